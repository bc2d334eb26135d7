// Replica-sync streaming kernels for MI355X (gfx950) and their C ABI.
//
// Every kernel here is HBM-bound elementwise work over a table of tensors.  The
// table is cut into chunks (a power-of-two number of elements of one tensor) and
// every chunk into slabs; one workgroup of 256 lanes (4 wavefronts of 64) owns
// exactly one slab: one, two or four 128-bit accesses per lane and per stream,
// i.e. 4-16 KiB per stream.  A workgroup finds its tensor with one scalar lookup
// (chunk_tensor[blockIdx >> shift]) followed by one round of scalar loads of
// that tensor's pointers.  Slabs are deliberately tiny and handed out by the
// hardware dispatcher in order: the set of workgroups in flight then covers a
// window of only a few MiB per stream, which keeps DRAM pages open across the
// 4-7 concurrent streams (measured on MI355X: 6.7 TB/s against 6.3 TB/s with
// 128 KiB per workgroup or a persistent grid-stride loop).  Nothing is reused,
// so accesses are non-temporal to keep L2 / Infinity Cache from being churned.
// No LDS, no MFMA: the arithmetic intensity is below 1 flop/byte.
//
// Entry points are declared and documented in include/torchft_amd.h.

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <string.h>

#include <mutex>

#include "torchft_amd.h"

namespace {

constexpr int kThreads = 256;
constexpr int kMaxCols = TFT_MAX_REPLICAS + 3;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

thread_local char g_err[512] = "";
#ifdef TFT_TUNING
thread_local uint32_t g_variant = 0;  // tuning builds only: overrides the launch shape
#endif

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// ---------------------------------------------------------------------------
// Element types: how a 16-byte vector is widened to fp32 lanes and back.
// ---------------------------------------------------------------------------
struct F32 {
  typedef float elem_t;
  typedef float acc_t;  // the type the arithmetic runs in
  static constexpr int kVec = 4;
  __device__ static inline void widen(const u32x4& raw, float (&v)[kVec]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __uint_as_float(raw[i]);
  }
  __device__ static inline u32x4 narrow(const float (&v)[kVec]) {
    u32x4 raw;
#pragma unroll
    for (int i = 0; i < 4; ++i) raw[i] = __float_as_uint(v[i]);
    return raw;
  }
  __device__ static inline float widen1(float x) { return x; }
  __device__ static inline float narrow1(float x) { return x; }
};

__device__ inline uint32_t f32_to_bf16_bits(float f) {
  // round to nearest even; NaN collapses to the canonical quiet NaN (what
  // c10::BFloat16's scalar conversion does on the host)
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

struct BF16 {
  typedef uint16_t elem_t;
  typedef float acc_t;
  static constexpr int kVec = 8;
  __device__ static inline void widen(const u32x4& raw, float (&v)[kVec]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(raw[i] << 16);
      v[2 * i + 1] = __uint_as_float(raw[i] & 0xffff0000u);
    }
  }
  // The vector body converts pairs with the hardware's round-to-nearest-even instruction
  // (v_cvt_pk_bf16_f32); the scalar path (narrow1) spells the same rounding with integer
  // arithmetic.  A NaN comes out as a quiet NaN either way; which one is unspecified (the
  // host's scalar conversion gives 0x7fc0, its vectorised one 0xffff).
  __device__ static inline u32x4 narrow(const float (&v)[kVec]) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    u32x4 raw;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const f32x2 pair = {v[2 * i], v[2 * i + 1]};
      raw[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2));
    }
    return raw;
  }
  __device__ static inline float widen1(uint16_t x) { return __uint_as_float((uint32_t)x << 16); }
  __device__ static inline uint16_t narrow1(float x) { return (uint16_t)f32_to_bf16_bits(x); }
};

struct F16 {
  typedef uint16_t elem_t;
  typedef float acc_t;
  static constexpr int kVec = 8;
  __device__ static inline float widen1(uint16_t x) { return __half2float(__ushort_as_half(x)); }
  __device__ static inline uint16_t narrow1(float x) {
    // The fp32 value is final before it is converted.  Without this barrier the
    // compiler folds a preceding fused multiply-add and the conversion into one
    // v_fma_mixlo_f16, which rounds the exact product-sum to fp16 directly and so
    // differs from "fp32 result, then round to nearest even" on (near-)ties.
    asm volatile("" : "+v"(x));
    return __half_as_ushort(__float2half_rn(x));
  }
  __device__ static inline void widen(const u32x4& raw, float (&v)[kVec]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = widen1((uint16_t)(raw[i] & 0xffffu));
      v[2 * i + 1] = widen1((uint16_t)(raw[i] >> 16));
    }
  }
  __device__ static inline u32x4 narrow(const float (&v)[kVec]) {
    u32x4 raw;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      raw[i] = (uint32_t)narrow1(v[2 * i]) | ((uint32_t)narrow1(v[2 * i + 1]) << 16);
    return raw;
  }
};

// fp64: two elements per 128-bit access, arithmetic in fp64 (only the replica
// average is instantiated for it: Manager.allreduce is dtype-generic in the
// reference, torchft/manager.py:267-287)
struct F64 {
  typedef double elem_t;
  typedef double acc_t;
  static constexpr int kVec = 2;
  __device__ static inline void widen(const u32x4& raw, double (&v)[kVec]) {
    v[0] = __hiloint2double((int)raw[1], (int)raw[0]);
    v[1] = __hiloint2double((int)raw[3], (int)raw[2]);
  }
  __device__ static inline u32x4 narrow(const double (&v)[kVec]) {
    u32x4 raw;
    raw[0] = (uint32_t)__double2loint(v[0]);
    raw[1] = (uint32_t)__double2hiint(v[0]);
    raw[2] = (uint32_t)__double2loint(v[1]);
    raw[3] = (uint32_t)__double2hiint(v[1]);
    return raw;
  }
  __device__ static inline double widen1(double x) { return x; }
  __device__ static inline double narrow1(double x) { return x; }
};

// round-to-nearest arithmetic the compiler may not contract or re-associate, by type
__device__ inline float add_rn(float a, float b) { return __fadd_rn(a, b); }
__device__ inline double add_rn(double a, double b) { return __dadd_rn(a, b); }
__device__ inline float mul_rn(float a, float b) { return __fmul_rn(a, b); }
__device__ inline double mul_rn(double a, double b) { return __dmul_rn(a, b); }
__device__ inline float div_rn(float a, float b) { return __fdiv_rn(a, b); }
__device__ inline double div_rn(double a, double b) { return __ddiv_rn(a, b); }

// Buffer instructions carry the cache policy of an access in their aux operand (bit 0 sc0,
// bit 1 nt, bit 4 sc1); the descriptor covers exactly the bytes a workgroup may touch, so
// the hardware also drops anything past their end.
constexpr int kBufferWord3 = 0x00020000;  // raw buffer, 32-bit data format
constexpr int kAuxNt = 2;                 // nt
constexpr int kAuxSc1 = 16;               // sc1
constexpr int kAuxNtSc1 = 18;             // nt | sc1

template <bool NT>
__device__ inline u32x4 load16(const void* p) {
  if (NT) return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return *reinterpret_cast<const u32x4*>(p);
}
template <bool NT>
__device__ inline void store16(void* p, const u32x4& v) {
  if (NT)
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
  else
    *reinterpret_cast<u32x4*>(p) = v;
}

// ---------------------------------------------------------------------------
// Locators: map a slab index to (column base pointers, element count).
// ---------------------------------------------------------------------------

// A launch of more than 2^31 work-items in one grid dimension is silently cut
// short by the runtime, so large slab counts are laid out as a 2-D grid with a
// bounded x extent (see grid_for); the dispatcher still hands workgroups out
// x-fastest, i.e. in workgroup-id order.
constexpr uint32_t kMaxGridX = 1u << 22;
constexpr uint32_t kMaxRunLog2 = 12;  // longest per-XCD run: 4096 slabs

// Workgroup id -> slab.  Ids go round-robin over the 8 XCDs; XCD x takes the
// x-th run of 2^run_log2 consecutive slabs out of every group of 8 runs.
__device__ inline uint32_t slab_index(uint32_t run_log2) {
  const uint32_t id = blockIdx.y * gridDim.x + blockIdx.x;
  const uint32_t xcd = id & 7u, j = id >> 3;
  const uint32_t within = j & ((1u << run_log2) - 1u), group = j >> run_log2;
  return (((group << 3) + xcd) << run_log2) + within;
}

struct TableArgs {
  void* const* ptrs;
  const uint64_t* numel;
  const uint32_t* chunk_start;
  const uint32_t* chunk_tensor;
  uint32_t n_tensors;
  uint32_t chunk_elems;
  uint32_t slab_shift;  // log2(slabs per chunk)
  uint32_t total_chunks;
  uint32_t run_log2;
};

struct FlatArgs {  // one tensor, pointers carried in the kernel arguments
  void* ptrs[kMaxCols];
  uint64_t numel;
  uint32_t run_log2;
};

// What one workgroup has to do: `n` elements starting at ptr, with 128-bit
// accesses if `vec`; the first slab of a misaligned tensor also has a head, the
// `head` elements starting at ptr - shift (the tensor's first elements, up to the
// 16-byte boundary or the tensor's end), done with scalar accesses.
struct SlabWork {
  uint32_t n;
  uint32_t head;
  uint32_t shift;  // elements from the tensor's base to the first aligned one
  bool vec;
};

// Shared by both locators: given the tensor's column base pointers, the slab's
// ordinal k inside the tensor and the tensor's size, computes the work and
// advances the active pointers to the first body element.
template <int NCOL>
__device__ inline SlabWork place_slab(char* (&ptr)[NCOL], uint32_t cols, uint64_t numel, uint64_t k,
                                      uint32_t slab_elems, uint32_t esize) {
  // common misalignment of the active columns (the shift keeps them aligned together)
  uint32_t mis = 0xffffffffu;
  bool same = true;
#pragma unroll
  for (int c = 0; c < NCOL; ++c) {
    if ((cols >> c) & 1u) {
      const uint32_t m = (uint32_t)(reinterpret_cast<uintptr_t>(ptr[c]) & 15u);
      if (mis == 0xffffffffu) mis = m;
      same = same && (m == mis);
    }
  }
  SlabWork w;
  w.vec = same && (mis % esize == 0);
  const uint32_t h = w.vec ? ((16u - mis) & 15u) / esize : 0u;  // elements up to the boundary
  const uint64_t begin = k * slab_elems + h;
  w.shift = h;
  w.head = (k == 0) ? (uint32_t)(numel < h ? numel : h) : 0u;
  w.n = 0;
  if (begin < numel) {
    const uint64_t left = numel - begin;
    w.n = left < slab_elems ? (uint32_t)left : slab_elems;
  }
#pragma unroll
  for (int c = 0; c < NCOL; ++c)
    ptr[c] = ((cols >> c) & 1u) ? ptr[c] + begin * esize : nullptr;
  return w;
}

template <int NCOL>
struct TableLocator {
  typedef TableArgs args_t;
  __device__ static inline SlabWork locate(const TableArgs& a, uint32_t slab_elems, uint32_t cols,
                                           char* (&ptr)[NCOL], uint32_t esize) {
    const uint32_t slab = slab_index(a.run_log2);
    const uint32_t chunk = slab >> a.slab_shift;
    if (chunk >= a.total_chunks) return SlabWork{0, 0, 0, false};  // padding of the grid
    const uint32_t sub = slab & ((1u << a.slab_shift) - 1u);
    const uint32_t t = a.chunk_tensor[chunk];
    const uint64_t numel = a.numel[t];
    const uint64_t k = ((uint64_t)(chunk - a.chunk_start[t]) << a.slab_shift) + sub;
#pragma unroll
    for (int c = 0; c < NCOL; ++c)
      ptr[c] = ((cols >> c) & 1u) ? static_cast<char*>(a.ptrs[(size_t)c * a.n_tensors + t]) : nullptr;
    return place_slab<NCOL>(ptr, cols, numel, k, slab_elems, esize);
  }
};

template <int NCOL>
struct FlatLocator {
  typedef FlatArgs args_t;
  __device__ static inline SlabWork locate(const FlatArgs& a, uint32_t slab_elems, uint32_t cols,
                                           char* (&ptr)[NCOL], uint32_t esize) {
    const uint64_t k = slab_index(a.run_log2);  // slabs past the end get n = 0 from place_slab
#pragma unroll
    for (int c = 0; c < NCOL; ++c) ptr[c] = ((cols >> c) & 1u) ? static_cast<char*>(a.ptrs[c]) : nullptr;
    return place_slab<NCOL>(ptr, cols, a.numel, k, slab_elems, esize);
  }
};

// ---------------------------------------------------------------------------
// The streaming skeleton.  Op supplies:
//   NCOL            number of pointer columns
//   rmask()/wmask() which columns are loaded / stored (uniform)
//   apply(v)        per-element arithmetic on v[NCOL] (fp32)
//   kHasFast, fast(), apply_fast(v)
//                   optionally, the same arithmetic for the common configuration with
//                   the uniform decisions (who participates, which SGD terms exist,
//                   whether the divisor is a power of two) taken once per workgroup
//                   instead of once per element; fast() is uniform and apply_fast
//                   returns bit for bit what apply returns whenever fast() holds
// ---------------------------------------------------------------------------
template <class E, class Op, int U, bool NT, bool CHECK, bool FAST = false>
__device__ inline void stream_block(char* const (&ptr)[Op::NCOL], const Op& op, uint32_t v0,
                                    uint32_t nvec, uint32_t rmask, uint32_t wmask) {
  constexpr int NCOL = Op::NCOL;
  constexpr int V = E::kVec;
  u32x4 raw[NCOL][U];
#pragma unroll
  for (int c = 0; c < NCOL; ++c) {
    if ((rmask >> c) & 1u) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t v = v0 + u * kThreads + threadIdx.x;
        if (!CHECK || v < nvec)
          raw[c][u] = load16<NT>(ptr[c] + (size_t)v * 16);
        else
          raw[c][u] = u32x4{0, 0, 0, 0};
      }
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) raw[c][u] = u32x4{0, 0, 0, 0};
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    typename E::acc_t lanes[NCOL][V];
#pragma unroll
    for (int c = 0; c < NCOL; ++c) E::widen(raw[c][u], lanes[c]);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      typename E::acc_t v[NCOL];
#pragma unroll
      for (int c = 0; c < NCOL; ++c) v[c] = lanes[c][i];
      if constexpr (FAST)
        op.apply_fast(v);
      else
        op.apply(v);
#pragma unroll
      for (int c = 0; c < NCOL; ++c) lanes[c][i] = v[c];
    }
#pragma unroll
    for (int c = 0; c < NCOL; ++c) raw[c][u] = E::narrow(lanes[c]);
  }
  // Stores of the kernels that write several streams (Op::kStoreSc1): sc1 WITHOUT nt.  Measured
  // on MI355X over all 81 pairs of load and store policies on the fused step, and per stream:
  // loads need nt on every stream (without it 0.76 instead of 0.79 of peak), and stores with sc1
  // alone beat non-temporal ones on every written stream (nt, nt|sc0, nt|sc1 and plain stores tie
  // among themselves).  In the library that is worth 0.5-1.5 % for the fused step, the outer SGD
  // and the LocalSGD average; the one-output replica average (three reads per write) is as fast
  // or faster with non-temporal stores and keeps them.
#pragma unroll
  for (int c = 0; c < NCOL; ++c) {
    if ((wmask >> c) & 1u) {
      if constexpr (NT && Op::kStoreSc1) {
        const __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(ptr[c], 0, nvec * 16, kBufferWord3);
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t v = v0 + u * kThreads + threadIdx.x;
          if (!CHECK || v < nvec) __builtin_amdgcn_raw_buffer_store_b128(raw[c][u], rd, v * 16, 0, kAuxSc1);
        }
      } else {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t v = v0 + u * kThreads + threadIdx.x;
          if (!CHECK || v < nvec) store16<NT>(ptr[c] + (size_t)v * 16, raw[c][u]);
        }
      }
    }
  }
}

template <class E, class Op>
__device__ inline void scalar_range(char* const (&ptr)[Op::NCOL], const Op& op, uint32_t begin,
                                    uint32_t end, uint32_t rmask, uint32_t wmask) {
  constexpr int NCOL = Op::NCOL;
  typedef typename E::elem_t T;
  for (uint32_t i = begin + threadIdx.x; i < end; i += kThreads) {
    typename E::acc_t v[NCOL];
#pragma unroll
    for (int c = 0; c < NCOL; ++c)
      v[c] = ((rmask >> c) & 1u) ? E::widen1(reinterpret_cast<const T*>(ptr[c])[i]) : 0;
    op.apply(v);
#pragma unroll
    for (int c = 0; c < NCOL; ++c)
      if ((wmask >> c) & 1u) reinterpret_cast<T*>(ptr[c])[i] = E::narrow1(v[c]);
  }
}

template <class E, class Op, class Loc, int U, bool NT>
__global__ __launch_bounds__(kThreads) void mt_stream_kernel(typename Loc::args_t args, Op op) {
  constexpr int NCOL = Op::NCOL;
  constexpr int V = E::kVec;
  constexpr uint32_t kSlab = kThreads * V * U;
  constexpr uint32_t kEsize = sizeof(typename E::elem_t);
  const uint32_t rmask = op.rmask();
  const uint32_t wmask = op.wmask();
  char* ptr[NCOL];
  const SlabWork w = Loc::locate(args, kSlab, rmask | wmask, ptr, kEsize);
  if (w.head) {  // first slab of a misaligned tensor: the elements before the boundary
    char* hp[NCOL];
#pragma unroll
    for (int c = 0; c < NCOL; ++c) hp[c] = ptr[c] ? ptr[c] - (size_t)w.shift * kEsize : nullptr;
    scalar_range<E, Op>(hp, op, 0, w.head, rmask, wmask);
  }
  if (w.n == 0) return;
  if (w.vec) {
    if (w.n == kSlab) {
      if constexpr (Op::kHasFast) {
        if (op.fast()) {
          stream_block<E, Op, U, NT, false, true>(ptr, op, 0, kSlab / V, rmask, wmask);
          return;
        }
      }
      stream_block<E, Op, U, NT, false>(ptr, op, 0, kSlab / V, rmask, wmask);
    } else {
      const uint32_t nvec = w.n / V;
      if (nvec) stream_block<E, Op, U, NT, true>(ptr, op, 0, nvec, rmask, wmask);
      if (nvec * V < w.n) scalar_range<E, Op>(ptr, op, nvec * V, w.n, rmask, wmask);
    }
  } else {
    scalar_range<E, Op>(ptr, op, 0, w.n, rmask, wmask);
  }
}

// ---------------------------------------------------------------------------
// Ops.  Division and the two-rounding momentum update are spelled with the
// round-to-nearest intrinsics so that the compiler cannot contract or
// re-associate them; the fused multiply-adds are the ones torch's own add(alpha)
// kernels perform.
// ---------------------------------------------------------------------------
// num_participants as the kernels see it.  Dividing by a power of two and multiplying by
// its (exact) reciprocal are the same real number rounded once, so the product replaces
// the IEEE division bit for bit: inv is that reciprocal, or 0 when n is no power of two.
struct Divisor {
  float n, inv;
  uint32_t count;  // the integer itself (fp64 arithmetic converts it exactly)
  __device__ inline float as(float) const { return n; }
  __device__ inline double as(double) const { return (double)count; }
  // the reciprocal is a power of two: exact in either type
  __device__ inline float inverse(float) const { return inv; }
  __device__ inline double inverse(double) const { return (double)inv; }
};

Divisor make_divisor(uint32_t num_participants) {
  const bool pow2 = num_participants && !(num_participants & (num_participants - 1u));
  return Divisor{(float)num_participants, pow2 ? 1.0f / (float)num_participants : 0.0f,
                 num_participants};
}

template <int NREP, class T>
__device__ inline T replica_sum(const T* x, uint32_t mask) {
  // sequential in replica order; a non-participant contributes +0
  T s = (mask & 1u) ? x[0] : T(0);
#pragma unroll
  for (int r = 1; r < NREP; ++r) s = add_rn(s, ((mask >> r) & 1u) ? x[r] : T(0));
  return s;
}

// columns: [out_0 .. out_{NOUT-1}, rep_0 .. rep_{NREP-1}]
template <int NOUT, int NREP>
struct ReduceAvgOp {
  static constexpr int NCOL = NOUT + NREP;
  static constexpr bool kHasFast = NREP > 0;
  static constexpr bool kStoreSc1 = NOUT > 1;
  uint32_t mask;  // participation bits
  Divisor d;      // num_participants
  __device__ inline uint32_t rmask() const { return mask << NOUT; }
  __device__ inline uint32_t wmask() const { return (1u << NOUT) - 1u; }
  template <class T>
  __device__ inline void apply(T (&v)[NCOL]) const {
    T s = T(0);
    if constexpr (NREP > 0) s = replica_sum<NREP, T>(&v[NOUT], mask);
    s = div_rn(s, d.as(T()));
#pragma unroll
    for (int o = 0; o < NOUT; ++o) v[o] = s;
  }
  // everybody participates and the divisor is a power of two
  __device__ inline bool fast() const { return mask == (1u << NREP) - 1u && d.inv != 0.0f; }
  template <class T>
  __device__ inline void apply_fast(T (&v)[NCOL]) const {
    T s = v[NOUT];
#pragma unroll
    for (int r = 1; r < NREP; ++r) s = add_rn(s, v[NOUT + r]);
    s = mul_rn(s, d.inverse(T()));
#pragma unroll
    for (int o = 0; o < NOUT; ++o) v[o] = s;
  }
};

struct SgdCoef {
  float neg_lr, momentum, one_minus_dampening, weight_decay;
  uint32_t nesterov, first_step;
};

__device__ inline float sgd_update(const SgdCoef& k, float g, float b, float& buf) {
  float d = g;
  if (k.weight_decay != 0.0f) d = __fmaf_rn(b, k.weight_decay, g);
  float e = d;
  if (k.momentum != 0.0f) {
    float nb = d;
    if (!k.first_step) nb = __fmaf_rn(d, k.one_minus_dampening, __fmul_rn(buf, k.momentum));
    buf = nb;
    e = k.nesterov ? __fmaf_rn(nb, k.momentum, d) : nb;
  }
  return __fmaf_rn(e, k.neg_lr, b);
}

// the usual outer optimizer: Nesterov momentum, no weight decay, not the first step
__device__ inline bool sgd_is_common(const SgdCoef& k) {
  return k.weight_decay == 0.0f && k.momentum != 0.0f && !k.first_step && k.nesterov;
}

__device__ inline float sgd_update_common(const SgdCoef& k, float g, float b, float& buf) {
  const float nb = __fmaf_rn(g, k.one_minus_dampening, __fmul_rn(buf, k.momentum));
  buf = nb;
  return __fmaf_rn(__fmaf_rn(nb, k.momentum, g), k.neg_lr, b);
}

// everybody participates and the divisor is a power of two
template <int NREP>
__device__ inline float pseudograd_avg_all(const float* x, float b, float inv) {
  float s = __fsub_rn(x[0], b);
#pragma unroll
  for (int r = 1; r < NREP; ++r) s = __fadd_rn(s, __fsub_rn(x[r], b));
  return __fmul_rn(s, inv);
}

template <int NREP>
__device__ inline float pseudograd_avg(const float* x, float b, uint32_t mask, float n) {
  // each replica subtracts the (shared) backup first, then the differences are summed
  float s = (mask & 1u) ? __fsub_rn(x[0], b) : 0.0f;
#pragma unroll
  for (int r = 1; r < NREP; ++r) s = __fadd_rn(s, ((mask >> r) & 1u) ? __fsub_rn(x[r], b) : 0.0f);
  return __fdiv_rn(s, n);
}

// columns: [p, b, buf, rep_0 ..]
template <int NREP>
struct DilocoFusedOp {
  static constexpr int NCOL = 3 + NREP;
  static constexpr bool kHasFast = NREP > 0;
  static constexpr bool kStoreSc1 = true;
  uint32_t mask;
  Divisor d;
  SgdCoef k;
  __device__ inline bool uses_buf() const { return k.momentum != 0.0f; }
  __device__ inline uint32_t rmask() const {
    return (mask << 3) | 2u | ((uses_buf() && !k.first_step) ? 4u : 0u);
  }
  __device__ inline uint32_t wmask() const { return 3u | (uses_buf() ? 4u : 0u); }
  __device__ inline void apply(float (&v)[NCOL]) const {
    const float g = pseudograd_avg<NREP>(&v[3], v[1], mask, d.n);
    const float p = sgd_update(k, g, v[1], v[2]);
    v[0] = p;
    v[1] = p;
  }
  __device__ inline bool fast() const {
    return mask == (1u << NREP) - 1u && d.inv != 0.0f && sgd_is_common(k);
  }
  __device__ inline void apply_fast(float (&v)[NCOL]) const {
    const float g = pseudograd_avg_all<NREP>(&v[3], v[1], d.inv);
    const float p = sgd_update_common(k, g, v[1], v[2]);
    v[0] = p;
    v[1] = p;
  }
};

// columns: [g, p, b, rep_0 ..]
template <int NREP>
struct PseudogradOp {
  static constexpr int NCOL = 3 + NREP;
  static constexpr bool kHasFast = NREP > 0;
  static constexpr bool kStoreSc1 = true;
  uint32_t mask;
  Divisor d;
  uint32_t restore_p;
  __device__ inline uint32_t rmask() const { return (mask << 3) | 4u; }
  __device__ inline uint32_t wmask() const { return 1u | (restore_p ? 2u : 0u); }
  __device__ inline void apply(float (&v)[NCOL]) const {
    v[0] = pseudograd_avg<NREP>(&v[3], v[2], mask, d.n);
    v[1] = v[2];
  }
  __device__ inline bool fast() const { return mask == (1u << NREP) - 1u && d.inv != 0.0f; }
  __device__ inline void apply_fast(float (&v)[NCOL]) const {
    v[0] = pseudograd_avg_all<NREP>(&v[3], v[2], d.inv);
    v[1] = v[2];
  }
};

// columns: [p, b, buf, g]
// With `divide` set, g holds the SUM of the replicas' pseudo-gradients as a collective left it
// and is divided by num_participants here, in registers, instead of by a pass of its own
// over the buffer.  The quotient is rounded to the storage type before it is used
// (`storage`: 0 fp32, 1 bf16, 2 fp16), as it would have been when that pass stored it.
struct OuterSgdOp {
  static constexpr int NCOL = 4;
  static constexpr bool kHasFast = true;
  static constexpr bool kStoreSc1 = true;
  SgdCoef k;
  Divisor d;
  uint32_t divide;
  uint32_t storage;
  __device__ inline bool uses_buf() const { return k.momentum != 0.0f; }
  __device__ inline uint32_t rmask() const {
    return 8u | 2u | ((uses_buf() && !k.first_step) ? 4u : 0u);
  }
  __device__ inline uint32_t wmask() const { return 3u | (uses_buf() ? 4u : 0u); }
  __device__ inline float grad(float g) const {
    if (!divide) return g;
    g = d.inv != 0.0f ? __fmul_rn(g, d.inv) : __fdiv_rn(g, d.n);
    if (storage == 1u) return BF16::widen1(BF16::narrow1(g));
    if (storage == 2u) return F16::widen1(F16::narrow1(g));
    return g;
  }
  __device__ inline void apply(float (&v)[NCOL]) const {
    const float p = sgd_update(k, grad(v[3]), v[1], v[2]);
    v[0] = p;
    v[1] = p;
  }
  __device__ inline bool fast() const { return sgd_is_common(k); }
  __device__ inline void apply_fast(float (&v)[NCOL]) const {
    const float p = sgd_update_common(k, grad(v[3]), v[1], v[2]);
    v[0] = p;
    v[1] = p;
  }
};

// columns: [a, scratch]; a is read and written back unchanged, scratch receives a
// copy (placement probe: one in-place stream next to one write stream).
// `key` is zero, but only at run time: storing back exactly what was loaded is
// something the compiler removes, and the probe exists to be timed.
struct ProbeOp {
  static constexpr int NCOL = 2;
  static constexpr bool kHasFast = false;
  static constexpr bool kStoreSc1 = false;  // the placement thresholds were measured with these stores
  uint32_t key;
  __device__ inline uint32_t rmask() const { return 1u; }
  __device__ inline uint32_t wmask() const { return 3u; }
  __device__ inline void apply(float (&v)[NCOL]) const {
    v[0] = __uint_as_float(__float_as_uint(v[0]) ^ key);
    v[1] = v[0];
  }
};

// ---------------------------------------------------------------------------
// Byte copy (gather / scatter).  columns: [dst, src]; numel counts bytes.
// ---------------------------------------------------------------------------
// Streaming stores of the copy go through buffer instructions so that they can carry
// the "nt sc1" policy (measured 2 % faster than plain non-temporal stores for a pure
// copy; for the mixed kernels the policies tie).  The descriptor covers exactly this
// workgroup's slab, so the hardware also drops anything past its end.

template <int U, bool NT>
__global__ __launch_bounds__(kThreads) void mt_copy_kernel(TableArgs args) {
  constexpr uint32_t kSlab = kThreads * 16 * U;  // bytes
  char* ptr[2];
  // esize 1: place_slab shifts the slabs to the common 16-byte boundary of dst and src
  const SlabWork w = TableLocator<2>::locate(args, kSlab, 3u, ptr, 1);
  char* dst = ptr[0];
  char* src = ptr[1];
  if (w.head) {
    for (uint32_t i = threadIdx.x; i < w.head; i += kThreads) (dst - w.shift)[i] = (src - w.shift)[i];
  }
  if (w.n == 0) return;
  const uint32_t n = w.n;
  uint32_t done = 0;
  if (w.vec) {
    const uint32_t nvec = n / 16;
    if (NT) {
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(src, 0, nvec * 16, kBufferWord3);
      const __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(dst, 0, nvec * 16, kBufferWord3);
      u32x4 raw[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t v = u * kThreads + threadIdx.x;
        if (v < nvec) raw[u] = __builtin_amdgcn_raw_buffer_load_b128(rs, v * 16, 0, kAuxNt);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t v = u * kThreads + threadIdx.x;
        if (v < nvec) __builtin_amdgcn_raw_buffer_store_b128(raw[u], rd, v * 16, 0, kAuxNtSc1);
      }
    } else {
      for (uint32_t v = threadIdx.x; v < nvec; v += kThreads)
        store16<false>(dst + (size_t)v * 16, load16<false>(src + (size_t)v * 16));
    }
    done = nvec * 16;
  } else {
    // dst and src are misaligned differently: widest access both sides allow
    const uintptr_t bits = reinterpret_cast<uintptr_t>(dst) ^ reinterpret_cast<uintptr_t>(src);
    if ((bits & 3u) == 0) {
      // bytes up to dst's 4-byte boundary, then words
      const uint32_t lead = (4u - (uint32_t)(reinterpret_cast<uintptr_t>(dst) & 3u)) & 3u;
      const uint32_t pre = lead < n ? lead : n;
      if (threadIdx.x < pre) dst[threadIdx.x] = src[threadIdx.x];
      const uint32_t nw = (n - pre) / 4;
      for (uint32_t i = threadIdx.x; i < nw; i += kThreads)
        reinterpret_cast<uint32_t*>(dst + pre)[i] = reinterpret_cast<const uint32_t*>(src + pre)[i];
      done = pre + nw * 4;
    }
  }
  for (uint32_t i = done + threadIdx.x; i < n; i += kThreads) dst[i] = src[i];
}

// ---------------------------------------------------------------------------
// Table built on the device, in a fixed array, for the allocation-free entry.
// ---------------------------------------------------------------------------
// Callers that cannot allocate device memory (code under graph capture, tight
// serving loops) cannot build a tensor table either.  For them the table lives in
// this file-scope array and is written by kernels whose arguments carry the
// entries, so the whole call is kernel launches on the caller's stream and
// nothing else.  Each GPU holds its own copy of the array at its own address.
constexpr size_t kScratchBytes = 8u << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr uint32_t kFillWords = 384;  // 64-bit entries carried by one fill launch (3 KiB)
struct FillArgs {
  uint64_t v[kFillWords];
  uint32_t n;
};

__global__ __launch_bounds__(kThreads) void table_fill_kernel(uint64_t* dst, FillArgs a) {
  for (uint32_t i = threadIdx.x; i < a.n; i += kThreads) dst[i] = a.v[i];
}

// chunk_tensor[c] = t for every chunk c of tensor t; one workgroup per tensor
__global__ __launch_bounds__(kThreads) void table_owner_kernel(const uint32_t* chunk_start,
                                                               uint32_t* chunk_tensor) {
  const uint32_t t = blockIdx.x;
  const uint32_t end = chunk_start[t + 1];
  for (uint32_t c = chunk_start[t] + threadIdx.x; c < end; c += kThreads) chunk_tensor[c] = t;
}

// ---------------------------------------------------------------------------
// Host side: validation, launch shape and dispatch.
// ---------------------------------------------------------------------------

// How a kernel is launched: 128-bit accesses per lane and stream (slab size in
// units of 4 KiB), per-XCD run length, unused dynamic LDS to cap residency.
struct Shape {
  int unroll;
  bool nt;
  uint32_t run_log2;
  uint32_t lds_bytes;
};

enum Family { kFamReduce, kFamDiloco, kFamPseudograd, kFamOuterSgd, kFamCopy };

// Tuned on MI355X with interleaved sweeps over (slab size, per-XCD run, residency cap) on
// the Llama-3-8B and GPT-2-small workloads.  `traffic` is the launch's algorithmic bytes.
// Launches that move less than a few GB finish in under a millisecond and are dominated by
// the ramp and tail of the in-flight window: short runs and 5 resident workgroups per CU
// (32 KiB of unused LDS each; 3 of 48 KiB for the fused step, whose workgroups hold seven
// to eleven streams in flight) are worth 5-10 % there.  Large launches still gain 1-5 % from
// runs of 128-256 slabs with 2-3 resident workgroups per CU; the plain copy only takes
// the runs.
Shape pick_shape(Family fam, uint64_t traffic, bool write_heavy = false) {
  const bool small = traffic < (16ull << 30);
  Shape s{2, true, 0, 0};
  if (fam == kFamCopy) {
    // 4 KiB slabs, no residency cap (a cap costs the copy 20-50 %); runs of 128 slabs per XCD
    // are worth 2.3 % over the Llama-3-8B tensor list (9.64 -> 9.41 ms for 64 GB moved; runs
    // of 64 and 256: 9.53 and 9.46 ms)
    s.unroll = 1;
    s.run_log2 = traffic < (256ull << 20) ? 0 : 7;
  } else if (small) {
    s.unroll = fam == kFamDiloco ? 1 : 2;
    s.run_log2 = fam == kFamDiloco ? 7 : 6;
    s.lds_bytes = (fam == kFamDiloco ? 48u : 32u) << 10;
  } else if (fam == kFamDiloco || fam == kFamOuterSgd) {
    s.run_log2 = 8;
    s.lds_bytes = 64u << 10;
  } else {
    s.run_log2 = 7;
    // more streams written than read (one summed buffer spread to parameters and backup):
    // measured 7 % faster with 24 KiB (6 workgroups per CU) than with the 48 KiB that suit
    // the other mixes (16.0 -> 14.3 ms over the Llama-3-8B parameters)
    s.lds_bytes = (write_heavy ? 24u : 48u) << 10;
  }
#ifdef TFT_TUNING
  // bits 0-3 unroll (1, 2, 4), bit 4 plain accesses, bits 8-11 run_log2 + 1,
  // bits 12-15 LDS bytes / 8 KiB + 1; a zero field keeps the default
  const uint32_t v = g_variant;
  if ((v & 0xfu) == 1 || (v & 0xfu) == 2 || (v & 0xfu) == 4) s.unroll = (int)(v & 0xfu);
  if (v & 0x10u) s.nt = false;
  if ((v >> 8) & 0xfu) s.run_log2 = ((v >> 8) & 0xfu) - 1;
  if ((v >> 12) & 0xfu) s.lds_bytes = (((v >> 12) & 0xfu) - 1) * 8192u;
#endif
  return s;
}

bool is_pow2(uint32_t x) { return x && !(x & (x - 1)); }

uint32_t log2u(uint32_t x) {
  uint32_t s = 0;
  while ((1u << s) < x) ++s;
  return s;
}

int check_chunk_elems(const char* what, uint32_t chunk_elems) {
  if (chunk_elems < TFT_MIN_CHUNK_ELEMS || !is_pow2(chunk_elems))
    return fail(TFT_ERR_INVALID_ARGUMENT, "%s: chunk_elems %u is not a power of two >= %u", what,
                chunk_elems, TFT_MIN_CHUNK_ELEMS);
  return TFT_OK;
}

// One workgroup per slab and slab indices are 32-bit, including the padding of the
// grid (up to one row of kMaxGridX and one group of 8 runs); the smallest slab any
// kernel uses is 1024 elements (4096 bytes for the copy kernel).
constexpr uint32_t kMaxSlabs = 0xffffffffu - 2u * kMaxGridX;
uint32_t max_chunks(uint32_t chunk_elems) { return kMaxSlabs / (chunk_elems / 1024u); }

// Grid for `slabs` workgroups, padded to whole groups of 8 runs (slab_index is a
// permutation of [0, padded)); kMaxGridX is a multiple of every group size.
dim3 grid_for(uint64_t slabs, uint32_t run_log2) {
  const uint64_t group = 8ull << run_log2;
  slabs = (slabs + group - 1) / group * group;
  const uint32_t x = (uint32_t)(slabs < kMaxGridX ? slabs : kMaxGridX);
  const uint32_t y = (uint32_t)((slabs + x - 1) / x);
  return dim3(x, y, 1);
}

// > 0: nothing to do; < 0: error
int check_table(const char* what, const tft_mt_table* t, uint32_t want_cols) {
  if (!t) return fail(TFT_ERR_INVALID_ARGUMENT, "%s: table is NULL", what);
  if (t->n_cols != want_cols)
    return fail(TFT_ERR_INVALID_ARGUMENT, "%s: table has %u columns, this call needs %u", what,
                t->n_cols, want_cols);
  if (int rc = check_chunk_elems(what, t->chunk_elems)) return rc;
  if (t->n_tensors == 0 || t->total_chunks == 0) return 1;
  if (!t->ptrs || !t->numel || !t->chunk_start || !t->chunk_tensor)
    return fail(TFT_ERR_INVALID_ARGUMENT, "%s: table arrays must not be NULL", what);
  if (t->total_chunks > max_chunks(t->chunk_elems))
    return fail(TFT_ERR_UNSUPPORTED, "%s: %u chunks do not fit one grid; raise chunk_elems", what,
                t->total_chunks);
  return TFT_OK;
}

int check_reduce(const char* what, uint32_t n_replicas, uint32_t mask, uint32_t num_participants) {
  if (n_replicas > TFT_MAX_REPLICAS)
    return fail(TFT_ERR_UNSUPPORTED, "%s: %u replicas, at most %d per launch", what, n_replicas,
                TFT_MAX_REPLICAS);
  if ((mask >> n_replicas) != 0)
    return fail(TFT_ERR_INVALID_ARGUMENT, "%s: participate_mask 0x%x names replicas >= %u", what,
                mask, n_replicas);
  if (num_participants == 0)
    return fail(TFT_ERR_INVALID_ARGUMENT, "%s: num_participants must be >= 1", what);
  return TFT_OK;
}

// fp64 exists for the replica average only (allow_f64)
int check_dtype(const char* what, int dtype, bool allow_f64 = false) {
  if (dtype == TFT_F64 && allow_f64) return TFT_OK;
  if (dtype == TFT_F64)
    return fail(TFT_ERR_UNSUPPORTED, "%s: fp64 is supported by the replica average only", what);
  if (dtype != TFT_F32 && dtype != TFT_BF16 && dtype != TFT_F16)
    return fail(TFT_ERR_UNSUPPORTED, "%s: dtype %d", what, dtype);
  return TFT_OK;
}

uint32_t popcount(uint32_t x) { return (uint32_t)__builtin_popcount(x); }

// The launch itself; the return code of hipLaunchKernel is this launch's own
// (the sticky "last error" may belong to somebody else's earlier call).
template <class Args, class Op>
int launch_kernel(const char* what, const void* kernel, dim3 grid, uint32_t lds, hipStream_t stream,
                  Args& a, Op& op) {
  void* params[] = {&a, &op};
  const hipError_t e = hipLaunchKernel(kernel, grid, dim3(kThreads), params, lds, stream);
  if (e != hipSuccess) return fail(TFT_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
  return TFT_OK;
}

// slab_elems always divides chunk_elems: both are powers of two and
// chunk_elems >= TFT_MIN_CHUNK_ELEMS >= the largest slab (256 lanes * 8 bf16 * 4;
// 256 lanes * 16 bytes * 4 for the byte copy, whose minimum is checked there).
TableArgs table_args(const tft_mt_table* t, uint32_t slab_elems, const Shape& shape, dim3* grid) {
  const uint32_t shift = log2u(t->chunk_elems / slab_elems);
  *grid = grid_for((uint64_t)t->total_chunks << shift, shape.run_log2);
  return TableArgs{static_cast<void* const*>(t->ptrs), t->numel, t->chunk_start, t->chunk_tensor,
                   t->n_tensors, t->chunk_elems, shift, t->total_chunks, shape.run_log2};
}

template <class E, class Op, int U, bool NT>
int launch_table(const char* what, const tft_mt_table* t, const Op& op, const Shape& shape,
                 hipStream_t stream) {
  dim3 grid;
  TableArgs a = table_args(t, kThreads * E::kVec * U, shape, &grid);
  Op o = op;
  return launch_kernel(what, reinterpret_cast<const void*>(
                                 &mt_stream_kernel<E, Op, TableLocator<Op::NCOL>, U, NT>),
                       grid, shape.lds_bytes, stream, a, o);
}

template <class E, class Op, int U, bool NT>
int launch_flat(const char* what, const FlatArgs& args, const Op& op, const Shape& shape,
                hipStream_t stream) {
  const uint64_t slab = (uint64_t)kThreads * E::kVec * U;
  FlatArgs a = args;
  a.run_log2 = shape.run_log2;
  // one extra slab: a misaligned buffer's body is shifted by up to 15 bytes
  const dim3 grid = grid_for((a.numel + slab - 1) / slab + 1, shape.run_log2);
  Op o = op;
  return launch_kernel(what, reinterpret_cast<const void*>(
                                 &mt_stream_kernel<E, Op, FlatLocator<Op::NCOL>, U, NT>),
                       grid, shape.lds_bytes, stream, a, o);
}

// rc = LAUNCHER<E, OP, U, NT>(what, ARGS, op, shape, stream) for the shape's unroll
// (plain instead of non-temporal accesses exist in tuning builds only).
#ifdef TFT_TUNING
#define TFT_DISPATCH_NT(LAUNCHER, E, OP, UU, what, ARGS, op, shape, stream)       \
  ((shape).nt ? LAUNCHER<E, OP, UU, true>(what, ARGS, op, shape, stream)          \
              : LAUNCHER<E, OP, UU, false>(what, ARGS, op, shape, stream))
#else
#define TFT_DISPATCH_NT(LAUNCHER, E, OP, UU, what, ARGS, op, shape, stream) \
  LAUNCHER<E, OP, UU, true>(what, ARGS, op, shape, stream)
#endif
// pick_shape only ever chooses 1 or 2; the 4-wide form exists in tuning builds
#ifdef TFT_TUNING
#define TFT_DISPATCH_U4(rc, LAUNCHER, E, OP, what, ARGS, op, shape, stream) \
  if ((shape).unroll == 4) rc = TFT_DISPATCH_NT(LAUNCHER, E, OP, 4, what, ARGS, op, shape, stream); else
#else
#define TFT_DISPATCH_U4(rc, LAUNCHER, E, OP, what, ARGS, op, shape, stream)
#endif
#define TFT_DISPATCH_U(rc, LAUNCHER, E, OP, what, ARGS, op, shape, stream)                          \
  do {                                                                                              \
    TFT_DISPATCH_U4(rc, LAUNCHER, E, OP, what, ARGS, op, shape, stream)                             \
    if ((shape).unroll == 2) rc = TFT_DISPATCH_NT(LAUNCHER, E, OP, 2, what, ARGS, op, shape, stream); \
    else rc = TFT_DISPATCH_NT(LAUNCHER, E, OP, 1, what, ARGS, op, shape, stream);                   \
  } while (0)
#define TFT_DISPATCH_DTYPE(rc, LAUNCHER, OP, dtype, what, ARGS, op, shape, stream)            \
  do {                                                                                        \
    if ((dtype) == TFT_F32) TFT_DISPATCH_U(rc, LAUNCHER, F32, OP, what, ARGS, op, shape, stream);        \
    else if ((dtype) == TFT_BF16) TFT_DISPATCH_U(rc, LAUNCHER, BF16, OP, what, ARGS, op, shape, stream); \
    else TFT_DISPATCH_U(rc, LAUNCHER, F16, OP, what, ARGS, op, shape, stream);                           \
  } while (0)

// The replica average also exists for fp64.
#define TFT_DISPATCH_DTYPE_F64(rc, LAUNCHER, OP, dtype, what, ARGS, op, shape, stream)           \
  do {                                                                                          \
    if ((dtype) == TFT_F64) TFT_DISPATCH_U(rc, LAUNCHER, F64, OP, what, ARGS, op, shape, stream); \
    else TFT_DISPATCH_DTYPE(rc, LAUNCHER, OP, dtype, what, ARGS, op, shape, stream);            \
  } while (0)

// Expands `CALL(N)` for the run-time replica count.
#define TFT_FOR_NREP(n, CALL) \
  switch (n) {                \
    case 0: CALL(0); break;   \
    case 1: CALL(1); break;   \
    case 2: CALL(2); break;   \
    case 3: CALL(3); break;   \
    case 4: CALL(4); break;   \
    case 5: CALL(5); break;   \
    case 6: CALL(6); break;   \
    case 7: CALL(7); break;   \
    default: CALL(8); break;  \
  }

SgdCoef make_coef(const tft_sgd_params* s) {
  SgdCoef k;
  k.neg_lr = -s->lr;
  k.momentum = s->momentum;
  k.one_minus_dampening = (float)(1.0 - (double)s->dampening);
  k.weight_decay = s->weight_decay;
  k.nesterov = s->nesterov ? 1u : 0u;
  k.first_step = s->first_step ? 1u : 0u;
  return k;
}

int check_sgd(const char* what, const tft_sgd_params* s) {
  if (!s) return fail(TFT_ERR_INVALID_ARGUMENT, "%s: sgd params are NULL", what);
  if (s->nesterov && (s->momentum <= 0.0f || s->dampening != 0.0f))
    return fail(TFT_ERR_INVALID_ARGUMENT,
                "%s: nesterov needs momentum > 0 and dampening == 0 (got %g, %g)", what,
                (double)s->momentum, (double)s->dampening);
  return TFT_OK;
}

uint64_t esize_of(int dtype) { return dtype == TFT_F64 ? 8 : dtype == TFT_F32 ? 4 : 2; }

// elements a table covers, rounded up to whole chunks (the host does not read the
// device-resident sizes); only used to choose the launch shape
uint64_t table_elems(const tft_mt_table* t) { return (uint64_t)t->total_chunks * t->chunk_elems; }

int diloco_outer(const char* what, const tft_mt_table* table, uint32_t n_replicas,
                 uint32_t participate_mask, uint32_t num_participants, int dtype,
                 const tft_sgd_params* sgd, void* stream) {
  const SgdCoef k = make_coef(sgd);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint32_t streams = popcount(participate_mask) + 2 + (k.momentum != 0.0f ? (k.first_step ? 1 : 2) : 0);
  const Shape shape = pick_shape(kFamDiloco, table_elems(table) * esize_of(dtype) * streams);
  int rc = TFT_OK;
#define TFT_CALL(N)                                                                     \
  do {                                                                                  \
    typedef DilocoFusedOp<N> Op;                                                        \
    const Op op{participate_mask, make_divisor(num_participants), k};                   \
    TFT_DISPATCH_DTYPE(rc, launch_table, Op, dtype, what, table, op, shape, s);         \
  } while (0)
  TFT_FOR_NREP(n_replicas, TFT_CALL)
#undef TFT_CALL
  return rc;
}


// Per-device address of `scratch` (the symbol's name is only a host-side handle).
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

int scratch_address(const char* what, void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(TFT_ERR_LAUNCH, "%s: hipGetDevice: %s", what, hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(TFT_ERR_UNSUPPORTED, "%s: device ordinal %d outside [0, %d)", what, dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return fail(TFT_ERR_LAUNCH, "%s: hipGetSymbolAddress(scratch) on device %d: %s", what, dev,
                  hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return TFT_OK;
}

// Writes `n` 64-bit entries to `dst` (device) with fill launches of kFillWords each.
int fill_words(const char* what, uint64_t* dst, const uint64_t* src, size_t n, hipStream_t stream) {
  for (size_t done = 0; done < n; done += kFillWords) {
    FillArgs a;
    a.n = (uint32_t)(n - done < kFillWords ? n - done : kFillWords);
    memcpy(a.v, src + done, a.n * sizeof(uint64_t));
    uint64_t* d = dst + done;
    void* params[] = {&d, &a};
    const hipError_t e = hipLaunchKernel(reinterpret_cast<const void*>(&table_fill_kernel), dim3(1),
                                         dim3(kThreads), params, 0, stream);
    if (e != hipSuccess)
      return fail(TFT_ERR_LAUNCH, "%s: table fill launch failed: %s", what, hipGetErrorString(e));
  }
  return TFT_OK;
}

size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

}  // namespace

extern "C" {

int tft_abi_version(void) { return TFT_ABI_VERSION; }

const char* tft_last_error(void) { return g_err; }

#ifdef TFT_TUNING
void tft_set_launch_variant(uint32_t variant) { g_variant = variant; }
#endif

uint32_t tft_default_chunk_elems(int dtype) {
  if (dtype < 0) return 256u * 1024u;  // bytes per copy chunk
  return 64u * 1024u;
}

int64_t tft_mt_plan(const uint64_t* numel, uint32_t n_tensors, uint32_t chunk_elems,
                    uint32_t* chunk_start, uint32_t* chunk_tensor) {
  static const char* what = "tft_mt_plan";
  if (n_tensors && !numel) return fail(TFT_ERR_INVALID_ARGUMENT, "%s: numel is NULL", what);
  if (!chunk_start) return fail(TFT_ERR_INVALID_ARGUMENT, "%s: chunk_start is NULL", what);
  if (int rc = check_chunk_elems(what, chunk_elems)) return rc;
  uint64_t total = 0;
  for (uint32_t t = 0; t < n_tensors; ++t) {
    chunk_start[t] = (uint32_t)total;
    const uint64_t chunks = numel[t] / chunk_elems + (numel[t] % chunk_elems ? 1 : 0);
    if (total + chunks > max_chunks(chunk_elems))
      return fail(TFT_ERR_UNSUPPORTED, "%s: too many chunks for one grid; raise chunk_elems", what);
    if (chunk_tensor)
      for (uint64_t c = 0; c < chunks; ++c) chunk_tensor[total + c] = t;
    total += chunks;
  }
  chunk_start[n_tensors] = (uint32_t)total;
  return (int64_t)total;
}

int tft_reduce_avg(void* out, const void* const* replicas, uint32_t n_replicas,
                   uint32_t participate_mask, uint32_t num_participants, uint64_t numel,
                   int dtype, void* stream) {
  static const char* what = "tft_reduce_avg";
  if (int rc = check_reduce(what, n_replicas, participate_mask, num_participants)) return rc;
  if (int rc = check_dtype(what, dtype, true)) return rc;
  if (numel == 0) return TFT_OK;
  if (!out) return fail(TFT_ERR_INVALID_ARGUMENT, "%s: out is NULL", what);
  if (n_replicas && !replicas) return fail(TFT_ERR_INVALID_ARGUMENT, "%s: replicas is NULL", what);
  if (numel > (1ull << 41)) return fail(TFT_ERR_UNSUPPORTED, "%s: numel too large", what);
  FlatArgs a{};
  a.ptrs[0] = out;
  for (uint32_t r = 0; r < n_replicas; ++r) {
    if (((participate_mask >> r) & 1u) && !replicas[r])
      return fail(TFT_ERR_INVALID_ARGUMENT, "%s: replica %u is NULL", what, r);
    a.ptrs[1 + r] = const_cast<void*>(replicas[r]);
  }
  a.numel = numel;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const Shape shape =
      pick_shape(kFamReduce, numel * esize_of(dtype) * (popcount(participate_mask) + 1));
  int rc = TFT_OK;
#define TFT_CALL(N)                                                             \
  do {                                                                          \
    typedef ReduceAvgOp<1, N> Op;                                               \
    const Op op{participate_mask, make_divisor(num_participants)};              \
    TFT_DISPATCH_DTYPE_F64(rc, launch_flat, Op, dtype, what, a, op, shape, s);  \
  } while (0)
  TFT_FOR_NREP(n_replicas, TFT_CALL)
#undef TFT_CALL
  return rc;
}

int tft_mt_reduce_avg(const tft_mt_table* table, uint32_t n_outs, uint32_t n_replicas,
                      uint32_t participate_mask, uint32_t num_participants, int dtype,
                      void* stream) {
  static const char* what = "tft_mt_reduce_avg";
  if (n_outs != 1 && n_outs != 2)
    return fail(TFT_ERR_INVALID_ARGUMENT, "%s: n_outs must be 1 or 2, got %u", what, n_outs);
  if (int rc = check_reduce(what, n_replicas, participate_mask, num_participants)) return rc;
  if (int rc = check_dtype(what, dtype, true)) return rc;
  if (int rc = check_table(what, table, n_outs + n_replicas)) return rc < 0 ? rc : TFT_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const Shape shape = pick_shape(
      kFamReduce, table_elems(table) * esize_of(dtype) * (popcount(participate_mask) + n_outs),
      n_outs > popcount(participate_mask));
  int rc = TFT_OK;
#define TFT_CALL2(O, N)                                                               \
  do {                                                                                \
    typedef ReduceAvgOp<O, N> Op;                                                     \
    const Op op{participate_mask, make_divisor(num_participants)};                    \
    TFT_DISPATCH_DTYPE_F64(rc, launch_table, Op, dtype, what, table, op, shape, s);   \
  } while (0)
#define TFT_CALL_O1(N) TFT_CALL2(1, N)
#define TFT_CALL_O2(N) TFT_CALL2(2, N)
  if (n_outs == 1) {
    TFT_FOR_NREP(n_replicas, TFT_CALL_O1)
  } else {
    TFT_FOR_NREP(n_replicas, TFT_CALL_O2)
  }
#undef TFT_CALL_O1
#undef TFT_CALL_O2
#undef TFT_CALL2
  return rc;
}

int tft_mt_diloco_outer(const tft_mt_table* table, uint32_t n_replicas, uint32_t participate_mask,
                        uint32_t num_participants, int dtype, const tft_sgd_params* sgd,
                        void* stream) {
  static const char* what = "tft_mt_diloco_outer";
  if (int rc = check_reduce(what, n_replicas, participate_mask, num_participants)) return rc;
  if (int rc = check_dtype(what, dtype)) return rc;
  if (int rc = check_sgd(what, sgd)) return rc;
  if (int rc = check_table(what, table, 3 + n_replicas)) return rc < 0 ? rc : TFT_OK;
  return diloco_outer(what, table, n_replicas, participate_mask, num_participants, dtype, sgd, stream);
}

int tft_mt_pseudograd_avg(const tft_mt_table* table, uint32_t n_replicas,
                          uint32_t participate_mask, uint32_t num_participants, int dtype,
                          int restore_p, void* stream) {
  static const char* what = "tft_mt_pseudograd_avg";
  if (int rc = check_reduce(what, n_replicas, participate_mask, num_participants)) return rc;
  if (int rc = check_dtype(what, dtype)) return rc;
  if (int rc = check_table(what, table, 3 + n_replicas)) return rc < 0 ? rc : TFT_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const Shape shape = pick_shape(
      kFamPseudograd,
      table_elems(table) * esize_of(dtype) * (popcount(participate_mask) + 2 + (restore_p ? 1 : 0)));
  int rc = TFT_OK;
#define TFT_CALL(N)                                                                   \
  do {                                                                                \
    typedef PseudogradOp<N> Op;                                                       \
    const Op op{participate_mask, make_divisor(num_participants), restore_p ? 1u : 0u}; \
    TFT_DISPATCH_DTYPE(rc, launch_table, Op, dtype, what, table, op, shape, s);       \
  } while (0)
  TFT_FOR_NREP(n_replicas, TFT_CALL)
#undef TFT_CALL
  return rc;
}

// grad_divisor 0: g is the averaged pseudo-gradient; otherwise g is a sum still to be divided
static int outer_sgd(const char* what, const tft_mt_table* table, uint32_t grad_divisor, int dtype,
                     const tft_sgd_params* sgd, void* stream) {
  if (int rc = check_dtype(what, dtype)) return rc;
  if (int rc = check_sgd(what, sgd)) return rc;
  if (int rc = check_table(what, table, 4)) return rc < 0 ? rc : TFT_OK;
  const uint32_t storage = dtype == TFT_BF16 ? 1u : dtype == TFT_F16 ? 2u : 0u;
  const OuterSgdOp op{make_coef(sgd), make_divisor(grad_divisor ? grad_divisor : 1u),
                      grad_divisor ? 1u : 0u, storage};
  hipStream_t s = static_cast<hipStream_t>(stream);
  const Shape shape = pick_shape(kFamOuterSgd, table_elems(table) * esize_of(dtype) * 6);
  int rc = TFT_OK;
  TFT_DISPATCH_DTYPE(rc, launch_table, OuterSgdOp, dtype, what, table, op, shape, s);
  return rc;
}

int tft_mt_outer_sgd(const tft_mt_table* table, int dtype, const tft_sgd_params* sgd,
                     void* stream) {
  return outer_sgd("tft_mt_outer_sgd", table, 0, dtype, sgd, stream);
}

int tft_mt_outer_sgd_of_sum(const tft_mt_table* table, uint32_t num_participants, int dtype,
                            const tft_sgd_params* sgd, void* stream) {
  static const char* what = "tft_mt_outer_sgd_of_sum";
  if (num_participants == 0)
    return fail(TFT_ERR_INVALID_ARGUMENT, "%s: num_participants must be at least 1", what);
  return outer_sgd(what, table, num_participants, dtype, sgd, stream);
}

int tft_mt_diloco_outer_noalloc(const void* const* ptrs, const uint64_t* numel, uint32_t n_tensors,
                                uint32_t n_replicas, uint32_t participate_mask,
                                uint32_t num_participants, int dtype, const tft_sgd_params* sgd,
                                void* stream) {
  static const char* what = "tft_mt_diloco_outer_noalloc";
  if (int rc = check_reduce(what, n_replicas, participate_mask, num_participants)) return rc;
  if (int rc = check_dtype(what, dtype)) return rc;
  if (int rc = check_sgd(what, sgd)) return rc;
  if (n_tensors == 0) return TFT_OK;
  if (!ptrs || !numel) return fail(TFT_ERR_INVALID_ARGUMENT, "%s: ptrs / numel are NULL", what);
  if (n_tensors > TFT_NOALLOC_MAX_TENSORS)
    return fail(TFT_ERR_UNSUPPORTED, "%s: %u tensors, at most %u fit the built-in table", what,
                n_tensors, (unsigned)TFT_NOALLOC_MAX_TENSORS);
  const uint32_t n_cols = 3 + n_replicas;
  const bool uses_buf = sgd->momentum != 0.0f;
  for (uint32_t t = 0; t < n_tensors; ++t) {
    if (numel[t] == 0)
      return fail(TFT_ERR_INVALID_ARGUMENT, "%s: tensor %u is empty; drop empty tensors", what, t);
    for (uint32_t c = 0; c < n_cols; ++c) {
      const bool used = c < 2 || (c == 2 && uses_buf) || (c >= 3 && ((participate_mask >> (c - 3)) & 1u));
      if (used && !ptrs[(size_t)c * n_tensors + t])
        return fail(TFT_ERR_INVALID_ARGUMENT, "%s: column %u of tensor %u is NULL", what, c, t);
    }
  }
  // host-side plan (stack / heap of the host only; nothing on the device is allocated)
  const uint32_t chunk_elems = tft_default_chunk_elems(dtype);
  uint32_t chunk_start[TFT_NOALLOC_MAX_TENSORS + 2] = {};
  const int64_t total = tft_mt_plan(numel, n_tensors, chunk_elems, chunk_start, nullptr);
  if (total < 0) return (int)total;
  const size_t off_numel = align_up((size_t)n_cols * n_tensors * 8, 256);
  const size_t off_start = align_up(off_numel + (size_t)n_tensors * 8, 256);
  const size_t off_owner = align_up(off_start + (size_t)(n_tensors + 2) * 4, 256);
  const size_t need = off_owner + (size_t)total * 4;
  if (need > kScratchBytes)
    return fail(TFT_ERR_UNSUPPORTED,
                "%s: the table needs %zu bytes (%lld chunks of %u elements), the built-in array holds %zu",
                what, need, (long long)total, chunk_elems, kScratchBytes);
  void* base_v = nullptr;
  if (int rc = scratch_address(what, &base_v)) return rc;
  unsigned char* base = static_cast<unsigned char*>(base_v);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (int rc = fill_words(what, reinterpret_cast<uint64_t*>(base),
                          reinterpret_cast<const uint64_t*>(ptrs), (size_t)n_cols * n_tensors, s))
    return rc;
  if (int rc = fill_words(what, reinterpret_cast<uint64_t*>(base + off_numel), numel, n_tensors, s))
    return rc;
  // (n_tensors + 1) 32-bit entries travel as 64-bit words; the array has one spare slot
  if (int rc = fill_words(what, reinterpret_cast<uint64_t*>(base + off_start),
                          reinterpret_cast<const uint64_t*>(chunk_start), (n_tensors + 2) / 2, s))
    return rc;
  {
    const uint32_t* cs = reinterpret_cast<const uint32_t*>(base + off_start);
    uint32_t* owner = reinterpret_cast<uint32_t*>(base + off_owner);
    void* params[] = {&cs, &owner};
    const hipError_t e = hipLaunchKernel(reinterpret_cast<const void*>(&table_owner_kernel),
                                         dim3(n_tensors), dim3(kThreads), params, 0, s);
    if (e != hipSuccess)
      return fail(TFT_ERR_LAUNCH, "%s: table owner launch failed: %s", what, hipGetErrorString(e));
  }
  tft_mt_table table;
  table.ptrs = base;
  table.numel = reinterpret_cast<const uint64_t*>(base + off_numel);
  table.chunk_start = reinterpret_cast<const uint32_t*>(base + off_start);
  table.chunk_tensor = reinterpret_cast<const uint32_t*>(base + off_owner);
  table.n_tensors = n_tensors;
  table.n_cols = n_cols;
  table.chunk_elems = chunk_elems;
  table.total_chunks = (uint32_t)total;
  return diloco_outer(what, &table, n_replicas, participate_mask, num_participants, dtype, sgd, stream);
}

int tft_probe_rw_pair(void* a, void* scratch, uint64_t bytes, void* stream) {
  static const char* what = "tft_probe_rw_pair";
  if (bytes == 0) return TFT_OK;
  if (!a || !scratch) return fail(TFT_ERR_INVALID_ARGUMENT, "%s: buffers must not be NULL", what);
  if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(scratch) | bytes) & 15u)
    return fail(TFT_ERR_INVALID_ARGUMENT, "%s: buffers and size must be multiples of 16 bytes", what);
  if (bytes > (1ull << 40)) return fail(TFT_ERR_UNSUPPORTED, "%s: size too large", what);
  FlatArgs args{};
  args.ptrs[0] = a;
  args.ptrs[1] = scratch;
  args.numel = bytes / 4;
  const Shape shape{2, true, 0, 0};
  const ProbeOp op{0u};
  return launch_flat<F32, ProbeOp, 2, true>(what, args, op, shape, static_cast<hipStream_t>(stream));
}

int tft_mt_copy_bytes(const tft_mt_table* table, void* stream) {
  static const char* what = "tft_mt_copy_bytes";
  if (int rc = check_table(what, table, 2)) return rc < 0 ? rc : TFT_OK;
  if (table->chunk_elems < kThreads * 16 * 4)
    return fail(TFT_ERR_INVALID_ARGUMENT, "%s: chunk_elems %u bytes is below %d", what,
                table->chunk_elems, kThreads * 16 * 4);
  const Shape shape = pick_shape(kFamCopy, table_elems(table) * 2);
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid;
  int rc = TFT_OK;
#define TFT_COPY(UU, NTT)                                                                      \
  do {                                                                                         \
    TableArgs a = table_args(table, kThreads * 16 * UU, shape, &grid);                         \
    void* params[] = {&a};                                                                     \
    const hipError_t e = hipLaunchKernel(reinterpret_cast<const void*>(&mt_copy_kernel<UU, NTT>), \
                                         grid, dim3(kThreads), params, shape.lds_bytes, s);    \
    if (e != hipSuccess) rc = fail(TFT_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e)); \
  } while (0)
#ifdef TFT_TUNING
  if (!shape.nt) {
    if (shape.unroll == 4) TFT_COPY(4, false);
    else if (shape.unroll == 2) TFT_COPY(2, false);
    else TFT_COPY(1, false);
    return rc;
  }
#endif
#ifdef TFT_TUNING
  if (shape.unroll == 4) TFT_COPY(4, true);
  else if (shape.unroll == 2) TFT_COPY(2, true);
  else
#endif
    TFT_COPY(1, true);
#undef TFT_COPY
  return rc;
}

}  // extern "C"
