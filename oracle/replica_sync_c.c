/*
 * TEST INFRASTRUCTURE - not part of the product.
 *
 * Plain-C restatement of the arithmetic of torchft's replica-sync path, one
 * element at a time, for checking the HIP kernels.  Only tests/, the smoke
 * check and the benchmark's cpu_baseline leg may load this file's library.
 *
 * The reference has no C code: the arithmetic below is what its Python loops
 * ask stock torch CPU kernels to do.  Each function cites the reference lines
 * it follows.  Build with -ffp-contract=off so that only the fmaf() calls
 * written here fuse (torch's add(alpha=...) CPU kernel fuses exactly there).
 *
 * Pinned by tests/test_oracle.py: against torch.optim.SGD (library routine),
 * closed forms, float64 brute force, and the reference's own known answers
 * (torchft/manager_test.py:520-543, torchft/process_group_test.py:185-203).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* torchft/manager.py:267-268 (zero when not participating), :274 (allreduce
 * SUM across replicas, taken here in replica order), :287 (tensor /= n). */
void oracle_reduce_avg_f32(float* out, const float* const* replicas, uint32_t n_replicas,
                           uint32_t participate_mask, uint32_t num_participants, uint64_t numel) {
  for (uint64_t i = 0; i < numel; ++i) {
    float s = 0.0f;
    for (uint32_t r = 0; r < n_replicas; ++r) {
      const float x = ((participate_mask >> r) & 1u) ? replicas[r][i] : 0.0f;
      s = r == 0 ? x : s + x;
    }
    out[i] = s / (float)num_participants;
  }
}

/* Same, bf16 storage with fp32 accumulation and one rounding on store. */
void oracle_reduce_avg_bf16(uint16_t* out, const uint16_t* const* replicas, uint32_t n_replicas,
                            uint32_t participate_mask, uint32_t num_participants,
                            uint64_t numel) {
  for (uint64_t i = 0; i < numel; ++i) {
    float s = 0.0f;
    for (uint32_t r = 0; r < n_replicas; ++r) {
      const float x = ((participate_mask >> r) & 1u) ? bf16_to_f32(replicas[r][i]) : 0.0f;
      s = r == 0 ? x : s + x;
    }
    out[i] = f32_to_bf16(s / (float)num_participants);
  }
}

typedef struct oracle_sgd {
  float lr, momentum, dampening, weight_decay;
  int32_t nesterov, first_step;
} oracle_sgd;

/* torch.optim.SGD single-tensor update as driven from torchft/local_sgd.py:223:
 * grad (+ wd * param); buf = grad on the first step, else buf*mu then
 * + (1-damp)*grad; nesterov: grad + mu*buf; param += -lr * grad. */
static float sgd_update(const oracle_sgd* k, float g, float p, float* buf) {
  float d = g;
  if (k->weight_decay != 0.0f) d = fmaf(p, k->weight_decay, g);
  float e = d;
  if (k->momentum != 0.0f) {
    float nb = d;
    if (!k->first_step) {
      const float scaled = *buf * k->momentum;
      nb = fmaf(d, (float)(1.0 - (double)k->dampening), scaled);
    }
    *buf = nb;
    e = k->nesterov ? fmaf(nb, k->momentum, d) : nb;
  }
  return fmaf(e, -k->lr, p);
}

/* torchft/local_sgd.py:212-215 (g_r = p_r - backup, per replica), :227-239 with
 * manager.py:267-287 (sum over replicas, / n). */
static float pseudograd_avg(const float* const* replicas, uint32_t n_replicas, uint32_t mask,
                            uint32_t num_participants, float b, uint64_t i) {
  float s = 0.0f;
  for (uint32_t r = 0; r < n_replicas; ++r) {
    const float x = ((mask >> r) & 1u) ? replicas[r][i] - b : 0.0f;
    s = r == 0 ? x : s + x;
  }
  return s / (float)num_participants;
}

void oracle_pseudograd_avg_f32(float* g, float* p, const float* b, const float* const* replicas,
                               uint32_t n_replicas, uint32_t participate_mask,
                               uint32_t num_participants, int restore_p, uint64_t numel) {
  for (uint64_t i = 0; i < numel; ++i) {
    const float gi = pseudograd_avg(replicas, n_replicas, participate_mask, num_participants, b[i], i);
    if (restore_p) p[i] = b[i]; /* torchft/local_sgd.py:219 */
    g[i] = gi;
  }
}

/* torchft/local_sgd.py:221-224: outer_optimizer.step() on params that were
 * just restored to the backup, then backup <- params. */
void oracle_outer_sgd_f32(float* p, float* b, float* buf, const float* g, const oracle_sgd* k,
                          uint64_t numel) {
  for (uint64_t i = 0; i < numel; ++i) {
    float m = buf ? buf[i] : 0.0f;
    const float np = sgd_update(k, g[i], b[i], &m);
    if (buf && k->momentum != 0.0f) buf[i] = m;
    p[i] = np;
    b[i] = np;
  }
}

/* torchft/local_sgd.py:205-225 in one pass (commit known to be true). */
void oracle_diloco_outer_f32(float* p, float* b, float* buf, const float* const* replicas,
                             uint32_t n_replicas, uint32_t participate_mask,
                             uint32_t num_participants, const oracle_sgd* k, uint64_t numel) {
  for (uint64_t i = 0; i < numel; ++i) {
    const float gi = pseudograd_avg(replicas, n_replicas, participate_mask, num_participants, b[i], i);
    float m = buf ? buf[i] : 0.0f;
    const float np = sgd_update(k, gi, b[i], &m);
    if (buf && k->momentum != 0.0f) buf[i] = m;
    p[i] = np;
    b[i] = np;
  }
}
