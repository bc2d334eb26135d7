#!/usr/bin/env python3
"""Replica-sync benchmark on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

The default workload (the headline one) is the fused DiLoCo outer step on
Llama-3-8B-shaped fp32 parameters: one step = one pass of the fused multi-tensor
kernel (pseudo-gradient of N replicas against the backup, average, Nesterov outer
SGD, backup refresh) over all 291 parameter tensors, steady state (momentum
buffers exist), everything resident in HBM before the timed region.  One JSON line
is printed with params/s, the kernel's achieved HBM bandwidth against the 8 TB/s
peak (HIP events around every launch, on the stream the kernel runs on), and the
reference's CPU loop (torch CPU ops + ProcessGroupGloo, world size 1) timed on a
bounded slice of the same workload on this box's host cores.

Other workloads measure the remaining kernels of the path with the same line
format: ``diloco_gpt2_small``, ``ddp_buckets_llama3_8b`` (bf16 gradient buckets, 4
contributions of which 3 participate), ``checkpoint_llama3_8b`` (pack / unpack of an
80 GB training state, plus the PCIe legs), ``localsgd_llama3_8b``.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from typing import Callable, Dict, List, Tuple

import torch

REPO_ROOT = os.path.dirname(os.path.abspath(__file__))
if REPO_ROOT not in sys.path:
    sys.path.insert(0, REPO_ROOT)

HBM_PEAK_GBS = 8000.0
LR, MOMENTUM = 0.7, 0.9
HEADLINE_METRIC = "outer-sync params/sec + achieved HBM GB/s (% peak), Llama-3-8B DiLoCo"
WORKLOADS = ["diloco_llama3_8b", "diloco_gpt2_small", "ddp_buckets_llama3_8b",
             "checkpoint_llama3_8b", "localsgd_llama3_8b", "diloco_llama3_8b_api",
             "diloco_two_phase_llama3_8b", "placement_llama3_8b_slice", "host_backup_llama3_8b",
             "diloco_bucketized_llama3_8b", "localsgd_bucketized_llama3_8b",
             "ddp_buckets_llama3_8b_two_streams", "ddp_whole_model_llama3_8b", "localsgd_llama3_8b_api",
             "ddp_hook_llama3_8b", "diloco_gpt2_small_api"]


def parse_args() -> argparse.Namespace:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", choices=WORKLOADS, default=WORKLOADS[0])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--recv-child", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("--api-child", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("--no-api", action="store_true",
                    help="headline workload: leave out the sub-record measured through DiLoCo.sync()")
    ap.add_argument("--cpu-layers", type=int, default=8,
                    help="decoder layers in the CPU baseline's slice of the Llama workload")
    ap.add_argument("--cpu-steps", type=int, default=4)
    ap.add_argument("--calibration-copy", action="store_true",
                    help="run one plain multi-tensor copy of known size before the timed loop "
                         "(reference point for hardware-counter runs)")
    ap.add_argument("--settle-seconds", type=float, default=8.0,
                    help="idle this long before the first device allocation: device memory freed by a "
                         "process that has just exited is handed out in a worse physical layout for a "
                         "few seconds (2-5 %% lower bandwidth for the whole run); 0 disables")
    ap.add_argument("--layout", default="",
                    help="comma list: alias_p (DiLoCo workloads: the live parameters are replica 0, "
                         "updated in place), flat_backup / flat_momentum (backup / momentum tensors are "
                         "views of one flat allocation, back to back without padding), misaligned (DiLoCo "
                         "workloads: every tensor re-allocated to start 4 bytes past a 16-byte boundary; moved: "
                         "the same re-allocation, 16 bytes past, as the aligned control; placed: backup "
                         "and momentum allocated by the library's bank-group placement), no_placement "
                         "(the library allocates backup / momentum / pseudo-gradients without looking "
                         "at HBM bank groups)")
    ap.add_argument("--launch-variant", default="",
                    help="route the launches through the tuning build of the library with this launch-shape "
                         "override (bits 0-3 accesses per lane: 1, 2, 4; bit 4 plain instead of non-temporal "
                         "accesses; bits 8-11 log2 of the per-XCD run + 1; bits 12-15 dynamic LDS per workgroup "
                         "in units of 8 KiB + 1, e.g. 0x1000 = no residency cap, 0x9000 = 64 KiB); for sweeps")
    ap.add_argument("--placement-all", action="store_true",
                    help="placement_llama3_8b_slice: every assignment of the streams to the three bank "
                         "groups (up to relabelling the groups) instead of a selection")
    ap.add_argument("--model-copies", type=int, default=1,
                    help="DiLoCo workloads: the tensor list repeated this many times in one launch "
                         "(separates the fixed cost of a launch from its streaming rate)")
    ap.add_argument("--storage-dtype", choices=("f32", "bf16"), default="f32",
                    help="DiLoCo workloads: dtype of parameters, backup, momentum and replicas "
                         "(arithmetic is fp32 either way; the named configurations are f32)")
    ap.add_argument("--arena", action="store_true",
                    help="carve all tensors of the DiLoCo workload out of one device allocation "
                         "instead of allocating each separately (makes no measurable difference)")
    return ap.parse_args()


class Timed:
    """K steps, wall clock bracketed by synchronize, HIP events around every launch group."""

    def __init__(self, steps: int, warmup: int) -> None:
        self.steps, self.warmup = steps, warmup

    def run(self, step: Callable[[], None]) -> Tuple[float, float]:
        for _ in range(self.warmup):
            step()
        torch.cuda.synchronize()
        starts = [torch.cuda.Event(enable_timing=True) for _ in range(self.steps)]
        stops = [torch.cuda.Event(enable_timing=True) for _ in range(self.steps)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(self.steps):
            starts[i].record()
            step()
            stops[i].record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / self.steps
        kernel_ms = sum(a.elapsed_time(b) for a, b in zip(starts, stops)) / self.steps
        return wall_ms, kernel_ms


# HBM bytes per step measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs per
# workload, each counter scaled by its reading for a plain copy of known size).  Counters
# cannot be read from inside this script: the figures, the scale factors and the commands
# that produced them are kept in one tracked data file, which this script quotes.
TRAFFIC_FILE = os.path.join(REPO_ROOT, "profiles", "hbm_traffic.json")


def measured_traffic(workload: str) -> Tuple[object, object]:
    """(HBM bytes per step from the hardware counters, where that figure comes from)."""
    try:
        with open(TRAFFIC_FILE) as f:
            entry = json.load(f)["workloads"][workload]
        return float(entry["read_bytes"]) + float(entry["write_bytes"]), "profiles/hbm_traffic.json"
    except (OSError, KeyError, ValueError):
        return None, None


def roofline(algo_bytes: float, kernel_ms: float, kernel: str, launches: int = 1,
             traffic: object = None, workload: str = "") -> Dict[str, object]:
    achieved = algo_bytes / (kernel_ms * 1e-3) / 1e9
    source = None
    if workload:
        traffic, source = measured_traffic(workload)
    return {
        "bound": "hbm",
        "achieved": achieved,
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": achieved / HBM_PEAK_GBS,
        "traffic": traffic,
        "traffic_source": source,
        "kernel": kernel,
        "kernel_ms_per_step": kernel_ms,
        "launches_per_step": launches,
        "algorithmic_bytes_per_step": algo_bytes,
    }


def base_line(args, metric: str, value: float, unit: str, ms_per_step: float, dtype: str,
              config: Dict[str, object]) -> Dict[str, object]:
    return {
        "metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
        "config": config,
    }


class CheckerReplay:
    """Output check of a timed DiLoCo run: the initial state of a few whole tensors is kept on
    the host, the CPU checker replays as many outer steps as the GPU ran, and parameters,
    backup and momentum must come out bit for bit.  ``in_place``: replica 0 is the live
    parameter tensor (what ``DiLoCo.sync()`` does), so every step reads the previous step's
    parameters."""

    MAX_ELEMS = 5_000_000

    def __init__(self, backup, bufs, replicas, in_place: bool, want: int = 3) -> None:
        small = [i for i, t in enumerate(backup) if t.numel() <= self.MAX_ELEMS]
        picks = sorted({small[0], small[len(small) // 2], small[-1]}) if small else []
        biggest_small = max(small, key=lambda i: backup[i].numel()) if small else None
        if biggest_small is not None:
            picks = sorted(set(picks[:want - 1]) | {biggest_small})
        self.picks = picks
        self.in_place = in_place
        self.backup = [backup[i].detach().cpu().clone() for i in picks]
        self.bufs = None if bufs is None else [bufs[i].detach().cpu().clone() for i in picks]
        self.replicas = [[rep[i].detach().cpu().clone() for i in picks] for rep in replicas]

    def check(self, steps: int, params, backup, bufs, dtype: torch.dtype) -> str:
        from oracle import replica_sync as O

        if not self.picks:
            return "skipped: no tensor small enough to replay on the host"
        n = len(self.replicas)
        acc = None if dtype == torch.float32 else torch.float32
        reps, b, m = self.replicas, self.backup, self.bufs
        for _ in range(steps):
            out = O.diloco_perform_sync(reps, b, m, [True] * n, n, True, lr=LR, momentum=MOMENTUM,
                                        nesterov=True, accumulate_dtype=acc)
            b, m = out["backup"], out["momentum"]
            if self.in_place:
                reps = [out["params"], *reps[1:]]
        for k, i in enumerate(self.picks):
            for got, want, what in ((params[i], out["params"][k], "parameters"),
                                    (backup[i], b[k], "backup"), (bufs[i], m[k], "momentum")):
                if not torch.equal(got.detach().cpu().view(torch.uint8), want.view(torch.uint8)):
                    raise RuntimeError(f"output check failed: {what} of tensor {i} differ from the "
                                       f"CPU checker after {steps} steps")
        elems = sum(t.numel() for t in self.backup)
        return (f"parameters, backup and momentum of tensors {self.picks} ({elems} elements) equal the CPU "
                f"checker's bit for bit after {steps} outer steps")


# ---------------------------------------------------------------------------
# CPU baseline: the reference's loop, timed
# ---------------------------------------------------------------------------

def cpu_baseline_diloco(args, shapes, n_rep: int, sample: str) -> Dict[str, object]:
    from oracle import replica_sync as O
    from torchft_amd import workloads

    # draw the values on the GPU (seconds) and move them to host memory: the CPU generator
    # needs minutes for a billion normals, and the values do not change the timing
    wl = workloads.make_diloco_workload(shapes, n_rep, torch.device("cuda", 0))
    wl.backup = [t.cpu() for t in wl.backup]
    wl.replicas = [[t.cpu() for t in rep] for rep in wl.replicas]
    torch.cuda.empty_cache()
    params = [torch.nn.Parameter(t) for t in wl.replicas[0]]
    opt = torch.optim.SGD(params, lr=LR, momentum=MOMENTUM, nesterov=True)
    pg = O.make_gloo_world1()
    peers = wl.replicas[1:]
    O.diloco_reference_loop_(pg, params, wl.backup, peers, opt, n_rep)  # creates momentum state
    t0 = time.perf_counter()
    for _ in range(args.cpu_steps):
        O.diloco_reference_loop_(pg, params, wl.backup, peers, opt, n_rep)
    dt = (time.perf_counter() - t0) / args.cpu_steps
    return {
        "value": wl.n_params / dt, "unit": "params/s", "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{sample}, {args.cpu_steps} steps after 1 warm-up; {wl.n_params} params, "
                  f"{dt * 1e3:.1f} ms/step; torch CPU ops + ProcessGroupGloo world size 1, "
                  f"os.cpu_count()={os.cpu_count()}",
    }


# ---------------------------------------------------------------------------
# Workloads
# ---------------------------------------------------------------------------

def bench_diloco(args, which: str) -> Dict[str, object]:
    from torchft_amd import ops, workloads
    from torchft_amd.multi_tensor import TensorTable

    dev = torch.device("cuda", 0)
    if which == "llama3_8b":
        shapes, n_rep = workloads.llama3_8b_shapes(), 2
    else:
        shapes, n_rep = workloads.gpt2_small_shapes(), 4
    if args.model_copies > 1:
        shapes = [(f"{k}.{name}", sh) for k in range(args.model_copies) for name, sh in shapes]
    dtype = torch.bfloat16 if args.storage_dtype == "bf16" else torch.float32
    esize = 2 if dtype == torch.bfloat16 else 4
    if args.arena and dtype != torch.float32:
        raise SystemExit("--arena is an fp32 layout experiment")
    if args.arena:
        per_set = sum(-(-workloads.numel(sh) * 4 // 256) * 256 for _, sh in shapes)
        arena = torch.empty((3 + n_rep) * per_set, dtype=torch.uint8, device=dev)
        cursor = [0]

        def carve(like):
            out = []
            for t in like:
                n = t.numel() * 4
                v = arena[cursor[0]:cursor[0] + n].view(torch.float32).view(t.shape)
                v.copy_(t)
                out.append(v)
                cursor[0] += -(-n // 256) * 256
            return out

        backup = carve(workloads.normal_tensors(shapes, 0.02, workloads.SEED_BACKUP, dev))
        replicas = [carve(workloads.drifted_replica(backup, 1e-3, workloads.SEED_REPLICA + r))
                    for r in range(n_rep)]
        wl = workloads.DilocoWorkload([n for n, _ in shapes], backup, replicas)
        params = carve([torch.zeros(1, device=dev).expand(workloads.numel(sh)).view(sh) for _, sh in shapes])
        bufs = carve(workloads.normal_tensors(shapes, 1e-3, 4000, dev))
        torch.cuda.empty_cache()
    else:
        wl = workloads.make_diloco_workload(shapes, n_rep, dev, dtype)
        params = [torch.empty_like(t) for t in wl.backup]
        bufs = workloads.normal_tensors(shapes, 1e-3, 4000, dev, dtype)
    layout = [x for x in args.layout.split(",") if x]
    if "misaligned" in layout or "moved" in layout:
        # misaligned: every tensor of every stream starts one element (4 bytes) past a 16-byte
        # boundary; moved: the same re-allocation with a shift of 16 bytes (the aligned control)
        first = 1 if "misaligned" in layout else 16 // esize

        def shifted(ts):
            for i, t in enumerate(ts):
                moved = torch.empty(t.numel() + 16, dtype=t.dtype, device=dev)[first:first + t.numel()].view(t.shape)
                moved.copy_(t)
                ts[i] = moved
            return ts

        for ts in (wl.backup, bufs, params, *wl.replicas):
            shifted(ts)
        torch.cuda.empty_cache()
        assert all(t.data_ptr() % 16 == (esize * first) % 16 for t in params + wl.backup + bufs)
    if "placed" in layout:
        # backup and momentum are the library's buffers: allocated the way DiLoCo allocates them
        from torchft_amd import hbm_placement

        placed_b, placed_buf = hbm_placement.model_copies(wl.replicas[0], 2)
        ops.mt_copy(placed_b, wl.backup)
        ops.mt_copy(placed_buf, bufs)
        torch.cuda.synchronize()
        wl.backup, bufs = placed_b, placed_buf
        torch.cuda.empty_cache()
    for item in layout:
        if item in ("misaligned", "moved", "placed"):
            continue
        if item == "alias_p":
            params = wl.replicas[0]
        elif item in ("flat_backup", "flat_momentum"):
            src = wl.backup if item == "flat_backup" else bufs
            flat = torch.empty(sum(t.numel() for t in src), dtype=dtype, device=dev)
            views = ops.flat_views(flat, src)
            ops.mt_copy(views, src)
            torch.cuda.synchronize()
            if item == "flat_backup":
                wl.backup = views
            else:
                bufs = views
            del src
            torch.cuda.empty_cache()
        elif item != "no_placement":
            raise SystemExit(f"unknown --layout item {item!r}")
    sgd = ops.OuterSGD(lr=LR, momentum=MOMENTUM, nesterov=True)
    table = TensorTable([params, wl.backup, bufs, *wl.replicas], what="bench")
    torch.cuda.synchronize()
    if args.calibration_copy:
        ops.mt_copy(params, wl.backup)
        torch.cuda.synchronize()

    # The reference computes the pseudo-gradient as params - backup and lets SGD subtract it
    # (torchft/local_sgd.py:214, :223), so with replicas that never move the backup runs away
    # from them geometrically and overflows fp32 after about 95 applications.  Real training
    # restarts the replicas from the new backup after every sync; a benchmark with static
    # inputs instead puts the pristine backup and momentum back every RESEED steps (two
    # multi-tensor copies, counted inside the timed region).  Runs of up to RESEED steps in
    # total (the default) never re-seed.
    RESEED = 64
    need_reseed = args.steps + args.warmup > RESEED
    pristine = None
    if need_reseed:
        pristine = ([t.clone() for t in wl.backup], [t.clone() for t in bufs])
    done = [0]
    reseeds = [0]
    replay = None if need_reseed else CheckerReplay(wl.backup, bufs, wl.replicas, in_place="alias_p" in layout)

    def step() -> None:
        if pristine is not None and done[0] and done[0] % RESEED == 0:
            ops.mt_copy(wl.backup, pristine[0])
            ops.mt_copy(bufs, pristine[1])
            reseeds[0] += 1
        ops.mt_diloco_outer(params, wl.backup, bufs, wl.replicas, sgd, False, table=table)
        done[0] += 1

    wall_ms, kernel_ms = Timed(args.steps, args.warmup).run(step)
    for probe in (0, len(params) // 2, len(params) - 1):
        same = torch.equal(params[probe].view(torch.uint8), wl.backup[probe].view(torch.uint8))
        if not same or not torch.isfinite(params[probe]).all():
            raise RuntimeError("output check failed: parameters are not finite or differ from the backup")
    checked = ("skipped: the state is re-seeded inside the timed region" if replay is None
               else replay.check(done[0], params, wl.backup, bufs, dtype))

    n_params = wl.n_params
    # read N replicas, backup, momentum; write momentum, parameters, backup
    algo_bytes = n_params * esize * (n_rep + 5)
    out = base_line(
        args, HEADLINE_METRIC if which == "llama3_8b" else "outer-sync params/sec, GPT-2-small DiLoCo",
        n_params / (wall_ms * 1e-3), "params/s", wall_ms, "f32",
        {"workload": f"DiLoCo outer step, {'fp32' if esize == 4 else 'bf16 storage with fp32 arithmetic'}, {which}-shaped params ({len(shapes)} tensors, "
                     f"{n_params} params), {n_rep} simulated replicas, Nesterov SGD lr={LR} "
                     f"momentum={MOMENTUM}, one fused multi-tensor launch per step",
         "n_tensors": len(shapes), "n_params": n_params, "n_replicas": n_rep,
         "allocation": ("every tensor is a contiguous view carved out of one device allocation"
                        if args.arena else "one device allocation per tensor"),
         "layout": layout, "model_copies": args.model_copies, "output_check": checked})
    out["roofline"] = roofline(algo_bytes, kernel_ms,
                               f"mt_stream_kernel<{'F32' if esize == 4 else 'BF16'}, DilocoFusedOp<{n_rep}>>",
                               workload="" if args.model_copies > 1 else
                               (f"diloco_{which}" if esize == 4 else f"diloco_{which}_bf16"))
    if reseeds[0]:
        out["config"]["state_reseeds_inside_timed_region"] = reseeds[0]
        out["roofline"]["note"] = ("steps that re-seed the state include two extra copy launches in "
                                   "kernel_ms_per_step")
    if not args.no_cpu_baseline:
        if which == "llama3_8b":
            cpu_shapes = workloads.llama3_8b_shapes(args.cpu_layers, with_embeddings=False)
            sample = f"{args.cpu_layers} of 32 decoder layers of the Llama-3-8B workload (no embeddings)"
        else:
            cpu_shapes, sample = shapes, "full GPT-2-small workload"
        out["cpu_baseline"] = cpu_baseline_diloco(args, cpu_shapes, n_rep, sample)
    return out


def bench_diloco_api(args, which: str = "llama3_8b") -> Dict[str, object]:
    """The same step driven through the torchft-shaped API: ``DiLoCo.sync()`` on a module
    with the model's parameters, this package's Manager on a local replica group; the timed
    step includes all host work (quorum, commit vote, validation of the kept launch).  The
    parameters are replica 0 and are updated in place, as the reference's ``p.data`` are."""
    from torch import nn

    from torchft_amd import DiLoCo, Manager, ProcessGroupLocalReplicas, StaticQuorum, workloads

    dev = torch.device("cuda", 0)
    if which == "llama3_8b":
        shapes, n_rep = workloads.llama3_8b_shapes(), 2
    else:
        shapes, n_rep = workloads.gpt2_small_shapes(), 4
    dtype = torch.bfloat16 if args.storage_dtype == "bf16" else torch.float32
    esize = 2 if dtype == torch.bfloat16 else 4

    class Bag(nn.Module):
        def __init__(self) -> None:
            super().__init__()
            self.ps = nn.ParameterList(
                [nn.Parameter(t) for t in workloads.normal_tensors(shapes, 0.02, 0, dev, dtype)])

    model = Bag()
    live = [p.data for p in model.parameters()]
    peers = [workloads.drifted_replica(live, 1e-3, 1001 + r) for r in range(n_rep - 1)]
    index = {p.data_ptr(): i for i, p in enumerate(model.parameters())}
    # the peers' buffers stay where they are for the whole run: the group may say so, and a
    # sync then does not ask for every tensor's peers again
    pg = ProcessGroupLocalReplicas(0, n_rep, peer_lookup=lambda t: [pr[index[t.data_ptr()]] for pr in peers],
                                   peers_are_stable=True)
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2, use_async_quorum=False,
                      quorum_client=StaticQuorum(0, n_rep))
    inner = torch.optim.SGD(model.parameters(), lr=0.1)
    outer = torch.optim.SGD(model.parameters(), lr=LR, momentum=MOMENTUM, nesterov=True)
    n_params = sum(p.numel() for p in model.parameters())
    if args.steps + args.warmup > 59:
        # static peers make the backup run away from them (see bench_diloco): fp32 overflows
        # after about 95 syncs, so a longer request is cut to 59 syncs and the line says so
        import copy

        args = copy.copy(args)
        args.warmup = min(args.warmup, 9)
        args.steps = min(args.steps, 59 - args.warmup)
        print(f"bench.py: diloco_{which}_api times {args.steps} syncs after {args.warmup} warm-up syncs "
              "(at most 59 in total)", file=sys.stderr)
    host_ms, isolated_ms = [], []
    with DiLoCo(manager, model, inner, outer, sync_every=10 ** 9) as diloco:
        backups = list(diloco._backup_parameters.values())
        replay = CheckerReplay(backups, None, [live, *peers], in_place=True)
        diloco.sync()  # first step creates the momentum state

        def timed_sync() -> None:
            t0 = time.perf_counter()
            diloco.sync()
            host_ms.append((time.perf_counter() - t0) * 1e3)

        wall_ms, kernel_ms = Timed(args.steps, args.warmup).run(timed_sync)
        n_syncs = 1 + args.warmup + args.steps
        if which != "llama3_8b":
            # a sync as a training loop sees it: device idle before, result awaited after
            for _ in range(10):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                diloco.sync()
                torch.cuda.synchronize()
                isolated_ms.append((time.perf_counter() - t0) * 1e3)
            n_syncs += 10
        bufs = [outer.state[p]["momentum_buffer"] for p in model.parameters()]
        checked = replay.check(n_syncs, [p.data for p in model.parameters()], backups, bufs, dtype)
        where = stream_groups(dev, {"p": [p.data for p in model.parameters()], "x1": peers[0],
                                    "b": backups, "buf": bufs})
    manager.shutdown(wait=False)
    metric = HEADLINE_METRIC if which == "llama3_8b" else "outer-sync params/sec, GPT-2-small DiLoCo"
    out = base_line(args, metric + " (through DiLoCo.sync())", n_params / (wall_ms * 1e-3),
                    "params/s", wall_ms, "f32",
                    {"workload": f"DiLoCo.sync() on a module with the {len(shapes)} {which} "
                                 f"{'fp32' if esize == 4 else 'bf16'} parameters, "
                                 f"Manager + ProcessGroupLocalReplicas(world {n_rep}), outer torch.optim.SGD "
                                 "Nesterov; parameters updated in place (the live parameters are "
                                 "replica 0); backup and momentum allocated by the library",
                     "n_tensors": len(shapes), "n_params": n_params, "n_replicas": n_rep,
                     "output_check": checked})
    out["roofline"] = roofline(n_params * (n_rep + 5) * esize, kernel_ms,
                               f"mt_stream_kernel<{'F32' if esize == 4 else 'BF16'}, DilocoFusedOp<{n_rep}>>")
    out["roofline"]["note"] = "kernel_ms_per_step here spans the whole sync() on the stream, host gaps included"
    if where:
        out["config"]["hbm_bank_groups"] = where
    timed = host_ms[args.warmup:]
    out["host_ms_per_sync"] = sum(timed) / len(timed)
    if isolated_ms:
        out["isolated_sync_ms"] = sum(isolated_ms) / len(isolated_ms)
    return out


def stream_groups(dev: torch.device, streams: Dict[str, List[torch.Tensor]], samples: int = 8) -> str:
    """Which HBM bank group (A, B, C in order of discovery; ? = none of the known ones) a
    few large tensors of every stream lie in, found with the library's own probe against the
    reference buffers its placement search has kept; empty if there was no search."""
    from torchft_amd import hbm_placement

    state = hbm_placement.device_state(dev)
    if len(state.map.anchors) < 2:
        return ""
    first = next(iter(streams.values()))
    big = [i for i, t in enumerate(first) if t.numel() * t.element_size() >= hbm_placement.MIN_PROBE_BYTES]
    if not big:
        return ""
    pick = big[:: max(1, len(big) // samples)][:samples]
    with state.lock:
        return " ".join(
            name + ":" + "".join("?" if g is None else "ABC"[g] for g in (state.map.group_of(ts[i]) for i in pick))
            for name, ts in streams.items())


def api_record(line: Dict[str, object]) -> Dict[str, object]:
    """The drop-in seat's figures as a sub-record of the headline line."""
    roof = line["roofline"]
    return {
        "workload": line["config"]["workload"],
        "steps": line["steps"],
        "warmup": line["warmup"],
        "ms_per_step": line["ms_per_step"],
        "params_per_s": line["value"],
        "kernel_ms_per_step": roof["kernel_ms_per_step"],
        "achieved_GBs": roof["achieved"],
        "frac": roof["frac"],
        "host_ms_per_sync": line["host_ms_per_sync"],
        "output_check": line["config"]["output_check"],
        "hbm_bank_groups": line["config"].get("hbm_bank_groups", ""),
    }


def bench_localsgd_api(args) -> Dict[str, object]:
    """The LocalSGD average driven through the torchft-shaped API: ``LocalSGD.sync()`` on a
    module with the 291 Llama-3-8B fp32 parameters, this package's Manager on a local replica
    group of 2 (quorum, table checks, commit vote, one launch that writes parameters and
    backup)."""
    from torch import nn

    from torchft_amd import LocalSGD, Manager, ProcessGroupLocalReplicas, StaticQuorum, workloads

    dev = torch.device("cuda", 0)
    shapes = workloads.llama3_8b_shapes()

    class Bag(nn.Module):
        def __init__(self) -> None:
            super().__init__()
            self.ps = nn.ParameterList(
                [nn.Parameter(t) for t in workloads.normal_tensors(shapes, 0.02, 0, dev)])

    model = Bag()
    peer = workloads.drifted_replica([p.data for p in model.parameters()], 1e-3, 1001)
    index = {p.data_ptr(): i for i, p in enumerate(model.parameters())}
    pg = ProcessGroupLocalReplicas(0, 2, peer_lookup=lambda t: [peer[index[t.data_ptr()]]])
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2, use_async_quorum=False,
                      quorum_client=StaticQuorum(0, 2))
    inner = torch.optim.SGD(model.parameters(), lr=0.1)
    n_params = sum(p.numel() for p in model.parameters())
    with LocalSGD(manager, model, inner, sync_every=10 ** 9) as local_sgd:
        wall_ms, kernel_ms = Timed(args.steps, args.warmup).run(local_sgd.sync)
    manager.shutdown(wait=False)
    out = base_line(args, "LocalSGD sync params/sec, Llama-3-8B (through LocalSGD.sync())",
                    n_params / (wall_ms * 1e-3), "params/s", wall_ms, "f32",
                    {"workload": "LocalSGD.sync() on a module with the 291 Llama-3-8B fp32 parameters, "
                                 "Manager + ProcessGroupLocalReplicas(world 2); parameters averaged in "
                                 "place, backup refreshed by the same launch",
                     "n_tensors": len(shapes), "n_params": n_params, "n_replicas": 2})
    out["roofline"] = roofline(n_params * 16, kernel_ms, "mt_stream_kernel<F32, ReduceAvgOp<2, 2>>")
    out["roofline"]["note"] = "kernel_ms_per_step here spans the whole sync() on the stream, host gaps included"
    return out


def bench_bucketized_api(args, kind: str) -> Dict[str, object]:
    """What one GPU does per sync when the replicas live on different GPUs: ``DiLoCo.sync()`` /
    ``LocalSGD.sync()`` over an ORDINARY process group (one collective per dtype on a flat
    buffer).  The collective itself is not this build's (one GPU): the group here returns at
    once, as if the peer had contributed zeros, so the timed sync is the local work around it.
    DiLoCo: pseudo-gradients into the flat buffer (12 B/param), the collective leaves the sum,
    the outer SGD divides on the way in and writes parameters, backup and momentum (24 B).
    LocalSGD: flatten (8 B), collective, then one launch that divides and writes parameters and
    backup (12 B)."""
    from torch import nn

    from oracle import replica_sync as O  # the checker of the first sync's output, nothing else
    from torchft_amd import DiLoCo, LocalSGD, Manager, ProcessGroup, StaticQuorum, workloads
    from torchft_amd.process_group import _DummyWork

    class SumWithAZeroPeer(ProcessGroup):
        def __init__(self) -> None:
            super().__init__(0, 2)
            self.calls = 0

        def configure(self, store_addr: str, rank: int, world_size: int) -> None:
            pass

        def allreduce(self, tensors, opts):
            self.calls += 1
            return _DummyWork(tensors)

        def size(self) -> int:
            return 2

        def getBackendName(self) -> str:
            return "sum-with-a-zero-peer"

    dev = torch.device("cuda", 0)
    shapes = workloads.llama3_8b_shapes()

    class Bag(nn.Module):
        def __init__(self) -> None:
            super().__init__()
            self.ps = nn.ParameterList(
                [nn.Parameter(t) for t in workloads.normal_tensors(shapes, 0.02, 0, dev)])

    model = Bag()
    pg = SumWithAZeroPeer()
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2, use_async_quorum=False,
                      quorum_client=StaticQuorum(0, 2))
    inner = torch.optim.SGD(model.parameters(), lr=0.1)
    n_params = sum(p.numel() for p in model.parameters())
    check = [2, 146]
    params = [p.data for p in model.parameters()]
    if kind == "diloco":
        outer = torch.optim.SGD(model.parameters(), lr=LR, momentum=MOMENTUM, nesterov=True)
        ctx = DiLoCo(manager, model, inner, outer, sync_every=10 ** 9)
        per_param = 36
    else:
        ctx = LocalSGD(manager, model, inner, sync_every=10 ** 9)
        per_param = 20
    with ctx:
        backups = list(ctx._backup_parameters.values())
        # the first sync, checked: a drift of the parameters against the backup
        for i in check:
            params[i].add_(1e-3)
        local = [params[i].cpu() for i in check]
        before = [backups[i].cpu() for i in check]
        ctx.sync()
        torch.cuda.synchronize()
        if kind == "diloco":
            want = O.diloco_perform_sync([local, before], before, None, [True, True], 2, True,
                                         lr=LR, momentum=MOMENTUM, nesterov=True)
        else:
            zeros = [torch.zeros_like(t) for t in local]
            want = O.localsgd_perform_sync([local, zeros], before, [True, True], 2, True)
        for k, i in enumerate(check):
            if not (torch.equal(params[i].cpu(), want["params"][k]) and torch.equal(backups[i].cpu(), want["backup"][k])):
                raise RuntimeError(f"output check failed: tensor {i} differs from the CPU checker's result")
        calls = pg.calls
        wall_ms, kernel_ms = Timed(args.steps, args.warmup).run(ctx.sync)
        per_sync = (pg.calls - calls) / (args.steps + args.warmup)
    manager.shutdown(wait=False)
    name = "DiLoCo" if kind == "diloco" else "LocalSGD"
    out = base_line(args, f"{name} sync over an ordinary process group, local work, params/sec, Llama-3-8B",
                    n_params / (wall_ms * 1e-3), "params/s", wall_ms, "f32",
                    {"workload": f"{name}.sync() on a module with the 291 Llama-3-8B fp32 parameters over an ordinary "
                                 "process group (bucketised: one collective per sync on a flat buffer; the "
                                 "collective returns at once, the peer contributing zeros), 2 replicas",
                     "n_tensors": len(shapes), "n_params": n_params, "n_replicas": 2,
                     "collectives_per_sync": per_sync,
                     "output_check": f"first sync: parameters and backup of tensors {check} equal the CPU checker's bit for bit"})
    out["roofline"] = roofline(n_params * per_param, kernel_ms,
                               "PseudogradOp<1> + OuterSgdOp" if kind == "diloco" else "mt_copy_kernel + ReduceAvgOp<2, 1>")
    out["roofline"]["launches_per_step"] = 2
    out["roofline"]["note"] = "kernel_ms_per_step spans the whole sync() on the stream: two launches and the host between them"
    return out


def bench_diloco_two_phase(args) -> Dict[str, object]:
    """The two-phase form used when the commit decision must come between reduction and
    update: phase 1 (pseudo-gradient average, in place on replica 0) and phase 2 (outer SGD +
    backup refresh), each one launch, timed separately.  Phase 1 leaves the parameters alone,
    as DiLoCo.sync() does with a fusable SGD (phase 2 overwrites them without reading them);
    the form that also restores them, used before any other optimizer, is timed beside it."""
    from torchft_amd import ops, workloads

    dev = torch.device("cuda", 0)
    shapes, n_rep = workloads.llama3_8b_shapes(), 2
    from torchft_amd import hbm_placement

    wl = workloads.make_diloco_workload(shapes, n_rep, dev)
    params = wl.replicas[0]  # live parameters are replica 0
    # backup, momentum and pseudo-gradients are the library's: allocated the way DiLoCo does
    backup, bufs, grads = hbm_placement.model_copies(params, 3)  # one search, as DiLoCo does
    ops.mt_copy(backup, wl.backup)
    ops.mt_copy(bufs, workloads.normal_tensors(shapes, 1e-3, 4000, dev))
    torch.cuda.synchronize()
    wl.backup = backup
    torch.cuda.empty_cache()
    sgd = ops.OuterSGD(lr=LR, momentum=MOMENTUM, nesterov=True)
    t1 = ops.mt_pseudograd_avg(grads, params, wl.backup, wl.replicas, False)
    t2 = ops.mt_outer_sgd(params, wl.backup, bufs, grads, sgd, False)
    pristine = [t.clone() for t in wl.backup]  # phase 2 moves the backup: put it back per step
    torch.cuda.synchronize()
    n_params = wl.n_params
    e = [[torch.cuda.Event(enable_timing=True) for _ in range(5)] for _ in range(args.steps)]
    for i in range(args.warmup + args.steps):
        k = i - args.warmup
        ops.mt_copy(wl.backup, pristine)
        ops.mt_copy(params, wl.replicas[1])  # some drift to average
        if k >= 0:
            e[k][3].record()
        ops.mt_pseudograd_avg(grads, params, wl.backup, wl.replicas, True, table=t1)
        if k >= 0:
            e[k][4].record()
        ops.mt_copy(params, wl.replicas[1])
        if k >= 0:
            e[k][0].record()
        ops.mt_pseudograd_avg(grads, params, wl.backup, wl.replicas, False, table=t1)
        if k >= 0:
            e[k][1].record()
        ops.mt_outer_sgd(params, wl.backup, bufs, grads, sgd, False, table=t2)
        if k >= 0:
            e[k][2].record()
    torch.cuda.synchronize()
    p1 = sum(a[0].elapsed_time(a[1]) for a in e) / args.steps
    p2 = sum(a[1].elapsed_time(a[2]) for a in e) / args.steps
    p1r = sum(a[3].elapsed_time(a[4]) for a in e) / args.steps
    out = base_line(args, "two-phase DiLoCo sync params/sec, Llama-3-8B", n_params / ((p1 + p2) * 1e-3),
                    "params/s", p1 + p2, "f32",
                    {"workload": "DiLoCo sync in two launches (pseudo-gradient average, then outer SGD + "
                                 "backup refresh), Llama-3-8B fp32, 2 replicas, in place on replica 0; "
                                 "ms_per_step is the sum of the two kernels (the state reset between steps "
                                 "is not counted)",
                     "n_tensors": len(shapes), "n_params": n_params, "n_replicas": n_rep})
    # phase 1: read x0, x1, b; write g (and p where it restores).
    # phase 2: read g, b, buf; write p, b, buf.
    out["roofline"] = roofline(n_params * 16, p1, "mt_stream_kernel<F32, PseudogradOp<2>>")
    out["phase2"] = roofline(n_params * 24, p2, "mt_stream_kernel<F32, OuterSgdOp>")
    out["phase1_with_restore"] = roofline(n_params * 20, p1r, "mt_stream_kernel<F32, PseudogradOp<2>>")
    return out


def bench_placement(args) -> Dict[str, object]:
    """How the kernels' speed depends on which HBM bank group each stream lies in: the fused
    DiLoCo step (separate output parameters, and parameters updated in place) and the LocalSGD
    average on an 8-layer slice of Llama-3-8B (7 GB per stream: any assignment fits a group),
    every stream placed in a chosen group through the library's own grouped pool."""
    from torchft_amd import hbm_placement, ops, workloads

    dev = torch.device("cuda", 0)
    shapes = workloads.llama3_8b_shapes(args.cpu_layers, with_embeddings=False)
    n_params = sum(workloads.numel(sh) for _, sh in shapes)
    per_stream = sum(-(-workloads.numel(sh) * 4 // 256) * 256 for _, sh in shapes)
    pool = hbm_placement.GroupedPool(dev)
    pool.limit = 280 << 30  # this workload wants all three groups, whatever that takes
    need = 5 * per_stream + (4 << 30)
    ok = pool.grow_until(lambda pl: len(pl.map.anchors) >= 3 and
                         all(pl.free_bytes(g) >= need for g in range(3)))
    if not ok or not pool.structured:
        have = {g: pool.free_bytes(g) >> 30 for g in range(len(pool.map.anchors))}
        raise SystemExit(f"placement_llama3_8b_slice: could not reserve {need >> 30} GiB in each of three "
                         f"HBM bank groups (GiB found per group: {have}, {len(pool._straddling)} blocks "
                         "across a boundary or unclassifiable)")
    sgd = ops.OuterSGD(lr=LR, momentum=MOMENTUM, nesterov=True)

    def column(group: int, init: float):
        out = []
        for _, sh in shapes:
            raw = pool.take(workloads.numel(sh) * 4, [group])
            assert raw is not None
            t = raw.view(torch.float32).view(sh)
            t.normal_(0.0, init) if init else t.zero_()
            out.append(t)
        return out

    def measure(step) -> float:
        _, kernel_ms = Timed(args.steps, args.warmup).run(step)
        return kernel_ms

    rows = []
    letters = "ABC"
    fused = ["AAAAA", "AABBB", "AABBA", "AACCA", "AABCA", "AAABA", "AAAAB", "AAABC", "AACAB", "ACACB"]
    in_place = ["AAAA", "ABBB", "AABB", "AABC", "AABA", "ABAB", "ABCA"]
    average = ["AAA", "ABB", "AAB", "ABA", "ABC"]
    if args.placement_all:
        # the first parameter stream (x0, or p where it is replica 0) fixed in group A: the
        # three groups are interchangeable
        import itertools

        fused = ["A" + "".join(t) for t in itertools.product(letters, repeat=4)]
        in_place = ["".join((t[0], "A", t[1], t[2])) for t in itertools.product(letters, repeat=3)]
        average = ["".join((t[0], "A", t[1])) for t in itertools.product(letters, repeat=2)]
    for lay in fused:  # streams x0 x1 b buf p
        pool.reset()
        x0, x1, b, buf, p = (column(letters.index(c), s) for c, s in zip(lay, (0.02, 0.02, 0.02, 0.0, 0.0)))
        ms = measure(lambda: ops.mt_diloco_outer(p, b, buf, [x0, x1], sgd, False))
        rows.append({"kernel": "fused DiLoCo, separate output", "streams": "x0 x1 b buf p", "groups": lay,
                     "kernel_ms": ms, "frac": n_params * 28 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS})
        del x0, x1, b, buf, p
    for lay in in_place:  # streams x1 p b buf (p is replica 0)
        pool.reset()
        x1, p, b, buf = (column(letters.index(c), s) for c, s in zip(lay, (0.02, 0.02, 0.02, 0.0)))
        ms = measure(lambda: ops.mt_diloco_outer(p, b, buf, [p, x1], sgd, False))
        rows.append({"kernel": "fused DiLoCo, parameters in place", "streams": "x1 p b buf", "groups": lay,
                     "kernel_ms": ms, "frac": n_params * 28 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS})
        del x1, p, b, buf
    for lay in average:  # streams x1 p b
        pool.reset()
        x1, p, b = (column(letters.index(c), 0.02) for c in lay)
        ms = measure(lambda: ops.mt_reduce_avg([p, b], [p, x1]))
        rows.append({"kernel": "LocalSGD average + backup", "streams": "x1 p b", "groups": lay,
                     "kernel_ms": ms, "frac": n_params * 16 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS})
        del x1, p, b
    best = max(r["frac"] for r in rows if r["kernel"].startswith("fused DiLoCo, separate"))
    out = base_line(args, "fused DiLoCo step by HBM bank-group assignment (best fraction of peak)", best,
                    "fraction of 8 TB/s", min(r["kernel_ms"] for r in rows), "f32",
                    {"workload": f"{args.cpu_layers} of 32 decoder layers of Llama-3-8B ({n_params} fp32 "
                                 f"params, {per_stream} bytes per stream), every stream placed in a chosen "
                                 "HBM bank group (A, B, C: three groups of 96 GiB)",
                     "n_params": n_params})
    out["placement_table"] = rows
    return out


def bench_localsgd(args) -> Dict[str, object]:
    from torchft_amd import ops, workloads

    dev = torch.device("cuda", 0)
    from torchft_amd import hbm_placement

    shapes, n_rep = workloads.llama3_8b_shapes(), 2
    wl = workloads.make_diloco_workload(shapes, n_rep, dev)
    # the backup is the library's: allocated the way LocalSGD does (outside the HBM bank
    # group of the parameters it shadows)
    backup = hbm_placement.model_copies(wl.replicas[0], 1)[0]
    ops.mt_copy(backup, wl.backup)
    torch.cuda.synchronize()
    wl.backup = backup
    torch.cuda.empty_cache()
    table = ops.reduce_avg_table([wl.replicas[0], wl.backup], wl.replicas)

    def step() -> None:
        ops.mt_reduce_avg([wl.replicas[0], wl.backup], wl.replicas, table=table)

    wall_ms, kernel_ms = Timed(args.steps, args.warmup).run(step)
    n_params = wl.n_params
    out = base_line(args, "LocalSGD sync params/sec, Llama-3-8B", n_params / (wall_ms * 1e-3),
                    "params/s", wall_ms, "f32",
                    {"workload": "LocalSGD weight average + backup refresh, fp32, Llama-3-8B-shaped "
                                 "params, 2 simulated replicas, one launch per step",
                     "n_tensors": len(shapes), "n_params": n_params, "n_replicas": n_rep})
    out["roofline"] = roofline(n_params * 4 * (n_rep + 2), kernel_ms,
                               "mt_stream_kernel<F32, ReduceAvgOp<2, 2>>",
                               workload="localsgd_llama3_8b")
    if not args.no_cpu_baseline:
        from oracle import replica_sync as O

        cpu_shapes = workloads.llama3_8b_shapes(args.cpu_layers, with_embeddings=False)
        cw = workloads.make_diloco_workload(cpu_shapes, n_rep, dev)
        backup = [t.cpu() for t in cw.backup]
        reps = [[t.cpu() for t in rep] for rep in cw.replicas]
        del cw
        O.localsgd_perform_sync(reps, backup, [True] * n_rep, n_rep, True)
        t0 = time.perf_counter()
        for _ in range(args.cpu_steps):
            O.localsgd_perform_sync(reps, backup, [True] * n_rep, n_rep, True)
        dt = (time.perf_counter() - t0) / args.cpu_steps
        n_cpu = sum(t.numel() for t in backup)
        out["cpu_baseline"] = {
            "value": n_cpu / dt, "unit": "params/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{args.cpu_layers} of 32 decoder layers (no embeddings), {args.cpu_steps} steps after "
                      f"1 warm-up; {n_cpu} params, {dt * 1e3:.1f} ms/step; per-tensor torch CPU ops "
                      f"(sum of replicas, divide, backup copy)"}
    return out


def bench_host_backup(args) -> Dict[str, object]:
    """LocalSGD's backup in pinned host memory (the reference's default placement): how long
    the training stream is held up by a save, and whether the transfer really overlaps
    compute.  The reference issues one copy per tensor on the training stream
    (torchft/local_sgd.py:121-125, with a TODO to use a separate stream); here one gather
    launch runs on the training stream and one PCIe transfer on a side stream."""
    from torchft_amd import ops, workloads
    from torchft_amd.local_sgd import _PackedHostBackup

    dev = torch.device("cuda", 0)
    shapes = workloads.llama3_8b_shapes(args.cpu_layers * 2, with_embeddings=False)
    params = workloads.normal_tensors(shapes, 0.02, workloads.SEED_BACKUP, dev)
    other = workloads.drifted_replica(params, 1e-3, workloads.SEED_REPLICA)
    out_t = [torch.empty_like(t) for t in params]
    n_params = sum(t.numel() for t in params)
    nbytes = 4 * n_params
    backup = _PackedHostBackup([(str(i), t) for i, t in enumerate(params)], pin_memory=True)
    def ev():
        return torch.cuda.Event(enable_timing=True)

    cached = [None]

    def compute():  # stand-in for the next inner steps: an HBM-bound launch over the model
        cached[0] = ops.mt_reduce_avg([out_t], [params, other], 0b11, 2, table=cached[0])

    for _ in range(2):
        compute()
    torch.cuda.synchronize()
    a, b = ev(), ev()
    a.record()
    for _ in range(10):
        compute()
    b.record()
    torch.cuda.synchronize()
    compute_alone_ms = a.elapsed_time(b) / 10

    held, total, overlapped = [], [], []
    for it in range(args.warmup + args.steps):
        torch.cuda.synchronize()
        a, b, c = ev(), ev(), ev()
        t0 = time.perf_counter()
        a.record()
        backup.save(params)
        b.record()
        for _ in range(10):
            compute()
        c.record()
        backup.wait()
        t_host = (time.perf_counter() - t0) * 1e3
        torch.cuda.synchronize()
        if it >= args.warmup:
            held.append(a.elapsed_time(b))
            total.append(t_host)
            overlapped.append(b.elapsed_time(c) / 10)
    for i in (0, len(params) // 2, len(params) - 1):
        if not torch.equal(backup.host_views[i], params[i].cpu()):
            raise RuntimeError("output check failed: the host backup differs from the parameters")

    # the reference's form: one copy per tensor into the pinned tensors, on the training stream
    per_tensor = []
    for it in range(2 + 3):
        torch.cuda.synchronize()
        a, b = ev(), ev()
        a.record()
        for h, p in zip(backup.host_views, params):
            h.copy_(p, non_blocking=True)
        b.record()
        torch.cuda.synchronize()
        if it >= 2:
            per_tensor.append(a.elapsed_time(b))
    mean = lambda xs: sum(xs) / len(xs)
    held_ms, total_ms = mean(held), mean(total)
    out = base_line(
        args, "LocalSGD host backup: bytes saved per second of training-stream time", nbytes / (held_ms * 1e-3) / 1e9,
        "GB/s", held_ms, "u8",
        {"workload": f"save of {len(shapes)} fp32 tensors ({n_params} params, {nbytes / 1e9:.1f} GB; "
                     f"{args.cpu_layers * 2} of 32 Llama-3-8B decoder layers) into pinned host memory: one "
                     "gather launch on the training stream, one transfer on a side stream",
         "n_tensors": len(shapes), "n_params": n_params})
    out["roofline"] = roofline(2 * nbytes, held_ms, "mt_copy_kernel")
    out["host_backup"] = {
        "training_stream_held_ms": held_ms,
        "save_complete_on_host_ms": total_ms,
        "pcie_GBps": nbytes / (total_ms * 1e-3) / 1e9,
        "compute_launch_alone_ms": compute_alone_ms,
        "compute_launch_during_transfer_ms": mean(overlapped),
        "per_tensor_copies_on_training_stream_ms": mean(per_tensor),
    }
    del backup, out_t
    torch.cuda.empty_cache()
    out["diloco_sync_with_host_backup"] = diloco_sync_with_host_backup(params, other, n_params)
    return out


def diloco_sync_with_host_backup(params: List[torch.Tensor], peer: List[torch.Tensor], n_params: int) -> Dict[str, object]:
    """``DiLoCo(..., backup_device="cpu").sync()`` on the same tensors: the backup comes from
    pinned host memory before the launch and goes back after it (the reference moves every
    backup tensor with ``.to(p.device)`` inside the sync, torchft/local_sgd.py:214)."""
    from torch import nn

    from torchft_amd import DiLoCo, Manager, ProcessGroupLocalReplicas, StaticQuorum

    class Bag(nn.Module):
        def __init__(self) -> None:
            super().__init__()
            self.ps = nn.ParameterList([nn.Parameter(t) for t in params])

    model = Bag()
    index = {p.data_ptr(): i for i, p in enumerate(model.parameters())}
    pg = ProcessGroupLocalReplicas(0, 2, peer_lookup=lambda t: [peer[index[t.data_ptr()]]], peers_are_stable=True)
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2, use_async_quorum=False,
                      quorum_client=StaticQuorum(0, 2))
    inner = torch.optim.SGD(model.parameters(), lr=0.1)
    outer = torch.optim.SGD(model.parameters(), lr=LR, momentum=MOMENTUM, nesterov=True)
    stream_ms, host_ms = [], []
    with DiLoCo(manager, model, inner, outer, sync_every=10 ** 9, backup_device=torch.device("cpu")) as diloco:
        diloco.sync()  # creates the momentum
        for it in range(2 + 4):
            diloco._host_backup.wait()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0 = time.perf_counter()
            a.record()
            diloco.sync()
            b.record()
            b.synchronize()
            diloco._host_backup.wait()
            if it >= 2:
                stream_ms.append(a.elapsed_time(b))
                host_ms.append((time.perf_counter() - t0) * 1e3)
        for i in (0, len(params) - 1):
            if not torch.equal(list(diloco._backup_parameters.values())[i], params[i].cpu()):
                raise RuntimeError("output check failed: host backup != parameters after a committed sync")
    manager.shutdown(wait=False)
    mean = lambda xs: sum(xs) / len(xs)
    nbytes = 4 * n_params
    return {
        "training_stream_held_ms": mean(stream_ms),
        "backup_on_host_again_after_ms": mean(host_ms),
        "GB": nbytes / 1e9,
        "note": "stream held = one host-to-device transfer of the backup + the fused launch; the "
                "transfer back overlaps what the stream does next",
    }


def bench_ddp_buckets(args, form: str = "hook_order") -> Dict[str, object]:
    from torchft_amd import GradBucketAverager, workloads

    dev = torch.device("cuda", 0)
    shapes = workloads.llama3_8b_shapes()
    grads = workloads.make_grad_replicas(shapes, 4, dev, torch.bfloat16)
    averager = GradBucketAverager(grads[0], grads)  # in place on replica 0, like a DDP bucket
    mask, n = 0b0111, 3  # replica 3 is a spare: zeroed, never read

    if form == "hook_order":
        def step() -> None:
            averager.average_all(mask, n, streams=1)  # what 162 hook calls in a row do
        how, launches = "one launch per bucket, in hook order on one stream", len(averager.buckets)
    elif form == "two_streams":
        def step() -> None:
            averager.average_all(mask, n, streams=2)  # the library's default for average_all
        how = ("one launch per bucket in hook order, alternating between two side streams; a step is "
               "timed from the fork to the join on the current stream")
        launches = len(averager.buckets)
    else:
        def step() -> None:
            averager.average_whole_model(mask, n)
        how, launches = "all buckets in one launch", 1

    wall_ms, kernel_ms = Timed(args.steps, args.warmup).run(step)
    n_elems = sum(g.numel() for g in grads[0])
    out = base_line(args, "DDP gradient-bucket average elements/sec, Llama-3-8B bf16",
                    n_elems / (wall_ms * 1e-3), "elements/s", wall_ms, "bf16 storage, f32 accumulate",
                    {"workload": f"bf16 gradients of Llama-3-8B ({len(shapes)} tensors, {n_elems} "
                                 f"elements) in {len(averager.buckets)} buckets by torch's 1 MiB / 25 MiB "
                                 f"rule, 4 contributions with 3 participating, {how}, "
                                 "over per-parameter views (no flatten / unflatten passes)",
                     "n_buckets": len(averager.buckets), "n_elements": n_elems})
    out["roofline"] = roofline(n_elems * 2 * (3 + 1), kernel_ms,
                               "mt_stream_kernel<BF16, ReduceAvgOp<1, 4>>", launches,
                               workload="ddp_buckets_llama3_8b" if form == "hook_order" else "")
    if form == "two_streams":
        out["roofline"]["note"] = ("launches on the two streams overlap: kernel_ms_per_step is the span from "
                                   "fork to join, not the sum of the kernels' durations")
    if not args.no_cpu_baseline:
        from oracle import replica_sync as O

        cpu_shapes = workloads.llama3_8b_shapes(args.cpu_layers, with_embeddings=False)
        cg = [[t.cpu() for t in rep]
              for rep in workloads.make_grad_replicas(cpu_shapes, 4, dev, torch.bfloat16)]
        buckets = O.bucket_assignment([t.numel() for t in cg[0]], 2)
        flags = [True, True, True, False]
        O.ddp_bucket_average(cg, flags, 3, buckets)
        t0 = time.perf_counter()
        for _ in range(args.cpu_steps):
            O.ddp_bucket_average(cg, flags, 3, buckets)
        dt = (time.perf_counter() - t0) / args.cpu_steps
        n_cpu = sum(t.numel() for t in cg[0])
        out["cpu_baseline"] = {
            "value": n_cpu / dt, "unit": "elements/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{args.cpu_layers} of 32 decoder layers (no embeddings), {len(buckets)} buckets, "
                      f"{args.cpu_steps} steps after 1 warm-up; {n_cpu} elements, {dt * 1e3:.1f} ms/step; "
                      f"torch CPU ops: flatten (cat), zero the spare, bf16 sum, divide, unflatten"}
    return out


def bench_ddp_hook(args) -> Dict[str, object]:
    """Gradient-bucket averaging through the reference's own seat (torchft/ddp.py:47-71): a module
    with the 291 Llama-3-8B bf16 parameters in ``DistributedDataParallel(manager, module,
    gradient_as_bucket_view=True)``; torch's Reducer owns the flat buckets and calls the
    communication hook as each fills during a real backward; the hook is
    ``manager.allreduce(bucket.buffer())`` on a local replica group of 4 of which one is a spare
    (3 participate).  Everything runs on one stream, so GPU time is additive: the same backward
    is timed with the averaging hook and with ``manager.allreduce`` replaced by a stand-in that
    only returns the bucket, and HIP events around every ``manager.allreduce`` call give the
    averaging kernels' own time (with the host kept ahead of the GPU, see ``backward``)."""
    from torch import nn

    from oracle import replica_sync as O
    from torchft_amd import (DistributedDataParallel, Manager, ProcessGroupLocalReplicas, StaticQuorum,
                             WorldSizeMode, workloads)

    dev = torch.device("cuda", 0)
    shapes = workloads.llama3_8b_shapes()
    n_rep, n_active = 4, 3

    class Bag(nn.Module):
        """loss = sum_i <p_i, w_i>: the backward hands the Reducer dense bf16 gradients (= w_i)."""

        def __init__(self) -> None:
            super().__init__()
            self.ps = nn.ParameterList(
                [nn.Parameter(t) for t in workloads.normal_tensors(shapes, 0.02, 0, dev, torch.bfloat16)])
            self.ws = workloads.normal_tensors(shapes, 1e-2, workloads.SEED_GRAD, dev, torch.bfloat16)

        def forward(self) -> torch.Tensor:
            total = torch.zeros((), device=dev, dtype=torch.float32)
            for p, w in zip(self.ps, self.ws):
                total = total + (p * w).sum(dtype=torch.float32)
            return total

    model = Bag()
    n_elems = sum(p.numel() for p in model.parameters())
    peer_bufs: Dict[int, List[torch.Tensor]] = {}
    gen = torch.Generator(device=dev).manual_seed(workloads.SEED_GRAD + 1)

    def peers_of(flat: torch.Tensor) -> List[torch.Tensor]:
        # the peers' copies of this bucket: drawn the first time the bucket is seen, then kept
        key = flat.data_ptr()
        if key not in peer_bufs:
            peer_bufs[key] = [
                torch.empty(flat.numel(), dtype=torch.float32, device=dev).normal_(0.0, 1e-2, generator=gen)
                .to(flat.dtype) for _ in range(n_rep - 1)]
        return peer_bufs[key]

    pg = ProcessGroupLocalReplicas(0, n_rep, peer_lookup=peers_of, peers_are_stable=True,
                                   peer_participating=[True, True, False])
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=n_active,
                      world_size_mode=WorldSizeMode.FIXED_WITH_SPARES, quorum_client=StaticQuorum(0, n_rep))
    ddp = DistributedDataParallel(manager, model, gradient_as_bucket_view=True)
    allreduce = manager.allreduce
    mode = {"average": True, "record": False}
    host_us: List[float] = []
    spans: List[Tuple[torch.cuda.Event, torch.cuda.Event]] = []
    buckets: Dict[int, torch.Tensor] = {}

    def instrumented(tensor: torch.Tensor):
        # sits one call below the hook itself (DistributedDataParallel._comm_hook stays in
        # its seat: a Reducer takes only one hook for its lifetime)
        if not mode["average"]:
            fut: torch.futures.Future = torch.futures.Future()
            fut.set_result(tensor)
            return fut
        buckets.setdefault(tensor.data_ptr(), tensor)
        if not mode["record"]:
            return allreduce(tensor)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        t0 = time.perf_counter()
        fut = allreduce(tensor)
        host_us.append((time.perf_counter() - t0) * 1e6)
        b.record()
        spans.append((a, b))
        return fut

    manager.allreduce = instrumented

    # This synthetic backward is host-bound (hundreds of tiny launches), a real one is not: the
    # host of a training step runs far ahead of the GPU.  To time GPU work rather than launch
    # gaps, a plug of plain copies is enqueued first, long enough for the host to issue the
    # whole backward while the GPU is still busy with the plug; everything behind it then
    # executes back to back, and an event pair around a launch measures that launch alone.
    plug_src = torch.empty(4 << 30, dtype=torch.uint8, device=dev)
    plug_dst = torch.empty_like(plug_src)
    plug_copies = [0]

    def backward(average: bool, record: bool = False) -> Tuple[float, float]:
        mode["average"], mode["record"] = average, record
        for p in model.parameters():
            p.grad = None
        manager.start_quorum()
        loss = ddp()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(plug_copies[0]):
            plug_dst.copy_(plug_src, non_blocking=True)
        t0 = time.perf_counter()
        a.record()
        loss.backward()
        b.record()
        wall = (time.perf_counter() - t0) * 1e3
        torch.cuda.synchronize()
        if not manager.should_commit():
            raise RuntimeError(f"the step did not commit: {manager.errored()!r}")
        return a.elapsed_time(b), wall

    host_walls = []
    for _ in range(max(args.warmup, 2)):
        host_walls.append(backward(True, record=True)[1])
        backward(False)
    # one 4 GiB copy takes about 1.4 ms; cover the host's time for one backward three times
    probe_a, probe_b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    probe_a.record()
    plug_dst.copy_(plug_src, non_blocking=True)
    probe_b.record()
    torch.cuda.synchronize()
    plug_copies[0] = min(int(3.0 * min(host_walls) / probe_a.elapsed_time(probe_b)) + 1, 96)
    with_hook, without, walls = [], [], []
    for _ in range(args.steps):
        gpu_ms, wall_ms = backward(True)  # no events inside: they would sit between the launches
        with_hook.append(gpu_ms)
        walls.append(wall_ms)
        without.append(backward(False)[0])
    # one more pass, instrumented, for the host's time per hook call (its GPU figures are not used)
    host_us.clear()
    spans.clear()
    backward(True, record=True)
    n_hooks, host_per_hook = len(spans), sum(host_us) / max(len(host_us), 1)
    in_situ = sum(a.elapsed_time(b) for a, b in spans)
    mean = lambda xs: sum(xs) / len(xs)

    # spot check of the last averaged backward against the checker: whole gradients of a few
    # parameters, located inside their bucket by address
    backward(True)
    params = list(model.parameters())
    small = [i for i, p in enumerate(params) if p.numel() <= 5_000_000]
    picks = sorted({small[0], small[len(small) // 2], small[-1], max(small, key=lambda i: params[i].numel())})
    for i in picks:
        g = params[i].grad
        home = next(((ptr, flat) for ptr, flat in buckets.items()
                     if ptr <= g.data_ptr() < ptr + flat.numel() * 2), None)
        if home is None:
            raise RuntimeError(f"output check failed: gradient {i} is not a view of a bucket")
        off = (g.data_ptr() - home[0]) // 2
        contributions = [model.ws[i].reshape(-1).cpu()] + [
            pb[off:off + g.numel()].cpu() for pb in peer_bufs[home[0]]]
        want = O.manager_allreduce_(contributions, [True, True, True, False], n_active, torch.float32)
        if not torch.equal(g.reshape(-1).cpu().view(torch.int16), want.view(torch.int16)):
            raise RuntimeError(f"output check failed: gradient {i} differs from the CPU checker")
    manager.shutdown(wait=False)

    hook_ms = mean(with_hook) - mean(without)
    out = base_line(args, "DDP gradient-bucket average elements/sec through the comm hook, Llama-3-8B bf16",
                    n_elems / (hook_ms * 1e-3), "elements/s", hook_ms, "bf16 storage, f32 accumulate",
                    {"workload": f"torch DistributedDataParallel(gradient_as_bucket_view=True) over the {len(shapes)} "
                                 f"Llama-3-8B bf16 parameters ({n_elems} elements), {n_hooks} buckets, comm hook = "
                                 "manager.allreduce(bucket.buffer()) on ProcessGroupLocalReplicas(world 4, one spare, "
                                 "3 participate); one step = one real backward; ms_per_step is the GPU time the "
                                 "averaging hook adds to that backward (same backward with a pass-through hook "
                                 "subtracted; one stream, host kept ahead of the GPU)",
                     "n_buckets": n_hooks, "n_elements": n_elems,
                     "output_check": f"gradients {picks} equal the CPU checker's bucket average bit for bit"})
    out["roofline"] = roofline(n_elems * 2 * (n_active + 1), hook_ms,
                               "mt_stream_kernel<BF16, ReduceAvgOp<1, 4>, FlatLocator>", n_hooks)
    out["roofline"]["note"] = ("kernel_ms_per_step is the GPU time added to one backward by the 162 averaging "
                               "launches, the gaps between them and their neighbours included; the kernels' own "
                               "durations are in the rocprofv3 summary of this command")
    out["hook_seat"] = {
        "backward_gpu_ms_with_averaging_hook": mean(with_hook),
        "backward_gpu_ms_with_pass_through_hook": mean(without),
        "difference_ms": hook_ms,
        "event_spans_around_the_hook_calls_ms": in_situ,
        "host_ms_to_issue_one_backward_with_averaging_hook": mean(walls),
        "plug_copies_of_4GiB_ahead_of_each_backward": plug_copies[0],
        "host_us_per_hook": host_per_hook,
        "hooks_per_backward": n_hooks,
    }
    return out


def bench_checkpoint(args) -> Dict[str, object]:
    from torchft_amd import state_pack, workloads

    dev = torch.device("cuda", 0)
    shapes = workloads.llama3_8b_shapes()
    state = workloads.make_training_state(shapes, dev)
    plan = state_pack.plan_pack(state)
    staging = torch.empty(plan.total_bytes, dtype=torch.uint8, device=dev)
    cache: Dict[str, object] = {}
    torch.cuda.synchronize()

    def pack_step() -> None:
        state_pack.pack(state, staging=staging, table_cache=cache)

    wall_ms, pack_ms = Timed(args.steps, args.warmup).run(pack_step)
    entries, total = list(plan.entries), plan.total_bytes
    payload = sum(e.nbytes for e in entries)
    # unpack into the tensors of a second state of the same layout (scatter kernel);
    # the source state is released first: 80 GB staging + 80 GB destination stay resident
    del state, plan
    cache.clear()
    torch.cuda.empty_cache()
    from torchft_amd import ops

    outs = [torch.empty(e.shape, dtype=state_pack._DTYPES[e.dtype], device=dev) for e in entries]
    srcs = [staging[e.offset:e.offset + e.nbytes] for e in entries]
    table = ops.mt_copy(outs, srcs)
    _, unpack_ms = Timed(args.steps, args.warmup).run(lambda: ops.mt_copy(outs, srcs, table=table))
    # PCIe legs through two pinned bounce buffers (bounded host memory)
    chunk = 1 << 30
    bounce = [torch.empty(chunk, dtype=torch.uint8, pin_memory=True) for _ in range(2)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i, lo in enumerate(range(0, total, chunk)):
        n = min(chunk, total - lo)
        bounce[i % 2][:n].copy_(staging[lo:lo + n], non_blocking=True)
    torch.cuda.synchronize()
    d2h_s = time.perf_counter() - t0
    t0 = time.perf_counter()
    for i, lo in enumerate(range(0, total, chunk)):
        n = min(chunk, total - lo)
        staging[lo:lo + n].copy_(bounce[i % 2][:n], non_blocking=True)
    torch.cuda.synchronize()
    h2d_s = time.perf_counter() - t0
    out = base_line(args, "checkpoint pack GB/s, Llama-3-8B training state",
                    payload / (wall_ms * 1e-3) / 1e9, "GB/s (payload bytes packed per second)", wall_ms,
                    "u8",
                    {"workload": f"training state of Llama-3-8B: bf16 params + fp32 AdamW exp_avg / "
                                 f"exp_avg_sq + int64 steps, {len(entries)} device tensors, "
                                 f"{payload} bytes, one gather launch into a contiguous staging buffer",
                     "n_tensors": len(entries), "payload_bytes": payload})
    out["roofline"] = roofline(2 * payload, pack_ms, "mt_copy_kernel (pack)", traffic=2.0 * payload)
    out["unpack"] = roofline(2 * payload, unpack_ms, "mt_copy_kernel (unpack)")
    if not args.no_cpu_baseline:
        from oracle import replica_sync as O

        del outs, srcs, table, staging
        torch.cuda.empty_cache()
        small = workloads.make_training_state(workloads.llama3_8b_shapes(1, with_embeddings=False), dev)
        small_bytes = sum(e.nbytes for e in state_pack.plan_pack(small).entries)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        O.state_dict_round_trip(small)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        out["cpu_baseline"] = {
            "value": small_bytes / dt / 1e9, "unit": "GB/s (payload bytes through save + load)",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"training state of 1 of 32 decoder layers on the GPU ({small_bytes} bytes), one "
                      f"torch.save into memory + torch.load (the reference's send / receive seats), "
                      f"{dt:.2f} s; includes its per-storage device-to-host copies"}
    out["http_recovery"] = http_recovery(dev, getattr(args, "child", None))
    out["pcie"] = {"d2h_GBs": total / d2h_s / 1e9, "h2d_GBs": total / h2d_s / 1e9,
                   "d2h_s": d2h_s, "h2d_s": h2d_s, "bytes": total,
                   "note": "staging buffer through two 1 GiB pinned bounce buffers; PCIe-bound, "
                           "reported separately from the HBM-bound kernels"}
    return out


class _Discard:
    """A sink that counts bytes (the socket taken out of the serving pipeline)."""

    def __init__(self) -> None:
        self.n = 0

    def write(self, view) -> int:
        self.n += len(view)
        return len(view)


def recv_child() -> int:
    """The receiving replica of ``http_recovery`` as a process of its own (started before the
    parent touches the GPU): reads one JSON command per line from stdin, answers one JSON line.
    ``fetch``: recover a state from a CheckpointServer address onto this process's GPU context;
    ``sink``: receive plain bytes over k loopback TCP connections into pinned buffers (what the
    kernel's loopback path allows a Python receiver, with no GPU and no HTTP involved)."""
    import socket
    import threading
    from datetime import timedelta

    from torchft_amd import CheckpointServer, state_pack

    torch.cuda.set_device(0)
    torch.zeros(1, device="cuda")  # context up before the first timed command
    for line in sys.stdin:
        cmd = json.loads(line)
        if cmd["op"] == "quit":
            break
        if cmd["op"] == "fetch":
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            got = CheckpointServer.load_from_address(cmd["address"], timedelta(seconds=120),
                                                     streams=cmd["streams"])
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            t = got["user"]["model"][cmd["name"]]
            checksum = int(t.view(torch.int16).sum(dtype=torch.int64))
            del got, t
            print(json.dumps({"seconds": dt, "checksum": checksum}), flush=True)
        elif cmd["op"] == "sink":
            k, per_conn, chunk = cmd["connections"], cmd["bytes_per_connection"], 64 << 20
            bufs = [state_pack.PINNED.acquire(chunk) for _ in range(k)]

            def drain(j: int) -> None:
                view = memoryview(bufs[j].numpy())
                with socket.create_connection(("127.0.0.1", cmd["port"])) as c:
                    left = per_conn
                    while left:
                        n = c.recv_into(view[:min(chunk, left)])
                        if not n:
                            raise EOFError("sender closed early")
                        left -= n

            threads = [threading.Thread(target=drain, args=(j,)) for j in range(k)]
            t0 = time.perf_counter()
            for t in threads:
                t.start()
            for t in threads:
                t.join()
            dt = time.perf_counter() - t0
            for b in bufs:
                state_pack.PINNED.release(b)
            print(json.dumps({"seconds": dt}), flush=True)
    return 0


def loopback_bound(child, connections: int, bytes_per_connection: int) -> float:
    """GB/s of plain loopback TCP from pinned buffers of this process into pinned buffers of
    the child over ``connections`` sockets: the ceiling of any recovery between two processes
    of one host, whatever is done on the GPU side."""
    import socket
    import threading

    from torchft_amd import state_pack

    chunk = 64 << 20
    srv = socket.socket(socket.AF_INET, socket.SOCK_STREAM)
    srv.setsockopt(socket.SOL_SOCKET, socket.SO_REUSEADDR, 1)
    srv.bind(("127.0.0.1", 0))
    srv.listen(connections)
    bufs = [state_pack.PINNED.acquire(chunk) for _ in range(connections)]

    def feed(conn, j: int) -> None:
        view = memoryview(bufs[j].numpy())
        with conn:
            left = bytes_per_connection
            while left:
                n = min(chunk, left)
                conn.sendall(view[:n])
                left -= n

    child.stdin.write(json.dumps({"op": "sink", "port": srv.getsockname()[1], "connections": connections,
                                  "bytes_per_connection": bytes_per_connection}) + "\n")
    child.stdin.flush()
    threads = []
    for j in range(connections):
        conn, _ = srv.accept()
        threads.append(threading.Thread(target=feed, args=(conn, j)))
        threads[-1].start()
    for t in threads:
        t.join()
    answer = json.loads(child.stdout.readline())
    srv.close()
    for b in bufs:
        state_pack.PINNED.release(b)
    return connections * bytes_per_connection / answer["seconds"] / 1e9


def http_recovery(dev: torch.device, child=None) -> Dict[str, object]:
    """Live recovery end to end on a bounded slice: CheckpointServer.send_checkpoint on one
    side, recv_checkpoint on the other over loopback HTTP: chunks gathered on the device into
    a ring, pinned D2H, socket, pinned H2D, views on the receiving GPU; with 1, 2, 4 and 8
    parallel connections.  The receiver runs once inside this process (sender and receiver
    share one interpreter lock) and once as a process of its own (``child``), next to what
    plain loopback TCP between the two processes carries.  Also the serving pipeline alone
    (same chunks into a sink instead of a socket), which is what PCIe allows."""
    from datetime import timedelta

    from torchft_amd import CheckpointServer, state_pack, workloads

    state = workloads.make_training_state(workloads.llama3_8b_shapes(4, with_embeddings=False), dev)
    plan = state_pack.plan_pack(state)
    nbytes = sum(e.nbytes for e in plan.entries)
    sink = _Discard()
    state_pack.stream_packed(plan, sink)  # warm-up: pins the bounce buffers
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    state_pack.stream_packed(plan, sink)
    pipeline_s = time.perf_counter() - t0
    rates, child_rates, bound = {}, {}, {}
    name = next(iter(state["user"]["model"]))
    want_sum = int(state["user"]["model"][name].view(torch.int16).sum(dtype=torch.int64))
    for streams in (1, 2, 4, 8):
        server = CheckpointServer(timeout=timedelta(seconds=120), fetch_streams=streams)
        try:
            server.send_checkpoint([1], 1, state, timedelta(seconds=120))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            got = server.recv_checkpoint(0, server.metadata(), 1, timedelta(seconds=120))
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            if not torch.equal(got["user"]["model"][name], state["user"]["model"][name]):
                raise RuntimeError("recovered state differs")
            rates[str(streams)] = nbytes / dt / 1e9
            del got
            if child is not None:
                for attempt in range(2):  # the first fetch of the child pins its buffers
                    child.stdin.write(json.dumps({"op": "fetch", "address": f"{server.metadata()}1",
                                                  "streams": streams, "name": name}) + "\n")
                    child.stdin.flush()
                    answer = json.loads(child.stdout.readline())
                    if answer["checksum"] != want_sum:
                        raise RuntimeError("state recovered by the child process differs")
                child_rates[str(streams)] = nbytes / answer["seconds"] / 1e9
        finally:
            server.shutdown()
    if child is not None:
        for k in (1, 4, 8):
            loopback_bound(child, k, 256 << 20)  # warm-up: pins, connects
            bound[str(k)] = loopback_bound(child, k, (8 << 30) // k)
    out = {"GBs_by_connections": rates, "serving_pipeline_to_pinned_host_GBs": nbytes / pipeline_s / 1e9,
           "bytes": nbytes,
           "note": "training state of 4 decoder layers served and fetched over loopback HTTP; one "
                   "connection is bound by one TCP stream's two copies through the kernel, "
                   "which is why a recovery fetches byte ranges over several; the serving pipeline "
                   "alone (device ring -> pinned host, no socket) shows the PCIe bound; the "
                   "reference's torch.save / torch.load seats are timed in cpu_baseline"}
    if child is not None:
        out["GBs_by_connections_receiver_in_its_own_process"] = child_rates
        out["plain_loopback_tcp_between_the_two_processes_GBs"] = bound
    return out


def api_child_main(args) -> int:
    """``DiLoCo.sync()`` on the headline model in a process of its own (what a training job is):
    started by the headline run before it touches the GPU, waits for its go-ahead on stdin (the
    parent has freed its device memory by then), pauses like any fresh bench process and prints
    the API line."""
    if not sys.stdin.readline().strip():
        return 1  # the parent went away
    if "no_placement" in args.layout.split(","):
        os.environ["TORCHFT_AMD_HBM_PLACEMENT"] = "0"
    if args.settle_seconds > 0:
        time.sleep(args.settle_seconds)
    torch.cuda.set_device(0)
    print(json.dumps(bench_diloco_api(args)), flush=True)
    return 0


def run_api_child(child) -> object:
    """Gives the child its go-ahead and returns the api sub-record, or None if it failed."""
    try:
        import queue
        import threading

        child.stdin.write("go\n")
        child.stdin.flush()
        lines: "queue.Queue[str]" = queue.Queue()

        def read_record() -> None:
            line = child.stdout.readline()
            while line and not line.startswith("{"):
                line = child.stdout.readline()
            lines.put(line)

        threading.Thread(target=read_record, daemon=True).start()
        line = lines.get(timeout=600)  # a child that hangs must not hang the headline line
        child.wait(timeout=60)
        record = api_record(json.loads(line))
        record["process"] = ("a process of its own, started before the headline run touched the GPU and "
                             "released after that run had freed its arrays")
        return record
    except Exception as e:
        print(f"bench.py: the API child failed ({e!r}); measuring in this process", file=sys.stderr)
        try:
            child.kill()
        except Exception:
            pass
        return None


def main() -> int:
    args = parse_args()
    if args.recv_child:
        return recv_child()
    if args.api_child:
        return api_child_main(args)
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU only (asked for --gpus {args.gpus}); "
              "the N-replica reduction is simulated over N buffers resident on that GPU",
              file=sys.stderr)
        return 2
    # Children are started before this process touches the GPU in any way.
    import subprocess

    def spawn(flag: str, *extra: str):
        return subprocess.Popen([sys.executable, "-u", os.path.abspath(__file__), flag, *extra],
                                stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)

    if args.workload == "checkpoint_llama3_8b":
        # the receiving replica of the recovery measurement: a process of its own
        args.child = spawn("--recv-child")
    api_child = None
    # under a profiler everything stays in this process, so that one trace holds all dispatches
    profiled = any("rocprof" in value for value in os.environ.values())
    if (args.workload == "diloco_llama3_8b" and not args.no_api and args.model_copies == 1
            and not args.arena and not args.launch_variant and not profiled):
        # the same step through DiLoCo.sync(), in a process of its own as a training job is:
        # it waits until this process has printed nothing yet but freed its device memory
        api_child = spawn("--api-child", "--steps", str(args.steps), "--warmup", str(args.warmup),
                          "--settle-seconds", str(args.settle_seconds), "--storage-dtype", args.storage_dtype,
                          "--layout", args.layout)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        for child in (getattr(args, "child", None), api_child):
            if child is not None:
                child.kill()
        return 2
    if "no_placement" in args.layout.split(","):
        os.environ["TORCHFT_AMD_HBM_PLACEMENT"] = "0"
    if args.settle_seconds > 0:
        time.sleep(args.settle_seconds)  # before anything is allocated on the device
    torch.cuda.set_device(0)
    from torchft_amd import ops

    if args.launch_variant:
        import ctypes

        from torchft_amd import _build, _native

        tuning = _native.load(_build.TUNING_LIB_PATH, {"tft_set_launch_variant": (None, [ctypes.c_uint32])})
        _native._lib = tuning
        tuning.tft_set_launch_variant(int(args.launch_variant, 0))  # thread-local: this thread launches

    if args.calibration_copy and not args.workload.startswith("diloco_llama3_8b"):
        # reference point for hardware-counter runs: a plain copy of exactly 8 GiB
        src = torch.zeros(8 << 30, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        ops.mt_copy([dst], [src])
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()
    if args.workload == "diloco_llama3_8b":
        out = bench_diloco(args, "llama3_8b")
        if not args.no_api and args.model_copies == 1 and not args.arena:
            # the same step through the reference's own seat; the kernel-level tensors are gone
            # by now (they were locals of bench_diloco)
            torch.cuda.synchronize()
            torch.cuda.empty_cache()
            record = run_api_child(api_child) if api_child is not None else None
            if record is None:  # no child (a launch-shape override lives in this process) or it failed
                record = api_record(bench_diloco_api(args))
                record["process"] = "the process of the headline run, after it had freed its arrays"
            out["api"] = record
    elif args.workload == "diloco_gpt2_small_api":
        out = bench_diloco_api(args, "gpt2_small")
    elif args.workload == "ddp_hook_llama3_8b":
        out = bench_ddp_hook(args)
    elif args.workload == "diloco_gpt2_small":
        out = bench_diloco(args, "gpt2_small")
    elif args.workload == "ddp_buckets_llama3_8b":
        out = bench_ddp_buckets(args)
    elif args.workload == "ddp_buckets_llama3_8b_two_streams":
        out = bench_ddp_buckets(args, "two_streams")
    elif args.workload == "ddp_whole_model_llama3_8b":
        out = bench_ddp_buckets(args, "one_launch")
    elif args.workload == "checkpoint_llama3_8b":
        out = bench_checkpoint(args)
    elif args.workload == "diloco_llama3_8b_api":
        out = bench_diloco_api(args)
    elif args.workload == "diloco_two_phase_llama3_8b":
        out = bench_diloco_two_phase(args)
    elif args.workload == "localsgd_llama3_8b_api":
        out = bench_localsgd_api(args)
    elif args.workload == "diloco_bucketized_llama3_8b":
        out = bench_bucketized_api(args, "diloco")
    elif args.workload == "localsgd_bucketized_llama3_8b":
        out = bench_bucketized_api(args, "localsgd")
    elif args.workload == "placement_llama3_8b_slice":
        out = bench_placement(args)
    elif args.workload == "host_backup_llama3_8b":
        out = bench_host_backup(args)
    else:
        out = bench_localsgd(args)
    child = getattr(args, "child", None)
    if child is not None:
        try:
            child.stdin.write(json.dumps({"op": "quit"}) + "\n")
            child.stdin.flush()
            child.wait(timeout=30)
        except Exception:
            child.kill()
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
