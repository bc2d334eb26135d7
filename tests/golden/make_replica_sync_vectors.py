"""Writes tests/golden/replica_sync_vectors.npz: small frozen input / output vectors for the
replica-sync arithmetic.

The reference ships no golden vectors for this path, and nothing of the reference is
imported here.  The expected outputs are produced by library routines only -
``torch.optim.SGD`` stepping real Parameters, plain tensor arithmetic in the reference's
order (subtract per replica, add in replica order, true divide), ``Tensor.to(bfloat16)`` -
and neither by the checker under oracle/ nor by the kernels, so both can be held to them.

    python tests/golden/make_replica_sync_vectors.py
"""

import os

import numpy as np
import torch

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "replica_sync_vectors.npz")
N = 2051  # not a multiple of 4: exercises the scalar tail


def u16(t: torch.Tensor) -> np.ndarray:
    return t.view(torch.int16).numpy().view(np.uint16)


def main() -> None:
    g = torch.Generator().manual_seed(20240607)
    backup = torch.randn(N, generator=g) * 0.02
    out = {"backup": backup.numpy()}
    # --- DiLoCo, 3 replicas of which replica 1 does not participate, n = 2, two syncs
    param = torch.nn.Parameter(backup.clone())
    opt = torch.optim.SGD([param], lr=0.7, momentum=0.9, nesterov=True)
    cur = backup.clone()
    for step in range(2):
        reps = [cur + torch.randn(N, generator=g) * 1e-3 for _ in range(3)]
        total = (reps[0] - cur) + torch.zeros(N)
        total = total + (reps[2] - cur)
        grad = total / 2
        param.data.copy_(cur)
        param.grad = grad.clone()
        opt.step()
        cur = param.data.clone()
        for r in range(3):
            out[f"diloco_step{step}_replica{r}"] = reps[r].numpy()
        out[f"diloco_step{step}_grad"] = grad.numpy()
        out[f"diloco_step{step}_params"] = cur.numpy()
        out[f"diloco_step{step}_momentum"] = opt.state[param]["momentum_buffer"].clone().numpy()
    # --- Manager.allreduce, fp32: 4 contributions, the last zeroed, divided by 3
    xs = [torch.randn(N, generator=g) for _ in range(4)]
    avg = ((xs[0] + xs[1]) + xs[2] + torch.zeros(N)) / 3
    for r in range(4):
        out[f"allreduce_f32_in{r}"] = xs[r].numpy()
    out["allreduce_f32_out"] = avg.numpy()
    # --- same in bf16 storage with fp32 accumulation
    bs = [(torch.randn(N, generator=g) * 1e-2).to(torch.bfloat16) for _ in range(4)]
    acc = ((bs[0].float() + bs[1].float()) + bs[2].float() + torch.zeros(N)) / 3
    for r in range(4):
        out[f"allreduce_bf16_in{r}"] = u16(bs[r])
    out["allreduce_bf16_out"] = u16(acc.to(torch.bfloat16))
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
