"""Synthetic replica-sync workloads: parameter shapes and seeded values.

Shapes follow ``named_parameters()`` order of the usual implementations.  Values
are drawn from seeded generators on the device asked for.  CPU and GPU
generators produce different streams, so a parity test draws on one device and
copies (a whole small workload, or slices of a full-size one) to the other.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Sequence, Tuple

import torch

Shape = Tuple[int, ...]
Named = List[Tuple[str, Shape]]

SEED_BACKUP = 0
SEED_REPLICA = 1000
SEED_GRAD = 2000
SEED_EXP_AVG = 3000
SEED_EXP_AVG_SQ = 3001


def mlp_shapes() -> Named:
    """3-layer MLP: Linear(1024,2048), Linear(2048,2048), Linear(2048,10); 6 316 042 params."""
    return [
        ("0.weight", (2048, 1024)),
        ("0.bias", (2048,)),
        ("2.weight", (2048, 2048)),
        ("2.bias", (2048,)),
        ("4.weight", (10, 2048)),
        ("4.bias", (10,)),
    ]


def gpt2_small_shapes() -> Named:
    """GPT-2 small: 148 tensors, 124 439 808 params."""
    d, ff, layers = 768, 3072, 12
    out: Named = [("wte.weight", (50257, d)), ("wpe.weight", (1024, d))]
    for i in range(layers):
        p = f"h.{i}."
        out += [
            (p + "ln_1.weight", (d,)),
            (p + "ln_1.bias", (d,)),
            (p + "attn.c_attn.weight", (d, 3 * d)),
            (p + "attn.c_attn.bias", (3 * d,)),
            (p + "attn.c_proj.weight", (d, d)),
            (p + "attn.c_proj.bias", (d,)),
            (p + "ln_2.weight", (d,)),
            (p + "ln_2.bias", (d,)),
            (p + "mlp.c_fc.weight", (d, ff)),
            (p + "mlp.c_fc.bias", (ff,)),
            (p + "mlp.c_proj.weight", (ff, d)),
            (p + "mlp.c_proj.bias", (d,)),
        ]
    out += [("ln_f.weight", (d,)), ("ln_f.bias", (d,))]
    return out


def llama3_8b_shapes(n_layers: int = 32, with_embeddings: bool = True) -> Named:
    """Llama-3-8B: 291 tensors, 8 030 261 248 params (``n_layers`` < 32 gives a slice)."""
    d, kv, ff, vocab = 4096, 1024, 14336, 128256
    out: Named = []
    if with_embeddings:
        out.append(("model.embed_tokens.weight", (vocab, d)))
    for i in range(n_layers):
        p = f"model.layers.{i}."
        out += [
            (p + "self_attn.q_proj.weight", (d, d)),
            (p + "self_attn.k_proj.weight", (kv, d)),
            (p + "self_attn.v_proj.weight", (kv, d)),
            (p + "self_attn.o_proj.weight", (d, d)),
            (p + "mlp.gate_proj.weight", (ff, d)),
            (p + "mlp.up_proj.weight", (ff, d)),
            (p + "mlp.down_proj.weight", (d, ff)),
            (p + "input_layernorm.weight", (d,)),
            (p + "post_attention_layernorm.weight", (d,)),
        ]
    if with_embeddings:
        out += [("model.norm.weight", (d,)), ("lm_head.weight", (vocab, d))]
    return out


def numel(shape: Shape) -> int:
    n = 1
    for s in shape:
        n *= s
    return n


def total_params(shapes: Named) -> int:
    return sum(numel(s) for _, s in shapes)


def _gen(device: torch.device, seed: int) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def normal_tensors(
    shapes: Named,
    std: float,
    seed: int,
    device: torch.device,
    dtype: torch.dtype = torch.float32,
    absolute: bool = False,
) -> List[torch.Tensor]:
    """One N(0, std) tensor per shape from a single seeded generator (fp32 draw, then cast)."""
    g = _gen(device, seed)
    out = []
    for _, shape in shapes:
        t = torch.empty(shape, dtype=torch.float32, device=device).normal_(0.0, std, generator=g)
        if absolute:
            t.abs_()
        out.append(t if dtype == torch.float32 else t.to(dtype))
    return out


def drifted_replica(
    backup: Sequence[torch.Tensor], std: float, seed: int
) -> List[torch.Tensor]:
    """backup + N(0, std): what a replica's live parameters look like after inner steps."""
    device = backup[0].device
    g = _gen(device, seed)
    out = []
    for b in backup:
        t = torch.empty(b.shape, dtype=torch.float32, device=device).normal_(0.0, std, generator=g)
        t.add_(b)
        out.append(t if b.dtype == torch.float32 else t.to(b.dtype))
    return out


@dataclass
class DilocoWorkload:
    names: List[str]
    backup: List[torch.Tensor]
    replicas: List[List[torch.Tensor]]  # [replica][tensor]

    @property
    def n_params(self) -> int:
        return sum(t.numel() for t in self.backup)


def make_diloco_workload(
    shapes: Named, n_replicas: int, device: torch.device, dtype: torch.dtype = torch.float32
) -> DilocoWorkload:
    """backup ~ N(0, 0.02); replica r = backup + N(0, 1e-3) with seed 1000 + r."""
    backup = normal_tensors(shapes, 0.02, SEED_BACKUP, device, dtype)
    replicas = [drifted_replica(backup, 1e-3, SEED_REPLICA + r) for r in range(n_replicas)]
    return DilocoWorkload([n for n, _ in shapes], backup, replicas)


def make_grad_replicas(
    shapes: Named, n_replicas: int, device: torch.device, dtype: torch.dtype = torch.bfloat16
) -> List[List[torch.Tensor]]:
    """Gradients ~ N(0, 1e-2), one set per replica (seed 2000 + r)."""
    return [normal_tensors(shapes, 1e-2, SEED_GRAD + r, device, dtype) for r in range(n_replicas)]


def make_training_state(
    shapes: Named, device: torch.device, step: int = 1000
) -> Dict[str, object]:
    """A training state dict shaped like what Manager ships during recovery:
    bf16 parameters, fp32 AdamW moments and an int64 step counter per parameter group."""
    params = normal_tensors(shapes, 0.02, SEED_BACKUP, device, torch.bfloat16)
    exp_avg = normal_tensors(shapes, 1e-3, SEED_EXP_AVG, device)
    exp_avg_sq = normal_tensors(shapes, 1e-6, SEED_EXP_AVG_SQ, device, absolute=True)
    names = [n for n, _ in shapes]
    return {
        "user": {
            "model": dict(zip(names, params)),
            "optim": {
                "state": {
                    i: {
                        "step": torch.tensor(step, dtype=torch.int64, device=device),
                        "exp_avg": exp_avg[i],
                        "exp_avg_sq": exp_avg_sq[i],
                    }
                    for i in range(len(names))
                },
                "param_groups": [
                    {
                        "lr": 4e-4,
                        "betas": (0.9, 0.95),
                        "eps": 1e-8,
                        "weight_decay": 0.1,
                        "params": list(range(len(names))),
                    }
                ],
            },
        },
        "torchft": {"step": step, "batches_committed": 2 * step},
    }
