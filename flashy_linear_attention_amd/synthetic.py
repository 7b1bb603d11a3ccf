"""Seeded synthetic inputs for the five benchmark/parity workloads.

All draws are made on the CPU in fp32 from one ``torch.Generator`` in the fixed
order q_raw, k_raw, v, dO; the feature map is applied in fp32; the result is
cast to the workload's dtype.  Tensors are contiguous ``(B, H, N, D)``.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, Tuple

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    dtype: torch.dtype
    batch: int
    heads: int
    seq: int
    d_qk: int
    d_v: int
    features: str  # "elu1" (elu(x)+1) or "taylor2" (x (x) x / sqrt 2 of a sqrt(d_qk)-dim x ~ 0.5 randn)
    backward: bool
    small_v: bool

    @property
    def flops_fwd(self) -> float:
        """Causal-counted forward FLOPs: N^2 (D_qk + D_v) per (b, h)."""
        return float(self.batch * self.heads) * self.seq * self.seq * (self.d_qk + self.d_v)

    @property
    def flops_bwd(self) -> float:
        """Causal-counted backward FLOPs: N^2 (3 D_qk + 2 D_v) per (b, h)."""
        return float(self.batch * self.heads) * self.seq * self.seq * (3 * self.d_qk + 2 * self.d_v)

    @property
    def bytes_fwd(self) -> float:
        e = self.batch * self.heads * self.seq
        return 2.0 * e * (2 * self.d_qk + 2 * self.d_v)

    @property
    def bytes_bwd(self) -> float:
        e = self.batch * self.heads * self.seq
        return 2.0 * e * (4 * self.d_qk + 3 * self.d_v)


WORKLOADS: Dict[str, Workload] = {
    "C1": Workload("C1", torch.float32, 1, 2, 256, 64, 64, "elu1", True, False),
    "C2": Workload("C2", torch.float16, 4, 16, 2048, 64, 64, "elu1", False, False),
    "C3": Workload("C3", torch.bfloat16, 4, 32, 4096, 128, 128, "elu1", True, False),
    "C4": Workload("C4", torch.bfloat16, 4, 16, 4096, 256, 64, "taylor2", True, True),
    "C5": Workload("C5", torch.bfloat16, 1, 16, 32768, 64, 64, "elu1", True, False),
}


def _features(kind: str, shape: Tuple[int, int, int], d_qk: int, gen: torch.Generator) -> torch.Tensor:
    if kind == "elu1":
        return torch.nn.functional.elu(torch.randn(*shape, d_qk, generator=gen)) + 1.0
    if kind == "taylor2":
        r = math.isqrt(d_qk)
        if r * r != d_qk:
            raise ValueError("taylor2 features need a square d_qk")
        x = 0.5 * torch.randn(*shape, r, generator=gen)
        return (x[..., :, None] * x[..., None, :]).flatten(-2) / math.sqrt(2.0)
    raise ValueError(kind)


def make_inputs(
    w: Workload, seed: int = 0, batch: int | None = None, heads: int | None = None, seq: int | None = None
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(q, k, v, dO) on the CPU in ``w.dtype``; batch/heads/seq may be overridden
    to draw a smaller sample of the same distribution."""
    b = w.batch if batch is None else batch
    h = w.heads if heads is None else heads
    n = w.seq if seq is None else seq
    gen = torch.Generator().manual_seed(seed)
    q = _features(w.features, (b, h, n), w.d_qk, gen)
    k = _features(w.features, (b, h, n), w.d_qk, gen)
    v = torch.randn(b, h, n, w.d_v, generator=gen)
    do = torch.randn(b, h, n, w.d_v, generator=gen)
    return tuple(t.to(w.dtype).contiguous() for t in (q, k, v, do))
