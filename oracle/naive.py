"""Naive CPU statement of causal linear attention and its gradients.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).

Layout everywhere: ``q, k : (B, H, N, D_qk)``, ``v, o, do : (B, H, N, D_v)``
(flashlinear/kernels/linear_attn_kernels.py:314,
flashlinear/kernels/linear_attn_kernels_smallv_hd.py:326-327).  Each (b, h)
pair is independent.

Mathematics (per (b, h); A and M are N x N and lower triangular, diagonal kept):

    A  = tril(Q K^T)        O  = A V            (linear_attn_kernels.py:74-82)
    M  = tril(dO V^T)       dV = A^T dO         (linear_attn_kernels.py:179-187)
                            dK = M^T Q          (linear_attn_kernels.py:189-197)
                            dQ = M K            (linear_attn_kernels.py:291-299)
"""

from __future__ import annotations

from typing import Tuple

import torch


def _tril_mask(n: int, device) -> torch.Tensor:
    return torch.ones(n, n, dtype=torch.bool, device=device).tril(0)


def causal_dot_product(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """O = tril(Q K^T) V as two matmuls and a mask, in the dtype of the inputs.

    The same three steps as the reference tests' ``linear_ref_torch``
    (flashlinear/test_attn.py:49-62): scores, multiply by a lower-triangular
    0/1 mask (diagonal=0), second matmul.
    """
    n = q.shape[-2]
    scores = torch.matmul(q, k.transpose(-2, -1))
    scores = scores * _tril_mask(n, q.device).to(scores.dtype)
    return torch.matmul(scores, v)


def causal_dot_product_recurrent(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """The same O written as a prefix-state recurrence (no N x N matrix):

        S_i = S_{i-1} + k_i v_i^T,   o_i = q_i S_i

    Deliberately shares no code with :func:`causal_dot_product`; the two must
    agree to rounding.  O(N D_qk D_v) memory, so meant for small N.
    """
    kv = torch.einsum("bhnd,bhne->bhnde", k, v).cumsum(dim=2)
    return torch.einsum("bhnd,bhnde->bhne", q, kv)


def causal_dot_product_grads(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, do: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dQ, dK, dV) from the closed-form expressions in the module docstring."""
    n = q.shape[-2]
    mask = _tril_mask(n, q.device)
    a = torch.matmul(q, k.transpose(-2, -1)) * mask.to(q.dtype)
    m = torch.matmul(do, v.transpose(-2, -1)) * mask.to(q.dtype)
    dv = torch.matmul(a.transpose(-2, -1), do)
    dk = torch.matmul(m.transpose(-2, -1), q)
    dq = torch.matmul(m, k)
    return dq, dk, dv


def causal_dot_product_grads_autograd(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, do: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dQ, dK, dV) by autograd through :func:`causal_dot_product`, the way the
    reference's tests obtain them (flashlinear/test_attn.py:107-110)."""
    q, k, v = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    causal_dot_product(q, k, v).backward(do)
    return q.grad, k.grad, v.grad


def linear_attention_normalised(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, eps: float = 1e-5
) -> torch.Tensor:
    """Full linear attention as the reference's README runs it (README.md:27-30):
    the un-normalised product divided by ``(q * cumsum(k)).sum(-1) + eps``."""
    out = causal_dot_product(q, k, v)
    denom = (q * k.cumsum(-2)).sum(dim=-1, keepdim=True) + eps
    return out / denom


def causal_dot_product_blocked(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, block: int = 1024
) -> torch.Tensor:
    """:func:`causal_dot_product` evaluated one block of query rows at a time so
    that long sequences never build the whole N x N score matrix.  Same
    arithmetic per element (one dot product per score, one per output)."""
    n = q.shape[-2]
    out = torch.empty(*q.shape[:-1], v.shape[-1], dtype=q.dtype, device=q.device)
    cols = torch.arange(n, device=q.device)
    for r0 in range(0, n, block):
        r1 = min(n, r0 + block)
        s = torch.matmul(q[..., r0:r1, :], k[..., :r1, :].transpose(-2, -1))
        keep = cols[None, :r1] <= torch.arange(r0, r1, device=q.device)[:, None]
        out[..., r0:r1, :] = torch.matmul(s * keep.to(s.dtype), v[..., :r1, :])
    return out


def causal_dot_product_grads_blocked(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, do: torch.Tensor, block: int = 1024
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Closed-form gradients, one block of query rows at a time (long N)."""
    n = q.shape[-2]
    dq = torch.zeros_like(q)
    dk = torch.zeros_like(k)
    dv = torch.zeros_like(v)
    cols = torch.arange(n, device=q.device)
    for r0 in range(0, n, block):
        r1 = min(n, r0 + block)
        keep = (cols[None, :r1] <= torch.arange(r0, r1, device=q.device)[:, None]).to(q.dtype)
        a = torch.matmul(q[..., r0:r1, :], k[..., :r1, :].transpose(-2, -1)) * keep
        m = torch.matmul(do[..., r0:r1, :], v[..., :r1, :].transpose(-2, -1)) * keep
        dv[..., :r1, :] += torch.matmul(a.transpose(-2, -1), do[..., r0:r1, :])
        dk[..., :r1, :] += torch.matmul(m.transpose(-2, -1), q[..., r0:r1, :])
        dq[..., r0:r1, :] = torch.matmul(m, k[..., :r1, :])
    return dq, dk, dv


def taylor2_features(x: torch.Tensor, coef: Tuple[float, float, float]) -> torch.Tensor:
    """Feature vector phi(x) with phi(x) . phi(y) = c0 + c1 (x . y) + c2 (x . y)^2 for
    non-negative (c0, c1, c2): [sqrt(c0), sqrt(c1) x, sqrt(c2) vec(x x^T)].  With (0, 0, 1/2) this
    is the map ``flatten(x (x) x) / sqrt 2`` of the reference's small-V use case (README.md:3 of
    the reference: Based / Taylor features in front of ``LinearAttentionSmallVHD``)."""
    c0, c1, c2 = coef
    parts = []
    if c0:
        parts.append(torch.full((*x.shape[:-1], 1), c0 ** 0.5, dtype=x.dtype, device=x.device))
    if c1:
        parts.append(c1 ** 0.5 * x)
    if c2:
        parts.append(c2 ** 0.5 * (x[..., :, None] * x[..., None, :]).flatten(-2))
    return torch.cat(parts, dim=-1)


def poly_causal_dot_product(
    xq: torch.Tensor, xk: torch.Tensor, v: torch.Tensor, coef: Tuple[float, float, float]
) -> torch.Tensor:
    """O = tril(f(Xq Xk^T)) V with f(u) = c0 + c1 u + c2 u^2 applied to every score: what
    :func:`causal_dot_product` gives on ``taylor2_features`` of xq and xk, with the features
    never built (the two must agree to rounding; tests/test_oracle.py checks it)."""
    c0, c1, c2 = coef
    n = xq.shape[-2]
    u = torch.matmul(xq, xk.transpose(-2, -1))
    scores = (c0 + c1 * u + c2 * u * u) * _tril_mask(n, xq.device).to(u.dtype)
    return torch.matmul(scores, v)


def poly_linear_attention_normalised(
    xq: torch.Tensor, xk: torch.Tensor, v: torch.Tensor, coef: Tuple[float, float, float], eps: float = 1e-5
) -> torch.Tensor:
    """:func:`linear_attention_normalised` on ``taylor2_features`` of xq and xk without the
    features: every row of :func:`poly_causal_dot_product` divided by the sum of its masked
    scores plus eps (differentiable; tests/test_oracle.py checks it against the explicit form)."""
    c0, c1, c2 = coef
    n = xq.shape[-2]
    u = torch.matmul(xq, xk.transpose(-2, -1))
    scores = (c0 + c1 * u + c2 * u * u) * _tril_mask(n, xq.device).to(u.dtype)
    return torch.matmul(scores, v) / (scores.sum(dim=-1, keepdim=True) + eps)


def poly_causal_dot_product_grads(
    xq: torch.Tensor, xk: torch.Tensor, v: torch.Tensor, do: torch.Tensor, coef: Tuple[float, float, float]
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dXq, dXk, dV) of :func:`poly_causal_dot_product` in closed form:
    dV = S^T dO,  dU = tril(dO V^T) * f'(U),  dXq = dU Xk,  dXk = dU^T Xq."""
    c0, c1, c2 = coef
    n = xq.shape[-2]
    mask = _tril_mask(n, xq.device).to(xq.dtype)
    u = torch.matmul(xq, xk.transpose(-2, -1))
    s = (c0 + c1 * u + c2 * u * u) * mask
    du = torch.matmul(do, v.transpose(-2, -1)) * mask * (c1 + 2.0 * c2 * u)
    return torch.matmul(du, xk), torch.matmul(du.transpose(-2, -1), xq), torch.matmul(s.transpose(-2, -1), do)


def feature_map(x: torch.Tensor, kind: str) -> torch.Tensor:
    """The element-wise positive maps callers put in front of the operators: ``"elu1"`` is
    elu(x) + 1 (= x + 1 for x > 0, e^x otherwise), ``"softplus"`` is log(1 + e^x), the map of the
    reference's tests (flashlinear/test_attn.py:36-40)."""
    if kind == "elu1":
        return torch.nn.functional.elu(x) + 1.0
    if kind == "softplus":
        return torch.nn.functional.softplus(x)
    raise ValueError(kind)


def feature_map_slope(x: torch.Tensor, kind: str) -> torch.Tensor:
    """d phi / d x in closed form: elu1 -> 1 for x > 0, e^x otherwise; softplus -> sigmoid(x)."""
    if kind == "elu1":
        return torch.where(x > 0, torch.ones_like(x), torch.exp(x))
    if kind == "softplus":
        return torch.sigmoid(x)
    raise ValueError(kind)


def feature_causal_dot_product(xq: torch.Tensor, xk: torch.Tensor, v: torch.Tensor, kind: str) -> torch.Tensor:
    """O = tril(phi(Xq) phi(Xk)^T) V: the caller's recipe (feature map, then the operator;
    README.md:27-30 of the reference) as one function of the raw xq, xk."""
    return causal_dot_product(feature_map(xq, kind), feature_map(xk, kind), v)


def feature_causal_dot_product_grads(
    xq: torch.Tensor, xk: torch.Tensor, v: torch.Tensor, do: torch.Tensor, kind: str
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dXq, dXk, dV) in closed form: the product's gradients with respect to phi(xq), phi(xk)
    times the slope of phi."""
    dq, dk, dv = causal_dot_product_grads(feature_map(xq, kind), feature_map(xk, kind), v, do)
    return dq * feature_map_slope(xq, kind), dk * feature_map_slope(xk, kind), dv


def feature_linear_attention_normalised(
    xq: torch.Tensor, xk: torch.Tensor, v: torch.Tensor, kind: str, eps: float = 1e-5
) -> torch.Tensor:
    """:func:`linear_attention_normalised` on phi(xq), phi(xk): the whole caller-side recipe
    (feature map, product, normaliser; README.md:27-30 of the reference) as a function of the raw
    xq, xk.  Differentiable; gradients by autograd."""
    return linear_attention_normalised(feature_map(xq, kind), feature_map(xk, kind), v, eps=eps)
