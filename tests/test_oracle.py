"""Pins the CPU oracle (runs without a GPU).

The reference holds no golden vectors for this path (its tests draw inputs at
run time on a GPU), so the oracle is pinned by what the mathematics fixes:
closed forms, special cases that reduce to textbook routines, invariants, and
agreement between forms written independently of each other (masked matmul,
prefix-state recurrence, C triple loop, autograd, finite differences).  Each
check is chosen so that a plausible slip -- strict instead of inclusive
diagonal, upper instead of lower triangle, a transposed operand, a dropped
term -- fails at least one of them.
"""

import numpy as np
import pytest
import torch

from oracle import c_oracle, naive


def _rand(shape, seed, dtype=torch.float64):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=dtype)


def test_all_ones_closed_form():
    """q = k = 1, v = 1: O[i, :] = (i + 1) * D_qk; an exclusive diagonal would give i * D_qk."""
    n, dqk, dv = 37, 5, 3
    q = torch.ones(1, 1, n, dqk, dtype=torch.float64)
    v = torch.ones(1, 1, n, dv, dtype=torch.float64)
    want = (torch.arange(1, n + 1, dtype=torch.float64) * dqk)[None, None, :, None].expand(1, 1, n, dv)
    assert torch.equal(naive.causal_dot_product(q, q, v), want)
    assert torch.equal(naive.causal_dot_product_recurrent(q, q, v), want)
    assert np.array_equal(c_oracle.fwd(q, q, v), want.numpy().astype(np.float32))


def test_one_hot_keys_give_prefix_sums_of_v():
    """With q_i = k_j = e_0 the scores are all 1 and O is the inclusive running sum of v:
    a flipped triangle would give suffix sums, a strict one would drop v_i."""
    n, dqk, dv = 23, 4, 6
    q = torch.zeros(1, 2, n, dqk, dtype=torch.float64)
    q[..., 0] = 1
    v = _rand((1, 2, n, dv), 1)
    want = v.cumsum(-2)
    torch.testing.assert_close(naive.causal_dot_product(q, q, v), want, rtol=0, atol=1e-12)
    np.testing.assert_allclose(c_oracle.fwd(q, q, v), want.numpy(), rtol=1e-6, atol=1e-6)


def test_matches_numpy_tril_gemm():
    """One head is just (tril(Q K^T)) V: check against numpy's tril and matmul."""
    q, k, v = _rand((1, 1, 19, 7), 2), _rand((1, 1, 19, 7), 3), _rand((1, 1, 19, 5), 4)
    want = np.tril(q[0, 0].numpy() @ k[0, 0].numpy().T) @ v[0, 0].numpy()
    np.testing.assert_allclose(naive.causal_dot_product(q, k, v)[0, 0].numpy(), want, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(c_oracle.fwd(q, k, v)[0, 0], want, rtol=2e-6, atol=2e-6)


def test_brute_force_python_loops():
    """o[i] = sum_{j<=i} (q_i . k_j) v_j spelled out in Python loops on a tiny case."""
    n, dqk, dv = 6, 3, 2
    q, k, v = _rand((1, 1, n, dqk), 5), _rand((1, 1, n, dqk), 6), _rand((1, 1, n, dv), 7)
    want = torch.zeros(n, dv, dtype=torch.float64)
    for i in range(n):
        for j in range(i + 1):
            a = sum(float(q[0, 0, i, d]) * float(k[0, 0, j, d]) for d in range(dqk))
            for e in range(dv):
                want[i, e] += a * float(v[0, 0, j, e])
    torch.testing.assert_close(naive.causal_dot_product(q, k, v)[0, 0], want, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("shape", [(2, 3, 65, 8, 8), (1, 2, 130, 16, 4), (1, 1, 64, 5, 9)])
def test_forms_agree(shape):
    b, h, n, dqk, dv = shape
    q, k, v = _rand((b, h, n, dqk), 8), _rand((b, h, n, dqk), 9), _rand((b, h, n, dv), 10)
    ref = naive.causal_dot_product(q, k, v)
    torch.testing.assert_close(naive.causal_dot_product_recurrent(q, k, v), ref, rtol=1e-11, atol=1e-11)
    torch.testing.assert_close(naive.causal_dot_product_blocked(q, k, v, block=48), ref, rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(c_oracle.fwd(q, k, v), ref.numpy(), rtol=1e-5, atol=1e-5)


def test_causality_invariant():
    """Changing token j leaves every output row < j untouched, bit for bit."""
    q, k, v = _rand((1, 2, 50, 6), 11), _rand((1, 2, 50, 6), 12), _rand((1, 2, 50, 6), 13)
    base = naive.causal_dot_product(q, k, v)
    j = 31
    k2, v2 = k.clone(), v.clone()
    k2[:, :, j] += 1.0
    v2[:, :, j] -= 2.0
    moved = naive.causal_dot_product(q, k2, v2)
    assert torch.equal(moved[:, :, :j], base[:, :, :j])
    assert not torch.equal(moved[:, :, j], base[:, :, j])


def test_heads_are_independent():
    q, k, v = _rand((2, 3, 40, 4), 14), _rand((2, 3, 40, 4), 15), _rand((2, 3, 40, 4), 16)
    perm = torch.tensor([2, 0, 1])
    a = naive.causal_dot_product(q, k, v)[:, perm]
    b = naive.causal_dot_product(q[:, perm], k[:, perm], v[:, perm])
    assert torch.equal(a, b)


def test_zero_padding_head_dims_changes_nothing():
    q, k, v = _rand((1, 2, 33, 5), 17), _rand((1, 2, 33, 5), 18), _rand((1, 2, 33, 3), 19)
    pad = torch.nn.functional.pad
    base = naive.causal_dot_product(q, k, v)
    wide = naive.causal_dot_product(pad(q, (0, 3)), pad(k, (0, 3)), pad(v, (0, 5)))
    assert torch.equal(wide[..., :3], base)
    assert torch.count_nonzero(wide[..., 3:]) == 0


def test_closed_form_grads_match_autograd_and_c():
    q, k, v, do = _rand((2, 2, 45, 6), 20), _rand((2, 2, 45, 6), 21), _rand((2, 2, 45, 4), 22), _rand((2, 2, 45, 4), 23)
    closed = naive.causal_dot_product_grads(q, k, v, do)
    auto = naive.causal_dot_product_grads_autograd(q, k, v, do)
    blocked = naive.causal_dot_product_grads_blocked(q, k, v, do, block=16)
    c = c_oracle.bwd(q, k, v, do)
    for a, b, bl, cc in zip(closed, auto, blocked, c):
        torch.testing.assert_close(a, b, rtol=1e-11, atol=1e-11)
        torch.testing.assert_close(a, bl, rtol=1e-11, atol=1e-11)
        np.testing.assert_allclose(cc, a.numpy(), rtol=1e-5, atol=1e-5)


def test_gradcheck_fp64():
    q, k, v = (_rand((1, 2, 9, 3), s).requires_grad_(True) for s in (24, 25, 26))
    assert torch.autograd.gradcheck(naive.causal_dot_product, (q, k, v), eps=1e-6, atol=1e-6)


def test_grads_by_finite_differences_of_the_recurrent_form():
    """Directional derivative of <dO, O> computed from the *recurrent* forward
    must equal <grad, direction> with grad from the closed-form expressions."""
    q, k, v, do = _rand((1, 1, 12, 4), 27), _rand((1, 1, 12, 4), 28), _rand((1, 1, 12, 5), 29), _rand((1, 1, 12, 5), 30)
    dq, dk, dv = naive.causal_dot_product_grads(q, k, v, do)
    dirs = [_rand(t.shape, 31 + i) for i, t in enumerate((q, k, v))]
    eps = 1e-6

    def f(q_, k_, v_):
        return float((naive.causal_dot_product_recurrent(q_, k_, v_) * do).sum())

    for idx, (grad, d) in enumerate(zip((dq, dk, dv), dirs)):
        plus = [q, k, v]
        minus = [q, k, v]
        plus[idx] = plus[idx] + eps * d
        minus[idx] = minus[idx] - eps * d
        fd = (f(*plus) - f(*minus)) / (2 * eps)
        assert abs(fd - float((grad * d).sum())) <= 1e-6 * max(1.0, abs(fd))


def test_normalised_recipe_is_a_weighted_average():
    """With positive features the README recipe divides by the row sums of
    tril(QK^T): constant v must come back unchanged (up to eps)."""
    g = torch.Generator().manual_seed(33)
    q = torch.rand(1, 2, 30, 4, generator=g, dtype=torch.float64) + 0.1
    k = torch.rand(1, 2, 30, 4, generator=g, dtype=torch.float64) + 0.1
    v = torch.full((1, 2, 30, 3), 2.5, dtype=torch.float64)
    out = naive.linear_attention_normalised(q, k, v, eps=1e-5)
    torch.testing.assert_close(out, v, rtol=1e-4, atol=0)
    rows = torch.tril(q @ k.transpose(-2, -1)).sum(-1, keepdim=True)
    torch.testing.assert_close((q * k.cumsum(-2)).sum(-1, keepdim=True), rows, rtol=1e-12, atol=1e-12)


def test_c_oracle_rejects_bad_arguments():
    lib = c_oracle._load()
    assert lib.oracle_causal_dot_product_fwd(None, None, None, None, 1, 1, 1, 1) == -1


@pytest.mark.parametrize("coef", [(0.0, 0.0, 0.5), (1.0, 1.0, 0.5), (0.25, 2.0, 0.0)], ids=["square", "taylor", "affine"])
def test_polynomial_score_map_equals_explicit_features(coef):
    """f(x . y) = phi(x) . phi(y): the polynomial form against the plain oracle on the explicit
    feature vectors, forward and all three gradients (the latter by autograd through the
    explicit features, an independent route), in fp64."""
    g = torch.Generator().manual_seed(3)
    xq = torch.randn(2, 2, 40, 6, generator=g, dtype=torch.float64)
    xk = torch.randn(2, 2, 40, 6, generator=g, dtype=torch.float64)
    v = torch.randn(2, 2, 40, 5, generator=g, dtype=torch.float64)
    do = torch.randn(2, 2, 40, 5, generator=g, dtype=torch.float64)
    a, b, c = (t.clone().requires_grad_(True) for t in (xq, xk, v))
    ref = naive.causal_dot_product(naive.taylor2_features(a, coef), naive.taylor2_features(b, coef), c)
    ref.backward(do)
    got = naive.poly_causal_dot_product(xq, xk, v, coef)
    assert torch.allclose(got, ref.detach(), rtol=1e-12, atol=1e-12)
    dxq, dxk, dv = naive.poly_causal_dot_product_grads(xq, xk, v, do, coef)
    for x, y in ((dxq, a.grad), (dxk, b.grad), (dv, c.grad)):
        assert torch.allclose(x, y, rtol=1e-11, atol=1e-11)
    # the reference's feature recipe for the small-V operator is the pure square with c2 = 1/2
    phi = (xq[..., :, None] * xq[..., None, :]).flatten(-2) / 2 ** 0.5
    assert torch.allclose(naive.taylor2_features(xq, (0.0, 0.0, 0.5)), phi)


def test_normalised_polynomial_equals_normalised_recipe_on_explicit_features():
    """The normalised polynomial form against the reference's README recipe (cumsum-based
    normaliser) applied to the explicit features: two routes to the row sums (masked scores
    summed / q . cumsum(k)), output and gradients by autograd on both, in fp64."""
    coef = (1.0, 1.0, 0.5)  # positive scores
    g = torch.Generator().manual_seed(8)
    xq = torch.randn(1, 3, 33, 5, generator=g, dtype=torch.float64)
    xk = torch.randn(1, 3, 33, 5, generator=g, dtype=torch.float64)
    v = torch.randn(1, 3, 33, 7, generator=g, dtype=torch.float64)
    do = torch.randn(1, 3, 33, 7, generator=g, dtype=torch.float64)
    a, b, c = (t.clone().requires_grad_(True) for t in (xq, xk, v))
    ref = naive.linear_attention_normalised(naive.taylor2_features(a, coef), naive.taylor2_features(b, coef), c, 1e-6)
    ref.backward(do)
    a2, b2, c2 = (t.clone().requires_grad_(True) for t in (xq, xk, v))
    got = naive.poly_linear_attention_normalised(a2, b2, c2, coef, 1e-6)
    got.backward(do)
    assert torch.allclose(got.detach(), ref.detach(), rtol=1e-11, atol=1e-11)
    for x, y in ((a2.grad, a.grad), (b2.grad, b.grad), (c2.grad, c.grad)):
        assert torch.allclose(x, y, rtol=1e-10, atol=1e-10)


# ------------------------------------------------------------------ feature maps
def test_feature_maps_closed_forms():
    """elu1: x + 1 right of zero, e^x left of it, 1 at zero, continuous with slope 1 there;
    softplus: log 2 at zero, softplus(x) - softplus(-x) = x, e^x far left, x far right.  A map
    written without the '+ 1', or with the branches swapped, fails."""
    import math

    x = torch.tensor([-30.0, -3.0, -0.5, 0.0, 0.25, 2.0, 30.0], dtype=torch.float64)
    e = naive.feature_map(x, "elu1")
    for xi, ei in zip(x.tolist(), e.tolist()):
        assert ei == pytest.approx(xi + 1.0 if xi > 0 else math.exp(xi), rel=1e-12)
    s = naive.feature_map(x, "softplus")
    assert s[3].item() == pytest.approx(math.log(2.0), rel=1e-12)
    torch.testing.assert_close(s - naive.feature_map(-x, "softplus"), x, rtol=1e-12, atol=1e-12)
    assert s[0].item() == pytest.approx(math.exp(-30.0), rel=1e-9) and s[-1].item() == pytest.approx(30.0, rel=1e-12)
    assert (e > 0).all() and (s > 0).all()
    with pytest.raises(ValueError):
        naive.feature_map(x, "relu")


@pytest.mark.parametrize("kind", ["elu1", "softplus"])
def test_feature_map_slopes_against_central_differences(kind):
    x = torch.linspace(-4.0, 4.0, 41, dtype=torch.float64) + 0.013  # keeps the elu kink off the grid
    h = 1e-6
    fd = (naive.feature_map(x + h, kind) - naive.feature_map(x - h, kind)) / (2 * h)
    torch.testing.assert_close(naive.feature_map_slope(x, kind), fd, rtol=1e-7, atol=1e-8)


@pytest.mark.parametrize("kind", ["elu1", "softplus"])
def test_feature_operator_gradients(kind):
    """Closed-form (dXq, dXk, dV) of O = tril(phi(Xq) phi(Xk)^T) V against autograd through the
    composed function and against central differences of <dO, O> through the *recurrent* form of
    the product: a missing slope factor, or the slope of the wrong operand, fails both."""
    xq, xk, v, do = _rand((1, 2, 9, 4), 31), _rand((1, 2, 9, 4), 32), _rand((1, 2, 9, 3), 33), _rand((1, 2, 9, 3), 34)
    got = naive.feature_causal_dot_product_grads(xq, xk, v, do, kind)
    a, b, c = (t.clone().requires_grad_(True) for t in (xq, xk, v))
    want = torch.autograd.grad(naive.feature_causal_dot_product(a, b, c, kind), (a, b, c), do)
    for g, w in zip(got, want):
        torch.testing.assert_close(g, w, rtol=1e-10, atol=1e-10)

    def scalar(xq_, xk_, v_):
        return (do * naive.causal_dot_product_recurrent(naive.feature_map(xq_, kind), naive.feature_map(xk_, kind), v_)).sum()

    h = 1e-6
    for which, g in enumerate(got):
        base = [xq, xk, v]
        for idx in [(0, 0, 0, 0), (0, 1, 4, 2), (0, 1, 8, 1)]:
            plus, minus = [t.clone() for t in base], [t.clone() for t in base]
            plus[which][idx] += h
            minus[which][idx] -= h
            fd = (scalar(*plus) - scalar(*minus)) / (2 * h)
            assert g[idx].item() == pytest.approx(fd.item(), rel=1e-6, abs=1e-8)


@pytest.mark.parametrize("kind", ["elu1", "softplus"])
def test_feature_recipe_is_a_weighted_average_under_the_map(kind):
    """feature_linear_attention_normalised by what the mathematics fixes, not by its formula:
    (i) both maps are positive, so the scores are positive weights and with eps = 0 every output
    row is a weighted AVERAGE of the value rows so far -- a constant v comes back unchanged, the
    first row is v_0 itself, and every entry lies between the running minimum and maximum of its
    column; (ii) the normaliser the recipe divides by equals the row sums of the masked scores of
    the MAPPED operands, summed by plain loops here; (iii) eps enters as out = O / (n + eps)."""
    xq, xk, v = _rand((1, 2, 11, 5), 41), _rand((1, 2, 11, 5), 42), _rand((1, 2, 11, 3), 43)
    const = torch.full_like(v, 0.75)
    torch.testing.assert_close(naive.feature_linear_attention_normalised(xq, xk, const, kind, eps=0.0), const,
                               rtol=1e-12, atol=1e-12)
    out = naive.feature_linear_attention_normalised(xq, xk, v, kind, eps=0.0)
    torch.testing.assert_close(out[:, :, 0], v[:, :, 0], rtol=1e-12, atol=1e-12)
    lo, hi = torch.cummin(v, dim=-2).values, torch.cummax(v, dim=-2).values
    assert (out >= lo - 1e-12).all() and (out <= hi + 1e-12).all()
    # (ii), (iii): out (n + eps) = unnormalised product, n by explicit loops over the mapped rows
    eps = 0.37
    fq, fk = naive.feature_map(xq, kind), naive.feature_map(xk, kind)
    n = torch.zeros(1, 2, 11, dtype=torch.float64)
    for h in range(2):
        for i in range(11):
            for j in range(i + 1):
                n[0, h, i] += float((fq[0, h, i] * fk[0, h, j]).sum())
    got = naive.feature_linear_attention_normalised(xq, xk, v, kind, eps=eps)
    want = naive.causal_dot_product_recurrent(fq, fk, v) / (n + eps).unsqueeze(-1)
    torch.testing.assert_close(got, want, rtol=1e-12, atol=1e-12)
    # the map matters: on operands with negative entries the unmapped recipe gives something else
    assert not torch.allclose(got, naive.linear_attention_normalised(xq, xk, v, eps=eps))
