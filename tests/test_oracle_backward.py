"""Pins the oracle's grouped products (the backward building blocks) against float64 math, one-hot selections and the
adjoint identity that ties a forward product to its two gradients."""
import numpy as np
import pytest

from oracle import binding as ob


def packed_case(rng, E, N, K, counts, dtype, gap=3):
    """Packed expert-major rows with `gap` unused rows behind the last expert (dropped pairs leave such rows)."""
    counts = np.asarray(counts, np.int32)
    offset = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.int32)
    R = int(counts.sum()) + gap
    a = ob.from_f32(rng.standard_normal((R, K)).astype(np.float32), dtype)
    dy = ob.from_f32(rng.standard_normal((R, N)).astype(np.float32), dtype)
    w = ob.from_f32((rng.standard_normal((E, N, K)) * 0.1).astype(np.float32), dtype)
    bias = ob.from_f32(rng.standard_normal((E, N)).astype(np.float32), dtype)
    return a, dy, w, bias, counts, offset


def rows_of(e, counts, offset):
    return slice(int(offset[e]), int(offset[e] + counts[e]))


@pytest.mark.parametrize("dtype", [ob.F32, ob.BF16, ob.F16])
def test_expert_gemm_against_float64(dtype):
    rng = np.random.default_rng(11)
    E, N, K = 5, 24, 40
    a, _, w, bias, counts, offset = packed_case(rng, E, N, K, [7, 0, 13, 1, 5], dtype)
    got = ob.to_f32(ob.expert_gemm(a, w, bias, counts, offset, dtype, ob.ACT_NONE), dtype)
    af, wf, bf = (ob.to_f32(v, dtype).astype(np.float64) for v in (a, w, bias))
    want = np.zeros_like(got, dtype=np.float64)
    for e in range(E):
        r = rows_of(e, counts, offset)
        want[r] = af[r] @ wf[e].T + bf[e]
    tol = {ob.F32: 2e-6, ob.BF16: 2.0 ** -8, ob.F16: 2.0 ** -11}[dtype]
    assert np.abs(got - want).max() <= tol * np.abs(want).max() + 1e-6
    assert not got[int(counts.sum()):].any()                      # rows of no expert are not written
    # a wrong expert for a row must show: evaluate every row with the next expert's weight
    wrong = np.zeros_like(want)
    for e in range(E):
        r = rows_of(e, counts, offset)
        wrong[r] = af[r] @ wf[(e + 1) % E].T + bf[(e + 1) % E]
    assert np.abs(got - wrong).max() > 0.1


@pytest.mark.parametrize("dtype", [ob.F32, ob.BF16, ob.F16])
def test_expert_wgrad_against_float64(dtype):
    rng = np.random.default_rng(12)
    E, N, K = 4, 20, 36
    a, dy, _, _, counts, offset = packed_case(rng, E, N, K, [9, 0, 130, 2], dtype)
    got = ob.to_f32(ob.expert_wgrad(dy, a, counts, offset, dtype), dtype)
    af, dyf = ob.to_f32(a, dtype).astype(np.float64), ob.to_f32(dy, dtype).astype(np.float64)
    want = np.stack([dyf[rows_of(e, counts, offset)].T @ af[rows_of(e, counts, offset)] for e in range(E)])
    tol = {ob.F32: 4e-6, ob.BF16: 2.0 ** -8, ob.F16: 2.0 ** -11}[dtype]
    assert np.abs(got - want).max() <= tol * np.abs(want).max() + 1e-6
    assert not got[1].any()                                       # an expert without rows gets zeros
    # swapped operands (a^T dy instead of dy^T a) have another shape; a shifted row window must show instead
    shifted = np.stack([dyf[int(offset[e]) + 1:int(offset[e] + counts[e]) + 1].T @
                        af[int(offset[e]) + 1:int(offset[e] + counts[e]) + 1] for e in range(E)])
    assert np.abs(got - shifted).max() > 0.1


def test_one_hot_rows_select_weight_columns_and_operand_rows():
    E, N, K = 3, 8, 16
    counts = np.array([2, 1, 3], np.int32); offset = np.array([0, 2, 3], np.int32)
    w = np.arange(E * N * K, dtype=np.float32).reshape(E, N, K)
    a = np.zeros((6, K), np.float32)
    for r in range(6):
        a[r, (5 * r + 1) % K] = 1.0
    out = ob.expert_gemm(a, w, None, counts, offset, ob.F32, ob.ACT_NONE)
    expert_of_row = [0, 0, 1, 2, 2, 2]
    for r in range(6):
        assert np.array_equal(out[r], w[expert_of_row[r], :, (5 * r + 1) % K])
    # wgrad with dy = one-hot(n_r): dw[e][n] is the sum of the operand rows that chose n
    dy = np.zeros((6, N), np.float32)
    choose = [3, 3, 0, 7, 1, 7]
    for r in range(6):
        dy[r, choose[r]] = 1.0
    arows = np.arange(6 * K, dtype=np.float32).reshape(6, K)
    dw = ob.expert_wgrad(dy, arows, counts, offset, ob.F32)
    want = np.zeros((E, N, K), np.float32)
    for r in range(6):
        want[expert_of_row[r], choose[r]] += arows[r]
    assert np.array_equal(dw, want)


def test_adjoint_identity_ties_forward_to_both_gradients():
    """<dY, X W^T> = <dY^T X, W> = <dY W, X>: the three products are each other's adjoints (float32, small integers so
    every sum is exact)."""
    rng = np.random.default_rng(13)
    E, N, K = 4, 12, 20
    counts = np.array([5, 0, 9, 2], np.int32); offset = np.array([0, 5, 5, 14], np.int32)
    R = 16
    x = rng.integers(-3, 4, (R, K)).astype(np.float32)
    dy = rng.integers(-3, 4, (R, N)).astype(np.float32)
    w = rng.integers(-3, 4, (E, N, K)).astype(np.float32)
    y = ob.expert_gemm(x, w, None, counts, offset, ob.F32, ob.ACT_NONE)
    dw = ob.expert_wgrad(dy, x, counts, offset, ob.F32)
    dx = ob.expert_gemm(dy, np.ascontiguousarray(w.transpose(0, 2, 1)), None, counts, offset, ob.F32, ob.ACT_NONE)
    lhs = float((dy.astype(np.float64) * y).sum())
    assert lhs == float((dw.astype(np.float64) * w).sum()) == float((dx.astype(np.float64) * x).sum())
    assert lhs != 0.0


def _f64_act(u, g, act):
    from scipy.special import erf
    if act == ob.ACT_SWIGLU:
        return g / (1 + np.exp(-g)) * u
    if act == ob.ACT_GELU:
        return 0.5 * u * (1 + erf(u / np.sqrt(2)))
    return np.maximum(u, 0)


@pytest.mark.parametrize("act", [ob.ACT_RELU, ob.ACT_GELU, ob.ACT_SWIGLU])
@pytest.mark.parametrize("dtype", [ob.F32, ob.BF16, ob.F16])
def test_act_backward_against_central_differences(dtype, act):
    """d act / d u (and d g) from central differences of the activation in float64: an independent derivative."""
    rng = np.random.default_rng(21)
    shape = (9, 40)
    u = ob.from_f32(rng.standard_normal(shape).astype(np.float32) * 2, dtype)
    g = ob.from_f32(rng.standard_normal(shape).astype(np.float32) * 2, dtype)
    dh = ob.from_f32(rng.standard_normal(shape).astype(np.float32), dtype)
    uf, gf, df = (ob.to_f32(v, dtype).astype(np.float64) for v in (u, g, dh))
    if act == ob.ACT_RELU:
        uf = np.where(np.abs(uf) < 1e-3, 0.5, uf)      # keep the finite difference off the kink
        u = ob.from_f32(uf.astype(np.float32), dtype); uf = ob.to_f32(u, dtype).astype(np.float64)
    du, dg = ob.act_backward(dh, u, g if act == ob.ACT_SWIGLU else None, dtype, act)
    eps = 1e-6
    want_du = df * (_f64_act(uf + eps, gf, act) - _f64_act(uf - eps, gf, act)) / (2 * eps)
    tol = {ob.F32: 2e-5, ob.BF16: 2.0 ** -8, ob.F16: 2.0 ** -10}[dtype]
    assert np.abs(ob.to_f32(du, dtype) - want_du).max() <= tol * max(np.abs(want_du).max(), 1) + 1e-6
    if act == ob.ACT_SWIGLU:
        want_dg = df * (_f64_act(uf, gf + eps, act) - _f64_act(uf, gf - eps, act)) / (2 * eps)
        assert np.abs(ob.to_f32(dg, dtype) - want_dg).max() <= tol * max(np.abs(want_dg).max(), 1) + 1e-6
        assert np.abs(ob.to_f32(dg, dtype) - want_du).max() > 0.05      # du and dg swapped would show
    else:
        assert dg is None


@pytest.mark.parametrize("dtype", [ob.F32, ob.BF16])
def test_bias_grad_is_the_column_sum_per_expert(dtype):
    rng = np.random.default_rng(22)
    E, N = 4, 24
    _, dy, _, _, counts, offset = packed_case(rng, E, N, 8, [7, 0, 130, 2], dtype)
    got = ob.to_f32(ob.bias_grad(dy, counts, offset, dtype), dtype)
    dyf = ob.to_f32(dy, dtype).astype(np.float64)
    want = np.stack([dyf[rows_of(e, counts, offset)].sum(0) for e in range(E)])
    tol = {ob.F32: 1e-5, ob.BF16: 2.0 ** -8}[dtype]
    assert np.abs(got - want).max() <= tol * np.abs(want).max() + 1e-6
    assert not got[1].any()


def test_combine_backward_is_the_adjoint_of_the_combine():
    """<dout, combine(y, w)> must equal <dy, y> and, per pair, dw = d<dout, out>/dw: exact with small integers."""
    rng = np.random.default_rng(23)
    S, k, H, rows = 12, 2, 16, 30
    pair_row = rng.permutation(rows)[:S * k].reshape(S, k).astype(np.int32)
    pair_row[3, 1] = -1; pair_row[7, 0] = -1                         # two dropped pairs
    w = rng.integers(-2, 3, (S, k)).astype(np.float32)
    y = rng.integers(-3, 4, (rows, H)).astype(np.float32)
    dout = rng.integers(-3, 4, (S, H)).astype(np.float32)
    out = ob.combine(y, pair_row, w, H, ob.F32)
    dy, dw = ob.combine_backward(dout, y, pair_row, w, ob.F32)
    want_out = np.zeros((S, H))
    for t in range(S):
        for r in range(k):
            if pair_row[t, r] >= 0:
                want_out[t] += w[t, r] * y[pair_row[t, r]]
    assert np.array_equal(out, want_out.astype(np.float32))      # the forward this is the adjoint of
    assert float((dout * want_out).sum()) == float((dy.astype(np.float64) * y).sum())
    for t in range(S):
        for r in range(k):
            want = float(dout[t] @ y[pair_row[t, r]]) if pair_row[t, r] >= 0 else 0.0
            assert dw[t, r] == want
    used = set(int(v) for v in pair_row.reshape(-1) if v >= 0)
    assert not dy[[i for i in range(rows) if i not in used]].any()
