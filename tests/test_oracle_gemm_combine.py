"""Pins the oracle's GEMM+epilogue and combine against the reference drivers' known answers and float64 math."""
import numpy as np
import pytest
from scipy.special import erf

from oracle import binding as ob


def collective_operands(dtype):
    """The operands the reference driver builds (mma.cuh:394-411): all zero except 2x2 corners and two biases."""
    M, N, K = 1536, 1152, 4096
    A = np.zeros((M, K), np.float32); B = np.zeros((N, K), np.float32); bias = np.zeros(N, np.float32)
    A[0, 0], A[0, 1], A[1, 0], A[1, 1] = 0, 1, 2, 3
    B[0, 0], B[0, 1], B[1, 0], B[1, 1] = 4, 5, 6, 7
    bias[0], bias[1] = 1, 2
    want = np.zeros((M, N), np.float32)
    want[:, 0] = 1; want[:, 1] = 2
    want[0, 0], want[0, 1], want[1, 0], want[1, 1] = 0 * 4 + 1 * 5 + 1, 0 * 6 + 1 * 7 + 2, 2 * 4 + 3 * 5 + 1, 2 * 6 + 3 * 7 + 2
    A, B, bias = ob.from_f32(A, dtype), ob.from_f32(B, dtype), ob.from_f32(bias, dtype)
    return A, B, bias, want


@pytest.mark.parametrize("dtype", [ob.F32, ob.BF16, ob.F16])
def test_reference_driver_known_answer(dtype):
    A, B, bias, want = collective_operands(dtype)
    C = ob.to_f32(ob.gemm_bias_act(A, B, bias, dtype, ob.ACT_RELU), dtype)
    assert C[0, 0] == 6 and C[0, 1] == 9 and C[1, 0] == 24 and C[1, 1] == 35
    assert np.array_equal(C, want)


@pytest.mark.parametrize("act", [ob.ACT_RELU, ob.ACT_GELU, ob.ACT_NONE])
@pytest.mark.parametrize("dtype", [ob.F32, ob.BF16])
def test_gemm_against_float64(dtype, act):
    rng = np.random.default_rng(3)
    M, N, K = 37, 53, 200
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((N, K)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    if dtype == ob.BF16:
        A, B, bias = ob.f32_to_bf16(A), ob.f32_to_bf16(B), ob.f32_to_bf16(bias)
    Af, Bf, bf = (ob.to_f32(v, dtype).astype(np.float64) for v in (A, B, bias))
    z = Af @ Bf.T + bf                      # add, then activate (processor/tiling.cuh:29-38)
    want = {ob.ACT_RELU: np.maximum(z, 0), ob.ACT_GELU: 0.5 * z * (1 + erf(z / np.sqrt(2))), ob.ACT_NONE: z}[act]
    got = ob.to_f32(ob.gemm_bias_act(A, B, bias, dtype, act), dtype)
    tol = 2e-6 if dtype == ob.F32 else 2.0 ** -8
    assert np.abs(got - want).max() <= tol * np.abs(want).max() + 1e-6
    # a transposed operand or a bias broadcast over rows instead of columns must fail
    assert np.abs(got - (Af @ Bf.T + bf[:M, None] if M <= N else 0)).max() > 0.1


def test_gemm_without_bias_and_operand_roles():
    A = np.zeros((2, 16), np.float32); B = np.zeros((3, 16), np.float32)
    A[1, 5] = 2.0; B[2, 5] = -3.0
    C = ob.gemm_bias_act(A, B, None, ob.F32, ob.ACT_NONE)
    want = np.zeros((2, 3), np.float32); want[1, 2] = -6.0
    assert np.array_equal(C, want)
    assert np.array_equal(ob.gemm_bias_act(A, B, None, ob.F32, ob.ACT_RELU), np.zeros((2, 3), np.float32))


def test_combine_reference_identity_case():
    """hostCombine (combine.cuh:220-231): identity indices, inputs[i][j] = i + 1, M=128, N=64."""
    M, N = 128, 64
    y = np.repeat(np.arange(1, M + 1, dtype=np.float32)[:, None], N, axis=1)
    rows = np.arange(M, dtype=np.int32)[:, None]
    w = np.ones((M, 1), np.float32)
    for dtype in (ob.F32, ob.BF16):
        yy = y if dtype == ob.F32 else ob.f32_to_bf16(y)
        out = ob.to_f32(ob.combine(yy, rows, w, N, dtype), dtype)
        assert np.array_equal(out, y)


def test_combine_permutation_weights_drops_and_linearity():
    rng = np.random.default_rng(4)
    S, k, H = 50, 3, 64
    A = S * k
    y = rng.standard_normal((A, H)).astype(np.float32)
    rows = rng.permutation(A).astype(np.int32).reshape(S, k)
    w = rng.random((S, k)).astype(np.float32)
    rows_d = rows.copy(); rows_d[::4, 1] = -1; rows_d[7, :] = -1
    want = np.zeros((S, H))
    for t in range(S):
        for r in range(k):
            if rows_d[t, r] >= 0:
                want[t] += np.float64(w[t, r]) * y[rows_d[t, r]]
    got = ob.combine(y, rows_d, w, H, ob.F32)
    assert np.abs(got - want).max() < 1e-5
    assert np.array_equal(got[7], np.zeros(H, np.float32))          # every pair dropped -> zero row
    # k = 1, unit weight: a pure row permutation, bit for bit
    p1 = rng.permutation(S).astype(np.int32)[:, None]
    assert np.array_equal(ob.combine(y[:S], p1, np.ones((S, 1), np.float32), H, ob.F32), y[:S][p1[:, 0]])
    # linear in y
    y2 = rng.standard_normal((A, H)).astype(np.float32)
    lhs = ob.combine(y + y2, rows_d, w, H, ob.F32)
    rhs = ob.combine(y, rows_d, w, H, ob.F32) + ob.combine(y2, rows_d, w, H, ob.F32)
    assert np.abs(lhs - rhs).max() < 1e-5
