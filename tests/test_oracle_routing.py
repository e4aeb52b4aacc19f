"""Pins the oracle's gate, top-k and slot assignment: exact-arithmetic restatement, brute force, invariants."""
from fractions import Fraction

import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from oracle import binding as ob


def round_f32(q: Fraction) -> np.float32:
    """Correctly rounded (nearest-even) float32 of an exact rational."""
    if q == 0:
        return np.float32(0.0)
    c = np.float32(float(q))                 # within an ulp or so; fix up exactly below
    cands = sorted({float(np.nextafter(c, np.float32(-np.inf))), float(c), float(np.nextafter(c, np.float32(np.inf)))})
    best = min(cands, key=lambda v: (abs(Fraction(v) - q), int(np.float32(v).view(np.uint32)) & 1))
    return np.float32(best)


def gate_dot_exact(x, w):
    """The documented summation order with every fmaf evaluated in exact rational arithmetic."""
    H = len(x)
    acc = [np.float32(0.0)] * 64
    for k in range(H):
        p = (k // 8) % 64
        acc[p] = round_f32(Fraction(float(x[k])) * Fraction(float(w[k])) + Fraction(float(acc[p])))
    off = 32
    while off >= 1:
        for p in range(off):
            acc[p] = np.float32(acc[p] + acc[p + off])
        off //= 2
    return acc[0]


@pytest.mark.parametrize("dtype,H", [(ob.F32, 64), (ob.F32, 576), (ob.BF16, 1088)])
def test_gate_logits_bit_pattern_and_value(dtype, H):
    rng = np.random.default_rng(5)
    S, E = 3, 4
    x = rng.standard_normal((S, H)).astype(np.float32)
    w = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    bias = rng.standard_normal(E).astype(np.float32)
    if dtype == ob.BF16:
        x, w = ob.f32_to_bf16(x), ob.f32_to_bf16(w)
    xf, wf = ob.to_f32(x, dtype), ob.to_f32(w, dtype)
    got = ob.gate_logits(x, w, bias, dtype)
    for t in range(S):
        for e in range(E):
            want = np.float32(gate_dot_exact(xf[t], wf[e]) + bias[e])
            assert got[t, e].view(np.uint32) == want.view(np.uint32), (t, e)
    ref = xf.astype(np.float64) @ wf.astype(np.float64).T + bias
    assert np.abs(got - ref).max() < 1e-5
    assert np.array_equal(ob.gate_logits(x, w, None, dtype) + bias, got)


def brute_topk(l, k):
    order = sorted(range(len(l)), key=lambda e: (-float(l[e]), e))     # score descending, index ascending
    return order[:k]


@pytest.mark.parametrize("gate_fn", [ob.GATE_SOFTMAX, ob.GATE_SIGMOID])
@pytest.mark.parametrize("norm", [0, 1])
def test_topk_against_brute_force_with_ties(gate_fn, norm):
    rng = np.random.default_rng(6)
    S, E, k = 200, 24, 5
    logits = np.round(rng.standard_normal((S, E)) * 2).astype(np.float32) / 2      # many exact ties
    idx, w = ob.topk(logits, k, gate_fn, norm)
    l64 = logits.astype(np.float64)
    if gate_fn == ob.GATE_SOFTMAX:
        p = np.exp(l64 - l64.max(1, keepdims=True)); p /= p.sum(1, keepdims=True)
    else:
        p = 1 / (1 + np.exp(-l64))
    for t in range(S):
        want = brute_topk(logits[t], k)
        assert list(idx[t]) == want
        pw = p[t, want]
        if norm:
            pw = pw / pw.sum()
        assert np.abs(w[t] - pw).max() < 1e-6
    if norm:
        assert np.abs(w.sum(1) - 1).max() < 1e-6
    # selection is invariant under a common shift of the logits; softmax weights too
    idx2, w2 = ob.topk(logits + np.float32(3.0), k, gate_fn, norm)
    assert np.array_equal(idx, idx2)
    if gate_fn == ob.GATE_SOFTMAX:
        assert np.abs(w - w2).max() < 1e-6


def test_top1_softmax_full_distribution():
    logits = np.array([[0.0, np.log(3.0)]], np.float32)
    idx, w = ob.topk(logits, 2, ob.GATE_SOFTMAX, 0)
    assert list(idx[0]) == [1, 0] and np.allclose(w[0], [0.75, 0.25], atol=1e-6)


def stable_sort_slots(idx, E, drop, cap):
    S, k = idx.shape
    flat = idx.reshape(-1)
    order = np.argsort(flat, kind="stable")
    slot = np.empty(S * k, np.int64)
    start = np.searchsorted(flat[order], np.arange(E))
    for pos, p in enumerate(order):
        slot[p] = pos - start[flat[p]]
    if drop:
        slot[slot >= cap] = -1
    return slot.reshape(S, k)


@settings(max_examples=60, deadline=None)
@given(st.integers(1, 40), st.integers(1, 9), st.integers(1, 4), st.booleans(), st.integers(1, 12), st.integers(0, 2 ** 31))
def test_route_equals_stable_sort(S, E, k, drop, cap, seed):
    k = min(k, E)
    rng = np.random.default_rng(seed)
    idx = np.stack([rng.permutation(E)[:k] for _ in range(S)]).astype(np.int32)
    r = ob.route_slots(idx, E, int(drop), cap)
    want = stable_sort_slots(idx, E, drop, cap)
    assert np.array_equal(r["slot"], want)
    kept = want >= 0
    cnt = np.array([(kept & (idx == e)).sum() for e in range(E)])
    assert np.array_equal(r["expert_count"], cnt)
    assert np.array_equal(r["expert_offset"], np.concatenate([[0], np.cumsum(cnt)[:-1]]))
    if drop:
        assert (r["slot"] < cap).all() and (cnt <= cap).all()
    # packed rows: every kept pair owns exactly one row, rows of an expert are 0..count-1 in pair order
    rows = r["pair_row"][kept]
    assert sorted(rows.tolist()) == list(range(int(cnt.sum())))
    tok = r["token_indices"]
    for t in range(S):
        for j in range(k):
            if kept[t, j]:
                assert tok[r["pair_row"][t, j]] == t
    assert (tok[int(cnt.sum()):] == -1).all()


def test_route_skew_all_tokens_one_expert():
    idx = np.zeros((100, 1), np.int32)
    r = ob.route_slots(idx, 4, 1, 25)
    assert np.array_equal(r["slot"][:25, 0], np.arange(25)) and (r["slot"][25:] == -1).all()
    assert list(r["expert_count"]) == [25, 0, 0, 0]
    r = ob.route_slots(idx, 4, 0, 25)
    assert np.array_equal(r["slot"][:, 0], np.arange(100)) and list(r["expert_count"]) == [100, 0, 0, 0]


# ---- router statistics (load-balancing loss) ----

def test_router_stats_closed_forms():
    S, E, k = 64, 8, 2
    # a uniform router: every score 1/E, assignments spread evenly -> loss exactly 1
    logits = np.zeros((S, E), np.float32)
    idx = np.stack([(np.arange(S) * k + r) % E for r in range(k)], axis=1).astype(np.int32)
    st = ob.router_stats(logits, idx, ob.GATE_SOFTMAX)
    assert np.allclose(st["mean_prob"], 1.0 / E, rtol=0, atol=1e-7)
    assert np.array_equal(st["load"], np.full(E, 1.0 / E, np.float32))
    assert abs(st["aux_loss"] - 1.0) <= 1e-6
    # a router that always picks expert 3 with probability ~1: load one-hot, loss ~E
    logits = np.full((S, E), -40.0, np.float32); logits[:, 3] = 40.0
    idx = np.full((S, 1), 3, np.int32)
    st = ob.router_stats(logits, idx, ob.GATE_SOFTMAX)
    assert st["load"][3] == 1.0 and st["load"].sum() == 1.0
    assert abs(st["mean_prob"][3] - 1.0) <= 1e-6 and abs(st["aux_loss"] - E) <= 1e-5
    # sigmoid scores at logit 0 are 1/2 each
    st = ob.router_stats(np.zeros((S, E), np.float32), idx, ob.GATE_SIGMOID)
    assert np.array_equal(st["mean_prob"], np.full(E, 0.5, np.float32))


@pytest.mark.parametrize("gate_fn", [ob.GATE_SOFTMAX, ob.GATE_SIGMOID])
def test_router_stats_vs_float64(gate_fn):
    rng = np.random.default_rng(5)
    S, E, k = 300, 24, 3
    logits = rng.standard_normal((S, E)).astype(np.float32) * 3
    idx, _ = ob.topk(logits, k, gate_fn, 0)
    st = ob.router_stats(logits, idx, gate_fn)
    l64 = logits.astype(np.float64)
    if gate_fn == ob.GATE_SOFTMAX:
        p = np.exp(l64 - l64.max(1, keepdims=True)); p /= p.sum(1, keepdims=True)
    else:
        p = 1.0 / (1.0 + np.exp(-l64))
    load = np.bincount(idx.reshape(-1), minlength=E) / (S * k)
    assert np.allclose(st["mean_prob"], p.mean(0), rtol=2e-6, atol=0)
    assert np.allclose(st["load"], load, rtol=1e-7, atol=0)
    assert abs(st["aux_loss"] - E * float((load * p.mean(0)).sum())) <= 2e-6 * E
    assert abs(st["load"].sum() - 1.0) <= 1e-6
    if gate_fn == ob.GATE_SOFTMAX:
        assert abs(st["mean_prob"].sum() - 1.0) <= 1e-6


def brute_topk_total(l, k):
    """The total order: NaN ranks as -inf; value descending, index ascending."""
    key = [(-np.inf if np.isnan(v) else float(v)) for v in l]
    return sorted(range(len(l)), key=lambda e: (-key[e], e))[:k]


def test_topk_is_total_with_nan_and_inf_logits():
    """A NaN logit ranks as -inf: every token gets k distinct valid experts, numbers first."""
    nan, inf = np.float32(np.nan), np.float32(np.inf)
    rows = np.array([
        [nan, nan, nan, nan, nan, nan],            # a token row that overflowed: experts 0..k-1
        [nan, 1.0, nan, 3.0, 2.0, nan],            # numbers first, then NaN by index
        [-inf, nan, -inf, 0.5, nan, -inf],         # NaN ties with a real -inf: lower index first
        [inf, nan, 1.0, inf, 0.0, -1.0],
        [0.1, 0.2, 0.3, 0.4, 0.5, 0.6],
    ], np.float32)
    for k in (1, 2, 4, 6):
        for fn in (ob.GATE_SOFTMAX, ob.GATE_SIGMOID):
            idx, w = ob.topk(rows, k, fn, 1)
            for t in range(rows.shape[0]):
                assert list(idx[t]) == brute_topk_total(rows[t], k), (t, k)
                assert len(set(idx[t])) == k and idx[t].min() >= 0 and idx[t].max() < rows.shape[1]
            assert np.isnan(w[0]).all()                       # weights follow the arithmetic: NaN in, NaN out
            assert np.isfinite(w[4]).all() and abs(w[4].sum() - 1) < 1e-6
    idx, _ = ob.topk(rows, 3, ob.GATE_SOFTMAX, 0)
    assert list(idx[0]) == [0, 1, 2] and list(idx[1]) == [3, 4, 1] and list(idx[2]) == [3, 0, 1]


def test_route_drops_expert_ids_outside_the_range():
    """Only a caller-supplied topk_idx can hold them; such a pair is dropped and counted nowhere."""
    E, k = 4, 2
    idx = np.array([[0, 1], [7, 1], [-3, 0], [1, 2**31 - 1], [1, 3]], np.int32)
    r = ob.route_slots(idx, E, 0, 100)
    good = (idx >= 0) & (idx < E)
    assert (r["slot"][~good] == -1).all() and (r["pair_row"][~good] == -1).all()
    assert list(r["expert_count"]) == [2, 4, 0, 1]
    assert r["expert_count"].sum() == good.sum()
    rows = r["pair_row"][good]
    assert sorted(rows) == list(range(good.sum()))
    assert (r["token_indices"][good.sum():] == -1).all()
    st_ = ob.router_stats(np.zeros((5, E), np.float32), idx, ob.GATE_SOFTMAX)
    assert np.allclose(st_["load"] * 10, [2, 4, 0, 1])
