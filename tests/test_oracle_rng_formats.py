"""Pins the oracle's generator and storage-format conversions against published vectors and torch CPU casts."""
import numpy as np
import pytest
import torch

from oracle import binding as ob

# Random123 known-answer vectors for philox4x32-10 (kat_vectors in the Random123 distribution)
KAT = [
    ([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
    ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
    ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
     [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
]


@pytest.mark.parametrize("ctr,key,want", KAT)
def test_philox_known_answers(ctr, key, want):
    assert [int(v) for v in ob.philox(ctr, key)] == want


def test_normal_is_counter_based_and_standard():
    a = ob.normal(100_003, 42, 7)
    b = ob.normal(50_000, 42, 7)
    assert np.array_equal(a[:50_000], b)            # element i does not depend on n
    assert not np.array_equal(a[:1000], ob.normal(1000, 42, 8))
    assert not np.array_equal(a[:1000], ob.normal(1000, 43, 7))
    z = ob.normal(2_000_000, 1, 1)
    assert abs(z.mean()) < 3e-3 and abs(z.std() - 1) < 3e-3
    assert abs((z ** 3).mean()) < 1e-2 and abs((z ** 4).mean() - 3) < 3e-2
    w = ob.normal(1_000_000, 1, 2, 0.0, 0.02)
    assert abs(w.std() - 0.02) < 1e-4


def test_bf16_every_code_point_round_trips():
    codes = np.arange(65536, dtype=np.uint16)
    f = ob.bf16_to_f32(codes)
    back = ob.f32_to_bf16(f)
    nan = np.isnan(f)
    assert np.array_equal(back[~nan], codes[~nan])
    assert np.isnan(ob.bf16_to_f32(back[nan])).all()


def test_bf16_rounding_matches_torch():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(200_000).astype(np.float32) * 10.0 ** rng.integers(-20, 20, 200_000),
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895e38, 1e-40], np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ob.f32_to_bf16(x), want)


def test_fp16_every_code_point_and_rounding_match_numpy():
    """IEEE binary16 (the reference's torch_dtype 3): every code widens as numpy's float16 does and rounds back to
    itself; round-to-nearest-even on random values over the whole range, on every kind of midpoint and its two
    neighbours, at the overflow threshold and in the subnormals -- against numpy's cast, a library routine."""
    codes = np.arange(65536, dtype=np.uint16)
    wide = ob.f16_to_f32(codes)
    ref = codes.view(np.float16).astype(np.float32)
    assert ((wide.view(np.uint32) == ref.view(np.uint32)) | (np.isnan(wide) & np.isnan(ref))).all()
    finite = ~np.isnan(ref)
    assert np.array_equal(ob.f32_to_f16(wide)[finite], codes[finite])
    rng = np.random.default_rng(0)
    x = rng.standard_normal(300000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 300000).astype(np.float32)
    h = rng.integers(0, 0x7BFF, 100000).astype(np.uint16)
    a = h.view(np.float16).astype(np.float64)
    b = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mid = ((a + b) / 2).astype(np.float32)
    edge = np.array([65504, 65519.996, 65520, 65536, 1e9, -1e9, np.inf, -np.inf, 0, -0.0, 5.96e-8, 2.98e-8,
                     2.9802322e-8, 2.9802326e-8, 6.1e-5, 6.097e-5], np.float32)
    x = np.concatenate([x, -x[:1000], mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)), edge])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(ob.f32_to_f16(x), want)
    nan = ob.f32_to_f16(np.array([np.nan], np.float32))
    assert (nan[0] & 0x7C00) == 0x7C00 and (nan[0] & 0x3FF) != 0


def test_e4m3_decode_matches_torch_for_all_codes():
    codes = np.arange(256, dtype=np.uint8)
    want = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    got = np.array([ob.lib().orc_e4m3_to_f32(int(c)) for c in codes], np.float32)
    nan = np.isnan(want)
    assert set(codes[nan]) == {0x7F, 0xFF}
    assert np.array_equal(got[~nan], want[~nan]) and np.isnan(got[nan]).all()
    assert got[0x7E] == 448.0 and got[0x01] == 2.0 ** -9 and got[0x08] == 2.0 ** -6


def test_e4m3_encode_round_trips_and_matches_torch():
    L = ob.lib()
    for c in range(256):
        if c & 0x7F == 0x7F:
            continue
        assert L.orc_f32_to_e4m3(L.orc_e4m3_to_f32(c)) == c
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(100_000) * 10.0 ** rng.uniform(-4, 2.5, 100_000)).astype(np.float32)
    x = x[np.abs(x) <= 448.0]
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = np.array([L.orc_f32_to_e4m3(float(v)) for v in x], np.uint8)
    assert np.array_equal(got, want)
    # ties go to even, values beyond the largest finite saturate
    assert L.orc_f32_to_e4m3(17.0) == L.orc_f32_to_e4m3(16.0)      # 17 is halfway between 16 and 18
    assert L.orc_f32_to_e4m3(19.0) == L.orc_f32_to_e4m3(20.0)
    assert L.orc_f32_to_e4m3(1e6) == 0x7E and L.orc_f32_to_e4m3(-1e6) == 0xFE


def test_block128_quantisation():
    rng = np.random.default_rng(2)
    w = (rng.standard_normal((2, 256, 384)) * 0.02).astype(np.float32)
    w[1, 128:, :128] = 0.0
    q, s = ob.quant_block128(w)
    assert q.shape == w.shape and s.shape == (2, 2, 3)
    for e in range(2):
        for i in range(2):
            for j in range(3):
                blk = w[e, i * 128:(i + 1) * 128, j * 128:(j + 1) * 128]
                amax = np.abs(blk).max()
                assert s[e, i, j] == (np.float32(amax) / np.float32(448.0) if amax > 0 else 1.0)
    d = ob.dequant_block128(q, s)
    scale = np.repeat(np.repeat(s, 128, axis=1), 128, axis=2)
    # normal range: half an ulp of a 3-bit mantissa = 2^-4 relative; subnormal range: half a step of scale*2^-9
    assert (np.abs(d - w) <= np.maximum(np.abs(w) * 2.0 ** -4, scale * 2.0 ** -10) * (1 + 1e-6)).all()
    assert np.array_equal(np.abs(d).reshape(2, 2, 128, 3, 128).max(axis=(2, 4)) > 0, s != 1.0)


def test_rows128_quantisation():
    """The activation operand of the e4m3 x e4m3 products: one scale per (row, 128 columns).  Pinned by the scale's
    definition computed independently, by torch's own e4m3 cast of x / scale, by every code point, by the error bound of
    a 3-bit significand, and by the independence of rows and column blocks."""
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((7, 300)) * np.exp(rng.uniform(-6, 6, (7, 1)))).astype(np.float32)     # ragged last block (44)
    x[2, 128:256] = 0.0                                                                               # an all-zero piece
    q, s = ob.quant_rows128(x)
    assert q.shape == (7, 300) and s.shape == (7, 3)
    for r in range(7):
        for j in range(3):
            piece = x[r, j * 128:(j + 1) * 128]
            amax = np.abs(piece).max()
            want_s = np.float32(amax) / np.float32(448.0) if amax > 0 else np.float32(1.0)
            assert s[r, j] == want_s
            want_q = torch.from_numpy((piece / want_s).astype(np.float32)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
            assert np.array_equal(q[r, j * 128:(j + 1) * 128], want_q), (r, j)
    assert not q[2, 128:256].any() and s[2, 1] == 1.0
    d = ob.dequant_rows128(q, s)
    scale = np.repeat(s, 128, axis=1)[:, :300]
    assert (np.abs(d - x) <= np.maximum(np.abs(x) * 2.0 ** -4, scale * 2.0 ** -10) * (1 + 1e-6)).all()
    # every finite code point: a piece that holds 448 has scale 1, so its values come back as their own codes
    codes = np.array([c for c in range(256) if c & 0x7F != 0x7F], np.uint8)
    vals = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    row = np.zeros((1, 256), np.float32)
    row[0, :codes.size] = vals
    q1, s1 = ob.quant_rows128(row)
    assert s1[0, 0] == 1.0 and s1[0, 1] == 1.0
    keep = vals != 0                                   # -0.0 and +0.0 may share a code
    assert np.array_equal(q1[0, :codes.size][keep], codes[keep])
    # a power-of-two multiple of the row scales exactly: same codes, scale times that power
    q2, s2 = ob.quant_rows128(row * np.float32(2.0 ** -5))
    assert np.array_equal(q2, q1) and s2[0, 0] == np.float32(2.0 ** -5)
    # rows and column blocks do not see each other
    y = x.copy()
    y[4, 130] = 1e6
    q3, s3 = ob.quant_rows128(y)
    same = np.ones((7, 300), bool)
    same[4, 128:256] = False
    assert np.array_equal(q3[same], q[same]) and s3[4, 1] == np.float32(1e6) / np.float32(448.0)
    assert q3[4, 130] == 0x7E and np.array_equal(np.delete(s3, 1, axis=1), np.delete(s, 1, axis=1))


def test_capacity_formula():
    assert ob.BASELINE["C1"].capacity == 16
    assert ob.BASELINE["C2"].capacity == 640
    assert ob.BASELINE["C3"].capacity == 4096
    assert ob.BASELINE["C4"].capacity == 1536
    assert ob.Cfg(S=10, H=64, I=64, E=3, k=1, capacity_factor=1.0).capacity == 4   # ceil(10/3)
