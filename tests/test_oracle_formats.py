"""Pins the oracle's number formats and roundings against torch's own casts
(a library, not the reference), closed forms and brute force."""
import numpy as np
import pytest
import torch

import oracle as orc


def _torch_table(dtype):
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    return codes.view(dtype).to(torch.float32).numpy()


def test_e4m3_decode_matches_torch():
    t = orc.decode_table(orc.E4M3)
    ref = _torch_table(torch.float8_e4m3fn)
    assert np.array_equal(np.isnan(t), np.isnan(ref))
    ok = ~np.isnan(ref)
    assert np.array_equal(t[ok].view(np.uint32), ref[ok].view(np.uint32))
    assert t[0x7E] == 448.0 and np.isnan(t[0x7F]) and t[0x01] == 2.0 ** -9


def test_e5m2_decode_matches_torch():
    t = orc.decode_table(orc.E5M2)
    ref = _torch_table(torch.float8_e5m2)
    assert np.array_equal(np.isnan(t), np.isnan(ref))
    ok = ~np.isnan(ref)
    assert np.array_equal(t[ok].view(np.uint32), ref[ok].view(np.uint32))


def test_e8m0_decode_matches_torch():
    t = orc.e8m0_table()
    ref = _torch_table(torch.float8_e8m0fnu)
    assert np.isnan(t[255]) and np.isnan(ref[255])
    assert np.array_equal(t[:255], ref[:255])
    assert t[127] == 1.0


def test_e2m1_table_closed_form():
    t = orc.decode_table(orc.E2M1)
    mags = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    assert list(t[:8]) == mags
    assert list(t[8:]) == [-m for m in mags]
    assert np.signbit(t[8])


def test_e1m2_table_closed_form():
    # one exponent bit, two mantissa bits, bias 1 (gen_mx_quant_allgather_data.py:65-72, :352-375):
    # subnormals m/4, normals 1 + m/4
    t = orc.decode_table(orc.E1M2)
    mags = [0.0, 0.25, 0.5, 0.75, 1.0, 1.25, 1.5, 1.75]
    assert list(t[:8]) == mags
    assert list(t[8:]) == [-m for m in mags]
    assert np.signbit(t[8])


def test_e1m2_ties_and_saturation():
    x = np.array([0.125, 0.375, 0.625, 0.875, 1.125, 1.375, 1.625, 1.8, 9.0, -0.125, -0.375, -1.625, -0.05, -0.0], dtype=np.float32)
    want_rne = [0, 2, 2, 4, 4, 6, 6, 7, 7, 8, 10, 14, 8, 8]
    want_lut = [0, 1, 2, 3, 4, 5, 6, 7, 7, 0, 9, 14, 0, 0]
    assert list(orc.encode(x, orc.E1M2, orc.RNE)) == want_rne
    assert list(orc.encode(x, orc.E1M2, orc.LUT)) == want_lut


def test_bf16_rounding_matches_torch():
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 100,
        rng.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32),
        np.array([0.0, -0.0, np.inf, -np.inf, 1.0 + 2 ** -8, 1.0 + 3 * 2 ** -8, 3.3895314e38], dtype=np.float32),
    ])
    x = x[~np.isnan(x)]
    ours = orc.f32_to_bf16(x)
    ref = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ours, ref)
    L = orc.lib()
    for v in x[:2000]:
        assert L.orc_f32_to_bf16(float(v)) == orc.f32_to_bf16(np.array([v]))[0]
    assert np.array_equal(orc.bf16_to_f32(ours), torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy())


def _sweep(table_pos, maxv):
    """Dense sweep: every code value, every midpoint, thirds between codes, beyond max."""
    pts = []
    for lo, hi in zip(table_pos[:-1], table_pos[1:]):
        d = hi - lo
        pts += [lo, lo + d / 3, lo + d / 2, lo + 2 * d / 3]
        pts += [np.nextafter(np.float32(lo + d / 2), np.float32(0)), np.nextafter(np.float32(lo + d / 2), np.float32(1e9))]
    pts += [table_pos[-1], maxv * 1.01, maxv * 1.07, maxv * 2, 1e30]
    p = np.array(pts, dtype=np.float32)
    return np.concatenate([p, -p])


@pytest.mark.parametrize("fmt,dtype,maxv", [(orc.E4M3, torch.float8_e4m3fn, 448.0), (orc.E5M2, torch.float8_e5m2, 57344.0)])
def test_fp8_rne_encode_matches_torch(fmt, dtype, maxv):
    tab = orc.decode_table(fmt)
    pos = np.sort(tab[:128][np.isfinite(tab[:128])])
    x = _sweep(pos, maxv)
    ours = orc.encode(x, fmt, orc.RNE)
    ref = torch.from_numpy(np.clip(x, -maxv, maxv)).to(dtype).view(torch.uint8).numpy()
    assert np.array_equal(ours, ref)
    # random values too
    rng = np.random.default_rng(1)
    y = (rng.standard_normal(50000) * rng.choice([1e-3, 1, 30, 400], 50000)).astype(np.float32)
    assert np.array_equal(orc.encode(y, fmt, orc.RNE),
                          torch.from_numpy(np.clip(y, -maxv, maxv)).to(dtype).view(torch.uint8).numpy())


@pytest.mark.parametrize("fmt", [orc.E4M3, orc.E5M2, orc.E2M1, orc.E1M2])
def test_lut_encode_is_first_argmin_over_full_table(fmt):
    """The reference's table rule: argmin |LUT - v| over the full signed table, first index wins
    (gen_mx_quant_allgather_data.py:198-247; gen_data_fp4_mx_alltoallv_gmm.py:216-217)."""
    tab = orc.decode_table(fmt).astype(np.float64)
    n = tab.size
    half = n // 2
    maxv = {orc.E4M3: 448.0, orc.E5M2: 57344.0, orc.E2M1: 6.0, orc.E1M2: 1.75}[fmt]
    lut = tab.copy()
    bad = ~np.isfinite(lut)
    lut[bad] = np.where(np.arange(n)[bad] < half, maxv, -maxv)  # reference maps NaN/Inf codes to +-max
    pos = np.sort(np.unique(np.abs(lut)))
    x = _sweep(pos.astype(np.float32), maxv)
    xc = np.clip(x.astype(np.float64), -maxv, maxv)
    brute = np.argmin(np.abs(xc[:, None] - lut[None, :]), axis=1).astype(np.uint8)
    ours = orc.encode(x, fmt, orc.LUT)
    assert np.array_equal(ours, brute)


@pytest.mark.parametrize("fmt", [orc.E4M3, orc.E5M2, orc.E2M1, orc.E1M2])
@pytest.mark.parametrize("rounding", [orc.RNE, orc.LUT])
def test_encode_decode_identity(fmt, rounding):
    tab = orc.decode_table(fmt)
    codes = np.arange(tab.size, dtype=np.uint8)
    ok = np.isfinite(tab)
    enc = orc.encode(tab[ok], fmt, rounding)
    want = codes[ok].copy()
    if rounding == orc.LUT:
        want[tab[ok] == 0] = 0  # table rule canonicalises -0
    assert np.array_equal(enc, want)


def test_e2m1_rne_ties_and_saturation():
    x = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 7.0, 100.0, -0.25, -0.75, -5.0, -0.1, 0.0, -0.0], dtype=np.float32)
    want_rne = [0, 2, 2, 4, 4, 6, 6, 7, 7, 8, 10, 14, 8, 0, 8]
    want_lut = [0, 1, 2, 3, 4, 5, 6, 7, 7, 0, 9, 14, 0, 0, 0]
    assert list(orc.encode(x, orc.E2M1, orc.RNE)) == want_rne
    assert list(orc.encode(x, orc.E2M1, orc.LUT)) == want_lut


def test_shared_exponent_invariant_all_bf16_maxima():
    """2^e <= amax / 2^emax < 2^(e+1) for every positive normal bf16 block maximum."""
    bits = np.arange(0x0080, 0x7F80, dtype=np.uint16)
    vals = orc.bf16_to_f32(bits)
    for emax in (8, 15, 2, 0):
        for v in vals[::37]:
            if v < 1e-12:
                continue
            e, nan = orc.shared_exp(v, emax)
            assert not nan
            if -128 < e < 127:
                r = float(v) / 2.0 ** emax
                assert 2.0 ** e <= r < 2.0 ** (e + 1)
    assert orc.shared_exp(0.0, 8) == (0, False)
    assert orc.shared_exp(5e-13, 8) == (0, False)
    assert orc.shared_exp(float("inf"), 8)[1] and orc.shared_exp(float("nan"), 8)[1]
    assert orc.shared_exp(448.0, 8) == (0, False)
    assert orc.shared_exp(512.0, 8) == (1, False)
    assert orc.shared_exp(1.0, 8) == (-8, False)


def test_round_through_f16_matches_torch():
    rng = np.random.default_rng(2)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * s for s in (1e-7, 1e-4, 1, 1e3, 7e4)])
    ref = torch.from_numpy(x).to(torch.float16).to(torch.float32).numpy()
    L = orc.lib()
    ours = np.array([L.orc_round_through_f16(float(v)) for v in x], dtype=np.float32)
    assert np.array_equal(ours.view(np.uint32), ref.view(np.uint32))
