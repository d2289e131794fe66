"""Pins the oracle's MX block quantiser with properties the mathematics fixes and with an
independent numpy/torch restatement of the OCP MX recipe the reference's golden follows
(examples/utils/gen_mx_quant_allgather_data.py:255-313, :385-449)."""
import numpy as np
import pytest
import torch

import oracle as orc

MAXV = {orc.E4M3: 448.0, orc.E5M2: 57344.0, orc.E2M1: 6.0, orc.E1M2: 1.75}
EMAX = {orc.E4M3: 8, orc.E5M2: 15, orc.E2M1: 2, orc.E1M2: 0}


def make_input(m, k, seed, outliers=True, scale=1.0):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, k)).astype(np.float32) * scale
    if outliers:
        x = np.where(rng.random((m, k)) < 0.001, x * 100, x).astype(np.float32)
    return orc.f32_to_bf16(x)


def unpack_fp4(p, k):
    lo, hi = p & 0xF, p >> 4
    return np.stack([lo, hi], axis=-1).reshape(p.shape[0], -1)[:, :k]


def independent_quant_fp8(x_bf16, fmt):
    """numpy + torch casts only: floor(log2(amax)) via frexp, torch RNE cast after clamp."""
    x = orc.bf16_to_f32(x_bf16).astype(np.float64)
    m, k = x.shape
    nb = (k + 31) // 32
    xp = np.zeros((m, nb * 32))
    xp[:, :k] = x
    blk = xp.reshape(m, nb, 32)
    amax = np.abs(blk).max(-1)
    mant, ex = np.frexp(amax)  # amax = mant * 2^ex, mant in [0.5,1) -> floor(log2) = ex-1
    e = np.where(amax < 1e-12, 0, np.clip(ex - 1 - EMAX[fmt], -128, 127)).astype(np.int64)
    y = blk / np.exp2(e)[..., None]
    y = np.clip(y, -MAXV[fmt], MAXV[fmt]).astype(np.float32)
    dt = torch.float8_e4m3fn if fmt == orc.E4M3 else torch.float8_e5m2
    q = torch.from_numpy(y).to(dt).view(torch.uint8).numpy().reshape(m, nb * 32)[:, :k]
    s = np.full((m, orc.scale_cols(k)), 127, dtype=np.uint8)
    s[:, :nb] = (e + 127).astype(np.uint8)
    return q, s


@pytest.mark.parametrize("fmt", [orc.E4M3, orc.E5M2])
@pytest.mark.parametrize("shape", [(64, 1024), (33, 224), (7, 96), (5, 70)])
def test_fp8_rows_match_independent_recipe(fmt, shape):
    x = make_input(*shape, seed=3)
    q, s = orc.mx_quant_rows(x, fmt, orc.RNE)
    qi, si = independent_quant_fp8(x, fmt)
    assert np.array_equal(s, si)
    assert np.array_equal(q, qi)


@pytest.mark.parametrize("fmt", [orc.E2M1, orc.E1M2])
def test_fp4_rows_match_bruteforce(fmt):
    x = make_input(48, 256, seed=4, scale=0.02)
    p, s = orc.mx_quant_rows(x, fmt, orc.RNE)
    q = unpack_fp4(p, 256)
    xf = orc.bf16_to_f32(x).astype(np.float64).reshape(48, 8, 32)
    amax = np.abs(xf).max(-1)
    e = np.floor(np.log2(amax)) - EMAX[fmt]
    assert np.array_equal(s, (e + 127).astype(np.uint8))
    y = np.clip(xf / np.exp2(e)[..., None], -MAXV[fmt], MAXV[fmt]).reshape(48, 256)
    tab = orc.decode_table(fmt).astype(np.float64)
    d = np.abs(y[..., None] - tab[None, None, :])
    best = d.min(-1)
    # the chosen code is a nearest one, and among ties it has an even mantissa bit
    chosen = tab[q]
    assert np.allclose(np.abs(y - chosen), best, rtol=0, atol=0)
    ties = (np.isclose(d, best[..., None], rtol=0, atol=0).sum(-1) > 1) & (y != 0)
    assert np.all((q[ties] & 1) == 0)
    neg = np.signbit(orc.bf16_to_f32(x))
    assert np.array_equal((q & 8) != 0, neg)  # RNE rule keeps the sign, also on zero results


@pytest.mark.parametrize("fmt", [orc.E4M3, orc.E5M2, orc.E2M1, orc.E1M2])
@pytest.mark.parametrize("rounding", [orc.RNE, orc.LUT])
def test_requantising_dequantised_data_is_identity(fmt, rounding):
    """The check the reference's own run.sh performs: its inputs are dequantised values
    (gen_mx_quant_allgather_data.py:529-534), so quant(dequant(q,s)) == (q,s)."""
    rng = np.random.default_rng(5)
    m, k = 32, 512
    x0 = orc.f32_to_bf16((rng.standard_normal((m, k)) * 10 - 5).astype(np.float32))
    p, s = orc.mx_quant_rows(x0, fmt, rounding)
    deq = orc.mx_dequant_rows(p, s, k, fmt)
    x1 = orc.f32_to_bf16(deq)
    assert np.array_equal(orc.bf16_to_f32(x1), deq)  # exact in bf16 (<=4 significant bits times 2^e)
    p2, s2 = orc.mx_quant_rows(x1, fmt, rounding)
    if rounding == orc.RNE:
        assert np.array_equal(p, p2)
    else:
        assert np.array_equal(p, p2)
    assert np.array_equal(s, s2)


@pytest.mark.parametrize("fmt", [orc.E4M3, orc.E2M1, orc.E1M2])
def test_power_of_two_scaling_shifts_only_the_scale(fmt):
    x = make_input(16, 256, seed=6)
    p, s = orc.mx_quant_rows(x, fmt)
    for sh in (-9, 3, 20):
        xs = orc.f32_to_bf16(orc.bf16_to_f32(x) * np.float32(2.0 ** sh))
        p2, s2 = orc.mx_quant_rows(xs, fmt)
        assert np.array_equal(p, p2)
        assert np.array_equal(s.astype(int) + sh, s2.astype(int))


def test_sign_flip_flips_sign_bits_only():
    x = make_input(16, 256, seed=7)
    p, s = orc.mx_quant_rows(x, orc.E4M3)
    p2, s2 = orc.mx_quant_rows(x ^ np.uint16(0x8000), orc.E4M3)
    assert np.array_equal(s, s2) and np.array_equal(p ^ 0x80, p2)


def test_special_blocks():
    x = np.zeros((1, 160), dtype=np.uint16)
    f = np.zeros((1, 160), dtype=np.float32)
    f[0, 32:64] = 500.0          # amax=500 -> e=0, 500 clamps to 448 (0x7E)
    f[0, 64] = -1e-30            # tiny negative: block below 1e-12 -> scale byte 127, payload -0
    f[0, 96] = np.inf            # Inf block -> scale 0xFF, payload NaN code
    f[0, 128] = 1.0
    f[0, 129] = -2.0 ** -12      # 1.0 sets e=-8; -2^-12*2^8 = -2^-4... representable
    f[0, 130] = -2.0 ** -20      # -2^-12 after scaling: below half the smallest subnormal -> -0
    x = orc.f32_to_bf16(f)
    p, s = orc.mx_quant_rows(x, orc.E4M3, orc.RNE)
    assert s.shape == (1, 6) and list(s[0]) == [127, 127, 127, 255, 119, 127]
    assert np.all(p[0, :32] == 0)
    assert np.all(p[0, 32:64] == 0x7E)
    assert p[0, 64] == 0x80 and np.all(p[0, 65:96] == 0)
    assert np.all((p[0, 96:128] & 0x7F) == 0x7F)
    assert p[0, 128] == orc.encode(np.float32(256.0), orc.E4M3)
    assert p[0, 130] == 0x80
    pl, sl = orc.mx_quant_rows(x, orc.E4M3, orc.LUT)
    assert pl[0, 64] == 0x00 and pl[0, 130] == 0x00 and np.array_equal(sl, s)


def test_ragged_k_zero_pads_last_block_and_pads_scales_with_one():
    x = make_input(4, 70, seed=8)
    p, s = orc.mx_quant_rows(x, orc.E4M3)
    xp = np.zeros((4, 96), dtype=np.uint16)
    xp[:, :70] = x
    pp, sp = orc.mx_quant_rows(xp, orc.E4M3)
    assert np.array_equal(p, pp[:, :70]) and np.array_equal(s[:, :3], sp[:, :3]) and np.all(s[:, 3] == 127)


@pytest.mark.parametrize("fmt", [orc.E4M3, orc.E2M1])
@pytest.mark.parametrize("trans_b", [0, 1])
def test_quant_b_equals_row_quant_of_transpose(fmt, trans_b):
    k, n = 128, 48
    b = make_input(k, n, seed=9, scale=0.5)
    pb, sb = orc.mx_quant_b(b, fmt, orc.RNE, trans_b)
    pt, st = orc.mx_quant_rows(np.ascontiguousarray(b.T), fmt)
    if trans_b:
        assert np.array_equal(pb, pt) and np.array_equal(sb, st)
    else:
        # scales: physical [K/64, N, 2] <- logical [N, K/32]
        assert np.array_equal(sb, st.reshape(n, k // 64, 2).transpose(1, 0, 2))
        if fmt == orc.E4M3:
            assert np.array_equal(pb, pt.T)
        else:
            qt = unpack_fp4(pt, k)          # [N,K] codes
            qb = unpack_fp4(pb, n)          # [K,N] codes
            assert np.array_equal(qb, qt.T)
