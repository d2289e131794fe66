"""Pins the oracle's half-input MX quantiser (the reference's MxQuantTraits<half> path,
include/catccos/epilogue/block/block_epilogue_dynamic_mx_quant.hpp:57-71; the reference holds no golden
for half input) with the independent numpy / torch recipe of the OCP rule on the widened values, with
half subnormals as block maxima, and against the bf16 oracle on values both types hold exactly."""
import numpy as np
import pytest
import torch

import oracle as orc
from test_oracle_quant import EMAX, MAXV, unpack_fp4


def half_input(m, k, seed, scale=1.0, outliers=True):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, k)).astype(np.float32) * scale
    if outliers:
        x = np.where(rng.random((m, k)) < 0.001, x * 100, x)
    return x.astype(np.float16)


def independent(x16, fmt):
    """floor(log2(amax)) via frexp on float64, then torch's RNE cast (FP8) or brute-force nearest code (FP4)."""
    x = x16.astype(np.float64)
    m, k = x.shape
    nb = (k + 31) // 32
    xp = np.zeros((m, nb * 32))
    xp[:, :k] = x
    blk = xp.reshape(m, nb, 32)
    amax = np.abs(blk).max(-1)
    _, ex = np.frexp(amax)
    e = np.where(amax < 1e-12, 0, np.clip(ex - 1 - EMAX[fmt], -128, 127)).astype(np.int64)
    y = np.clip(blk / np.exp2(e)[..., None], -MAXV[fmt], MAXV[fmt]).reshape(m, nb * 32)[:, :k]
    s = np.full((m, orc.scale_cols(k)), 127, dtype=np.uint8)
    s[:, :nb] = (e + 127).astype(np.uint8)
    return y, s


@pytest.mark.parametrize("fmt", [orc.E4M3, orc.E5M2])
@pytest.mark.parametrize("shape,scale", [((64, 1024), 1.0), ((33, 224), 30.0), ((7, 96), 1e-3), ((5, 70), 1e-6)])
def test_fp8_matches_independent_recipe(fmt, shape, scale):
    x = half_input(*shape, seed=5, scale=scale)      # scale 1e-6: every value a half subnormal
    q, s = orc.mx_quant_rows_f16(x, fmt, orc.RNE)
    y, si = independent(x, fmt)
    dt = torch.float8_e4m3fn if fmt == orc.E4M3 else torch.float8_e5m2
    qi = torch.from_numpy(y.astype(np.float32)).to(dt).view(torch.uint8).numpy()
    assert np.array_equal(s, si)
    assert np.array_equal(q, qi)


@pytest.mark.parametrize("fmt", [orc.E2M1, orc.E1M2])
def test_fp4_matches_bruteforce_nearest_code(fmt):
    x = half_input(40, 256, seed=6, scale=0.02)
    p, s = orc.mx_quant_rows_f16(x, fmt, orc.RNE)
    y, si = independent(x, fmt)
    assert np.array_equal(s, si)
    tab = orc.decode_table(fmt).astype(np.float64)
    got = tab[unpack_fp4(p, 256)]
    d = np.abs(y[..., None] - tab[None, None, :]).min(-1)
    assert np.array_equal(np.abs(got - y), d)        # a nearest code every time


@pytest.mark.parametrize("fmt", [orc.E4M3, orc.E2M1])
@pytest.mark.parametrize("rounding", [orc.RNE, orc.LUT])
def test_equals_the_bf16_quantiser_where_both_types_hold_the_values(fmt, rounding):
    """Values with 8 significant bits inside half's normal range are exact in bf16 and in half."""
    rng = np.random.default_rng(7)
    x = np.ldexp(rng.integers(-255, 256, (32, 160)).astype(np.float32), rng.integers(-12, 6, (32, 160)))
    xb, xh = orc.f32_to_bf16(x), x.astype(np.float16)
    assert np.array_equal(orc.bf16_to_f32(xb), x) and np.array_equal(xh.astype(np.float32), x)
    qb, sb = orc.mx_quant_rows(xb, fmt, rounding)
    qh, sh = orc.mx_quant_rows_f16(xh, fmt, rounding)
    assert np.array_equal(qb, qh) and np.array_equal(sb, sh)


def test_special_blocks_and_ragged_rows():
    x = np.zeros((3, 70), np.float16)
    x[0, :32] = 0.0                                   # all-zero block: scale byte 127, payload 0
    x[1, 3] = np.inf                                  # Inf block: scale 0xFF, NaN payload
    x[2, 40] = np.nan
    x[2, 69] = 3.0                                    # ragged last block of 6 elements
    q, s = orc.mx_quant_rows_f16(x, orc.E4M3, orc.RNE)
    assert s.shape == (3, 4) and s[0, 0] == 127 and s[1, 0] == 0xFF and s[2, 1] == 0xFF and (s[:, 3] == 127).all()
    assert (q[0] == 0).all() and (q[1, :32] == 0x7F).all() and (q[2, 32:64] == 0x7F).all()
    assert s[2, 2] == 127 + 1 - 8 and q[2, 69] == orc.encode(np.array([3.0 / 2.0 ** -7], np.float32), orc.E4M3)[0]
