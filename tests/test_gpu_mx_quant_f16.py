"""GPU parity of the half-input MX quantiser (cch_mx_quant_rows_f16) against the oracle: bit-exact
payload and scale bytes for every format and both rounding rules, on vector and ragged row lengths,
on every half bit pattern under several block maxima, on special blocks and at config-1 size."""
import numpy as np
import pytest
import torch

import oracle as orc
import catccos_amd as cc

pytestmark = pytest.mark.gpu
FMTS = {"e4m3": orc.E4M3, "e5m2": orc.E5M2, "e2m1": orc.E2M1, "e1m2": orc.E1M2}


def run(x16, fmt, rounding):
    xd = torch.from_numpy(np.ascontiguousarray(x16).view(np.int16)).cuda().view(torch.float16)
    q, s = cc.mx_quant(xd, fmt, rounding)
    torch.cuda.synchronize()
    return q.cpu().numpy(), s.cpu().numpy()


def check(x16, fmt, rounding=orc.RNE):
    q, s = run(x16, fmt, rounding)
    qo, so = orc.mx_quant_rows_f16(x16, FMTS[fmt], rounding)
    assert np.array_equal(s, so), (fmt, rounding, "scales")
    assert np.array_equal(q, qo), (fmt, rounding, "payload")


@pytest.mark.parametrize("fmt", list(FMTS))
@pytest.mark.parametrize("rounding", [orc.RNE, orc.LUT])
@pytest.mark.parametrize("shape", [(64, 1024), (130, 7168), (33, 224), (9, 70), (5, 33), (3, 1), (17, 96)])
def test_random_rows(fmt, rounding, shape):
    rng = np.random.default_rng([FMTS[fmt], rounding, shape[0], shape[1]])
    x = rng.standard_normal(shape).astype(np.float32) * rng.choice([1e-6, 1e-3, 1.0, 50.0], size=(shape[0], 1))
    x = np.where(rng.random(shape) < 0.001, x * 100, x)
    check(x.astype(np.float16), fmt, rounding)


@pytest.mark.parametrize("fmt", list(FMTS))
def test_every_half_pattern_under_several_block_maxima(fmt):
    """All 65536 bit patterns (Inf/NaN included: their blocks turn into NaN blocks), 31 per block next to
    one element that sets the block maximum: a large, a mid, a small normal and a subnormal one."""
    pats = np.arange(65536, dtype=np.uint16)
    pad = (-len(pats)) % 31
    body = np.concatenate([pats, np.zeros(pad, np.uint16)]).reshape(-1, 31)
    for top in (0x7BFF, 0x5640, 0x3C00, 0x0400, 0x0003):     # 65504, 100, 1, 2^-14, 3 * 2^-24
        x = np.concatenate([np.full((body.shape[0], 1), top, np.uint16), body], axis=1).reshape(-1, 32 * 5)   # 2115 blocks = 423 rows of 5
        check(x.view(np.float16), fmt)


def test_special_blocks():
    x = np.zeros((4, 96), np.float16)
    x[1, 5] = np.inf
    x[2, 40] = -np.inf
    x[3, 70] = np.nan
    x[3, :32] = 65504.0
    for fmt in FMTS:
        check(x, fmt)


def test_config1_size_sampled_rows_and_scale_shift():
    """[4096, 7168] as config 1: a sample of rows against the oracle, and the power-of-two shift
    property on the whole tensor (payload unchanged, scale bytes moved by the shift)."""
    rng = np.random.default_rng(1)
    x = rng.standard_normal((4096, 7168)).astype(np.float32)
    x = np.where(rng.random(x.shape) < 0.001, x * 100, x).astype(np.float16)
    q, s = run(x, "e4m3", orc.RNE)
    rows = rng.choice(4096, 64, replace=False)
    qo, so = orc.mx_quant_rows_f16(x[rows], orc.E4M3, orc.RNE)
    assert np.array_equal(q[rows], qo) and np.array_equal(s[rows], so)
    q2, s2 = run((x.astype(np.float32) * 0.25).astype(np.float16), "e4m3", orc.RNE)   # exact in half away from subnormals
    big = np.abs(x.astype(np.float32)).reshape(4096, -1, 32).min(-1) > 1e-3          # blocks without tiny values
    assert np.array_equal(q.reshape(4096, -1, 32)[big], q2.reshape(4096, -1, 32)[big])
    assert np.array_equal(s[:, :224][big].astype(np.int32) - 2, s2[:, :224][big].astype(np.int32))
