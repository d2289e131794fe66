"""Pins of the oracle's per-token dynamic int8 quantiser (CPU only).

The oracle restates examples/aux_ops/moe_init_routing_quant_v2/moe_v2_gather_dynamic_quant.h:117-150
(mode DQ_DEVICE) and gen_data_dispatch_gmm_dequant_swiglu.py:275-280 (mode DQ_GOLDEN).  It is checked
here against torch's own abs/max/round (golden mode), against a numpy restatement whose half
truncation is a brute-force search over all 65536 half patterns (device mode), and through
properties that hold for any correct implementation."""
import numpy as np
import torch

import oracle as orc


def rand_rows(rng, rows, k, sigma=1.0):
    return orc.f32_to_bf16((rng.standard_normal((rows, k)) * sigma).astype(np.float32))


def all_halves():
    h = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    return np.sort(np.unique(np.abs(h[np.isfinite(h)])))


def test_half_truncation_against_brute_force():
    mags = all_halves()
    rng = np.random.default_rng(0)
    vals = np.concatenate([rng.uniform(-130, 130, 4000), rng.uniform(-1e-4, 1e-4, 500), mags[::97], -mags[::89],
                           np.nextafter(mags[100:2000:7], np.inf), np.nextafter(mags[100:2000:7], -np.inf)]).astype(np.float32)
    L = orc.lib()
    for v in vals:
        want = mags[np.searchsorted(mags, abs(v), side="right") - 1] * (-1.0 if v < 0 else 1.0)
        got = L.orc_trunc_through_f16(float(v))
        assert got == np.float32(want), (v, got, want)


def test_golden_mode_against_torch():
    rng = np.random.default_rng(1)
    for rows, k in [(7, 64), (33, 1000), (4, 7168)]:
        xb = rand_rows(rng, rows, k, 3.0)
        q, s = orc.dyn_quant_i8_rows(xb, mode=orc.DQ_GOLDEN)
        x = torch.from_numpy(orc.bf16_to_f32(xb))
        amax = torch.max(torch.abs(x), dim=-1).values
        want_q = torch.round(x * 127.0 / amax[:, None]).to(torch.int8).numpy()
        want_s = (amax / 127.0).to(torch.float32).numpy()
        assert np.array_equal(q, want_q)
        assert np.array_equal(s, want_s)


def test_device_mode_against_numpy_restatement():
    mags = all_halves()
    rng = np.random.default_rng(2)
    xb = rand_rows(rng, 9, 512, 2.0)
    q, s = orc.dyn_quant_i8_rows(xb, mode=orc.DQ_DEVICE)
    x = orc.bf16_to_f32(xb)
    amax = np.abs(x).max(axis=1)
    sc = (amax / np.float32(127.0)).astype(np.float32)
    y = (x / sc[:, None]).astype(np.float32)
    t = mags[np.searchsorted(mags, np.abs(y), side="right") - 1] * np.sign(y)          # toward zero, to half
    want = (np.sign(t) * np.floor(np.abs(t) + 0.5)).astype(np.int8)                    # halves away from zero
    assert np.array_equal(s, sc)
    assert np.array_equal(q, want)


def test_properties_and_gather():
    rng = np.random.default_rng(3)
    xb = rand_rows(rng, 20, 256)
    xb[5] = 0                                   # an all-zero row
    x = orc.bf16_to_f32(xb)
    for mode, bound in [(orc.DQ_DEVICE, 1.0), (orc.DQ_GOLDEN, 0.5)]:
        q, s = orc.dyn_quant_i8_rows(xb, mode=mode)
        assert np.all(q[5] == 0) and s[5] == 0
        live = np.arange(20) != 5
        assert np.all(np.abs(q[live].astype(np.int32)).max(axis=1) == 127)
        err = np.abs(x - q.astype(np.float32) * s[:, None])
        assert np.all(err[live] <= (bound + 1e-3) * s[live, None])   # fp32 rounding of x*127/amax and of q*scale
    # gather: expanded rows of a top-2 routing, with a dropped and an out-of-range entry
    src = np.array([6, 7, 0, 1, -1, 39, 40, 12], np.int32)
    q, s = orc.dyn_quant_i8_rows(xb, src=src, topk=2)
    q0, s0 = orc.dyn_quant_i8_rows(xb)
    for i, sidx in enumerate(src):
        if sidx < 0 or sidx // 2 >= 20:
            assert np.all(q[i] == 0) and s[i] == 0
        else:
            assert np.array_equal(q[i], q0[sidx // 2]) and s[i] == s0[sidx // 2]


def test_smoothing_against_the_two_restatements():
    """Smoothing multiplies in fp32 first (moe_v2_gather_dynamic_quant.h:127-130); everything after is
    the unsmoothed arithmetic on the products."""
    mags = all_halves()
    rng = np.random.default_rng(4)
    rows, k, experts = 12, 384, 3
    xb = rand_rows(rng, rows, k, 2.0)
    smooth = rng.uniform(0.25, 4.0, (experts, k)).astype(np.float32)
    idx = rng.integers(0, experts, rows).astype(np.int32)
    y = (orc.bf16_to_f32(xb) * smooth[idx]).astype(np.float32)
    amax = np.abs(y).max(axis=1)
    sc = (amax / np.float32(127.0)).astype(np.float32)
    # golden mode against torch
    q, s = orc.dyn_quant_i8_rows(xb, mode=orc.DQ_GOLDEN, smooth=smooth, smooth_rows=idx)
    yt = torch.from_numpy(y)
    want = torch.round(yt * 127.0 / torch.from_numpy(amax)[:, None]).to(torch.int8).numpy()
    assert np.array_equal(q, want) and np.array_equal(s, sc)
    # device mode against the brute-force half truncation
    q, s = orc.dyn_quant_i8_rows(xb, mode=orc.DQ_DEVICE, smooth=smooth, smooth_rows=idx)
    d = (y / sc[:, None]).astype(np.float32)
    t = mags[np.searchsorted(mags, np.abs(d), side="right") - 1] * np.sign(d)
    assert np.array_equal(q, (np.sign(t) * np.floor(np.abs(t) + 0.5)).astype(np.int8)) and np.array_equal(s, sc)
    # one vector for all rows = vector 0
    q1, s1 = orc.dyn_quant_i8_rows(xb, smooth=smooth[0])
    q2, s2 = orc.dyn_quant_i8_rows(xb, smooth=smooth, smooth_rows=np.zeros(rows, np.int32))
    assert np.array_equal(q1, q2) and np.array_equal(s1, s2)


def test_power_of_two_smoothing_equals_prescaled_input():
    """Products with powers of two are exact bf16 values, so the smoothed result is the unsmoothed
    one of the pre-scaled rows; a vector index out of range gives a zero row."""
    rng = np.random.default_rng(5)
    rows, k = 10, 200
    xb = rand_rows(rng, rows, k)
    smooth = np.exp2(rng.integers(-3, 4, (4, k))).astype(np.float32)
    idx = rng.integers(0, 4, rows).astype(np.int32)
    pre = orc.f32_to_bf16(orc.bf16_to_f32(xb) * smooth[idx])
    src = rng.permutation(rows * 2).astype(np.int32)[:rows]       # top-2 expanded rows
    idx[3] = 4
    idx[7] = -1
    for mode in (orc.DQ_DEVICE, orc.DQ_GOLDEN):
        q, s = orc.dyn_quant_i8_rows(xb, src=src, topk=2, mode=mode, smooth=smooth, smooth_rows=idx)
        for i in range(rows):
            if idx[i] < 0 or idx[i] >= 4:
                assert np.all(q[i] == 0) and s[i] == 0
                continue
            row = (orc.bf16_to_f32(xb[src[i] // 2]) * smooth[idx[i]]).astype(np.float32)
            q0, s0 = orc.dyn_quant_i8_rows(orc.f32_to_bf16(row)[None, :], mode=mode)
            assert np.array_equal(q[i], q0[0]) and s[i] == s0[0]
    assert pre.shape == xb.shape
