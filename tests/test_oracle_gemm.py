"""Pins the oracle's GEMM goldens against numpy/torch library routines on small shapes."""
import numpy as np
import pytest
import torch

import oracle as orc
from test_oracle_quant import make_input, unpack_fp4


def test_int8_gemm_dequant_exact_vs_int64():
    rng = np.random.default_rng(10)
    m, k, n = 37, 300, 53
    a = rng.integers(-127, 128, (m, k)).astype(np.int8)
    b = rng.integers(-127, 128, (k, n)).astype(np.int8)
    pt = rng.uniform(0.001, 0.02, m).astype(np.float32)
    pc = rng.uniform(0.001, 0.02, n).astype(np.float32)
    acc = a.astype(np.int64) @ b.astype(np.int64)
    want = acc.astype(np.float32) * pt[:, None] * pc[None, :]
    got, got16 = orc.gemm_i8_dequant(a, b, pt, pc, want_bf16=True)
    assert np.array_equal(got, want)
    assert np.array_equal(got16, orc.f32_to_bf16(want))
    got_t = orc.gemm_i8_dequant(a, np.ascontiguousarray(b.T), pt, pc, trans_b=1)
    assert np.array_equal(got_t, want)
    rows = np.array([5, 0, 36])
    assert np.array_equal(orc.gemm_i8_dequant(a, b, pt, pc, rows=rows), want[rows])


def test_gmm_swiglu_vs_torch():
    rng = np.random.default_rng(11)
    e, k, n = 4, 96, 64
    gs = np.array([5, 0, 9, 3], dtype=np.int32)
    t = int(gs.sum()) + 2  # two rows past the groups stay zero
    x = rng.integers(-127, 128, (t, k)).astype(np.int8)
    w = rng.integers(-127, 128, (e, k, n)).astype(np.int8)
    pt = rng.uniform(0.001, 0.02, t).astype(np.float32)
    pc = rng.uniform(0.001, 0.02, (e, n)).astype(np.float32)
    got = orc.gmm_i8_dequant_swiglu(x, w, gs, pt, pc)
    got_h = orc.gmm_i8_dequant_swiglu(x, w, gs, pt, pc, fp16_step=True)
    want = np.zeros((t, n // 2), dtype=np.float32)
    want_h = np.zeros_like(want)
    r = 0
    for g in range(e):
        for _ in range(gs[g]):
            acc = x[r].astype(np.int64) @ w[g].astype(np.int64)
            c0 = torch.from_numpy(acc.astype(np.float32) * pc[g])
            for half, dst in ((False, want), (True, want_h)):
                c = c0.to(torch.float16).to(torch.float32) if half else c0
                c = c * float(pt[r])
                gate, up = c.chunk(2)
                dst[r] = (torch.nn.functional.silu(gate) * up).numpy()
            r += 1
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-30)
    np.testing.assert_allclose(got_h, want_h, rtol=2e-6, atol=1e-30)
    assert np.all(got[r:] == 0)
    # each group equals the dense routine followed by swiglu
    off = 0
    for g in range(e):
        if gs[g] == 0:
            continue
        sl = slice(off, off + gs[g])
        dense = orc.gemm_i8_dequant(x[sl], w[g], pt[sl], pc[g])
        gate, up = dense[:, : n // 2], dense[:, n // 2:]
        np.testing.assert_allclose(got[sl], gate / (1 + np.exp(-gate.astype(np.float64))) * up, rtol=1e-5)
        off += gs[g]


def _deq_a(p, s, k, fmt):
    tab = orc.decode_table(fmt).astype(np.float64)
    q = unpack_fp4(p, k) if fmt == orc.E2M1 else p
    sc = np.exp2(s.astype(np.float64) - 127)
    return tab[q] * np.repeat(sc, 32, axis=1)[:, :k]


def _deq_b(pb, sb, k, n, fmt, trans_b):
    tab = orc.decode_table(fmt).astype(np.float64)
    if trans_b:
        q = unpack_fp4(pb, k) if fmt == orc.E2M1 else pb          # [N,K]
        sc = np.exp2(sb.astype(np.float64) - 127)                 # [N,K/32]
        return (tab[q] * np.repeat(sc, 32, axis=1)[:, :k]).T
    q = unpack_fp4(pb, n) if fmt == orc.E2M1 else pb              # [K,N]
    logical = sb.transpose(0, 2, 1).reshape(-1, n)                # [K/64,N,2] -> [K/32,N]
    sc = np.exp2(logical.astype(np.float64) - 127)
    return tab[q] * np.repeat(sc, 32, axis=0)[:k]


@pytest.mark.parametrize("fmt", [orc.E4M3, orc.E2M1])
@pytest.mark.parametrize("trans_b", [0, 1])
def test_mx_gemm_vs_fp64(fmt, trans_b):
    m, k, n = 24, 192, 40
    a0 = make_input(m, k, seed=12, outliers=False)
    b0 = make_input(k, n, seed=13, outliers=False)
    pa, sa = orc.mx_quant_rows(a0, fmt)
    pb, sb = orc.mx_quant_b(b0, fmt, orc.RNE, trans_b)
    got, got64 = orc.mx_gmm(pa, sa, pb, sb, n, k, fmt, trans_b, want_f64=True)
    want = _deq_a(pa, sa, k, fmt) @ _deq_b(pb, sb, k, n, fmt, trans_b)
    np.testing.assert_allclose(got64, want, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)
    # the quantised product is close to the unquantised one (sanity of the whole chain)
    full = orc.bf16_to_f32(a0).astype(np.float64) @ orc.bf16_to_f32(b0).astype(np.float64)
    rel = np.abs(want - full).max() / np.abs(full).max()
    assert rel < (0.08 if fmt == orc.E4M3 else 0.4)


def test_mx_gemm_unit_scales_is_plain_fp8_gemm():
    rng = np.random.default_rng(14)
    m, k, n = 8, 64, 16
    pa = rng.integers(0, 0x7F, (m, k)).astype(np.uint8) | (rng.integers(0, 2, (m, k)).astype(np.uint8) << 7)
    pa[(pa & 0x7F) == 0x7F] = 0
    pb = rng.integers(0, 0x7F, (k, n)).astype(np.uint8)
    sa = np.full((m, 2), 127, np.uint8)
    sb = np.full((1, n, 2), 127, np.uint8)
    got = orc.mx_gmm(pa, sa, pb, sb, n, k, orc.E4M3, 0, want_f64=True)[1]
    ta = torch.from_numpy(pa).view(torch.float8_e4m3fn).to(torch.float64)
    tb = torch.from_numpy(pb).view(torch.float8_e4m3fn).to(torch.float64)
    np.testing.assert_allclose(got, (ta @ tb).numpy(), rtol=1e-13)


def test_mx_gemm_one_hot_rows_copy_scaled_b_rows():
    k, n = 64, 24
    b0 = make_input(k, n, seed=15, outliers=False)
    pb, sb = orc.mx_quant_b(b0, orc.E4M3, orc.RNE, 0)
    pa = np.zeros((2, k), np.uint8)
    pa[0, 5] = 0x38   # 1.0
    pa[1, 40] = 0xC0  # -2.0
    sa = np.array([[127, 127], [127, 130]], np.uint8)  # second row: block 1 scaled by 8
    got = orc.mx_gmm(pa, sa, pb, sb, n, k, orc.E4M3, 0)
    bd = _deq_b(pb, sb, k, n, orc.E4M3, 0)
    assert np.array_equal(got[0], bd[5].astype(np.float32))
    assert np.array_equal(got[1], (-16.0 * bd[40]).astype(np.float32))


def test_grouped_mx_equals_per_group_dense():
    fmt = orc.E2M1
    e, k, n = 3, 128, 32
    gs = np.array([4, 0, 7], np.int32)
    t = 13
    a0 = make_input(t, k, seed=16, outliers=False, scale=0.02)
    pa, sa = orc.mx_quant_rows(a0, fmt)
    pbs, sbs = [], []
    for g in range(e):
        pb, sb = orc.mx_quant_b(make_input(k, n, seed=17 + g, outliers=False, scale=0.02), fmt, orc.RNE, 0)
        pbs.append(pb), sbs.append(sb)
    got = orc.mx_gmm(pa, sa, np.stack(pbs), np.stack(sbs), n, k, fmt, 0, group_sizes=gs)
    off = 0
    for g in range(e):
        sl = slice(off, off + gs[g])
        if gs[g]:
            dense = orc.mx_gmm(pa[sl], sa[sl], pbs[g], sbs[g], n, k, fmt, 0)
            assert np.array_equal(got[sl], dense)
        off += gs[g]
    assert np.all(got[off:] == 0)
    rows = np.array([10, 2])
    assert np.array_equal(orc.mx_gmm(pa, sa, np.stack(pbs), np.stack(sbs), n, k, fmt, 0, group_sizes=gs, rows=rows), got[rows])


def test_compare_metrics_vs_numpy():
    rng = np.random.default_rng(18)
    g = rng.standard_normal(1000).astype(np.float32) * 3
    d = g + rng.standard_normal(1000).astype(np.float32) * 0.01
    m = orc.compare(d, g, rtol=2 ** -7)
    f1 = np.maximum(np.abs(g.astype(np.float64)), 1)
    rms = np.sqrt(np.mean(g.astype(np.float64) ** 2))
    diff = np.abs(d.astype(np.float64) - g)
    assert np.isclose(m["max_rel_floor1"], (diff / f1).max())
    assert np.isclose(m["max_rel_floor_rms"], (diff / np.maximum(np.abs(g), rms)).max())
    assert np.isclose(m["eb"], ((d.astype(np.float64) - g) / f1).mean())
    assert np.isclose(m["rms_golden"], rms)


def test_double_golden_metric_vs_torch_restatement_and_closed_forms():
    """The reference's acceptance metric for the MXFP8 dense operator (examples/utils/verify_result.py:198-246 with the
    verdict of :105-117): pinned by a torch restatement of those lines in fp32 (NaN and Inf replaced by zero first) and
    by what the formulas fix: a result equal to the golden has zero ratios, a result equal to the low-precision golden
    has ratios of exactly one wherever that golden's own error lies above the 2^-8 floor, and below the floor the
    denominator is the floor."""
    import torch
    rng = np.random.default_rng(19)
    g = (rng.standard_normal(5000) * 30).astype(np.float32)
    g[:5] = [0.0, 1e-6, -3e-5, np.inf, np.nan]
    low = orc.bf16_to_f32(orc.f32_to_bf16(g))
    d = (g * (1 + rng.standard_normal(5000) * 2e-3)).astype(np.float32)
    d[7] = np.nan
    got = orc.compare_double(d, g, low)
    td, tg, tl = (torch.nan_to_num(torch.from_numpy(x), nan=0.0, posinf=0.0, neginf=0.0) for x in (d, g, low))
    da, dl = td - tg, tl - tg
    ra, rl = da.abs() / (tg.abs() + 1e-7), dl.abs() / (tg.abs() + 1e-7)
    thr = 2.0 ** -8
    want = {
        "max_rel_ratio": float(ra.max()) / max(float(rl.max()), thr),
        "mean_rel_ratio": float(ra.mean()) / max(float(rl.mean()), thr),
        "rmse_ratio": float((da ** 2).mean().sqrt()) / max(float((dl ** 2).mean().sqrt()), thr),
        "eb_percent": abs(float((da / torch.maximum(torch.ones_like(tg), tg.abs())).mean())) / 2.0 ** -7 * 100,
    }
    for key, val in want.items():
        assert np.isclose(got[key], val, rtol=1e-4), (key, got[key], val)
    same = orc.compare_double(g, g, low)
    assert same["max_rel_ratio"] == 0 and same["mean_rel_ratio"] == 0 and same["rmse_ratio"] == 0 and same["eb_percent"] == 0 and same["ok"]
    # a coarse "low" golden (error above the floor): a result equal to it has ratios of one
    coarse = (g * (1 + 0.05 * np.sign(rng.standard_normal(5000)))).astype(np.float32)
    one = orc.compare_double(coarse, g, coarse)
    assert one["max_rel_ratio"] == 1 and one["mean_rel_ratio"] == 1 and one["rmse_ratio"] == 1
    # below the floor the floor is the denominator: the bf16 golden's mean relative error is about 2^-10
    fl = orc.compare_double(low, g, low)
    assert fl["mean_rel_low"] < thr and np.isclose(fl["mean_rel_ratio"], fl["mean_rel"] / thr)
    # the verdict's four limits
    bad = orc.compare_double((g * 1.2).astype(np.float32), g, low)
    assert not bad["ok"] and bad["mean_rel_ratio"] > 2 and bad["rmse_ratio"] > 2
    # a constant offset of 1 on goldens of magnitude 4: eb = 1/4 of 2^-7 scaled to percent, far past 100
    four = np.where(rng.standard_normal(64) > 0, 4.0, -4.0).astype(np.float32)
    off = orc.compare_double(four + 1, four, four)
    assert np.isclose(off["eb_percent"], 0.25 / 2.0 ** -7 * 100) and not off["ok"]


def test_swiglu_bf16_against_torch_and_closed_forms():
    """The SwiGLU of a bf16 tile (gate | up halves): torch's silu on the widened values, rounded to
    bf16, is the independent check.  The oracle divides gate by 1 + exp(-gate) where torch multiplies by a
    sigmoid: both are fp32 and may round one fp32 step apart, which moves the bf16 result by at most one
    step and only on a small share of the inputs."""
    import torch
    rng = np.random.default_rng(8)
    t, n = 300, 256
    c = orc.f32_to_bf16((rng.standard_normal((t, n)) * 3.0).astype(np.float32))
    got = orc.swiglu_bf16(c)
    cf = torch.from_numpy(orc.bf16_to_f32(c))
    want = (torch.nn.functional.silu(cf[:, : n // 2]) * cf[:, n // 2:]).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    diff = np.abs(got.astype(np.int32) - want.astype(np.int32))
    assert diff.max() <= 1 and np.mean(diff == 0) > 0.99, (diff.max(), np.mean(diff == 0))
    # closed forms: gate 0 -> 0; gate = 40 -> gate * up exactly (exp(-40) vanishes against 1); gate = -100 -> -0 * up
    z = np.zeros((1, 4), np.float32)
    z[0] = [0.0, 40.0, 3.0, -2.5]            # gates 0 and 40, ups 3 and -2.5
    out = orc.bf16_to_f32(orc.swiglu_bf16(orc.f32_to_bf16(z)))
    assert out[0, 0] == 0.0 and out[0, 1] == -100.0
    z[0] = [-100.0, 1.0, 7.0, 2.0]
    out = orc.bf16_to_f32(orc.swiglu_bf16(orc.f32_to_bf16(z)))
    assert out[0, 0] == 0.0 and abs(out[0, 1] - 2.0 * 0.7310586) < 0.01
    # a swapped gate and up would fail this one: silu(1) * 2 != silu(2) * 1
    assert abs(out[0, 1] - 2.0 / (1.0 + np.exp(-1.0))) < 0.01 and abs(out[0, 1] - 2.0 / (1.0 + np.exp(-2.0))) > 0.1
