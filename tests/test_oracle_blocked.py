"""The cache-blocked CPU GEMMs (the benchmark's CPU baseline) against the row-at-a-time goldens.

Both accumulate every output in ascending k with one fused multiply-add per term (fp32) or in
exact int32, so the blocked routines must give the same bits: ragged shapes (K, N and row counts
that are no multiples of the block sizes), both layouts of B, every payload format, row samples in
arbitrary order, empty groups and rows that belong to no group."""
import numpy as np
import pytest

import oracle as orc

FMT = {"e4m3": orc.E4M3, "e5m2": orc.E5M2, "e2m1": orc.E2M1}


def rand_bf16(rng, shape, sigma=1.0):
    return orc.f32_to_bf16((rng.standard_normal(shape) * sigma).astype(np.float32))


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e2m1"])
@pytest.mark.parametrize("trans_b", [0, 1])
@pytest.mark.parametrize("shape", [(37, 200, 320), (130, 136, 96), (5, 384, 1216)])
def test_mx_dense_blocked_equals_golden(fmt, trans_b, shape):
    m, n, k = shape
    rng = np.random.default_rng(m + n + k + trans_b)
    sigma = 0.02 if fmt == "e2m1" else 1.0
    pa, sa = orc.mx_quant_rows(rand_bf16(rng, (m, k), sigma), FMT[fmt])
    pb, sb = orc.mx_quant_b(rand_bf16(rng, (k, n), sigma), FMT[fmt], orc.RNE, trans_b)
    want, want16 = orc.mx_gmm(pa, sa, pb, sb, n, k, FMT[fmt], trans_b, want_bf16=True)
    got, got16 = orc.mx_gmm(pa, sa, pb, sb, n, k, FMT[fmt], trans_b, want_bf16=True, blocked=True)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(got16, want16)


@pytest.mark.parametrize("fmt", ["e4m3", "e2m1"])
@pytest.mark.parametrize("trans_b", [0, 1])
def test_mx_grouped_blocked_equals_golden(fmt, trans_b):
    e, t, n, k = 5, 300, 264, 448
    gs = np.array([0, 140, 1, 0, 150], np.int32)   # 9 rows belong to no group
    rng = np.random.default_rng(3 + trans_b)
    sigma = 0.02 if fmt == "e2m1" else 1.0
    pa, sa = orc.mx_quant_rows(rand_bf16(rng, (t, k), sigma), FMT[fmt])
    pbs, sbs = zip(*[orc.mx_quant_b(rand_bf16(rng, (k, n), sigma), FMT[fmt], orc.RNE, trans_b) for _ in range(e)])
    pb, sb = np.stack(pbs), np.stack(sbs)
    want = orc.mx_gmm(pa, sa, pb, sb, n, k, FMT[fmt], trans_b, group_sizes=gs)
    got = orc.mx_gmm(pa, sa, pb, sb, n, k, FMT[fmt], trans_b, group_sizes=gs, blocked=True)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.all(got[291:] == 0)
    rows = rng.permutation(t)[:77].astype(np.int64)   # unsorted sample, rows of no group included
    got = orc.mx_gmm(pa, sa, pb, sb, n, k, FMT[fmt], trans_b, group_sizes=gs, rows=rows, blocked=True)
    assert np.array_equal(got.view(np.uint32), want[rows].view(np.uint32))


@pytest.mark.parametrize("trans_b", [0, 1])
def test_i8_dequant_blocked_equals_golden(trans_b):
    m, n, k = 67, 200, 300
    rng = np.random.default_rng(9 + trans_b)
    a = rng.integers(-128, 128, (m, k)).astype(np.int8)
    b = rng.integers(-128, 128, (k, n)).astype(np.int8)
    pt = rng.uniform(0.001, 0.02, m).astype(np.float32)
    pc = rng.uniform(0.001, 0.02, n).astype(np.float32)
    bb = np.ascontiguousarray(b.T) if trans_b else b
    want = orc.gemm_i8_dequant(a, bb, pt, pc, trans_b)
    got = orc.gemm_i8_dequant(a, bb, pt, pc, trans_b, blocked=True)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # exact integer sums, independently: int64 matmul
    ref = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32) * pt[:, None] * pc[None, :]
    assert np.array_equal(got, ref)
    rows = np.array([66, 0, 13], np.int64)
    got = orc.gemm_i8_dequant(a, bb, pt, pc, trans_b, rows=rows, blocked=True)
    assert np.array_equal(got, want[rows])


@pytest.mark.parametrize("fp16_step", [False, True])
def test_gmm_swiglu_blocked_equals_golden(fp16_step):
    e, t, k, n = 4, 150, 264, 272
    gs = np.array([70, 0, 9, 60], np.int32)
    rng = np.random.default_rng(21)
    x = rng.integers(-127, 128, (t, k)).astype(np.int8)
    w = rng.integers(-127, 128, (e, k, n)).astype(np.int8)
    pt = rng.uniform(0.001, 0.02, t).astype(np.float32)
    pc = rng.uniform(0.001, 0.02, (e, n)).astype(np.float32)
    want, want16 = orc.gmm_i8_dequant_swiglu(x, w, gs, pt, pc, fp16_step, want_bf16=True)
    got, got16 = orc.gmm_i8_dequant_swiglu(x, w, gs, pt, pc, fp16_step, want_bf16=True, blocked=True)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(got16, want16)
    rows = np.array([149, 3, 75, 139], np.int64)
    got = orc.gmm_i8_dequant_swiglu(x, w, gs, pt, pc, fp16_step, rows=rows, blocked=True)
    assert np.array_equal(got.view(np.uint32), want[rows].view(np.uint32))
