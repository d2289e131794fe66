"""GPU parity of the per-token dynamic int8 quantiser against the oracle: bit-exact int8 rows and
fp32 scales, both rounding modes, register path and two-pass path, gather with dropped rows."""
import numpy as np
import pytest
import torch

import oracle as orc
import catccos_amd as cc

pytestmark = pytest.mark.gpu


def rand_rows(rng, rows, k, sigma=1.0):
    return orc.f32_to_bf16((rng.standard_normal((rows, k)) * sigma).astype(np.float32))


def dev_bf16(bits):
    return torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16)


@pytest.mark.parametrize("mode", [cc.DQ_DEVICE, cc.DQ_GOLDEN])
@pytest.mark.parametrize("shape", [(64, 512), (300, 7168), (17, 1000), (5, 8200), (3, 12288), (9, 8), (2, 7),
                                   (10, 4096), (7, 3000), (5, 2048), (3, 16384), (2, 20000), (1, 7168)])
def test_dyn_quant_bit_exact(shape, mode):
    rows, k = shape
    rng = np.random.default_rng(rows * 131 + k + mode)
    xb = rand_rows(rng, rows, k, 2.5)
    xb[rows // 2] = 0
    xb[0, : min(k, 3)] = orc.f32_to_bf16(np.array([100.0, -100.0, 0.5], np.float32))[: min(k, 3)]
    q, s = cc.dynamic_quant_i8(dev_bf16(xb), mode=mode)
    torch.cuda.synchronize()
    wq, ws = orc.dyn_quant_i8_rows(xb, mode=mode)
    assert np.array_equal(s.cpu().numpy(), ws)
    assert np.array_equal(q.cpu().numpy(), wq)


def test_dyn_quant_ties_and_extremes():
    # rows built so that x / scale lands on .5 boundaries and on half-precision truncation edges
    k = 512
    base = np.zeros((4, k), np.float32)
    base[:, 0] = 127.0                                  # amax = 127 -> scale = 1
    base[0, 1:200] = np.arange(1, 200) * 0.5            # exact halves
    base[1, 1:200] = -np.arange(1, 200) * 0.5
    base[2, 1:300] = np.linspace(0.01, 126.99, 299)
    base[3, 1:300] = -np.linspace(63.5, 126.99, 299)
    xb = orc.f32_to_bf16(base)
    for mode in (cc.DQ_DEVICE, cc.DQ_GOLDEN):
        q, s = cc.dynamic_quant_i8(dev_bf16(xb), mode=mode)
        torch.cuda.synchronize()
        wq, ws = orc.dyn_quant_i8_rows(xb, mode=mode)
        assert np.array_equal(q.cpu().numpy(), wq) and np.array_equal(s.cpu().numpy(), ws)


def test_dyn_quant_gather():
    rng = np.random.default_rng(7)
    rows, k, topk = 100, 1024, 2
    xb = rand_rows(rng, rows, k)
    src = rng.permutation(rows * topk).astype(np.int32)
    src[3] = -1
    src[10] = rows * topk + 5
    q, s = cc.dynamic_quant_i8(dev_bf16(xb), torch.from_numpy(src).cuda(), topk)
    torch.cuda.synchronize()
    wq, ws = orc.dyn_quant_i8_rows(xb, src=src, topk=topk)
    assert np.array_equal(q.cpu().numpy(), wq) and np.array_equal(s.cpu().numpy(), ws)


def test_dyn_quant_feeds_grouped_gemm():
    """bf16 tokens -> dynamic int8 quant -> grouped int8 GEMM + dequant + SwiGLU, against the oracle chain."""
    rng = np.random.default_rng(11)
    e, t, k, n = 3, 520, 512, 512
    gs = np.array([300, 0, 213], np.int32)
    xb = rand_rows(rng, t, k)
    w = rng.integers(-127, 128, (e, k, n)).astype(np.int8)
    pc = rng.uniform(0.001, 0.02, (e, n)).astype(np.float32)
    q, s = cc.dynamic_quant_i8(dev_bf16(xb))
    out = cc.gmm_dequant_swiglu(q, torch.from_numpy(w).cuda(), torch.from_numpy(gs).cuda(), s, torch.from_numpy(pc).cuda(), 0)
    torch.cuda.synchronize()
    wq, ws = orc.dyn_quant_i8_rows(xb)
    want = orc.gmm_i8_dequant_swiglu(wq, w, gs, ws, pc)
    m = orc.compare(out.float().cpu().numpy(), want)
    assert m["max_rel_floor1"] <= 1e-2 and m["max_rel_floor_rms"] <= 1e-2, m


@pytest.mark.parametrize("mode", [cc.DQ_DEVICE, cc.DQ_GOLDEN])
@pytest.mark.parametrize("shape", [(64, 512), (200, 7168), (17, 1000), (5, 8200), (3, 12288), (2, 7), (3, 16384), (2, 20000)])
@pytest.mark.parametrize("per_row", [False, True])
def test_dyn_quant_smoothing_bit_exact(shape, mode, per_row):
    """Smoothing vectors (one for all rows, or one per expert picked by row), with a gather, a dropped row
    and vector indices out of range."""
    rows, k = shape
    experts, topk = 5, 2
    rng = np.random.default_rng(rows * 7 + k + mode)
    xb = rand_rows(rng, rows, k, 2.5)
    xb[rows // 2] = 0
    t = rows * topk
    src = rng.permutation(t).astype(np.int32)
    src[1] = -1
    smooth = (rng.uniform(0.2, 5.0, (experts, k)) * np.where(rng.random((experts, k)) < 0.5, -1, 1)).astype(np.float32)
    idx = None
    if per_row:
        idx = rng.integers(0, experts, t).astype(np.int32)
        idx[0] = experts
        idx[t - 1] = -3
    q, s = cc.dynamic_quant_i8(dev_bf16(xb), torch.from_numpy(src).cuda(), topk, mode,
                               smooth=torch.from_numpy(smooth).cuda(),
                               smooth_rows=torch.from_numpy(idx).cuda() if per_row else None)
    torch.cuda.synchronize()
    wq, ws = orc.dyn_quant_i8_rows(xb, src=src, topk=topk, mode=mode, smooth=smooth, smooth_rows=idx)
    assert np.array_equal(s.cpu().numpy(), ws)
    assert np.array_equal(q.cpu().numpy(), wq)


def test_dyn_quant_smoothing_arguments():
    x = torch.zeros(4, 64, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        cc.dynamic_quant_i8(x, smooth_rows=torch.zeros(4, dtype=torch.int32, device="cuda"))
    with pytest.raises(ValueError):
        cc.dynamic_quant_i8(x, smooth=torch.ones(2, 32, device="cuda"))
