"""GPU parity of the MoE routing sort against the oracle (exact integers), and the chain
routing -> gather + dynamic quantisation -> un-permute on the device."""
import numpy as np
import pytest
import torch

import oracle as orc
import catccos_amd as cc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("cumsum", [False, True])
@pytest.mark.parametrize("case", [(64, 4), (1000, 16), (1024, 8), (1025, 8), (16384, 32), (50000, 256), (3, 1), (70000, 1024)])
def test_routing_exact(case, cumsum):
    rows, e = case
    rng = np.random.default_rng(rows + e)
    idx = rng.integers(0, e, rows).astype(np.int32)
    if rows > 10:
        idx[rng.integers(0, rows, 3)] = -1          # dropped entries
        idx[rng.integers(0, rows, 2)] = e
        idx[idx == e // 2] = (e // 2 + 1) % e       # an expert nobody routes to (when e > 1)
    d2s, s2d, cnt = cc.moe_init_routing(torch.from_numpy(idx).cuda(), e, cumsum)
    torch.cuda.synchronize()
    wd, ws, wc = orc.moe_init_routing(idx, e, cumsum)
    assert np.array_equal(cnt.cpu().numpy(), wc)
    assert np.array_equal(s2d.cpu().numpy(), ws)
    assert np.array_equal(d2s.cpu().numpy(), wd)


@pytest.mark.parametrize("case", [(1, 1), (63, 3), (64, 256), (1000, 16), (4097, 200), (8192, 256), (8192, 1), (8193, 256), (500, 257)])
def test_routing_one_workgroup_equals_three_launches(case):
    """Up to 8192 rows and 256 experts one workgroup does the whole sort in one launch; the general path (three launches,
    `routing_three_launches`) and the oracle give the same integers, also just past either limit and with dropped routes."""
    rows, e = case
    rng = np.random.default_rng(rows * 7 + e)
    idx = rng.integers(-1, e + 1, rows).astype(np.int32)      # -1 and e are dropped
    want = orc.moe_init_routing(idx, e)
    for cumsum in (False, True):
        res = []
        for three in (0, 1):
            cc.set_option("routing_three_launches", three)
            try:
                res.append([t.cpu().numpy() for t in cc.moe_init_routing(torch.from_numpy(idx).cuda(), e, cumsum)])
            finally:
                cc.set_option("routing_three_launches", 0)
        for a, b in zip(*res):
            assert np.array_equal(a, b)
        if not cumsum:
            for a, w in zip(res[0], want):
                assert np.array_equal(a, w)


def test_routing_skewed_and_sorted_inputs():
    for idx in (np.zeros(5000, np.int32), np.arange(5000, dtype=np.int32) % 7, np.sort(np.arange(5000, dtype=np.int32) % 7)[::-1].copy()):
        d2s, s2d, cnt = cc.moe_init_routing(torch.from_numpy(idx).cuda(), 7)
        torch.cuda.synchronize()
        wd, ws, wc = orc.moe_init_routing(idx, 7)
        assert np.array_equal(d2s.cpu().numpy(), wd) and np.array_equal(s2d.cpu().numpy(), ws) and np.array_equal(cnt.cpu().numpy(), wc)


def test_routing_empty_and_errors():
    d2s, s2d, cnt = cc.moe_init_routing(torch.zeros(0, dtype=torch.int32, device="cuda"), 4)
    torch.cuda.synchronize()
    assert d2s.numel() == 0 and list(cnt.cpu().numpy()) == [0, 0, 0, 0]
    with pytest.raises(cc.CatccosError):
        cc.moe_init_routing(torch.zeros(8, dtype=torch.int32, device="cuda"), 2000)


def test_routing_feeds_gather_quant_and_unpermute():
    """tokens -> routing -> expert-sorted int8 rows; the same maps bring expert-order rows back to token order."""
    rng = np.random.default_rng(4)
    tokens, k, topk, e = 200, 1024, 2, 8
    xb = orc.f32_to_bf16(rng.standard_normal((tokens, k)).astype(np.float32))
    expert_idx = rng.integers(0, e, (tokens, topk)).astype(np.int32)
    x = torch.from_numpy(xb.view(np.int16)).cuda().view(torch.bfloat16)
    d2s, s2d, cnt = cc.moe_init_routing(torch.from_numpy(expert_idx).cuda(), e)
    q, s = cc.dynamic_quant_i8(x, d2s, topk)
    torch.cuda.synchronize()
    wd, ws, wc = orc.moe_init_routing(expert_idx, e)
    wq, wsc = orc.dyn_quant_i8_rows(xb, wd, topk)
    assert np.array_equal(q.cpu().numpy(), wq) and np.array_equal(s.cpu().numpy(), wsc)
    # rows in expert order are the tokens themselves here; un-permute with the inverse map sums each token topk times
    permuted = x[(d2s // topk).long()]
    back = cc.moe_token_unpermute(permuted, s2d, None, topk)
    torch.cuda.synchronize()
    want = orc.f32_to_bf16(orc.bf16_to_f32(xb) * np.float32(topk))
    assert np.array_equal(back.view(torch.int16).cpu().numpy().view(np.uint16), want)
