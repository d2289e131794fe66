"""torch.ops.catccos.* on the GPU: the dispatcher reaches the HIP library (results equal the oracle's,
bit-exact for the quantiser, within the GEMM gate otherwise) and refuses to run before init, as the
reference's binding does (examples/torch_binding/src/torch_bindings.cpp:131-133)."""
import numpy as np
import pytest
import torch

import oracle as orc
import catccos_amd.torch_library  # noqa: F401

pytestmark = pytest.mark.gpu
OPS = torch.ops.catccos


def dev(x):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def close(got, want):
    m = orc.compare(got.float().cpu().numpy(), want)
    assert m["max_rel_floor1"] <= 1e-2 and m["max_rel_floor_rms"] <= 1e-2, m


def test_ops_need_init_then_match_the_oracle():
    rng = np.random.default_rng(3)
    e, t, k, n = 3, 333, 512, 256
    gs = np.array([200, 0, 133], np.int32)
    x = orc.f32_to_bf16(rng.standard_normal((t, k)).astype(np.float32))
    xd = torch.from_numpy(x.view(np.int16)).cuda().view(torch.bfloat16)
    assert OPS.finalize() == 0
    with pytest.raises(RuntimeError, match="not initialized"):
        OPS.mx_quant(xd, "e4m3", 0)
    assert OPS.init(0, 1, 1 << 20, "tcp://127.0.0.1:8666") == 0
    try:
        a, sa = OPS.mx_quant(xd, "e4m3", 0)
        pa, psa = orc.mx_quant_rows(x, orc.E4M3)
        assert np.array_equal(a.cpu().numpy(), pa) and np.array_equal(sa.cpu().numpy(), psa)
        pbs, sbs = zip(*[orc.mx_quant_b(orc.f32_to_bf16(rng.standard_normal((k, n)).astype(np.float32)), orc.E4M3, orc.RNE, 0)
                         for _ in range(e)])
        pb, sb = np.stack(pbs), np.stack(sbs)
        close(OPS.mx_grouped_matmul(a, sa, dev(pb), dev(sb), dev(gs), "e4m3", 0),
              orc.mx_gmm(pa, psa, pb, sb, n, k, orc.E4M3, 0, group_sizes=gs))
        close(OPS.mx_matmul(a, sa, dev(pb[0]), dev(sb[0]), "e4m3", 0), orc.mx_gmm(pa, psa, pb[:1], sb[:1], n, k, orc.E4M3, 0))
        xi = rng.integers(-127, 128, (t, k)).astype(np.int8)
        wi = rng.integers(-127, 128, (e, k, n)).astype(np.int8)
        pt = rng.uniform(0.001, 0.02, t).astype(np.float32)
        pc = rng.uniform(0.001, 0.02, (e, n)).astype(np.float32)
        close(OPS.gmm_dequant_swiglu(dev(xi), dev(wi), dev(gs), dev(pt), dev(pc), 0), orc.gmm_i8_dequant_swiglu(xi, wi, gs, pt, pc))
        close(OPS.w8a8_matmul_dequant(dev(xi), dev(wi[0]), dev(pt), dev(pc[0]), 0), orc.gemm_i8_dequant(xi, wi[0], pt, pc[0]))
        act = OPS.gmm_dequant_swiglu(dev(xi), dev(wi), dev(gs), dev(pt), dev(pc), 0)
        pq, sq = OPS.gmm_dequant_swiglu_mx(dev(xi), dev(wi), dev(gs), dev(pt), dev(pc), 0, "e4m3")
        torch.cuda.synchronize()
        want_p, want_s = orc.mx_quant_rows(act.view(torch.int16).cpu().numpy().view(np.uint16), orc.E4M3)
        assert np.array_equal(pq.cpu().numpy(), want_p) and np.array_equal(sq.cpu().numpy(), want_s)
        # the whole MXFP8 FFN in one op equals the chain of the single calls, to the bit (same launches)
        import catccos_amd as cc
        m, topk, n1 = 100, 2, 512
        idx = dev(np.argsort(rng.random((m, e)), axis=1)[:, :topk].astype(np.int32))
        probs = torch.softmax(torch.randn(m, topk, device="cuda"), dim=-1)
        w1 = [cc.mx_quant_b(torch.randn(k, n1, device="cuda").to(torch.bfloat16) / k ** 0.5, "e4m3", trans_b=1) for _ in range(e)]
        w2 = [cc.mx_quant_b(torch.randn(n1 // 2, k, device="cuda").to(torch.bfloat16) / (n1 // 2) ** 0.5, "e4m3", trans_b=1) for _ in range(e)]
        b1, s1, b2, s2 = (torch.stack([w[i] for w in ws]) for ws in (w1, w2) for i in (0, 1))
        out = OPS.moe_ffn_mxfp8(xd[:m], idx, probs, b1, s1, b2, s2, 1)
        _, s2d, cnt = cc.moe_init_routing(idx, e)
        packed = torch.empty((m * topk, cc.packed_row_bytes(k)), dtype=torch.uint8, device="cuda")
        cc.mx_quant_scatter_packed(xd[:m], s2d, packed, topk)
        a2, sa2 = cc.mx_grouped_matmul_swiglu(packed[:, :k].contiguous(), packed[:, k:].contiguous(), b1, s1, cnt, "e4m3", 1, out_fmt="e4m3")
        want = cc.moe_token_unpermute(cc.mx_grouped_matmul(a2, sa2, b2, s2, cnt, "e4m3", 1), s2d, probs, topk)
        assert out.shape == (m, k) and torch.equal(out, want)
    finally:
        assert OPS.finalize() == 0


def test_a_host_tensor_among_gpu_arguments_is_refused_before_any_launch():
    """The dispatcher picks the GPU kernel as soon as one argument is a GPU tensor.  Every other tensor argument must then
    be on that GPU too (the reference's binding checks the same, examples/torch_binding/src/torch_bindings.cpp:140-144):
    a host tensor's address must never reach a kernel.  The check throws on the host, so nothing is launched."""
    rng = np.random.default_rng(4)
    e, t, k, n = 2, 64, 128, 64
    gs = np.array([40, 24], np.int32)
    a8 = rng.integers(0, 120, (t, k)).astype(np.uint8)
    sa = np.full((t, 4), 127, np.uint8)
    b8 = rng.integers(0, 120, (e, k, n)).astype(np.uint8)
    sb = np.full((e, 2, n, 2), 127, np.uint8)
    xi = rng.integers(-127, 128, (t, k)).astype(np.int8)
    wi = rng.integers(-127, 128, (e, k, n)).astype(np.int8)
    pt = rng.uniform(0.001, 0.02, t).astype(np.float32)
    pc = rng.uniform(0.001, 0.02, (e, n)).astype(np.float32)
    idx = np.zeros((t, 1), np.int32)
    probs = np.ones((t, 1), np.float32)
    xb = torch.zeros((t, k), dtype=torch.bfloat16)
    w1, s1 = np.zeros((e, 64, k), np.uint8), np.full((e, 64, 4), 127, np.uint8)
    w2, s2 = np.zeros((e, k, 32), np.uint8), np.full((e, k, 2), 127, np.uint8)
    calls = {
        "w8a8_matmul_dequant": (lambda a: OPS.w8a8_matmul_dequant(*a, 0), [xi, wi[0], pt, pc[0]]),
        "mx_matmul": (lambda a: OPS.mx_matmul(*a, "e4m3", 0), [a8, sa, b8[0], sb[0]]),
        "gmm_dequant_swiglu": (lambda a: OPS.gmm_dequant_swiglu(*a, 0), [xi, wi, gs, pt, pc]),
        "gmm_dequant_swiglu_mx": (lambda a: OPS.gmm_dequant_swiglu_mx(*a, 0, "e4m3"), [xi, wi, gs, pt, pc]),
        "mx_grouped_matmul": (lambda a: OPS.mx_grouped_matmul(*a, "e4m3", 0), [a8, sa, b8, sb, gs]),
        "mx_grouped_matmul_swiglu_mx": (lambda a: OPS.mx_grouped_matmul_swiglu_mx(*a, "e4m3", 0, "e4m3"), [a8, sa, b8, sb, gs]),
        "moe_ffn_mxfp8": (lambda a: OPS.moe_ffn_mxfp8(*a, 1), [xb, idx, probs, w1, s1, w2, s2]),
    }
    assert OPS.init(0, 1, 1 << 20, "tcp://127.0.0.1:8666") == 0
    try:
        for name, (call, host_args) in calls.items():
            as_t = [x if isinstance(x, torch.Tensor) else torch.from_numpy(x) for x in host_args]
            for on_host in range(len(as_t)):
                mixed = [x if i == on_host else x.cuda() for i, x in enumerate(as_t)]
                with pytest.raises(RuntimeError, match="must be a GPU tensor"):
                    call(mixed)
    finally:
        assert OPS.finalize() == 0
