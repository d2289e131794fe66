"""The compute entry points only enqueue kernels on the caller's stream (no allocation, no memset, no
synchronisation inside the library), so a chain of them can be recorded into a HIP graph: MX quantise ->
MXFP8 grouped matmul and the int8 SwiGLU path are captured once and replayed several times, with eager
work and synchronisations between the replays; every replay must equal the eager result bit for bit,
also after the inputs were overwritten in place."""
import numpy as np
import pytest
import torch

import catccos_amd as cc

pytestmark = pytest.mark.gpu


def test_captured_chain_replays_like_eager():
    torch.manual_seed(0)
    e, t, k, n = 4, 1500, 1024, 1024
    gs = torch.tensor([700, 0, 290, 510], dtype=torch.int32, device="cuda")
    x = torch.randn(t, k, device="cuda").to(torch.bfloat16)
    w = torch.randn(e * k, n, device="cuda").to(torch.bfloat16)
    xi = torch.randint(-127, 128, (t, k), dtype=torch.int8, device="cuda")
    wi = torch.randint(-127, 128, (e, k, n), dtype=torch.int8, device="cuda")
    pt = torch.rand(t, device="cuda") * 0.019 + 0.001
    pc = torch.rand(e, n, device="cuda") * 0.019 + 0.001
    pb, sb = zip(*[cc.mx_quant_b(w[i * k:(i + 1) * k], "e4m3", 0, 0) for i in range(e)])
    pb, sb = torch.stack(pb), torch.stack(sb)

    def chain():
        a, sa = cc.mx_quant(x, "e4m3")
        y = cc.mx_grouped_matmul(a, sa, pb, sb, gs, "e4m3", 0)
        z = cc.gmm_dequant_swiglu(xi, wi, gs, pt, pc, 0)
        return a, sa, y, z

    cc.set_option("require_tiled_gemm", 1)
    try:
        eager = [o.clone() for o in chain()]       # also the first launch of each kernel, outside the capture
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            outs = chain()
        for rep in range(4):
            if rep == 2:
                # new input values in the captured buffers: the replay must follow them
                x.copy_((torch.randn(t, k, device="cuda") * 3).to(torch.bfloat16))
                xi.copy_(torch.randint(-127, 128, (t, k), dtype=torch.int8, device="cuda"))
                eager = [o.clone() for o in chain()]
            for o in outs:
                o.fill_(0)                          # eager work between the replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for got, want in zip(outs, eager):
                assert torch.equal(got, want), rep
    finally:
        cc.set_option("require_tiled_gemm", 0)


def test_captured_ffn_follows_new_routing():
    """The whole MXFP8 FFN (routing sort, quantise-and-scatter, both grouped matmuls, un-permute) in one graph: the
    group sizes and row maps are device data that the graph's own kernels produce, so a replay follows new routes
    and new tokens written into the captured input buffers; every replay equals the eager result bit for bit."""
    torch.manual_seed(1)
    m, k, n, e, topk = 200, 512, 1024, 8, 2
    x = torch.randn(m, k, device="cuda").to(torch.bfloat16)
    idx = torch.argsort(torch.rand(m, e, device="cuda"), dim=1)[:, :topk].to(torch.int32).contiguous()
    probs = torch.softmax(torch.randn(m, topk, device="cuda"), dim=-1)
    w1 = [cc.mx_quant_b(torch.randn(k, n, device="cuda").to(torch.bfloat16) / k ** 0.5, "e4m3", trans_b=1) for _ in range(e)]
    w2 = [cc.mx_quant_b(torch.randn(n // 2, k, device="cuda").to(torch.bfloat16) / (n // 2) ** 0.5, "e4m3", trans_b=1) for _ in range(e)]
    b1, s1, b2, s2 = (torch.stack([w[i] for w in ws]) for ws in (w1, w2) for i in (0, 1))
    cc.set_option("require_tiled_gemm", 1)
    try:
        eager = cc.moe_ffn_mxfp8(x, idx, probs, b1, s1, b2, s2).clone()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = cc.moe_ffn_mxfp8(x, idx, probs, b1, s1, b2, s2)
        for rep in range(4):
            if rep == 2:
                # other tokens, and routes that leave three experts empty
                x.copy_((torch.randn(m, k, device="cuda") * 2).to(torch.bfloat16))
                idx.copy_(torch.argsort(torch.rand(m, e - 3, device="cuda"), dim=1)[:, :topk].to(torch.int32))
                eager = cc.moe_ffn_mxfp8(x, idx, probs, b1, s1, b2, s2).clone()
            out.fill_(0)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager), rep
    finally:
        cc.set_option("require_tiled_gemm", 0)
