"""The grouped int8 matmul + dequant + SwiGLU whose activation leaves MX-quantised from the kernel's
epilogue: its bytes must equal the oracle's row quantiser applied to the bf16 tensor that the unfused
entry point writes, bit for bit (payload and scales, padding bytes, rows that belong to no group)."""
import numpy as np
import pytest
import torch

import oracle as orc
import catccos_amd as cc

pytestmark = pytest.mark.gpu
FMT = {"e4m3": orc.E4M3, "e5m2": orc.E5M2, "e2m1": orc.E2M1}


def bits(t):
    torch.cuda.synchronize()
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def case(e, t, k, n, gs, seed):
    rng = np.random.default_rng(seed)
    x = torch.from_numpy(rng.integers(-127, 128, (t, k)).astype(np.int8)).cuda()
    w = rng.integers(-127, 128, (e, k, n)).astype(np.int8)
    pt = torch.from_numpy(rng.uniform(0.001, 0.02, t).astype(np.float32)).cuda()
    # a wide range of channel scales, so that blocks differ in their shared exponents
    pc = torch.from_numpy((rng.uniform(0.001, 0.02, (e, n)) * 2.0 ** rng.integers(-6, 3, (e, n))).astype(np.float32)).cuda()
    return x, w, pt, pc, torch.from_numpy(np.array(gs, np.int32)).cuda()


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e2m1"])
@pytest.mark.parametrize("trans_b", [0, 1])
@pytest.mark.parametrize("cfg", [(4, 700, 512, 1088, [300, 0, 143, 250]),     # n/2 = 544: 17 blocks (odd: a padding byte), 7 rows of no group
                                 (3, 300, 256, 512, [1, 0, 299]),
                                 (6, 2000, 768, 2048, [700, 13, 0, 256, 900, 131])])
def test_fused_bytes_equal_quantised_bf16_tiled(fmt, trans_b, cfg):
    e, t, k, n, gs = cfg
    x, w, pt, pc, gsd = case(e, t, k, n, gs, seed=t + k + trans_b)
    wd = torch.from_numpy(np.ascontiguousarray(w.transpose(0, 2, 1)) if trans_b else w).cuda()
    cc.set_option("require_tiled_gemm", 1)
    try:
        plain = cc.gmm_dequant_swiglu(x, wd, gsd, pt, pc, trans_b)
        pay, sc = cc.gmm_dequant_swiglu_mx(x, wd, gsd, pt, pc, trans_b, fmt)
    finally:
        cc.set_option("require_tiled_gemm", 0)
    want_p, want_s = orc.mx_quant_rows(bits(plain), FMT[fmt])
    assert np.array_equal(sc.cpu().numpy(), want_s)
    assert np.array_equal(pay.cpu().numpy(), want_p)
    # and the device's own row quantiser agrees (the same bytes by another kernel)
    p2, s2 = cc.mx_quant(plain, fmt)
    assert torch.equal(p2, pay) and torch.equal(s2, sc)


@pytest.mark.parametrize("fmt", ["e4m3", "e2m1"])
@pytest.mark.parametrize("trans_b", [0, 1])
def test_fused_bytes_generic_path_and_ragged_blocks(fmt, trans_b):
    """n/2 = 100: three whole blocks and one of four columns, outside what the tiled kernels take."""
    e, t, k, n, gs = 3, 70, 96, 200, [30, 0, 33]
    x, w, pt, pc, gsd = case(e, t, k, n, gs, seed=5 + trans_b)
    wd = torch.from_numpy(np.ascontiguousarray(w.transpose(0, 2, 1)) if trans_b else w).cuda()
    plain = cc.gmm_dequant_swiglu(x, wd, gsd, pt, pc, trans_b)
    pay, sc = cc.gmm_dequant_swiglu_mx(x, wd, gsd, pt, pc, trans_b, fmt)
    want_p, want_s = orc.mx_quant_rows(bits(plain), FMT[fmt])
    assert np.array_equal(sc.cpu().numpy(), want_s)
    assert np.array_equal(pay.cpu().numpy(), want_p)


def test_fused_generic_equals_oracle_chain():
    """Generic kernels at a tiled-capable shape against the oracle end to end: oracle GEMM + SwiGLU to bf16,
    then the oracle's quantiser (the generic kernel's exp and division are the IEEE ones; a one-ulp bf16
    difference from the oracle's libm moves at most that element's code by one step)."""
    e, t, k, n, gs = 2, 96, 128, 256, [40, 56]
    x, w, pt, pc, gsd = case(e, t, k, n, gs, seed=77)
    cc.set_option("force_generic_gemm", 1)
    try:
        pay, sc = cc.gmm_dequant_swiglu_mx(x, torch.from_numpy(w).cuda(), gsd, pt, pc, 0, "e4m3")
    finally:
        cc.set_option("force_generic_gemm", 0)
    _, gold16 = orc.gmm_i8_dequant_swiglu(x.cpu().numpy(), w, np.array(gs, np.int32), pt.cpu().numpy(), pc.cpu().numpy(), want_bf16=True)
    want_p, want_s = orc.mx_quant_rows(gold16, orc.E4M3)
    got = orc.mx_dequant_rows(pay.cpu().numpy(), sc.cpu().numpy(), n // 2, orc.E4M3)
    want = orc.mx_dequant_rows(want_p, want_s, n // 2, orc.E4M3)
    assert np.mean(sc.cpu().numpy() == want_s) > 0.99
    assert np.mean(pay.cpu().numpy() == want_p) > 0.99
    m = orc.compare(got, want)
    assert m["max_rel_floor_rms"] <= 0.15, m   # one code step of E4M3 is 1/8 relative


def test_bad_arguments():
    x, w, pt, pc, gsd = case(2, 8, 32, 64, [4, 4], seed=1)
    wd = torch.from_numpy(w).cuda()
    with pytest.raises(ValueError):
        cc.gmm_dequant_swiglu_mx(x, wd, gsd, pt, pc, 0, "e1m2x")
    with pytest.raises(cc.CatccosError):
        cc.gmm_dequant_swiglu_mx(x, wd, gsd, pt, pc, 0, "e1m2")


# ---------------------------------------------------------------- MX up projection + SwiGLU

def mx_case(e, t, k, n, gs, fmt, trans_b, seed):
    rng = np.random.default_rng(seed)
    sigma = 0.05 if fmt == "e2m1" else 0.5
    pa, sa = orc.mx_quant_rows(orc.f32_to_bf16((rng.standard_normal((t, k)) * sigma).astype(np.float32)), FMT[fmt])
    pbs, sbs = zip(*[orc.mx_quant_b(orc.f32_to_bf16((rng.standard_normal((k, n)) * sigma).astype(np.float32)), FMT[fmt], orc.RNE, trans_b)
                     for _ in range(e)])
    return pa, sa, np.stack(pbs), np.stack(sbs), np.array(gs, np.int32)


def to_dev(x):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e2m1"])
@pytest.mark.parametrize("trans_b", [0, 1])
@pytest.mark.parametrize("cfg", [(4, 700, 512, 1088, [300, 0, 143, 250]),     # n/2 = 544: ragged last column tile, odd block count
                                 (3, 300, 1216, 512, [1, 0, 299]),            # K tail, scale rows off 4-byte boundaries
                                 (5, 1500, 768, 2048, [700, 13, 0, 256, 531])])
@pytest.mark.parametrize("tiled", [True, False], ids=["tiled", "generic"])
def test_mx_gmm_swiglu_against_oracle_chain_and_fused_bytes(fmt, trans_b, cfg, tiled):
    """bf16 result against the oracle chain (grouped MX GEMM -> bf16 -> SwiGLU of the bf16 tile), then the
    fused MX-quantised activation byte for byte against the oracle's row quantiser of that bf16 result."""
    e, t, k, n, gs = cfg
    if not tiled:
        t, gs = 120, [50, 0, 70][:e] + [0] * (e - 3)     # one thread per output: a few rows of the same N and K
    pa, sa, pb, sb, gsh = mx_case(e, t, k, n, gs, fmt, trans_b, seed=t + k + n + trans_b)
    cc.set_option("require_tiled_gemm" if tiled else "force_generic_gemm", 1)
    try:
        args = (to_dev(pa), to_dev(sa), to_dev(pb), to_dev(sb), to_dev(gsh), fmt, trans_b)
        plain = cc.mx_grouped_matmul_swiglu(*args)
        outs = {of: cc.mx_grouped_matmul_swiglu(*args, out_fmt=of) for of in ("e4m3", "e2m1")}
        full = cc.mx_grouped_matmul(*args)
    finally:
        cc.set_option("require_tiled_gemm" if tiled else "force_generic_gemm", 0)
    # (a) the activation, given the tile: the kernel rounds its accumulators to bf16 exactly as the plain grouped
    # GEMM does (same accumulators), so the oracle's SwiGLU of that kernel's bf16 output must reproduce the result -
    # to the bit, but for the hardware's exp and reciprocal: at most one bf16 step on at most one element in 10 000
    want16 = orc.swiglu_bf16(bits(full))
    got16 = bits(plain)
    d16 = np.abs(got16.astype(np.int32) - want16.astype(np.int32))
    assert d16.max() <= 1 and np.mean(d16 != 0) <= 1e-4, (int(d16.max()), float(np.mean(d16 != 0)))
    # (b) end to end against the oracle chain (its own GEMM, bf16, SwiGLU): the two GEMMs agree to about 1e-6 of
    # their terms, which flips the bf16 rounding of gate or up on one element in a hundred and swings sums that
    # cancel to nearly zero; against the tensor's rms that stays inside the GEMM gate
    _, c16 = orc.mx_gmm(pa, sa, pb, sb, n, k, FMT[fmt], trans_b, group_sizes=gsh, want_bf16=True)
    want = orc.bf16_to_f32(orc.swiglu_bf16(c16))
    got = plain.float().cpu().numpy()
    m = orc.compare(got, want)
    assert m["max_rel_floor_rms"] <= 3e-2 and m["frac_bad"] <= 1e-2 and abs(m["eb"]) <= 2.0 ** -7, m
    assert np.all(got[int(gsh.sum()):] == 0)
    for of, (pay, sc) in outs.items():
        want_p, want_s = orc.mx_quant_rows(bits(plain), FMT[of])
        assert np.array_equal(sc.cpu().numpy(), want_s), of
        assert np.array_equal(pay.cpu().numpy(), want_p), of


@pytest.mark.parametrize("tiled", [True, False], ids=["tiled", "generic"])
def test_edge_cases_of_the_fused_outputs(tiled):
    """All groups empty (every row is a row of no group: zero codes, scale bytes 127), group sizes that run past
    the rows (clipped, as the GEMMs do), one row, and no rows at all."""
    e, k, n = 3, 256, 512
    rng = np.random.default_rng(99)
    cc.set_option("require_tiled_gemm" if tiled else "force_generic_gemm", 1)
    try:
        for t, gs in ((5, [0, 0, 0]), (70, [40, 0, 100]), (1, [0, 1, 0]), (0, [0, 0, 0])):
            pa, sa, pb, sb, gsh = mx_case(e, max(t, 1), k, n, gs, "e4m3", 0, seed=t)
            pa, sa = pa[:t], sa[:t]
            args = (to_dev(pa), to_dev(sa), to_dev(pb), to_dev(sb), to_dev(gsh), "e4m3", 0)
            plain = cc.mx_grouped_matmul_swiglu(*args)
            pay, sc = cc.mx_grouped_matmul_swiglu(*args, out_fmt="e4m3")
            torch.cuda.synchronize()
            assert plain.shape == (t, n // 2) and pay.shape == (t, n // 2) and sc.shape == (t, 8)
            if t == 0:
                continue
            want_p, want_s = orc.mx_quant_rows(bits(plain), orc.E4M3)
            assert np.array_equal(pay.cpu().numpy(), want_p) and np.array_equal(sc.cpu().numpy(), want_s), (t, gs)
            used = min(t, int(np.sum(gs)))
            assert np.all(bits(plain)[used:] == 0) and np.all(pay.cpu().numpy()[used:] == 0) and np.all(sc.cpu().numpy()[used:] == 127)
            # int8 twin on the same grouping
            x = torch.from_numpy(rng.integers(-127, 128, (t, k)).astype(np.int8)).cuda()
            w = torch.from_numpy(rng.integers(-127, 128, (e, k, n)).astype(np.int8)).cuda()
            pt = torch.from_numpy(rng.uniform(0.001, 0.02, t).astype(np.float32)).cuda()
            pc = torch.from_numpy(rng.uniform(0.001, 0.02, (e, n)).astype(np.float32)).cuda()
            p8, s8 = cc.gmm_dequant_swiglu_mx(x, w, to_dev(gsh), pt, pc, 0, "e2m1")
            w_p, w_s = orc.mx_quant_rows(bits(cc.gmm_dequant_swiglu(x, w, to_dev(gsh), pt, pc, 0)), orc.E2M1)
            assert np.array_equal(p8.cpu().numpy(), w_p) and np.array_equal(s8.cpu().numpy(), w_s), (t, gs)
    finally:
        cc.set_option("require_tiled_gemm" if tiled else "force_generic_gemm", 0)
