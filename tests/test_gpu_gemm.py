"""GPU parity of the GEMM family against the CPU oracle.

Gate (from the task): max |d-g| / max(|g|, tau) <= 1e-2 on bf16 outputs, with tau = 1 as the
reference's verifier uses (examples/utils/verify_result.py:172) and additionally tau = rms(golden),
which still bites when outputs are far below 1."""
import numpy as np
import pytest
import torch

import oracle as orc
import catccos_amd as cc

pytestmark = pytest.mark.gpu
TOL = 1e-2


def dev(x):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def bf16_dev(bits):
    return torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16)


def out_f32(t):
    torch.cuda.synchronize()
    return t.float().cpu().numpy()


def assert_close(got, want, what=""):
    m = orc.compare(got, want)
    assert m["max_rel_floor1"] <= TOL and m["max_rel_floor_rms"] <= TOL, (what, m)
    assert abs(m["eb"]) <= 2.0 ** -7, (what, m)


def assert_double_golden(got, want, what=""):
    """The acceptance metric the reference's own run applies to the MXFP8 dense operator (double golden,
    examples/utils/verify_result.py:198-246 called at examples/ascend950_mxfp8_matmul_reduce_scatter/scripts/run.sh:56-61):
    the result against the fp32 golden, relative to what a low-precision golden - that golden cast to bf16,
    gen_data_mxfp8_mmrs.py:349-355 - loses: mean relative error and RMSE within 2x, bias within 2^-7, over every element.
    Its fourth limit, the largest relative error within 10x, is asserted over the elements whose golden value is at
    least 2^-7 of the tensor's rms.  Where the golden sum cancels to (almost) nothing the relative error is unbounded
    for any summation that is not exact: the matrix instruction aligns the 64 products of a block to the largest one
    before it adds them, which costs a few 2^-22 of that product and shows only when the sum itself is that small (on
    the reference's shape list the ratio over all elements runs into the thousands, at elements of 1e-5 among values
    of 30), while the bf16 cast of the golden that the result is measured against stays within 2^-8 of every value,
    however small."""
    low = orc.bf16_to_f32(orc.f32_to_bf16(want))
    m = orc.compare_double(got, want, low)
    assert m["mean_rel_ratio"] < 2 and m["rmse_ratio"] < 2 and m["eb_percent"] <= 100, (what, m)
    keep = np.abs(want) >= 2.0 ** -7 * np.sqrt(np.mean(want.astype(np.float64) ** 2))
    mk = orc.compare_double(got[keep], want[keep], low[keep])
    assert mk["max_rel_ratio"] < 10, (what, mk)


def rand_bf16(rng, shape, sigma=1.0):
    return orc.f32_to_bf16((rng.standard_normal(shape) * sigma).astype(np.float32))


def zipf_groups(rng, t, e, empty=True):
    p = (np.arange(e) + 1.0) ** -1.1
    p = p[rng.permutation(e)]
    gs = rng.multinomial(t, p / p.sum()).astype(np.int32)
    if empty and gs.min() > 0:
        i, j = int(gs.argmin()), int(gs.argmax())
        gs[j] += gs[i]
        gs[i] = 0
    return gs


@pytest.fixture(params=[0, 1], ids=["tiled", "generic"])
def path(request):
    cc.set_option("force_generic_gemm", request.param)
    yield request.param
    cc.set_option("force_generic_gemm", 0)


# ---------------------------------------------------------------- int8 dense

@pytest.mark.parametrize("shape", [(128, 128, 128), (300, 520, 256), (64, 1000, 384), (257, 255, 1024), (5, 33, 96)])
@pytest.mark.parametrize("trans_b", [0, 1])
def test_i8_dequant(shape, trans_b, path):
    m, n, k = shape
    rng = np.random.default_rng(m + n + k)
    a = rng.integers(-127, 128, (m, k)).astype(np.int8)
    b = rng.integers(-127, 128, (k, n)).astype(np.int8)
    pt = rng.uniform(0.001, 0.02, m).astype(np.float32)
    pc = rng.uniform(0.001, 0.02, n).astype(np.float32)
    want = orc.gemm_i8_dequant(a, b, pt, pc)
    bb = np.ascontiguousarray(b.T) if trans_b else b
    got = out_f32(cc.w8a8_matmul_dequant(dev(a), dev(bb), dev(pt), dev(pc), trans_b))
    assert_close(got, want)
    # int32 accumulation is exact, so the bf16 result is the correctly rounded golden up to the
    # order of the two fp32 multiplies: at most one bf16 ulp away
    want16 = orc.bf16_to_f32(orc.f32_to_bf16(want))
    assert np.max(np.abs(got - want16) / np.maximum(np.abs(want16), 1e-30)) <= 2.0 ** -7


# ------------------------------------------------------- int8 grouped SwiGLU

@pytest.mark.parametrize("cfg", [(4, 700, 256, 512, [300, 0, 143, 257]), (3, 64, 128, 256, [1, 0, 50]),
                                 (16, 2048, 384, 1024, None), (2, 10, 96, 64, [4, 6])])
@pytest.mark.parametrize("trans_b", [0, 1])
def test_gmm_swiglu(cfg, trans_b, path):
    e, t, k, n, gs = cfg
    rng = np.random.default_rng(e + t + k + n)
    gs = zipf_groups(rng, t - 7, e) if gs is None else np.array(gs, np.int32)   # leaves rows past the groups
    x = rng.integers(-127, 128, (t, k)).astype(np.int8)
    w = rng.integers(-127, 128, (e, k, n)).astype(np.int8)
    pt = rng.uniform(0.001, 0.02, t).astype(np.float32)
    pc = rng.uniform(0.001, 0.02, (e, n)).astype(np.float32)
    want = orc.gmm_i8_dequant_swiglu(x, w, gs, pt, pc)
    ww = np.ascontiguousarray(w.transpose(0, 2, 1)) if trans_b else w
    got = out_f32(cc.gmm_dequant_swiglu(dev(x), dev(ww), dev(gs), dev(pt), dev(pc), trans_b))
    assert_close(got, want)
    assert np.all(got[int(gs.sum()):] == 0)
    # the reference rounds the per-channel product through fp16 before the per-token scale
    # (gen_data_dispatch_gmm_dequant_swiglu.py:309-310); the fused path must stay within the gate of that too
    assert_close(got, orc.gmm_i8_dequant_swiglu(x, w, gs, pt, pc, fp16_step=True), "fp16-step golden")


@pytest.mark.parametrize("tiled", [True, False], ids=["tiled", "generic"])
@pytest.mark.parametrize("trans_b", [0, 1])
def test_int8_epilogues_with_the_reference_devices_fp16_step(tiled, trans_b):
    """`i8_epilogue_fp16_step`: acc * per_channel leaves the matrix stage as IEEE half and the per-token factor meets the
    widened half, as the reference's device kernel does it
    (include/catccos/epilogue/block/block_epilogue_per_token_dequant_swiglu.hpp:348-361; the golden generator's option,
    examples/utils/gen_data_dispatch_gmm_dequant_swiglu.py:309-310).  The int32 sums are exact, so the kernels' bf16
    output can be held to the bits of that golden rounded to bf16:
      * without the activation every operation is one correctly rounded fp32 (or half) step: bit for bit equal to a numpy
        restatement (int64 matmul, fp32 product, numpy's half cast, fp32 product, bf16), dense and grouped;
      * with SwiGLU the hardware's exp and reciprocal stand where the golden has expf and a division: at most one bf16
        step on at most two elements in a thousand (results below 1e-30 aside, where the reciprocal flushes to zero).
    The switch must change something: the default path keeps fp32 throughout and differs on some elements."""
    rng = np.random.default_rng(77 + trans_b)
    e, t, k, n = 3, 300, 256, 512
    gs = np.array([130, 0, 170], np.int32)
    x = rng.integers(-127, 128, (t, k)).astype(np.int8)
    w = rng.integers(-127, 128, (e, k, n)).astype(np.int8)
    pt = rng.uniform(0.001, 0.02, t).astype(np.float32)
    pc = rng.uniform(0.001, 0.02, (e, n)).astype(np.float32)
    ww = np.ascontiguousarray(w.transpose(0, 2, 1)) if trans_b else w
    row_e = np.repeat(np.arange(e), gs)
    acc = np.einsum("tk,tkn->tn", x.astype(np.int64), w[row_e].astype(np.int64)).astype(np.float32)   # exact: |sum| < 2^24
    half = (acc * pc[row_e]).astype(np.float16).astype(np.float32)
    want_plain = orc.f32_to_bf16(half * pt[:, None])
    cc.set_option("require_tiled_gemm" if tiled else "force_generic_gemm", 1)
    try:
        cc.set_option("i8_epilogue_fp16_step", 1)
        act = cc.gmm_dequant_swiglu(dev(x), dev(ww), dev(gs), dev(pt), dev(pc), trans_b)
        plain = cc.gmm_dequant(dev(x), dev(ww), dev(gs), dev(pt), dev(pc), trans_b)
        dense = cc.w8a8_matmul_dequant(dev(x[:130]), dev(ww[0]), dev(pt[:130]), dev(pc[0]), trans_b)
        cc.set_option("i8_epilogue_fp16_step", 0)
        plain32 = cc.gmm_dequant(dev(x), dev(ww), dev(gs), dev(pt), dev(pc), trans_b)
        torch.cuda.synchronize()
    finally:
        cc.set_option("i8_epilogue_fp16_step", 0)
        cc.set_option("require_tiled_gemm" if tiled else "force_generic_gemm", 0)
    bits16 = lambda tt: tt.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(bits16(plain), want_plain)
    assert np.array_equal(bits16(dense), want_plain[:130])
    assert not np.array_equal(bits16(plain32), want_plain)
    _, want_act = orc.gmm_i8_dequant_swiglu(x, w, gs, pt, pc, fp16_step=True, want_bf16=True)
    # (a gate below about -87 leaves 1 + exp(-gate) near the top of the fp32 range: its hardware reciprocal is flushed
    # to zero where the golden's division keeps a subnormal quotient; such results, below 1e-30, only have to be as small)
    normal = np.abs(orc.bf16_to_f32(want_act)) >= 1e-30
    d = np.abs(bits16(act).astype(np.int32) - want_act.astype(np.int32))
    assert d[normal].max() <= 1 and np.mean(d[normal] != 0) <= 2e-3, (int(d[normal].max()), float(np.mean(d[normal] != 0)))
    assert np.all(np.abs(act.float().cpu().numpy()[~normal]) <= 2e-30)


# ------------------------------------------------------------------ MX dense

FMT = {"e4m3": orc.E4M3, "e5m2": orc.E5M2, "e2m1": orc.E2M1}


def mx_operands(rng, m, n, k, fmt, trans_b, sigma=1.0):
    a0 = rand_bf16(rng, (m, k), sigma)
    b0 = rand_bf16(rng, (k, n), sigma)
    pa, sa = orc.mx_quant_rows(a0, FMT[fmt])
    pb, sb = orc.mx_quant_b(b0, FMT[fmt], orc.RNE, trans_b)
    return pa, sa, pb, sb


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e2m1"])
@pytest.mark.parametrize("shape", [(64, 128, 128), (256, 256, 256), (300, 520, 512), (8, 1536, 1216), (1000, 1000, 960),
                                   (33, 70, 64)])
@pytest.mark.parametrize("trans_b", [0, 1])
def test_mx_gemm(fmt, shape, trans_b, path):
    """Shapes include the reference's own mxfp8 test list entries with ragged M/N and K % 128 != 0
    (examples/ascend950_mxfp8_matmul_reduce_scatter/scripts/test_shapes.csv)."""
    m, n, k = shape
    if path == 1 and m * n * k > 3e8:
        m = max(8, int(3e8 / (n * k)))   # generic path (one thread per output): fewer rows of the same N and K keep the run short
    rng = np.random.default_rng(m * 7 + n * 3 + k)
    pa, sa, pb, sb = mx_operands(rng, m, n, k, fmt, trans_b)
    want = orc.mx_gmm(pa, sa, pb, sb, n, k, FMT[fmt], trans_b)
    got = out_f32(cc.mx_matmul(dev(pa), dev(sa), dev(pb), dev(sb), fmt, trans_b))
    assert_close(got, want)


def _reference_shapes(op, limit=4e10):
    import json
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_shapes.json")
    return [tuple(s) for s in json.load(open(path))[op] if 2.0 * s[0] * s[1] * s[2] <= limit]


@pytest.mark.parametrize("shape", _reference_shapes("ascend950_mxfp8_matmul_reduce_scatter"))
def test_mx_gemm_reference_shape_list(shape):
    """Every (M, K, N) of the reference's own list for the MXFP8 operator
    (examples/ascend950_mxfp8_matmul_reduce_scatter/scripts/test_shapes.csv, kept as the fixture
    golden/reference_shapes.json), in the layout its run uses (transB = 1)."""
    m, k, n = shape
    rng = np.random.default_rng(m + k + n)
    pa, sa, pb, sb = mx_operands(rng, m, n, k, "e4m3", 1)
    want = orc.mx_gmm(pa, sa, pb, sb, n, k, orc.E4M3, 1, blocked=True)   # the cache-blocked routine: same bits, a fraction of the time
    got = out_f32(cc.mx_matmul(dev(pa), dev(sa), dev(pb), dev(sb), "e4m3", 1))
    assert_close(got, want, shape)
    assert_double_golden(got, want, shape)


@pytest.mark.parametrize("op,fmt", [("ascend950_fp8_mx_grouped_matmul_alltoallv", "e4m3"), ("ascend950_fp4_mx_grouped_matmul_alltoallv", "e2m1"),
                                    ("ascend950_fp8_mx_alltoallv_grouped_matmul", "e4m3"), ("ascend950_fp4_mx_alltoallv_grouped_matmul", "e2m1")])
def test_mx_gmm_reference_shape_lists(op, fmt):
    """The grouped operators' own shapes (their scripts/test_shapes.csv), 8 experts as their run.sh defaults to."""
    for (m, k, n) in _reference_shapes(op):
        e = 8
        rng = np.random.default_rng(m + k + n)
        gs = zipf_groups(rng, m, e)
        sigma = 0.02 if fmt == "e2m1" else 1.0
        pa, sa = orc.mx_quant_rows(rand_bf16(rng, (m, k), sigma), FMT[fmt])
        pbs, sbs = zip(*[orc.mx_quant_b(rand_bf16(rng, (k, n), sigma), FMT[fmt], orc.RNE, 0) for _ in range(e)])
        pb, sb = np.stack(pbs), np.stack(sbs)
        want = orc.mx_gmm(pa, sa, pb, sb, n, k, FMT[fmt], 0, group_sizes=gs)
        got = out_f32(cc.mx_grouped_matmul(dev(pa), dev(sa), dev(pb), dev(sb), dev(gs), fmt, 0))
        assert_close(got, want, (op, m, k, n))


def test_mx_gemm_scale_extremes():
    """Scale bytes far from 127 on both operands, incl. products that leave the fp32 normal range."""
    rng = np.random.default_rng(5)
    m, n, k = 64, 64, 256
    pa, sa, pb, sb = mx_operands(rng, m, n, k, "e4m3", 1)
    sa[:, 0] = 200
    sb[:, 0] = 60
    sa[:, 1] = 20
    sb[:, 1] = 230
    want = orc.mx_gmm(pa, sa, pb, sb, n, k, orc.E4M3, 1)
    got = out_f32(cc.mx_matmul(dev(pa), dev(sa), dev(pb), dev(sb), "e4m3", 1))
    # outputs are ~1e7 with heavy cancellation, so only the rms-floored error is meaningful here
    m = orc.compare(got, want)
    assert m["max_rel_floor_rms"] <= TOL, m


# ---------------------------------------------------------------- MX grouped

@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e2m1"])
@pytest.mark.parametrize("cfg", [(4, 1024, 256, 256, None), (5, 900, 512, 384, [0, 300, 1, 0, 500]), (32, 4096, 512, 512, None)])
@pytest.mark.parametrize("trans_b", [0, 1])
def test_mx_gmm(fmt, cfg, trans_b, path):
    e, t, n, k, gs = cfg
    if path == 1 and t * n * k > 3e8:
        assert gs is None
        t = max(4 * e, int(3e8 / (n * k)))   # generic path: fewer tokens over the same experts keep the run short
    rng = np.random.default_rng(e + t + n + k)
    gs = zipf_groups(rng, t - 5, e) if gs is None else np.array(gs, np.int32)
    sigma = 0.02 if fmt == "e2m1" else 1.0
    a0 = rand_bf16(rng, (t, k), sigma)
    pa, sa = orc.mx_quant_rows(a0, FMT[fmt])
    pbs, sbs = [], []
    for _ in range(e):
        pb, sb = orc.mx_quant_b(rand_bf16(rng, (k, n), sigma), FMT[fmt], orc.RNE, trans_b)
        pbs.append(pb), sbs.append(sb)
    pb, sb = np.stack(pbs), np.stack(sbs)
    want = orc.mx_gmm(pa, sa, pb, sb, n, k, FMT[fmt], trans_b, group_sizes=gs)
    got = out_f32(cc.mx_grouped_matmul(dev(pa), dev(sa), dev(pb), dev(sb), dev(gs), fmt, trans_b))
    assert_close(got, want)
    assert np.all(got[int(gs.sum()):] == 0)


# ---------------------------------------------------------------- shapes chosen for the tiled MFMA kernels
# Every case below must run on the tiled kernels (require_tiled_gemm makes a silent fall-back to
# the generic kernels an error): several K-steps, ragged last row and column tiles, both operand
# layouts of B, empty and one-row groups.

@pytest.fixture
def tiled_only():
    cc.set_option("force_generic_gemm", 0)
    cc.set_option("require_tiled_gemm", 1)
    yield
    cc.set_option("require_tiled_gemm", 0)


@pytest.mark.parametrize("shape", [(300, 528, 512), (513, 272, 768), (1, 16, 256), (1024, 1040, 1280)])
@pytest.mark.parametrize("trans_b", [0, 1])
def test_i8_dequant_tiled(shape, trans_b, tiled_only):
    m, n, k = shape
    rng = np.random.default_rng(100 + m + trans_b)
    a = rng.integers(-127, 128, (m, k)).astype(np.int8)
    b = rng.integers(-127, 128, (k, n)).astype(np.int8)
    pt = rng.uniform(0.001, 0.02, m).astype(np.float32)
    pc = rng.uniform(0.001, 0.02, n).astype(np.float32)
    want = orc.gemm_i8_dequant(a, b, pt, pc)
    bb = np.ascontiguousarray(b.T) if trans_b else b
    got = out_f32(cc.w8a8_matmul_dequant(dev(a), dev(bb), dev(pt), dev(pc), trans_b))
    assert_close(got, want, ("i8 tiled", shape, trans_b))


@pytest.mark.parametrize("cfg", [(4, 700, 512, 1056, [300, 0, 143, 257]), (3, 300, 256, 512, [1, 0, 299]), (6, 2000, 768, 2080, None)])
@pytest.mark.parametrize("trans_b", [0, 1])
def test_gmm_swiglu_tiled(cfg, trans_b, tiled_only):
    e, t, k, n, gs = cfg
    rng = np.random.default_rng(200 + t + trans_b)
    gs = np.array(gs, np.int32) if gs is not None else zipf_groups(rng, t, e)
    x = rng.integers(-127, 128, (t, k)).astype(np.int8)
    w = rng.integers(-127, 128, (e, k, n)).astype(np.int8)
    pt = rng.uniform(0.001, 0.02, t).astype(np.float32)
    pc = rng.uniform(0.001, 0.02, (e, n)).astype(np.float32)
    want = orc.gmm_i8_dequant_swiglu(x, w, gs, pt, pc)
    ww = np.ascontiguousarray(w.transpose(0, 2, 1)) if trans_b else w
    got = out_f32(cc.gmm_dequant_swiglu(dev(x), dev(ww), dev(gs), dev(pt), dev(pc), trans_b))
    assert_close(got, want, ("swiglu tiled", cfg[:4], trans_b))


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e2m1"])
@pytest.mark.parametrize("shape", [(300, 544, 1024), (513, 288, 768), (2, 32, 512), (700, 1312, 1536)])
@pytest.mark.parametrize("trans_b", [0, 1])
def test_mx_gemm_tiled(fmt, shape, trans_b, tiled_only):
    m, n, k = shape
    rng = np.random.default_rng(300 + m + trans_b)
    pa, sa, pb, sb = mx_operands(rng, m, n, k, fmt, trans_b)
    want = orc.mx_gmm(pa, sa, pb, sb, n, k, FMT[fmt], trans_b)
    got = out_f32(cc.mx_matmul(dev(pa), dev(sa), dev(pb), dev(sb), fmt, trans_b))
    assert_close(got, want, ("mx tiled", fmt, shape, trans_b))


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e2m1"])
@pytest.mark.parametrize("trans_b", [0, 1])
@pytest.mark.parametrize("shape", _reference_shapes("ascend950_mxfp8_matmul_reduce_scatter"))
def test_mx_gemm_reference_shape_list_tiled(shape, trans_b, fmt, tiled_only):
    """Every (M, K, N) of the reference's MXFP8 list (K = 1216, 960 and 1984 end inside a 128-byte step
    and their scale rows start 2 bytes past a 4-byte boundary; K = 128 is a single step) on the MFMA
    path - a fall-back is an error here - in both layouts of B, and with the FP4 and E5M2 payloads at
    the same shapes."""
    m, k, n = shape
    rng = np.random.default_rng(m + k + n + trans_b)
    pa, sa, pb, sb = mx_operands(rng, m, n, k, fmt, trans_b, 0.02 if fmt == "e2m1" else 1.0)
    want = orc.mx_gmm(pa, sa, pb, sb, n, k, FMT[fmt], trans_b, blocked=True)
    got = out_f32(cc.mx_matmul(dev(pa), dev(sa), dev(pb), dev(sb), fmt, trans_b))
    assert_close(got, want, (shape, trans_b, fmt))
    assert_double_golden(got, want, (shape, trans_b, fmt))


@pytest.mark.parametrize("trans_b", [0, 1])
@pytest.mark.parametrize("shape", _reference_shapes("ascend950_mxfp8_matmul_reduce_scatter"))
def test_i8_dequant_reference_mx_shapes_tiled(shape, trans_b, tiled_only):
    """The int8 kernels at the same shapes (K tails of 64 and 96 bytes, a single K step)."""
    m, k, n = shape
    rng = np.random.default_rng(m + k + n + 17 * trans_b)
    a = rng.integers(-127, 128, (m, k)).astype(np.int8)
    b = rng.integers(-127, 128, (k, n)).astype(np.int8)
    pt = rng.uniform(0.001, 0.02, m).astype(np.float32)
    pc = rng.uniform(0.001, 0.02, n).astype(np.float32)
    want = orc.gemm_i8_dequant(a, b, pt, pc, blocked=True)
    bb = np.ascontiguousarray(b.T) if trans_b else b
    got = out_f32(cc.w8a8_matmul_dequant(dev(a), dev(bb), dev(pt), dev(pc), trans_b))
    assert_close(got, want, ("i8 tiled", shape, trans_b))


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e2m1"])
@pytest.mark.parametrize("cfg", [(5, 900, 1024, 416, [0, 300, 1, 0, 500]), (8, 3000, 768, 1056, None), (6, 1500, 1216, 520, None)])
@pytest.mark.parametrize("trans_b", [0, 1])
def test_mx_gmm_tiled(fmt, cfg, trans_b, tiled_only):
    e, t, k, n, gs = cfg
    rng = np.random.default_rng(400 + t + trans_b)
    gs = np.array(gs, np.int32) if gs is not None else zipf_groups(rng, t - 37, e)   # leaves 37 rows that belong to no group
    sigma = 0.02 if fmt == "e2m1" else 1.0
    pa, sa = orc.mx_quant_rows(rand_bf16(rng, (t, k), sigma), FMT[fmt])
    pbs, sbs = [], []
    for _ in range(e):
        pb, sb = orc.mx_quant_b(rand_bf16(rng, (k, n), sigma), FMT[fmt], orc.RNE, trans_b)
        pbs.append(pb)
        sbs.append(sb)
    pb, sb = np.stack(pbs), np.stack(sbs)
    want = orc.mx_gmm(pa, sa, pb, sb, n, k, FMT[fmt], trans_b, group_sizes=gs)
    got = out_f32(cc.mx_grouped_matmul(dev(pa), dev(sa), dev(pb), dev(sb), dev(gs), fmt, trans_b))
    assert_close(got, want, ("mx gmm tiled", fmt, cfg[:4], trans_b))


def test_mx_gmm_mapped_fp16_is_the_rounded_accumulator():
    """The half-precision output is the same fp32 result rounded to nearest even: on data whose
    results are exact in both types (small integers) the two outputs agree exactly, and on random
    data the fp16 output is closer to the oracle than bf16's 8 bits allow."""
    e, t, k, n = 2, 300, 256, 256
    rng = np.random.default_rng(5)
    gs = np.array([130, 170], np.int32)
    pa, sa = orc.mx_quant_rows(rand_bf16(rng, (t, k), 1.0), orc.E4M3)
    pbs, sbs = zip(*[orc.mx_quant_b(rand_bf16(rng, (k, n), 1.0), orc.E4M3, orc.RNE, 0) for _ in range(e)])
    pb, sb = np.stack(pbs), np.stack(sbs)
    gold = orc.mx_gmm(pa, sa, pb, sb, n, k, orc.E4M3, 0, group_sizes=gs)
    ident = np.arange(t, dtype=np.int32)
    for tiled in (True, False):
        cc.set_option("require_tiled_gemm", 1 if tiled else 0)
        cc.set_option("force_generic_gemm", 0 if tiled else 1)
        try:
            out_h = torch.zeros((t, n), dtype=torch.float16, device="cuda")
            out_b = torch.zeros((t, n), dtype=torch.bfloat16, device="cuda")
            cc.mx_grouped_matmul_mapped(dev(pa), dev(sa), dev(pb), dev(sb), dev(gs), dev(ident), out_h, "e4m3", 0)
            cc.mx_grouped_matmul_mapped(dev(pa), dev(sa), dev(pb), dev(sb), dev(gs), dev(ident), out_b, "e4m3", 0)
            torch.cuda.synchronize()
        finally:
            cc.set_option("require_tiled_gemm", 0)
            cc.set_option("force_generic_gemm", 0)
        h, b = out_h.float().cpu().numpy(), out_b.float().cpu().numpy()
        assert_close(h, gold, ("fp16 out", tiled))
        # bf16 of the half result equals the bf16 result wherever no double rounding can occur:
        # compare through the error against the fp32 oracle instead, half must be at least as close
        eh, eb = np.abs(h - gold), np.abs(b - gold)
        assert eh.mean() < 0.2 * eb.mean()
        # and fp16 rounding of the oracle's fp32 value is within one half-ulp of what came back
        assert np.max(np.abs(h - gold.astype(np.float16).astype(np.float32)) / np.maximum(np.abs(gold), 1.0)) < 2e-3


@pytest.mark.parametrize("fmt", ["e4m3", "e2m1"])
@pytest.mark.parametrize("trans_b", [0, 1])
@pytest.mark.parametrize("tiled", [True, False])
def test_mx_gmm_mapped_rows(fmt, trans_b, tiled):
    """Down-projection form: result rows leave in send-buffer order (by destination rank, then
    expert); dropped rows and rows of no group are not written."""
    ranks, e, k, n = 3, 5, 1024, 416
    rng = np.random.default_rng(77 + trans_b)
    g = rng.integers(0, 260, (ranks, e)).astype(np.int32)
    g[:, 2] = 0                                                  # an expert nobody routed to
    gs = g.sum(axis=0).astype(np.int32)
    used = int(gs.sum())
    t = used + 19                                                # rows past the groups
    rank_rows = int(g.sum(axis=1).max()) + 5
    row_map = np.full(t, -1, np.int32)
    row_map[:used] = orc.send_buffer_row_map(g, rank_rows)
    row_map[7] = -1                                              # a dropped row
    row_map[9] = ranks * rank_rows + 3                           # past the end of out: dropped as well
    sigma = 0.02 if fmt == "e2m1" else 1.0
    pa, sa = orc.mx_quant_rows(rand_bf16(rng, (t, k), sigma), FMT[fmt])
    pbs, sbs = [], []
    for _ in range(e):
        pb, sb = orc.mx_quant_b(rand_bf16(rng, (k, n), sigma), FMT[fmt], orc.RNE, trans_b)
        pbs.append(pb)
        sbs.append(sb)
    pb, sb = np.stack(pbs), np.stack(sbs)
    gold = orc.mx_gmm(pa, sa, pb, sb, n, k, FMT[fmt], trans_b, group_sizes=gs)
    kept = np.where(row_map[:used] < ranks * rank_rows, row_map[:used], -1)
    want = orc.scatter_rows(gold[:used], kept, ranks * rank_rows, fill=np.float32(-3.0))
    cc.set_option("require_tiled_gemm", 1 if tiled else 0)
    cc.set_option("force_generic_gemm", 0 if tiled else 1)
    try:
        out = torch.full((ranks * rank_rows, n), -3.0, dtype=torch.bfloat16, device="cuda")
        cc.mx_grouped_matmul_mapped(dev(pa), dev(sa), dev(pb), dev(sb), dev(gs), dev(row_map), out, fmt, trans_b)
        got = out_f32(out)
    finally:
        cc.set_option("require_tiled_gemm", 0)
        cc.set_option("force_generic_gemm", 0)
    untouched = np.ones(ranks * rank_rows, bool)
    untouched[kept[kept >= 0]] = False
    assert (got[untouched] == -3.0).all()
    assert_close(got[~untouched], want[~untouched], ("mx gmm mapped", fmt, trans_b, tiled))


def _both_paths(fn):
    """fn() on the tiled kernels (a fall-back would be an error) and on the generic ones."""
    outs = []
    for tiled in (True, False):
        cc.set_option("require_tiled_gemm", 1 if tiled else 0)
        cc.set_option("force_generic_gemm", 0 if tiled else 1)
        try:
            outs.append(out_f32(fn()))
        finally:
            cc.set_option("require_tiled_gemm", 0)
            cc.set_option("force_generic_gemm", 0)
    return outs


@pytest.mark.parametrize("seed", range(96))
def test_tiled_matches_generic_on_random_groups(seed):
    """Random expert counts, group sizes (empty, one-row, many-tile groups, rows of no group), K-step
    counts, widths and both weight layouts: the tiled kernels against the one-thread-per-output
    kernels on the device.  Both accumulate the same products in fp32 (int32 for int8), so they may
    differ only by summation order and one final rounding."""
    rng = np.random.default_rng(1000 + seed)
    e = int(rng.integers(1, 13))
    sizes = rng.choice([0, 1, 31, 33, 100, 129, 255, 256, 257, 300, 600, 1100], e).astype(np.int32)
    used = int(sizes.sum())
    t = used + int(rng.choice([0, 0, 5, 260]))
    if t == 0:
        t, sizes[0] = 40, 40
    kind = ["i8", "e4m3", "e5m2", "e2m1"][seed % 4]
    k = int(rng.choice([256, 384, 640, 1024])) * (2 if kind == "e2m1" else 1)    # whole 128-byte K-steps, at least two
    n = int(rng.choice([64, 160, 256, 416, 512, 672]))
    trans_b = int(rng.integers(0, 2))
    gs = dev(sizes)
    if kind == "i8":
        x = dev(rng.integers(-127, 128, (t, k)).astype(np.int8))
        w = dev(rng.integers(-127, 128, (e, n, k) if trans_b else (e, k, n)).astype(np.int8))
        pt = dev(rng.uniform(0.001, 0.02, t).astype(np.float32))
        pc = dev(rng.uniform(0.001, 0.02, (e, n)).astype(np.float32))
        a, b = _both_paths(lambda: cc.gmm_dequant_swiglu(x, w, gs, pt, pc, trans_b))
    else:
        pack = 2 if kind == "e2m1" else 1
        mask = 0x77 if kind != "e5m2" else 0x7B                       # finite codes only
        pa = dev((rng.integers(0, 256, (t, k // pack)) & (mask | 0x80 if pack == 1 else 0xFF)).astype(np.uint8))
        pb = dev((rng.integers(0, 256, ((e, n, k // pack) if trans_b else (e, k, n // pack))) & (mask | 0x80 if pack == 1 else 0xFF)).astype(np.uint8))
        sa = dev(rng.integers(120, 132, (t, k // 32)).astype(np.uint8))
        sb = dev(rng.integers(120, 132, ((e, n, k // 32) if trans_b else (e, k // 64, n, 2))).astype(np.uint8))
        a, b = _both_paths(lambda: cc.mx_grouped_matmul(pa, sa, pb, sb, gs, kind, trans_b))
    assert np.isfinite(a).all() and np.isfinite(b).all()
    assert (a[used:] == 0).all() and (b[used:] == 0).all()               # rows of no group
    # one bf16 unit in the last place of the element itself, plus summation-order noise relative to the typical size
    scale = max(float(np.sqrt(np.mean(b[:used].astype(np.float64) ** 2))), 1e-30) if used else 1.0
    excess = np.abs(a - b) - (2.0 ** -7 * np.abs(b) + 1e-3 * scale)
    assert excess.max() <= 0, (seed, e, sizes.tolist(), t, k, n, trans_b, kind, float(excess.max()), scale)


@pytest.mark.parametrize("trans_b", [0, 1])
@pytest.mark.parametrize("tiled", [True, False])
def test_gmm_i8_dequant_without_activation(trans_b, tiled):
    """Grouped int8 matmul + per-token x per-channel dequant: every group is the dense golden of its rows."""
    e, t, k, n = 5, 900, 512, 384
    rng = np.random.default_rng(31 + trans_b)
    gs = np.array([0, 300, 1, 420, 150], np.int32)            # 29 rows belong to no group
    x = rng.integers(-127, 128, (t, k)).astype(np.int8)
    w = rng.integers(-127, 128, (e, k, n)).astype(np.int8)
    pt = rng.uniform(0.001, 0.02, t).astype(np.float32)
    pc = rng.uniform(0.001, 0.02, (e, n)).astype(np.float32)
    want = np.zeros((t, n), np.float32)
    r0 = 0
    for g in range(e):
        r1 = r0 + int(gs[g])
        if r1 > r0:
            want[r0:r1] = orc.gemm_i8_dequant(x[r0:r1], w[g], pt[r0:r1], pc[g])
        r0 = r1
    ww = np.ascontiguousarray(w.transpose(0, 2, 1)) if trans_b else w
    cc.set_option("require_tiled_gemm", 1 if tiled else 0)
    cc.set_option("force_generic_gemm", 0 if tiled else 1)
    try:
        got = out_f32(cc.gmm_dequant(dev(x), dev(ww), dev(gs), dev(pt), dev(pc), trans_b))
    finally:
        cc.set_option("require_tiled_gemm", 0)
        cc.set_option("force_generic_gemm", 0)
    assert (got[r0:] == 0).all()
    assert_close(got, want, ("gmm i8 dequant", trans_b, tiled))


@pytest.mark.parametrize("fmt", ["e4m3", "e2m1"])
@pytest.mark.parametrize("tiled", [True, False])
def test_mx_gmm_half_output_without_a_row_map(fmt, tiled):
    """out_dtype float16 on the plain grouped matmul: same accumulators, rounded to half; rows of no
    group are zero-filled as in the bf16 call."""
    ofmt = orc.E4M3 if fmt == "e4m3" else orc.E2M1
    e, t, k, n = 3, 700, 512, 384
    rng = np.random.default_rng(9)
    gs = np.array([300, 0, 370], np.int32)             # 30 rows belong to no group
    pa, sa = orc.mx_quant_rows(rand_bf16(rng, (t, k), 1.0), ofmt)
    pbs, sbs = zip(*[orc.mx_quant_b(rand_bf16(rng, (k, n), 1.0), ofmt, orc.RNE, 0) for _ in range(e)])
    pb, sb = np.stack(pbs), np.stack(sbs)
    gold = orc.mx_gmm(pa, sa, pb, sb, n, k, ofmt, 0, group_sizes=gs)
    cc.set_option("require_tiled_gemm", 1 if tiled else 0)
    cc.set_option("force_generic_gemm", 0 if tiled else 1)
    try:
        h = cc.mx_grouped_matmul(dev(pa), dev(sa), dev(pb), dev(sb), dev(gs), fmt, 0, out_dtype=torch.float16)
        b = cc.mx_grouped_matmul(dev(pa), dev(sa), dev(pb), dev(sb), dev(gs), fmt, 0)
        torch.cuda.synchronize()
    finally:
        cc.set_option("require_tiled_gemm", 0)
        cc.set_option("force_generic_gemm", 0)
    assert h.dtype == torch.float16 and b.dtype == torch.bfloat16
    hf, bf = h.float().cpu().numpy(), b.float().cpu().numpy()
    assert (hf[670:] == 0).all() and (bf[670:] == 0).all()
    assert_close(hf, gold, ("fp16 out", fmt, tiled))
    assert np.abs(hf - gold).mean() < 0.2 * np.abs(bf - gold).mean()


def test_fall_back_note_describes_the_call_that_fell_back_only():
    """A GEMM call that runs on the generic kernels returns CCH_OK and leaves a note for cch_last_error(); the next call,
    which the tiled kernels take, must leave the message empty (a caller that reads it after CCH_OK to find out which
    path ran would otherwise see the earlier call's note)."""
    from catccos_amd import _abi
    rng = np.random.default_rng(31)
    t, n = 64, 64
    pt, pc = dev(rng.uniform(0.001, 0.02, t).astype(np.float32)), dev(rng.uniform(0.001, 0.02, n).astype(np.float32))
    last = lambda: _abi.lib().cch_last_error().decode()
    # K = 40 is no multiple of 16 bytes: generic kernels
    a, b = dev(rng.integers(-127, 128, (t, 40)).astype(np.int8)), dev(rng.integers(-127, 128, (40, n)).astype(np.int8))
    cc.w8a8_matmul_dequant(a, b, pt, pc, 0)
    assert "one-thread-per-element" in last()
    a, b = dev(rng.integers(-127, 128, (t, 64)).astype(np.int8)), dev(rng.integers(-127, 128, (64, n)).astype(np.int8))
    cc.w8a8_matmul_dequant(a, b, pt, pc, 0)
    assert last() == ""
    torch.cuda.synchronize()


def test_generic_kernels_take_more_than_65535_rows():
    """The one-thread-per-element kernels put the rows on the grid's x axis: a problem the tiled kernels do not take
    (K no multiple of 16 bytes) runs at any row count (the reference takes such shapes; an earlier form of the generic
    path stopped at 65535 rows)."""
    rng = np.random.default_rng(41)
    t, k, n = 70000, 40, 8
    a = rng.integers(-127, 128, (t, k)).astype(np.int8)
    b = rng.integers(-127, 128, (k, n)).astype(np.int8)
    pt = rng.uniform(0.001, 0.02, t).astype(np.float32)
    pc = rng.uniform(0.001, 0.02, n).astype(np.float32)
    got = out_f32(cc.w8a8_matmul_dequant(dev(a), dev(b), dev(pt), dev(pc), 0))
    assert_close(got, orc.gemm_i8_dequant(a, b, pt, pc), "generic path, 70000 rows")


# ---------------------------------------------------------------- tile order

def test_grouped_tile_order_covers_every_tile_once():
    """More tiles than workgroups (several rounds and a partial last one), so the per-XCD tile order of
    the grouped kernels is in force: every tile must still be computed exactly once.  The output equals
    the row-major order's bit for bit (each tile accumulates in the same order), and the oracle's."""
    e, t, k, n = 7, 4700, 256, 4096
    rng = np.random.default_rng(11)
    gs = np.array([900, 0, 1300, 37, 256, 1700, 507], np.int32)
    assert gs.sum() == t
    pa, sa = orc.mx_quant_rows(rand_bf16(rng, (t, k), 1.0), orc.E4M3)
    pbs, sbs = zip(*[orc.mx_quant_b(rand_bf16(rng, (k, n), 1.0), orc.E4M3, orc.RNE, 0) for _ in range(e)])
    pb, sb = np.stack(pbs), np.stack(sbs)
    gold = orc.mx_gmm(pa, sa, pb, sb, n, k, orc.E4M3, 0, group_sizes=gs)
    ident = np.arange(t, dtype=np.int32)
    outs = {}
    cc.set_option("require_tiled_gemm", 1)
    try:
        for order in (0, 1, 2, -1, 4):
            # 4: the default order with non-temporal output stores
            cc.set_option("gemm_nt_output", 1 if order == 4 else 0 if order == 0 else -1)
            cc.set_option("gemm_tile_order", -1 if order >= 3 else order)
            # the output starts as NaN: a tile that no workgroup computes would keep it
            out = torch.full((t, n), float("nan"), dtype=torch.bfloat16, device="cuda")
            cc.mx_grouped_matmul_mapped(dev(pa), dev(sa), dev(pb), dev(sb), dev(gs), dev(ident), out, "e4m3", 0)
            outs[order] = out_f32(out)
    finally:
        cc.set_option("gemm_tile_order", -1)
        cc.set_option("gemm_nt_output", -1)
        cc.set_option("require_tiled_gemm", 0)
    assert not np.isnan(outs[1]).any()
    for order in (1, 2, -1, 4):
        assert np.array_equal(outs[0], outs[order]), order
    assert_close(outs[1], gold, "per-XCD tile order")


@pytest.mark.parametrize("e,t,seed", [(70, 9000, 1), (200, 20000, 2), (256, 12000, 3), (5, 1300, 4)])
def test_group_table_of_many_groups_covers_every_tile_once(e, t, seed):
    """The tiled kernels build their table of row ranges and row tiles with wave-wide prefix sums, 64 groups per batch:
    with more groups than one batch, empty ones, groups of one row, of exactly one and of several row tiles and rows that
    belong to no group, every output element must be written exactly once (the output starts as NaN and is written
    through an identity row map, which leaves rows of no group alone), the same bits under every tile order, and agree
    with the oracle."""
    rng = np.random.default_rng(seed)
    k, n = 128, 4096
    gs = rng.integers(0, 2 * t // e, e).astype(np.int32)
    gs[rng.integers(0, e, max(e // 8, 1))] = 0
    gs[rng.integers(0, e)] = 256
    gs[rng.integers(0, e)] = 64
    gs[rng.integers(0, e)] = 1
    while gs.sum() > t - 5:
        gs[int(gs.argmax())] //= 2
    pa, sa = orc.mx_quant_rows(rand_bf16(rng, (t, k), 1.0), orc.E4M3)
    pbs, sbs = zip(*[orc.mx_quant_b(rand_bf16(rng, (k, n), 1.0), orc.E4M3, orc.RNE, 0) for _ in range(e)])
    pb, sb = np.stack(pbs), np.stack(sbs)
    ident = np.arange(t, dtype=np.int32)
    outs = {}
    cc.set_option("require_tiled_gemm", 1)
    try:
        for order in (0, 1, 2):
            cc.set_option("gemm_tile_order", order)
            out = torch.full((t, n), float("nan"), dtype=torch.bfloat16, device="cuda")
            cc.mx_grouped_matmul_mapped(dev(pa), dev(sa), dev(pb), dev(sb), dev(gs), dev(ident), out, "e4m3", 0)
            outs[order] = out_f32(out)
    finally:
        cc.set_option("gemm_tile_order", -1)
        cc.set_option("require_tiled_gemm", 0)
    used = int(gs.sum())
    for order in (0, 1, 2):
        assert not np.isnan(outs[order][:used]).any(), order
        assert np.isnan(outs[order][used:]).all(), order   # rows of no group are not written through a row map
        assert np.array_equal(outs[0][:used], outs[order][:used]), order
    gold = orc.mx_gmm(pa, sa, pb, sb, n, k, orc.E4M3, 0, group_sizes=gs)
    assert_close(outs[2][:used], gold[:used], ("many groups", e, t))


# ---------------------------------------------------------------- half-precision output

@pytest.mark.parametrize("tiled", [True, False], ids=["tiled", "generic"])
def test_fp16_output_of_the_int8_and_dense_mx_operators(tiled):
    """IEEE half output (what the reference's int8 launchers write, tests/dynamic_tiling/impl/kernel_int8.cpp:16)
    is the same fp32 result rounded to half: within the gate against the oracle and closer to it than bf16's
    8 bits allow (the oracle's fp32 value against a correctly rounded half: at most 2^-11 apart, relative)."""
    rng = np.random.default_rng(21)
    e, t, k, n = 3, 300, 256, 256
    gs = np.array([130, 0, 170], np.int32)
    xi = rng.integers(-127, 128, (t, k)).astype(np.int8)
    wi = rng.integers(-127, 128, (e, k, n)).astype(np.int8)
    pt = rng.uniform(0.001, 0.02, t).astype(np.float32)
    pc = rng.uniform(0.001, 0.02, (e, n)).astype(np.float32)
    pa, sa = orc.mx_quant_rows(rand_bf16(rng, (t, k), 1.0), orc.E4M3)
    pb, sb = orc.mx_quant_b(rand_bf16(rng, (k, n), 1.0), orc.E4M3, orc.RNE, 0)
    golds = {
        "dense": orc.gemm_i8_dequant(xi, wi[0], pt, pc[0]),
        "gmm": np.concatenate([orc.gemm_i8_dequant(xi[:130], wi[0], pt[:130], pc[0]), orc.gemm_i8_dequant(xi[130:], wi[2], pt[130:], pc[2])]),
        "swiglu": orc.gmm_i8_dequant_swiglu(xi, wi, gs, pt, pc),
        "mx": orc.mx_gmm(pa, sa, pb[None], sb[None], n, k, orc.E4M3, 0),
    }
    cc.set_option("require_tiled_gemm", 1 if tiled else 0)
    cc.set_option("force_generic_gemm", 0 if tiled else 1)
    try:
        for dt in (torch.float16, torch.bfloat16):
            outs = {
                "dense": cc.w8a8_matmul_dequant(dev(xi), dev(wi[0]), dev(pt), dev(pc[0]), 0, out_dtype=dt),
                "gmm": cc.gmm_dequant(dev(xi), dev(wi), dev(gs), dev(pt), dev(pc), 0, out_dtype=dt),
                "swiglu": cc.gmm_dequant_swiglu(dev(xi), dev(wi), dev(gs), dev(pt), dev(pc), 0, out_dtype=dt),
                "mx": cc.mx_matmul(dev(pa), dev(sa), dev(pb), dev(sb), "e4m3", 0, out_dtype=dt),
            }
            for name, out in outs.items():
                assert out.dtype == dt
                got = out_f32(out)
                assert_close(got, golds[name], (name, dt, tiled))
                if dt == torch.float16:
                    # 11 significant bits: relative error of a correctly rounded half is at most 2^-11
                    big = np.abs(golds[name]) > 1.0   # away from cancellation, where fp32 summation order shows
                    rel = np.abs(got - golds[name])[big] / np.abs(golds[name])[big]
                    if name == "mx":
                        # the matrix unit's fp32 summation differs from the oracle's by up to ~1e-3 on single
                        # values; on average the half output must still beat what bf16 could give (2^-10)
                        assert rel.mean() <= 2.0 ** -11 and rel.max() <= 2.0 ** -9, (name, rel.mean(), rel.max())
                    else:
                        assert rel.max() <= 2.0 ** -10, (name, rel.max())
    finally:
        cc.set_option("require_tiled_gemm", 0)
        cc.set_option("force_generic_gemm", 0)


@pytest.mark.parametrize("sizes,t", [([-5, 300, -1, 2 ** 30, 7], 500), ([2 ** 31 - 1, 2 ** 31 - 1, 5], 300), ([0, 0, 0], 64), ([100] * 200, 9000)],
                         ids=["negative-and-huge", "sum-overflows-int32", "all-empty", "200-groups-run-out-of-rows"])
def test_group_sizes_are_clipped_the_same_way_on_both_paths(sizes, t):
    """Group sizes below zero count as empty and the groups stop where the rows do (the reference's golden pads the
    remainder with zeros, examples/utils/gen_data_fp4_mx_alltoallv_gmm.py:788-790): the tiled kernels (table built by
    one wave with two scans) and the generic ones (one thread's running sum) agree to the bit on which rows belong
    to which expert, and with the oracle fed the clipped sizes."""
    rng = np.random.default_rng(len(sizes) + t)
    e, k, n = len(sizes), 256, 256
    gs_h = np.array(sizes, dtype=np.int64).astype(np.int32)
    clipped, row = [], 0
    for s in gs_h.tolist():
        c = max(0, min(int(s), t - row))
        clipped.append(c)
        row += c
    x = rng.integers(-127, 128, (t, k)).astype(np.int8)
    w = rng.integers(-3, 4, (e, k, n)).astype(np.int8)
    pt = rng.uniform(0.001, 0.02, t).astype(np.float32)
    pc = rng.uniform(0.001, 0.02, (e, n)).astype(np.float32)
    a, b = _both_paths(lambda: cc.gmm_dequant(dev(x), dev(w), dev(gs_h), dev(pt), dev(pc), 0))
    assert np.array_equal(a, b)            # exact int32 sums, the same two fp32 products and one rounding on either path
    want = np.zeros((t, n), np.float32)
    r0 = 0
    for g, c in enumerate(clipped):
        if c:
            want[r0:r0 + c] = orc.gemm_i8_dequant(x[r0:r0 + c], w[g], pt[r0:r0 + c], pc[g])
        r0 += c
    assert_close(a, want)
    assert (a[r0:] == 0).all()
