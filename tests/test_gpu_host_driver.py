"""End-to-end through the C++ operator surface, the way the reference's run.sh scripts test an
operator: write input .bin files, run the driver binary, compare the output files with the golden
(here: the CPU oracle)."""
import json
import os
import subprocess

import numpy as np
import pytest

import oracle as orc
from test_gpu_gemm import assert_close, rand_bf16, zipf_groups

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "catccos_amd", "catccos_run")


def drive(tmp_path, *args):
    r = subprocess.run([DRIVER, *map(str, args)], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "error num: 0" in r.stdout and "[ERROR]" not in r.stdout, r.stdout
    assert "[PERF] Avg latency" in r.stdout


def bf16_file(path, shape):
    return orc.bf16_to_f32(np.fromfile(path, dtype=np.uint16)).reshape(shape)


def test_mx_quant_files_byte_exact(tmp_path):
    """Shapes of the reference's own list (ascend950_mx_quant_allgather/scripts/test_shapes.csv), shrunk in M."""
    for m, n in ((512, 1024), (510, 1024)):
        d = tmp_path / str(m)   # result files are written in place (no truncation), so one directory per shape
        d.mkdir()
        rng = np.random.default_rng(m)
        x = rand_bf16(rng, (m, n))
        x.tofile(d / "rank_0_input.bin")
        drive(d, "mxqtag", m, 0, n, d, "--iters", 1, "--warmup", 1)
        q, s = orc.mx_quant_rows(x, orc.E4M3)
        assert np.array_equal(np.fromfile(d / "rank_0_output.bin", dtype=np.uint8).reshape(m, n), q)
        assert np.array_equal(np.fromfile(d / "rank_0_mxscale.bin", dtype=np.uint8).reshape(m, n // 32), s)


@pytest.mark.parametrize("fixpipe_words", [False, True])
def test_int8_dequant_files(tmp_path, fixpipe_words):
    m, k, n = 384, 512, 640
    rng = np.random.default_rng(1)
    a = rng.integers(-16, 16, (m, k)).astype(np.int8)      # the reference's data range
    b = rng.integers(-16, 16, (k, n)).astype(np.int8)
    pc = rng.uniform(0.001, 0.02, n).astype(np.float32)
    pt = rng.uniform(0.001, 0.02, m).astype(np.float32)
    a.tofile(tmp_path / "a_gm_rank0.bin")
    b.tofile(tmp_path / "b_gm_rank0.bin")
    if fixpipe_words:   # 64-bit words, low half = fp32 scale with 13 mantissa bits cleared
        pc = (pc.view(np.uint32) & 0xFFFFE000).view(np.float32)
        pc.view(np.uint32).astype(np.uint64).tofile(tmp_path / "scale_gm.bin")
        pt[:] = 1.0
    else:
        pc.tofile(tmp_path / "scale_gm.bin")
        pt.tofile(tmp_path / "pertoken_scale_gm_rank0.bin")
    drive(tmp_path, "agmmdq", m, k, n, tmp_path, "--iters", 1, "--warmup", 0)
    assert_close(bf16_file(tmp_path / "output_rank0.bin", (m, n)), orc.gemm_i8_dequant(a, b, pt, pc))


def test_mxfp8_dense_files_rank_offset(tmp_path):
    m, k, n = 256, 256, 384
    rng = np.random.default_rng(2)
    pa, sa = orc.mx_quant_rows(rand_bf16(rng, (m, k)), orc.E4M3)
    pb, sb = orc.mx_quant_b(rand_bf16(rng, (k, n)), orc.E4M3, orc.RNE, 1)   # the reference's run uses transB=1
    for name, arr in (("a", pa), ("b", pb), ("a_scale", sa), ("b_scale", sb)):
        arr.tofile(tmp_path / f"rank_1_{name}.bin")
    drive(tmp_path, "a5mxfp8mmrs", m, k, n, tmp_path, "--transB", 1, "--rank", 1, "--iters", 1, "--warmup", 0)
    out = orc.bf16_to_f32(np.fromfile(tmp_path / "output.bin", dtype=np.uint16))
    assert out.size == 2 * m * n                      # rank 1 wrote the second slice
    assert_close(out[m * n:].reshape(m, n), orc.mx_gmm(pa, sa, pb, sb, n, k, orc.E4M3, 1))


def test_dispatch_gmm_swiglu_files(tmp_path):
    e, t, k, n = 4, 700, 256, 512
    rng = np.random.default_rng(3)
    gs = zipf_groups(rng, t, e)
    x = rng.integers(-127, 128, (t, k)).astype(np.int8)
    w = rng.integers(-16, 16, (e, k, n)).astype(np.int8)
    pt = rng.uniform(0.001, 0.02, t).astype(np.float32)
    pc = rng.uniform(0.001, 0.02, (e, n)).astype(np.float32)
    x.tofile(tmp_path / "a_gm_0.bin"); w.tofile(tmp_path / "b_gm_0.bin"); pc.tofile(tmp_path / "scale_gm_0.bin")
    pt.tofile(tmp_path / "pertoken_scale_0.bin"); gs.tofile(tmp_path / "group_list_0.bin")
    drive(tmp_path, "dgds", t, k, n, tmp_path, "--experts", e, "--iters", 1, "--warmup", 0)
    assert_close(bf16_file(tmp_path / "output_0.bin", (t, n // 2)), orc.gmm_i8_dequant_swiglu(x, w, gs, pt, pc))


@pytest.mark.parametrize("fp16", [0, 1])
@pytest.mark.parametrize("kernel,fmt", [("a5fp4mxatavgmm", orc.E2M1), ("a5fp8mxatavgmm", orc.E4M3)])
def test_mx_grouped_files(tmp_path, kernel, fmt, fp16):
    """The reference's own shape for this operator: 1024 x 256 x 256, 4 experts (test_shapes.csv)."""
    e, t, k, n = 4, 1024, 256, 256
    rng = np.random.default_rng(4)
    gs = zipf_groups(rng, t, e)
    pa, sa = orc.mx_quant_rows(rand_bf16(rng, (t, k), 0.5), fmt)
    pbs, sbs = zip(*[orc.mx_quant_b(rand_bf16(rng, (k, n), 0.5), fmt, orc.RNE, 0) for _ in range(e)])
    pb, sb = np.stack(pbs), np.stack(sbs)
    pa.tofile(tmp_path / "input_a_0.bin"); pb.tofile(tmp_path / "input_b_0.bin")
    sa.tofile(tmp_path / "input_a_scale_0.bin"); sb.tofile(tmp_path / "input_b_scale_0.bin")
    gs.tofile(tmp_path / "global_tokens_per_local_expert_0.bin")
    drive(tmp_path, kernel, t, k, n, tmp_path, "--experts", e, "--fp16", fp16, "--iters", 1, "--warmup", 0)
    if fp16:
        got = np.fromfile(tmp_path / "output_0.bin", dtype=np.float16).astype(np.float32).reshape(t, n)
    else:
        got = bf16_file(tmp_path / "output_0.bin", (t, n))
    assert_close(got, orc.mx_gmm(pa, sa, pb, sb, n, k, fmt, 0, group_sizes=gs))


@pytest.mark.parametrize("fp16", [0, 1])
@pytest.mark.parametrize("kernel,fmt", [("a5fp4gmmata", orc.E2M1), ("a5fp8gmmata", orc.E4M3)])
def test_mx_grouped_down_projection_files(tmp_path, kernel, fmt, fp16):
    """Down projection with two source ranks: rows arrive by (expert, rank) and leave by (rank, expert),
    rank r's rows in region r of the output (file names of ascend950_fp8_mx_grouped_matmul_alltoallv_host.h)."""
    ranks, e, t, k, n = 2, 4, 1024, 256, 256
    rng = np.random.default_rng(6)
    g = rng.multinomial(t - 24, np.ones(ranks * e) / (ranks * e)).reshape(ranks, e).astype(np.int32)
    g[1, 2] = 0
    gs = g.sum(axis=0).astype(np.int32)
    used = int(gs.sum())
    pa, sa = orc.mx_quant_rows(rand_bf16(rng, (t, k), 0.5), fmt)
    pbs, sbs = zip(*[orc.mx_quant_b(rand_bf16(rng, (k, n), 0.5), fmt, orc.RNE, 0) for _ in range(e)])
    pb, sb = np.stack(pbs), np.stack(sbs)
    pa.tofile(tmp_path / "a_gm_0.bin"); pb.tofile(tmp_path / "b_gm_0.bin")
    sa.tofile(tmp_path / "a_scale_0.bin"); sb.tofile(tmp_path / "b_scale_0.bin")
    g.tofile(tmp_path / "global_tokens_per_local_expert_0.bin")
    np.zeros(e, np.int32).tofile(tmp_path / "local_tokens_per_expert_0.bin")
    drive(tmp_path, kernel, t, k, n, tmp_path, "--experts", e, "--ranks", ranks, "--fp16", fp16, "--iters", 1, "--warmup", 0)
    gold = orc.mx_gmm(pa, sa, pb, sb, n, k, fmt, 0, group_sizes=gs)
    want = orc.scatter_rows(gold[:used], orc.send_buffer_row_map(g, rank_rows=t), ranks * t, fill=np.float32(0))
    if fp16:     # the type the reference registers this operator for
        got = np.fromfile(tmp_path / "output_0.bin", dtype=np.float16).astype(np.float32).reshape(ranks * t, n)
    else:
        got = bf16_file(tmp_path / "output_0.bin", (ranks * t, n))
    assert_close(got, want)


@pytest.mark.parametrize("words", [True, False])
def test_dispatch_gmm_swiglu_from_bf16_tokens(tmp_path, words):
    """The reference's own file set for this operator: bf16 tokens + expert_idx [m, topK] + per-channel
    scales as 64-bit fix-pipe words (dispatch_gmm_dequant_swiglu_host.h:21-71).  Routing on the host,
    dynamic int8 quantisation with the expert-sorted gather and the grouped matmul on the device."""
    e, m, topk, k, n = 8, 300, 2, 512, 512
    rng = np.random.default_rng(8)
    xb = rand_bf16(rng, (m, k), 1.5)
    expert_idx = rng.integers(0, e, (m, topk)).astype(np.int32)
    expert_idx[expert_idx == 5] = 4                                   # an expert nobody routes to
    w = rng.integers(-16, 16, (e, k, n)).astype(np.int8)
    pc = rng.uniform(0.001, 0.02, (e, n)).astype(np.float32)
    xb.tofile(tmp_path / "a_gm_0.bin"); w.tofile(tmp_path / "b_gm_0.bin"); expert_idx.tofile(tmp_path / "expert_idx_0.bin")
    if words:
        raw = np.zeros((e, n), np.uint64)
        raw[:] = pc.view(np.uint32)
        raw.tofile(tmp_path / "scale_gm_0.bin")
    else:
        pc.tofile(tmp_path / "scale_gm_0.bin")
    drive(tmp_path, "dgds", m, k, n, tmp_path, "--experts", e, "--topk", topk, "--iters", 1, "--warmup", 0)
    flat = expert_idx.reshape(-1)
    order = np.argsort(flat, kind="stable").astype(np.int32)          # moe_init_routing: sorted position -> flat index
    gs = np.bincount(flat, minlength=e).astype(np.int32)
    q, s = orc.dyn_quant_i8_rows(xb, order, topk, orc.DQ_DEVICE)
    want = orc.gmm_i8_dequant_swiglu(q, w, gs, s, pc)
    assert_close(bf16_file(tmp_path / "output_0.bin", (m * topk, n // 2)), want)


def test_shape_list_walk(tmp_path):
    """One process walks a test_shapes.csv (header + M,K,N lines, the loop of the reference's run.sh):
    per-shape data directories, outputs against the oracle."""
    shapes = [(256, 256, 384), (130, 512, 256)]
    csv = tmp_path / "test_shapes.csv"
    csv.write_text("M,K,N\n" + "".join(f"{m},{k},{n}\n" for m, k, n in shapes) + "\n")
    want = {}
    for i, (m, k, n) in enumerate(shapes):
        d = tmp_path / f"{m}_{k}_{n}"
        d.mkdir()
        rng = np.random.default_rng(40 + i)
        pa, sa = orc.mx_quant_rows(rand_bf16(rng, (m, k)), orc.E4M3)
        pb, sb = orc.mx_quant_b(rand_bf16(rng, (k, n)), orc.E4M3, orc.RNE, 1)
        for name, arr in (("a", pa), ("b", pb), ("a_scale", sa), ("b_scale", sb)):
            arr.tofile(d / f"rank_0_{name}.bin")
        want[(m, k, n)] = orc.mx_gmm(pa, sa, pb, sb, n, k, orc.E4M3, 1)
    r = subprocess.run([DRIVER, "a5mxfp8mmrs", "--shapes", str(csv), str(tmp_path), "--transB", "1", "--iters", "1", "--warmup", "0"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count("Processing test case") == 2 and "2 shapes finished" in r.stdout, r.stdout
    for (m, k, n), w in want.items():
        assert_close(bf16_file(tmp_path / f"{m}_{k}_{n}" / "output.bin", (m, n)), w)
    # perf mode over the same list, and a list that cannot be read
    r = subprocess.run([DRIVER, "a5mxfp8mmrs", "--shapes", str(csv), "-", "--iters", "2"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.count("[PERF] Avg latency") == 2, r.stdout + r.stderr
    r = subprocess.run([DRIVER, "a5mxfp8mmrs", "--shapes", str(tmp_path / "missing.csv"), "-"], capture_output=True, text=True, timeout=60)
    assert r.returncode != 0


@pytest.mark.parametrize("m,k,n,e,topk", [(4, 512, 1024, 16, 6), (300, 256, 512, 8, 2), (256, 7168, 1024, 16, 6)],
                         ids=["m4-top6", "m300-top2", "reference-shape-256x7168x1024"])
def test_dispatch_ffn_combine_files(tmp_path, m, k, n, e, topk):
    """The reference's file set of the MXFP8 FFN example (ascend950_dispatch_ffn_combine_host.h:15-150, written the way
    examples/utils/gen_data_moe.py:460-616 writes it: weights transposed, gate weights a softmax, routes distinct per
    token) through the driver; the golden is that generator's chain restated with the oracle's routines.  The third case
    is a line of the example's own shape list (scripts/test_shapes.csv) with its run.sh's 16 experts and top-6."""
    rng = np.random.default_rng(m + e)
    x = rand_bf16(rng, (m, k))
    expert_idx = np.argsort(rng.random((m, e)), axis=1)[:, :topk].astype(np.int32)
    logits = rng.standard_normal((m, topk)).astype(np.float32)
    probs = (np.exp(logits) / np.exp(logits).sum(1, keepdims=True)).astype(np.float32)
    h = n // 2
    w1 = [orc.f32_to_bf16((rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32)) for _ in range(e)]
    w2 = [orc.f32_to_bf16((rng.standard_normal((h, k)) / np.sqrt(h)).astype(np.float32)) for _ in range(e)]
    b1, sb1 = map(np.stack, zip(*[orc.mx_quant_b(w, orc.E4M3, orc.RNE, 1) for w in w1]))      # [E, n, k], scales [E, n, k/32]
    b2, sb2 = map(np.stack, zip(*[orc.mx_quant_b(w, orc.E4M3, orc.RNE, 1) for w in w2]))      # [E, k, h], scales [E, k, h/32]
    for name, arr in (("in_routing_matrix_a", x), ("in_routing_expert_idx", expert_idx), ("in_gather_gate_weight", probs),
                      ("in_gmm_matrix_b", b1), ("in_gmm_matrix_b_scale", sb1), ("in_gmm_matrix_b2", b2), ("in_gmm_matrix_b2_scale", sb2)):
        arr.tofile(tmp_path / f"{name}_0.bin")
    drive(tmp_path, "a5moe", m, k, n, tmp_path, "--experts", e, "--topk", topk, "--iters", 1, "--warmup", 1)
    rows = m * topk
    _, s2d, cnt = orc.moe_init_routing(expert_idx, e)
    packed = orc.mx_quant_scatter_packed(x, s2d, rows, topk, orc.E4M3)
    _, c1 = orc.mx_gmm(packed[:, :k], packed[:, k:], b1, sb1, n, k, orc.E4M3, 1, group_sizes=cnt, want_bf16=True, blocked=True)
    a2, sa2 = orc.mx_quant_rows(orc.swiglu_bf16(c1), orc.E4M3)
    _, y = orc.mx_gmm(a2, sa2, b2, sb2, k, h, orc.E4M3, 1, group_sizes=cnt, want_bf16=True, blocked=True)
    want = orc.bf16_to_f32(orc.moe_token_unpermute(y, s2d, probs, topk))
    got = bf16_file(tmp_path / "output_0.bin", (m, k))
    # two implementations of this chain agree to about 1 % of the tensor's rms: a bf16 step in GMM1's result moves a code
    # of the quantised activation (tests/test_gpu_ffn_chain.py checks the stages one by one, to the bit where they are bytes)
    rms = np.sqrt(np.mean(want ** 2))
    assert np.sqrt(np.mean((got - want) ** 2)) <= 2e-2 * rms and np.abs(got - want).max() <= 0.12 * rms
    # perf mode: constant inputs, nothing written
    drive(tmp_path, "a5moe", m, k, n, "-", "--experts", e, "--topk", topk, "--iters", 2, "--warmup", 1)
    # the reference's own shape rule and message (ascend950_dispatch_ffn_combine_host.h:180-184); one rank only
    r = subprocess.run([DRIVER, "a5moe", "64", "7168", "1000", "-", "--experts", "8", "--topk", "2"], capture_output=True, text=True, timeout=60)
    assert r.returncode != 0 and "MXFP8 FFN requires K % 256 == 0 and N % 512 == 0" in r.stdout
    r = subprocess.run([DRIVER, "a5moe", "64", "256", "512", "-", "--experts", "8", "--topk", "2", "--ranks", "2"], capture_output=True, text=True, timeout=60)
    assert r.returncode != 0 and "one rank" in r.stdout


def test_dispatch_ffn_combine_reference_shape_list_perf_mode(tmp_path):
    """Every line of the example's own shape list (tests/golden/reference_shapes.json, from its scripts/test_shapes.csv) with
    its run.sh's 16 experts and top-6, on constant inputs: the driver's shape walk, all five launches on the tiled kernels."""
    shapes = json.load(open(os.path.join(ROOT, "tests", "golden", "reference_shapes.json")))["ascend950_dispatch_ffn_combine"]
    assert [256, 7168, 1024] in shapes and len(shapes) == 4
    csv = tmp_path / "test_shapes.csv"
    csv.write_text("M,K,N\n" + "".join("%d,%d,%d\n" % tuple(s) for s in shapes))
    r = subprocess.run([DRIVER, "a5moe", "--shapes", str(csv), "-", "--experts", "16", "--topk", "6", "--iters", "3", "--warmup", "2"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.count("[PERF] Avg latency") == 4 and "4 shapes finished" in r.stdout, r.stdout + r.stderr
    assert "[ERROR]" not in r.stdout and "generic" not in r.stderr, r.stdout + r.stderr
    print(r.stdout)


def test_run_examples_walks_every_operator(tmp_path):
    """`python -m catccos_amd.run_examples` (the counterpart of the reference's examples/run_all_examples.sh): every operator
    over its reference shape list in perf mode, log patterns checked, summary line, exit status."""
    import sys
    r = subprocess.run([sys.executable, "-m", "catccos_amd.run_examples", "--iters", "2", "--warmup", "1", "--logs", str(tmp_path)],
                       capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "summary: 9 of 9 operators ran every shape of their lists" in r.stdout, r.stdout
    assert r.stdout.count("a5moe") == 4 and r.stdout.count("a5mxfp8mmrs") == 6
    # an operator that fails is reported and sets the exit status (a kernel name the driver does not know)
    r = subprocess.run([sys.executable, "-c", "import catccos_amd.run_examples as m, sys; m.OPERATORS[:] = [('ascend950_mx_quant_allgather', 'nosuch', [])]; "
                        "sys.argv = ['x']; sys.exit(m.main())"], capture_output=True, text=True, timeout=120, cwd=ROOT)
    assert r.returncode == 1 and "FAILED" in r.stdout and "failed: ascend950_mx_quant_allgather" in r.stdout, r.stdout
