#!/usr/bin/env python3
"""Headline benchmark: MXFP8 grouped GEMM (the MoE expert matmul of the
ascend950_fp8_mx_alltoallv_grouped_matmul operator, one rank's share) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the grouped GEMM over one batch of synthetic input that is already
resident in HBM: 16384 received tokens, 32 local experts with Zipf(1.1)-skewed group sizes
(at least one empty), K = 7168, N = 4096, E4M3 payload with one E8M0 scale per 32 elements,
fp32 accumulation, bf16 output.  Input quantisation is data preparation and is not timed.

Prints ONE JSON line.  `value` is TFLOP/s of the whole job; `roofline` prices the GEMM kernel
against the dense FP8 MFMA peak from HIP-event timing of the launches themselves;
`cpu_baseline` is the CPU oracle (test infrastructure, used here only as the timed baseline)
on a bounded sample of output rows of the same workload; `extra` carries the MX-quantiser
line (HBM-bound) and the other configurations measured with the same library.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP8_PEAK_TFLOPS = 5000.0   # MI355X dense FP8 / INT8 MFMA, published
FP4_PEAK_TFLOPS = 10100.0  # MI355X dense FP4 MFMA, published
HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published
# Bytes per launch of the headline kernel between the L2s and the fabric (Infinity Cache and HBM behind it), from two
# rocprofv3 --pmc runs of this script (FETCH_SIZE 1 128 767 KiB x 2.000, WRITE_SIZE 131 072 KiB x 1.000; the factors are
# what the same counters read for a 512 MiB device copy, `--only copy`).  Algorithmic bytes: 1 224 212 480.
GMM_TRAFFIC_BYTES = 2445932544


def zipf_groups(rng, t, e):
    """multinomial(t, p_e ~ (e+1)^-1.1) over permuted expert ids, with at least one empty group."""
    import numpy as np
    p = (np.arange(e) + 1.0) ** -1.1
    p = p[rng.permutation(e)]
    gs = rng.multinomial(t, p / p.sum()).astype(np.int32)
    if gs.min() > 0:
        i, j = int(gs.argmin()), int(gs.argmax())
        gs[j] += gs[i]
        gs[i] = 0
    return gs


def sample_rows(rng, group_sizes, want):
    """Output rows for a CPU check: the first and the last row of every non-empty group and the first row
    of its last 256-row tile (so every expert and every ragged last tile is hit), then random rows up to
    `want`; all rows if `want` covers them."""
    import numpy as np
    used = int(np.sum(group_sizes))
    if want >= used:
        return np.arange(used, dtype=np.int64)
    must, r0 = [], 0
    for g in group_sizes:
        g = int(g)
        if g > 0:
            must += [r0, r0 + g - 1, r0 + ((g - 1) // 256) * 256]
        r0 += g
    must = np.unique(np.array(must, dtype=np.int64))
    rest = np.setdiff1d(np.arange(used, dtype=np.int64), must)
    more = rng.choice(rest, max(0, min(rest.size, want - must.size)), replace=False)
    return np.sort(np.concatenate([must, more]))


def cpu_leg(run_rows, all_rows_flop, nrows_all, pick_rows, budget_s, unit):
    """Times run_rows(rows) -> golden rows (the CPU oracle's cache-blocked routine) on as many output rows
    as `budget_s` seconds allow, judged from a probe of 256 rows; returns (rows, golden, record)."""
    import oracle as orc
    rows = pick_rows(min(256, nrows_all))
    for _ in range(3):
        t0 = time.perf_counter()
        gold = run_rows(rows)
        dt = time.perf_counter() - t0
        # a small sample amortises the weight decode badly: more rows only get cheaper per row
        want = int(min(nrows_all, rows.size * budget_s / max(dt, 1e-3)))
        if rows.size == nrows_all or want < rows.size * 2:
            break
        rows = pick_rows(want)
    rec = {"value": round(all_rows_flop * rows.size / nrows_all / dt / 1e12, 4), "unit": unit, "cores": orc.num_threads(), "kind": "port",
           "sample": "%d of %d output rows (all columns, full K) of the same workload, %.1f s, cache-blocked CPU routine" % (rows.size, nrows_all, dt)}
    return rows, gold, rec


def parity_record(got, gold):
    import oracle as orc
    m = orc.compare(got, gold)
    return {"max_rel_err_floor1": m["max_rel_floor1"], "max_rel_err_floor_rms": m["max_rel_floor_rms"], "rows_checked": int(gold.shape[0]),
            "within_1e-2": bool(m["max_rel_floor1"] <= 1e-2 and m["max_rel_floor_rms"] <= 1e-2)}


LAST_WARM = {"launches": 0, "ms": 0.0}   # what the last event_time_ms() call ran untimed


def event_time_ms(fn, steps, warmup, warm_ms=0.0):
    """Wall time per step, average launch duration over the timed region and per-launch durations of fn()
    on the current stream, the latter two by HIP events.

    The shader clock needs some tens of milliseconds of load to reach its steady state (launch
    durations fall by 15-20 % over the first 50 ms after an idle period), so the untimed part must
    be long enough: `warmup` launches, then more until `warm_ms` of wall time have passed.
    """
    import torch
    t0 = time.perf_counter()
    launches = 0
    for _ in range(warmup):
        fn()
    launches += warmup
    torch.cuda.synchronize()
    while (time.perf_counter() - t0) * 1e3 < warm_ms:
        for _ in range(10):
            fn()
        launches += 10
        torch.cuda.synchronize()
    LAST_WARM["launches"], LAST_WARM["ms"] = launches, (time.perf_counter() - t0) * 1e3
    # the timed region: exactly `steps` launches queued back to back between one pair of events
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    region = e0.elapsed_time(e1) / steps
    # the same launches again, each between its own events: the spread (an event pair adds about 1 %)
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    for i in range(steps):
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    per = [s.elapsed_time(e) for s, e in zip(starts, ends)]
    return wall, region, per


def measurement_build_clocks(ksteps, group_sizes=None):
    """With a measurement build of the library (`--lib`, built with -DCCH_PROF): what the tiled GEMM kernel's last launch
    noted down - per wave the shader clocks spent in each wait and barrier of the K loops, per workgroup the clocks from
    kernel entry to the first K-step, and per tile its rows, its group and the clocks of its K loop and its epilogue,
    summarised by rows (in classes of 64) and, for whole tiles, by the rows of their group and by their place in the
    workgroup's sequence.  {} with the shipped library, which has none of this."""
    import collections
    import ctypes
    import numpy as np
    from catccos_amd import _abi
    lib = _abi.lib()
    try:
        rd, rdt, rde = lib.cch_prof_read, lib.cch_prof_read_tiles, lib.cch_prof_read_entry
    except AttributeError:
        return {}
    for f in (rd, rdt, rde):
        f.argtypes = [ctypes.c_void_p]
    pt = 12   # PROF_TILES of the kernel
    wbuf, tbuf, ebuf = (ctypes.c_uint64 * (256 * 64))(), (ctypes.c_uint64 * (256 * 2 * pt * 6))(), (ctypes.c_uint64 * (256 * 8))()
    if rd(wbuf) != 0 or rdt(tbuf) != 0 or rde(ebuf) != 0:
        return {}
    out = {}
    wd = np.frombuffer(wbuf, dtype=np.uint64).reshape(256, 8, 8).astype(np.float64)
    names = ["total", "lgkm_wait_L0", "barrier_after_L0", "vm_wait_a", "barrier_after_C0", "vm_wait_b", "barrier_after_L1", "barrier_after_C1"]
    out["shader_cycles_per_wave"] = {g: {n: int(v) for n, v in zip(names, wd[:, sl, :].mean(axis=(0, 1)))}
                                     for g, sl in (("waves_0_3", slice(0, 4)), ("waves_4_7", slice(4, 8)))}
    en = np.frombuffer(ebuf, dtype=np.uint64).reshape(256, 8).astype(np.int64)
    en = en[en[:, 5] > 0]
    st = (en[:, 1:6] - en[:, 0:5]).mean(axis=0)
    out["kernel_entry_cycles"] = dict(zip(["group_table", "per_lane_set_up", "first_decode", "first_requests_issued", "wait_and_barrier"],
                                          (int(v) for v in st)), total=int((en[:, 5] - en[:, 0]).mean()))
    d = np.frombuffer(tbuf, dtype=np.uint64).reshape(256, 2, pt, 6)
    recs = []
    for w in range(256):
        for i in range(pt):
            v, k0, k1, e1, dec, ent = (int(x) for x in d[w, 0, i])
            if k1 == 0 or (i > 0 and k0 <= int(d[w, 0, i - 1][1])):
                break
            recs.append({"wg": w, "idx": i, "rows": (v >> 32) & 0xFFFF, "group": v >> 48, "kloop": k1 - k0, "epi": e1 - k1, "dec": dec, "span": e1 - ent})
    out["tiles_noted"] = len(recs)
    by_wg = collections.defaultdict(list)
    for r in recs:
        by_wg[r["wg"]].append(r)
    out["decode_of_next_tile_cycles_per_tile"] = int(np.mean([max(r["dec"] for r in rs) / len(rs) for rs in by_wg.values()]))
    span = np.array([max(r["span"] for r in rs) for rs in by_wg.values()])
    out["entry_to_last_epilogue_cycles_per_workgroup"] = {"mean": int(span.mean()), "min": int(span.min()), "max": int(span.max())}
    by_rows = collections.defaultdict(list)
    for r in recs:
        by_rows[(r["rows"] + 63) // 64].append(r)
    out["k_loop_cycles_by_rows_div_64"] = {
        str(c): {"tiles": len(rs), "mean": int(np.mean([r["kloop"] for r in rs])), "min": int(min(r["kloop"] for r in rs)), "max": int(max(r["kloop"] for r in rs)),
                 "per_step": int(np.mean([r["kloop"] for r in rs]) / ksteps), "epilogue_mean": int(np.mean([r["epi"] for r in rs]))}
        for c, rs in sorted(by_rows.items())}
    whole = [r for r in recs if r["rows"] == 256]
    if group_sizes is not None and len(group_sizes) > 1:
        out["whole_tiles_by_rows_of_their_group"] = [
            {"group_rows": int(group_sizes[g]), "tiles": len(ks), "k_loop_mean": int(np.mean(ks))}
            for g in np.argsort(group_sizes) for ks in [[r["kloop"] for r in whole if r["group"] == g]] if ks]
    out["whole_tiles_by_place_in_the_workgroups_sequence"] = [
        {"place": i, "tiles": len(ks), "k_loop_mean": int(np.mean(ks))} for i in range(pt) for ks in [[r["kloop"] for r in whole if r["idx"] == i]] if ks]
    return out


def clock_under_load(fn, seconds=1.5):
    """Shader clock and power as rocm-smi reports them while fn() runs back to back: the figure that prices
    the published peak (quoted at the 2.4 GHz boost clock) for this kernel.  Returns {} where rocm-smi is
    missing or prints something else."""
    import re
    import subprocess
    import torch
    out = {}
    t0 = time.perf_counter()
    texts = []
    try:
        while time.perf_counter() - t0 < seconds:
            for _ in range(200):
                fn()
            if time.perf_counter() - t0 > 0.6 and len(texts) < 2:
                texts.append(subprocess.run(["rocm-smi", "--showclocks", "--showpower"], capture_output=True, text=True, timeout=20).stdout)
        torch.cuda.synchronize()
        sclk = [int(m) for t in texts for m in re.findall(r"sclk clock level: \d+: \((\d+)Mhz\)", t)]
        power = [float(m) for t in texts for m in re.findall(r"Power \(W\): ([0-9.]+)", t)]
        if sclk:
            out["sclk_mhz_under_load"] = sclk
        if power:
            out["power_w_under_load"] = power
    except Exception as exc:   # a reporting aid only
        torch.cuda.synchronize()
        out["error"] = repr(exc)[:120]
    return out


def queue_time_ms(fn, launches, warm_ms):
    """Average duration of fn() over a queue of back-to-back launches between one pair of events
    (gaps between kernels included), after at least warm_ms of the same load."""
    import torch
    t0 = time.perf_counter()
    while True:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        if (time.perf_counter() - t0) * 1e3 >= warm_ms:
            break
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(launches):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / launches


def quant_inputs(dev, m, k, nsets):
    """Config-1 inputs: N(0,1) with 0.1 % of the elements multiplied by 100, as bf16."""
    import torch
    out = []
    for _ in range(nsets):
        x = torch.randn(m, k, device=dev)
        x = torch.where(torch.rand(m, k, device=dev) < 0.001, x * 100.0, x)
        out.append(x.to(torch.bfloat16))
    return out


def quant_batch_time_us(sets, launches, warmup, entry="cch_mx_quant_rows"):
    """Average duration of the config-1 MX quantiser over a queue of back-to-back launches.

    One launch lasts about 16 us, the same order as the cost of a pair of events or of two tensor
    allocations, so the launches are queued through the C ABI into preallocated outputs and timed
    as one region: the figure includes the gaps between consecutive kernels, as a caller's would.
    """
    import torch
    from catccos_amd import _abi
    lib = _abi.lib()
    m, k = sets[0].shape
    payload = torch.empty((m, k), dtype=torch.uint8, device=sets[0].device)
    scales = torch.empty((m, k // 32), dtype=torch.uint8, device=sets[0].device)
    stream = torch.cuda.current_stream().cuda_stream

    def launch(i):
        _abi.check(getattr(lib, entry)(sets[i % len(sets)].data_ptr(), payload.data_ptr(), scales.data_ptr(), m, k, 0, 0, stream))

    for i in range(warmup):
        launch(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(launches):
        launch(i)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / launches


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=100, help="untimed launches (about 55 ms: the clock's ramp from idle)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true")
    ap.add_argument("--no-clock", action="store_true", help="skip the 1.5 s of back-to-back launches under which rocm-smi is asked for the clock")
    ap.add_argument("--set-option", action="append", default=[], metavar="NAME=VALUE",
                    help="library switch for an A/B run, e.g. gemm_tile_order=0 (cch_set_option)")
    ap.add_argument("--groups", metavar="E:ROWS", help="the headline kernel on E equal groups of ROWS rows each (E * ROWS tokens) instead of the "
                    "Zipf-sized groups: how the time follows the tiles and the weight bytes per tile (profiles/)")
    ap.add_argument("--lib", metavar="PATH", help="another build of libcatccos_hip.so (a measurement build, see catccos_amd/build.py)")
    ap.add_argument("--only", choices=["copy", "quant", "cfg2", "cfg3", "cfg4", "cfg5"], help="profiling aid: run only a 512 MiB device copy "
                    "(counter calibration), only the config-1 MX quantiser, or only one of the other configurations' GEMMs; "
                    "print a short JSON line and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU's share of the grouped GEMM; this build has no multi-GPU path "
                 "(the reference's communication stages are out of scope). Run with --gpus 1.")

    import numpy as np
    import torch
    if args.lib:
        from catccos_amd import _abi as abi0
        abi0.LIB_PATH = os.path.abspath(args.lib)
    import catccos_amd as cc
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (MI355X); none is visible")
    dev = "cuda"
    torch.manual_seed(5)
    rng = np.random.default_rng(5)
    rng_s = np.random.default_rng(55)   # row samples of the CPU legs (kept apart: the inputs do not depend on whether those run)

    if args.only == "copy":
        src = torch.empty(512 << 20, dtype=torch.uint8, device=dev).fill_(7)
        dst = torch.empty_like(src)
        _, _, ms = event_time_ms(lambda: dst.copy_(src), args.steps, args.warmup)
        print(json.dumps({"only": "copy", "bytes_read": src.numel(), "bytes_written": src.numel(), "ms": float(np.mean(ms))}))
        return
    if args.only == "quant":
        sets = quant_inputs(dev, 4096, 7168, 6)
        us = quant_batch_time_us(sets, args.steps, args.warmup)
        qb = 4096 * 7168 * 3 + 4096 * 224
        print(json.dumps({"only": "quant", "bytes": qb, "us": us, "gb_per_s": qb / (us * 1e-6) / 1e9}))
        return

    # ------------------------------------------------------------ workload (config 5 shapes, E4M3 payload)
    E, T, K, N = 32, 16384, 7168, 4096
    TRANS_B = 0   # W stored [E, K, N] as the configurations name it (B scales [E, K/64, N, 2])
    cc.set_option("require_tiled_gemm", 1)   # a fall-back to the generic kernels is an error here, not a slow number
    for kv in args.set_option:
        name, _, val = kv.partition("=")
        cc.set_option(name, int(val))
    gs_host = zipf_groups(rng, T, E)
    if args.groups:
        E, rows_each = (int(v) for v in args.groups.split(":"))
        T = E * rows_each
        gs_host = np.full(E, rows_each, dtype=np.int32)
    gs = torch.from_numpy(gs_host).to(dev)
    only_cfg = args.only if args.only in ("cfg2", "cfg3", "cfg4", "cfg5") else None
    flop = 2.0 * T * N * K
    cpu = not args.no_cpu_baseline and only_cfg is None
    result = {"only": only_cfg}
    if only_cfg is None:
        x0 = (torch.randn(T, K, device=dev) * 0.02).to(torch.bfloat16)
        a, sa = cc.mx_quant(x0, "e4m3")
        b = torch.empty((E, K, N), dtype=torch.uint8, device=dev)
        sb = torch.empty((E, K // 64, N, 2), dtype=torch.uint8, device=dev)
        for e in range(E):
            w0 = (torch.randn(K, N, device=dev) * 0.02).to(torch.bfloat16)
            b[e], sb[e] = cc.mx_quant_b(w0, "e4m3", trans_b=TRANS_B)
        del x0, w0
        torch.cuda.synchronize()

        out = [None]

        def step():
            out[0] = cc.mx_grouped_matmul(a, sa, b, sb, gs, "e4m3", TRANS_B)

        # `warmup` launches as asked for, then more of the same until the shader clock has settled (see event_time_ms)
        wall_ms, kernel_ms, per_ms = event_time_ms(step, args.steps, args.warmup, warm_ms=100.0)
        warm_run = dict(LAST_WARM)
        flop = 2.0 * T * N * K
        value = flop / (wall_ms * 1e-3) / 1e12
        achieved = flop / (kernel_ms * 1e-3) / 1e12

        clk = clock_under_load(step) if not args.no_clock else {}
        # an instrumented build of the library (--lib, built with -DCCH_PROF) notes clocks per wave, workgroup and tile
        step()
        torch.cuda.synchronize()
        clk.update(measurement_build_clocks((K + 127) // 128, gs_host))
        # size-independent sanity of the timed result: sampled rows against the oracle happen in the CPU leg below
        result = {
            "metric": "MXFP8 GMM TFLOP/s (% MFMA peak); MX-quant HBM GB/s (% of peak)",
            "value": round(value, 2),
            "unit": "TFLOP/s",
            "n_gpus": 1,
            "steps": args.steps,
            "warmup": args.warmup,
            # the untimed part is the `warmup` launches asked for plus more of the same until 100 ms have passed (the shader
            # clock settles after about 50 ms of load): what actually ran before the timed region
            "warmup_launches_run": warm_run["launches"],
            "warm_ms": round(warm_run["ms"], 1),
            "ms_per_step": round(wall_ms, 4),
            "higher_is_better": True,
            "scaling": "weak",
            "vs_baseline": None,
            "dtype": "mxfp8 (e4m3 x e4m3, e8m0 scales, f32 accumulate, bf16 out)",
            "data": "synthetic",
            "config": {"workload": "MXFP8 grouped matmul, config-5 shapes with E4M3 payload" + (" but equal groups (--groups)" if args.groups else ""), "experts": E, "tokens": T, "k": K,
                       "n": N, "trans_b": TRANS_B, "group_sizes": gs_host.tolist()},
            "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(achieved / FP8_PEAK_TFLOPS, 4), "traffic": GMM_TRAFFIC_BYTES,
                         # (a constant of this script, from the counter runs summarised in that file: not measured by this run)
                         "traffic_source": "profiles/gemm_tile_mxfp8_grouped_cfg5_e4m3.md",
                         "kernel": "gemm_tile_kernel<KIND_F8, EPI_PLAIN, E4M3, TB=0, UA=0>", "algorithmic_flop_per_launch": flop,
                         "kernel_ms_min": round(float(np.min(per_ms)), 4), "kernel_ms_median": round(float(np.median(per_ms)), 4),
                         "kernel_ms_mean": round(kernel_ms, 4), "kernel_ms_mean_single_launches": round(float(np.mean(per_ms)), 4), **clk},
        }

        # ------------------------------------------------------------ CPU baseline on a bounded sample of rows
        if cpu:
            import oracle as orc
            a_h, sa_h = a.cpu().numpy(), sa.cpu().numpy()
            b_h, sb_h = b.cpu().numpy(), sb.cpu().numpy()
            out_h = out[0].float().cpu().numpy()
            used = int(gs_host.sum())
            rows, gold, rec = cpu_leg(lambda r: orc.mx_gmm(a_h, sa_h, b_h, sb_h, N, K, orc.E4M3, TRANS_B, group_sizes=gs_host, rows=r, blocked=True),
                                      2.0 * used * N * K, used, lambda n: sample_rows(rng_s, gs_host, n), 20.0, "TFLOP/s")
            rec["parity_on_sample"] = parity_record(out_h[rows], gold)
            rec["parity_on_sample"]["rows_past_the_groups_are_zero"] = bool(np.all(out_h[used:] == 0))
            result["cpu_baseline"] = rec
            del a_h, sa_h, b_h, sb_h, out_h, gold

        # ------------------------------------------------------------ the other configurations, same library
    if not args.no_extra or only_cfg:
        extra = {}
        if only_cfg is None:
            # config 1: MX quantiser, rotating buffer sets larger than the 256 MB Infinity Cache
            M1, K1 = 4096, 7168
            sets = quant_inputs(dev, M1, K1, 6)
            q_us = quant_batch_time_us(sets, 120, 1500)
            qbytes = M1 * K1 * 2 + M1 * K1 + M1 * K1 // 32
            q_gbs = qbytes / (q_us * 1e-6) / 1e9
            extra["mx_quant_cfg1"] = {"gb_per_s": round(q_gbs, 1), "frac_of_hbm_peak": round(q_gbs / HBM_PEAK_GBS, 4),
                                      "us": round(q_us, 2), "bytes": qbytes, "buffers": "6 rotating input sets (352 MB), 120 queued launches"}
            # the same kernel on one input set that stays in the Infinity Cache: the rate a caller sees whose tensor was just written
            hot_us = quant_batch_time_us(sets[:1], 120, 1500)
            extra["mx_quant_cfg1"]["hot_cache"] = {"gb_per_s": round(qbytes / (hot_us * 1e-6) / 1e9, 1), "us": round(hot_us, 2),
                                                   "buffers": "one input set (59 MB) read again and again"}
            if cpu:
                # whole-tensor check and CPU rate of the same tensor
                x_h = sets[0].view(torch.int16).cpu().numpy().view(np.uint16)
                t0 = time.perf_counter()
                pq_h, sq_h = orc.mx_quant_rows(x_h, orc.E4M3)
                dt = time.perf_counter() - t0
                pq_d, sq_d = cc.mx_quant(sets[0], "e4m3")
                extra["mx_quant_cfg1"]["cpu_baseline"] = {"value": round(qbytes / dt / 1e9, 2), "unit": "GB/s", "cores": orc.num_threads(), "kind": "port",
                                                          "sample": "the whole [4096, 7168] tensor, %.2f s" % dt}
                extra["mx_quant_cfg1"]["parity"] = {"bit_exact_whole_tensor": bool(np.array_equal(pq_d.cpu().numpy(), pq_h) and
                                                                                   np.array_equal(sq_d.cpu().numpy(), sq_h)),
                                                    "payload_bytes": int(pq_h.size), "scale_bytes": int(sq_h.size)}
            # the half-input twin of the quantiser on the same values
            sets16 = [x.to(torch.float16) for x in sets]
            h_us = quant_batch_time_us(sets16, 120, 1500, "cch_mx_quant_rows_f16")
            extra["mx_quant_f16_input_cfg1_shape"] = {"gb_per_s": round(qbytes / (h_us * 1e-6) / 1e9, 1),
                                                      "frac_of_hbm_peak": round(qbytes / (h_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                                                      "us": round(h_us, 2), "bytes": qbytes}
            if cpu:
                t0 = time.perf_counter()
                ph_h, sh_h = orc.mx_quant_rows_f16(sets16[0].view(torch.int16).cpu().numpy().view(np.uint16), orc.E4M3)
                dt = time.perf_counter() - t0
                ph_d, sh_d = cc.mx_quant(sets16[0], "e4m3")
                extra["mx_quant_f16_input_cfg1_shape"]["cpu_baseline"] = {"value": round(qbytes / dt / 1e9, 2), "unit": "GB/s", "cores": orc.num_threads(),
                                                                          "kind": "port", "sample": "the whole [4096, 7168] tensor, %.2f s" % dt}
                extra["mx_quant_f16_input_cfg1_shape"]["parity"] = {"bit_exact_whole_tensor": bool(np.array_equal(ph_d.cpu().numpy(), ph_h) and
                                                                                                 np.array_equal(sh_d.cpu().numpy(), sh_h))}
            del sets16
            # the same rows quantised once and scattered as packed [payload | scales] rows to their top-2 destinations
            idx1 = torch.randperm(M1 * 2, device=dev).to(torch.int32)
            packed1 = torch.empty((M1 * 2, cc.packed_row_bytes(K1)), dtype=torch.uint8, device=dev)
            st1 = torch.cuda.current_stream().cuda_stream
            from catccos_amd import _abi as abi1

            def sc_launch(i):
                abi1.check(abi1.lib().cch_mx_quant_scatter_packed(sets[i % len(sets)].data_ptr(), idx1.data_ptr(), packed1.data_ptr(),
                                                                  M1, K1, 2, 0, 0, st1))

            for i in range(600):
                sc_launch(i)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(120):
                sc_launch(i)
            e1.record()
            torch.cuda.synchronize()
            sc_us = e0.elapsed_time(e1) * 1e3 / 120
            sc_bytes = M1 * K1 * 2 + 2 * M1 * cc.packed_row_bytes(K1)
            extra["mx_quant_scatter_top2_cfg1_rows"] = {"gb_per_s": round(sc_bytes / sc_us / 1e3, 1),
                                                        "frac_of_hbm_peak": round(sc_bytes / sc_us / 1e3 / HBM_PEAK_GBS, 4),
                                                        "us": round(sc_us, 2), "bytes": sc_bytes}
            if cpu:
                sc_launch(0)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                pk_h = orc.mx_quant_scatter_packed(x_h, idx1.cpu().numpy(), M1 * 2, 2, orc.E4M3)
                dt = time.perf_counter() - t0
                extra["mx_quant_scatter_top2_cfg1_rows"]["cpu_baseline"] = {"value": round(sc_bytes / dt / 1e9, 2), "unit": "GB/s", "cores": orc.num_threads(),
                                                                            "kind": "port", "sample": "all 4096 tokens, top-2, %.2f s" % dt}
                extra["mx_quant_scatter_top2_cfg1_rows"]["parity"] = {"bit_exact_whole_tensor": bool(np.array_equal(packed1.cpu().numpy(), pk_h))}
            del sets, packed1
        if only_cfg in (None, "cfg2"):
            # config 2: int8 W8A8 + dequant
            m2, k2, n2 = 8192, 4096, 8192
            a2 = torch.randint(-127, 128, (m2, k2), dtype=torch.int8, device=dev)
            b2 = torch.randint(-127, 128, (k2, n2), dtype=torch.int8, device=dev)
            pt2 = torch.rand(m2, device=dev) * 0.019 + 0.001
            pc2 = torch.rand(n2, device=dev) * 0.019 + 0.001
            t2 = [queue_time_ms(lambda: cc.w8a8_matmul_dequant(a2, b2, pt2, pc2, TRANS_B), 30, 60.0)]
            extra["w8a8_dequant_cfg2"] = {"tops": round(2.0 * m2 * n2 * k2 / (np.mean(t2) * 1e-3) / 1e12, 1), "us": round(float(np.mean(t2)) * 1e3, 1)}
            extra["w8a8_dequant_cfg2"]["frac_of_int8_peak"] = round(extra["w8a8_dequant_cfg2"]["tops"] / FP8_PEAK_TFLOPS, 4)
            extra["w8a8_dequant_cfg2"].update(measurement_build_clocks(k2 // 128))
            if cpu:
                o2 = cc.w8a8_matmul_dequant(a2, b2, pt2, pc2, TRANS_B).float().cpu().numpy()
                a2h, b2h, pt2h, pc2h = a2.cpu().numpy(), b2.cpu().numpy(), pt2.cpu().numpy(), pc2.cpu().numpy()
                rows, gold, rec = cpu_leg(lambda r: orc.gemm_i8_dequant(a2h, b2h, pt2h, pc2h, TRANS_B, rows=r, blocked=True), 2.0 * m2 * n2 * k2, m2,
                                          lambda n: np.sort(rng_s.choice(m2, n, replace=False)).astype(np.int64), 6.0, "TOP/s")
                extra["w8a8_dequant_cfg2"]["cpu_baseline"] = rec
                extra["w8a8_dequant_cfg2"]["parity"] = parity_record(o2[rows], gold)
                del o2, a2h, b2h, gold
            del a2, b2
        if only_cfg in (None, "cfg3"):
            # config 3: MXFP8 dense
            m3, k3, n3 = 4096, 2048, 7168
            a3, sa3 = cc.mx_quant(torch.randn(m3, k3, device=dev).to(torch.bfloat16), "e4m3")
            b3, sb3 = cc.mx_quant_b(torch.randn(k3, n3, device=dev).to(torch.bfloat16), "e4m3", trans_b=TRANS_B)
            t3 = [queue_time_ms(lambda: cc.mx_matmul(a3, sa3, b3, sb3, "e4m3", TRANS_B), 30, 60.0)]
            extra["mxfp8_dense_cfg3"] = {"tflops": round(2.0 * m3 * n3 * k3 / (np.mean(t3) * 1e-3) / 1e12, 1), "us": round(float(np.mean(t3)) * 1e3, 1)}
            extra["mxfp8_dense_cfg3"]["frac_of_fp8_peak"] = round(extra["mxfp8_dense_cfg3"]["tflops"] / FP8_PEAK_TFLOPS, 4)
            extra["mxfp8_dense_cfg3"].update(measurement_build_clocks(k3 // 128))
            if cpu:
                o3 = cc.mx_matmul(a3, sa3, b3, sb3, "e4m3", TRANS_B).float().cpu().numpy()
                h3 = [t.cpu().numpy() for t in (a3, sa3, b3, sb3)]
                rows, gold, rec = cpu_leg(lambda r: orc.mx_gmm(h3[0], h3[1], h3[2], h3[3], n3, k3, orc.E4M3, TRANS_B, rows=r, blocked=True), 2.0 * m3 * n3 * k3, m3,
                                          lambda n: np.sort(rng_s.choice(m3, n, replace=False)).astype(np.int64), 6.0, "TFLOP/s")
                extra["mxfp8_dense_cfg3"]["cpu_baseline"] = rec
                extra["mxfp8_dense_cfg3"]["parity"] = parity_record(o3[rows], gold)
                del o3, h3, gold
        if only_cfg in (None, "cfg4"):
            # config 4: MoE W8A8 grouped + dequant + SwiGLU
            e4, t4, k4, n4 = 16, 8192, 7168, 4096
            gs4 = torch.from_numpy(zipf_groups(rng, t4, e4)).to(dev)
            x4 = torch.randint(-127, 128, (t4, k4), dtype=torch.int8, device=dev)
            w4 = torch.randint(-127, 128, (e4, k4, n4), dtype=torch.int8, device=dev)
            pt4 = torch.rand(t4, device=dev) * 0.019 + 0.001
            pc4 = torch.rand(e4, n4, device=dev) * 0.019 + 0.001
            tt4 = [queue_time_ms(lambda: cc.gmm_dequant_swiglu(x4, w4, gs4, pt4, pc4, TRANS_B), 30, 60.0)]
            extra["moe_w8a8_swiglu_cfg4"] = {"tops": round(2.0 * t4 * n4 * k4 / (np.mean(tt4) * 1e-3) / 1e12, 1), "us": round(float(np.mean(tt4)) * 1e3, 1)}
            extra["moe_w8a8_swiglu_cfg4"]["frac_of_int8_peak"] = round(extra["moe_w8a8_swiglu_cfg4"]["tops"] / FP8_PEAK_TFLOPS, 4)
            extra["moe_w8a8_swiglu_cfg4"].update(measurement_build_clocks(k4 // 128, gs4.cpu().numpy()))
            # the same with the activation leaving as MXFP8 from the epilogue, against the two-kernel chain it replaces
            tf4 = queue_time_ms(lambda: cc.gmm_dequant_swiglu_mx(x4, w4, gs4, pt4, pc4, TRANS_B, "e4m3"), 30, 60.0)
            tc4 = queue_time_ms(lambda: cc.mx_quant(cc.gmm_dequant_swiglu(x4, w4, gs4, pt4, pc4, TRANS_B), "e4m3"), 30, 60.0)
            pf4, sf4 = cc.gmm_dequant_swiglu_mx(x4, w4, gs4, pt4, pc4, TRANS_B, "e4m3")
            pq4, sq4 = cc.mx_quant(cc.gmm_dequant_swiglu(x4, w4, gs4, pt4, pc4, TRANS_B), "e4m3")
            extra["moe_w8a8_swiglu_mxfp8_out_cfg4"] = {"us": round(tf4 * 1e3, 1), "two_kernel_chain_us": round(tc4 * 1e3, 1),
                                                       "tops": round(2.0 * t4 * n4 * k4 / (tf4 * 1e-3) / 1e12, 1),
                                                       "parity": {"bit_exact_vs_quantised_bf16_output": bool(torch.equal(pf4, pq4) and torch.equal(sf4, sq4))}}
            del pf4, sf4, pq4, sq4
            if cpu:
                o4 = cc.gmm_dequant_swiglu(x4, w4, gs4, pt4, pc4, TRANS_B).float().cpu().numpy()
                h4 = [t.cpu().numpy() for t in (x4, w4, gs4, pt4, pc4)]
                used4 = int(h4[2].sum())
                rows, gold, rec = cpu_leg(lambda r: orc.gmm_i8_dequant_swiglu(h4[0], h4[1], h4[2], h4[3], h4[4], rows=r, blocked=True), 2.0 * used4 * n4 * k4,
                                          used4, lambda n: sample_rows(rng_s, h4[2], n), 8.0, "TOP/s")
                extra["moe_w8a8_swiglu_cfg4"]["cpu_baseline"] = rec
                extra["moe_w8a8_swiglu_cfg4"]["parity"] = parity_record(o4[rows], gold)
                extra["moe_w8a8_swiglu_cfg4"]["parity"]["rows_past_the_groups_are_zero"] = bool(np.all(o4[used4:] == 0))
                del o4, h4, gold
            del x4, w4
        if only_cfg is None:
            # input side of config 4: per-token dynamic int8 quantisation of the bf16 tokens (queued launches through the C ABI)
            from catccos_amd import _abi
            xs4 = [torch.randn(t4, k4, device=dev).to(torch.bfloat16) for _ in range(4)]
            q4 = torch.empty((t4, k4), dtype=torch.int8, device=dev)
            s4 = torch.empty((t4,), dtype=torch.float32, device=dev)
            st4 = torch.cuda.current_stream().cuda_stream

            def dq_launch(i):
                _abi.check(_abi.lib().cch_dyn_quant_i8_rows(xs4[i % 4].data_ptr(), None, q4.data_ptr(), s4.data_ptr(), t4, t4, k4, 1, 0, st4))

            for i in range(800):
                dq_launch(i)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(60):
                dq_launch(i)
            e1.record()
            torch.cuda.synchronize()
            dq_us = e0.elapsed_time(e1) * 1e3 / 60
            dq_bytes = t4 * k4 * 3 + t4 * 4
            extra["dyn_quant_i8_cfg4_tokens"] = {"gb_per_s": round(dq_bytes / dq_us / 1e3, 1), "frac_of_hbm_peak": round(dq_bytes / dq_us / 1e3 / HBM_PEAK_GBS, 4),
                                                 "us": round(dq_us, 2), "bytes": dq_bytes}
            if cpu:
                dq_launch(0)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                qh, sh = orc.dyn_quant_i8_rows(xs4[0].view(torch.int16).cpu().numpy().view(np.uint16))
                dt = time.perf_counter() - t0
                extra["dyn_quant_i8_cfg4_tokens"]["cpu_baseline"] = {"value": round(dq_bytes / dt / 1e9, 2), "unit": "GB/s", "cores": orc.num_threads(),
                                                                     "kind": "port", "sample": "all 8192 tokens, %.2f s" % dt}
                extra["dyn_quant_i8_cfg4_tokens"]["parity"] = {"bit_exact_whole_tensor": bool(np.array_equal(q4.cpu().numpy(), qh) and
                                                                                            np.array_equal(s4.cpu().numpy(), sh))}
            del xs4, q4
            # combine side: top-2 weighted un-permute of 8192 expert-output rows back to 4096 tokens
            tok_u, hid_u, topk_u = 4096, 7168, 2
            ys = [torch.randn(tok_u * topk_u, hid_u, device=dev).to(torch.bfloat16) for _ in range(3)]
            idx_u = torch.randperm(tok_u * topk_u, device=dev).to(torch.int32)
            pr_u = torch.rand(tok_u * topk_u, device=dev)
            out_u = torch.empty((tok_u, hid_u), dtype=torch.bfloat16, device=dev)

            def un_launch(i):
                _abi.check(_abi.lib().cch_moe_token_unpermute(ys[i % 3].data_ptr(), idx_u.data_ptr(), pr_u.data_ptr(), out_u.data_ptr(),
                                                              tok_u * topk_u, tok_u, hid_u, topk_u, st4))

            for i in range(600):
                un_launch(i)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(60):
                un_launch(i)
            e1.record()
            torch.cuda.synchronize()
            un_us = e0.elapsed_time(e1) * 1e3 / 60
            un_bytes = tok_u * topk_u * hid_u * 2 + tok_u * hid_u * 2 + tok_u * topk_u * 8
            extra["moe_token_unpermute_top2"] = {"gb_per_s": round(un_bytes / un_us / 1e3, 1), "frac_of_hbm_peak": round(un_bytes / un_us / 1e3 / HBM_PEAK_GBS, 4),
                                                 "us": round(un_us, 2), "bytes": un_bytes}
            if cpu:
                un_launch(0)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                uh = orc.moe_token_unpermute(ys[0].view(torch.int16).cpu().numpy().view(np.uint16), idx_u.cpu().numpy(), pr_u.cpu().numpy(), topk_u)
                dt = time.perf_counter() - t0
                extra["moe_token_unpermute_top2"]["cpu_baseline"] = {"value": round(un_bytes / dt / 1e9, 2), "unit": "GB/s", "cores": orc.num_threads(),
                                                                     "kind": "port", "sample": "all 4096 tokens, %.2f s" % dt}
                extra["moe_token_unpermute_top2"]["parity"] = {"bit_exact_whole_tensor": bool(np.array_equal(
                    out_u.view(torch.int16).cpu().numpy().view(np.uint16), uh))}
            del ys, out_u
            # routing sort of config 4's routes (8192 tokens, top-2, 16 experts): three short launches through the C ABI
            rt_rows, rt_e = 8192 * 2, 16
            rt_idx = torch.randint(0, rt_e, (rt_rows,), dtype=torch.int32, device=dev)
            rt_d2s = torch.empty(rt_rows, dtype=torch.int32, device=dev)
            rt_s2d = torch.empty_like(rt_d2s)
            rt_cnt = torch.empty(rt_e, dtype=torch.int32, device=dev)
            rt_wsb = int(_abi.lib().cch_moe_init_routing_workspace_bytes(rt_rows, rt_e))
            rt_ws = torch.empty(max(rt_wsb, 4), dtype=torch.uint8, device=dev)

            def rt_launch():
                _abi.check(_abi.lib().cch_moe_init_routing(rt_idx.data_ptr(), rt_rows, rt_e, rt_d2s.data_ptr(), rt_s2d.data_ptr(),
                                                           rt_cnt.data_ptr(), 0, rt_ws.data_ptr(), rt_wsb, st4))

            for _ in range(200):
                rt_launch()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(100):
                rt_launch()
            e1.record()
            torch.cuda.synchronize()
            extra["moe_init_routing_cfg4_routes"] = {"us": round(e0.elapsed_time(e1) * 1e3 / 100, 2), "routes": rt_rows, "experts": rt_e,
                                                     "launches_per_call": 3}
            if cpu:
                t0 = time.perf_counter()
                d2s_h, s2d_h, cnt_h = orc.moe_init_routing(rt_idx.cpu().numpy(), rt_e)
                dt = time.perf_counter() - t0
                extra["moe_init_routing_cfg4_routes"]["cpu_baseline"] = {"value": round(dt * 1e6, 1), "unit": "us", "cores": 1, "kind": "port",
                                                                         "sample": "all 16384 routes (numpy stable argsort and bincount)"}
                extra["moe_init_routing_cfg4_routes"]["parity"] = {"bit_exact_whole_tensor": bool(
                    np.array_equal(rt_d2s.cpu().numpy(), d2s_h) and np.array_equal(rt_s2d.cpu().numpy(), s2d_h) and np.array_equal(rt_cnt.cpu().numpy(), cnt_h))}
        if only_cfg in (None, "cfg5"):
            # config 5: MXFP4 grouped (same groups as the headline)
            a5, sa5 = cc.mx_quant((torch.randn(T, K, device=dev) * 0.02).to(torch.bfloat16), "e2m1")
            b5 = torch.empty((E, K, N // 2), dtype=torch.uint8, device=dev)
            sb5 = torch.empty((E, K // 64, N, 2), dtype=torch.uint8, device=dev)
            for e in range(E):
                b5[e], sb5[e] = cc.mx_quant_b((torch.randn(K, N, device=dev) * 0.02).to(torch.bfloat16), "e2m1", trans_b=TRANS_B)
            t5 = [queue_time_ms(lambda: cc.mx_grouped_matmul(a5, sa5, b5, sb5, gs, "e2m1", TRANS_B), 30, 60.0)]
            extra["mxfp4_grouped_cfg5"] = {"tflops": round(flop / (np.mean(t5) * 1e-3) / 1e12, 1), "us": round(float(np.mean(t5)) * 1e3, 1)}
            extra["mxfp4_grouped_cfg5"]["frac_of_fp4_peak"] = round(extra["mxfp4_grouped_cfg5"]["tflops"] / FP4_PEAK_TFLOPS, 4)
            extra["mxfp4_grouped_cfg5"].update(measurement_build_clocks(K // 256, gs_host))
            if cpu:
                o5 = cc.mx_grouped_matmul(a5, sa5, b5, sb5, gs, "e2m1", TRANS_B).float().cpu().numpy()
                h5 = [t.cpu().numpy() for t in (a5, sa5, b5, sb5)]
                used5 = int(gs_host.sum())
                rows, gold, rec = cpu_leg(lambda r: orc.mx_gmm(h5[0], h5[1], h5[2], h5[3], N, K, orc.E2M1, TRANS_B, group_sizes=gs_host, rows=r, blocked=True),
                                          2.0 * used5 * N * K, used5, lambda n: sample_rows(rng_s, gs_host, n), 10.0, "TFLOP/s")
                extra["mxfp4_grouped_cfg5"]["cpu_baseline"] = rec
                extra["mxfp4_grouped_cfg5"]["parity"] = parity_record(o5[rows], gold)
                del o5, h5, gold
            del a5, sa5, b5, sb5
        if only_cfg is None:
            # the headline's operands as the up projection of the MX FFN chain: SwiGLU on the bf16 tile in the epilogue, and the
            # same with the activation leaving as MXFP8 (what the down projection reads), against the kernel chain it replaces
            tu = queue_time_ms(lambda: cc.mx_grouped_matmul_swiglu(a, sa, b, sb, gs, "e4m3", TRANS_B), 30, 60.0)
            tq = queue_time_ms(lambda: cc.mx_grouped_matmul_swiglu(a, sa, b, sb, gs, "e4m3", TRANS_B, out_fmt="e4m3"), 30, 60.0)
            tch = queue_time_ms(lambda: cc.mx_quant(cc.mx_grouped_matmul_swiglu(a, sa, b, sb, gs, "e4m3", TRANS_B), "e4m3"), 30, 60.0)
            pu, su = cc.mx_grouped_matmul_swiglu(a, sa, b, sb, gs, "e4m3", TRANS_B, out_fmt="e4m3")
            pv, sv = cc.mx_quant(cc.mx_grouped_matmul_swiglu(a, sa, b, sb, gs, "e4m3", TRANS_B), "e4m3")
            extra["mxfp8_up_projection_swiglu_headline_shapes"] = {
                "bf16_out_us": round(tu * 1e3, 1), "mxfp8_out_us": round(tq * 1e3, 1), "two_kernel_chain_us": round(tch * 1e3, 1),
                "tflops_mxfp8_out": round(flop / (tq * 1e-3) / 1e12, 1),
                "parity": {"bit_exact_vs_quantised_bf16_output": bool(torch.equal(pu, pv) and torch.equal(su, sv))}}
            del pu, su, pv, sv
            # The MXFP8 FFN of one rank from routing to combine, at the largest shape of the reference example's own list
            # (examples/ascend950_dispatch_ffn_combine/scripts/test_shapes.csv: 512 tokens, K 7168, N 4096) with its run.sh's
            # 16 experts and top-6: seven launches (routing sort x3, quantise-and-scatter, GMM1 + SwiGLU + quantise, GMM2,
            # un-permute), eager and as one HIP graph.  Weight bytes per pass: 16 x (29.4 + 14.7) MB + scales = 0.73 GB.
            mf, ef, topf = 512, 16, 6
            xf = torch.randn(mf, K, device=dev).to(torch.bfloat16)
            idf = torch.argsort(torch.rand(mf, ef, device=dev), dim=1)[:, :topf].to(torch.int32).contiguous()
            prf = torch.softmax(torch.randn(mf, topf, device=dev), dim=-1)
            w1f = [cc.mx_quant_b((torch.randn(K, N, device=dev) / K ** 0.5).to(torch.bfloat16), "e4m3", trans_b=1) for _ in range(ef)]
            w2f = [cc.mx_quant_b((torch.randn(N // 2, K, device=dev) / (N // 2) ** 0.5).to(torch.bfloat16), "e4m3", trans_b=1) for _ in range(ef)]
            b1f, s1f, b2f, s2f = (torch.stack([w[i] for w in ws]) for ws in (w1f, w2f) for i in (0, 1))
            del w1f, w2f
            ffn = lambda: cc.moe_ffn_mxfp8(xf, idf, prf, b1f, s1f, b2f, s2f)   # noqa: E731
            t_eager = queue_time_ms(ffn, 30, 60.0)
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                out_g = ffn()
            t_graph = queue_time_ms(gr.replay, 30, 60.0)
            ffn_flop = 2.0 * mf * topf * (K * N + (N // 2) * K)
            wbytes = b1f.numel() + s1f.numel() + b2f.numel() + s2f.numel()
            ent = {"us_eager": round(t_eager * 1e3, 1), "us_graph": round(t_graph * 1e3, 1), "tflops_graph": round(ffn_flop / (t_graph * 1e-3) / 1e12, 1),
                   "weight_tb_s_graph": round(wbytes / (t_graph * 1e-3) / 1e12, 2),
                   "workload": "%d tokens, top-%d of %d experts, K %d, N %d, weights [E,N,K] / [E,K,N/2] as the reference's files" % (mf, topf, ef, K, N)}
            if cpu:
                gr.replay()
                torch.cuda.synchronize()
                got = out_g.float().cpu().numpy()
                xh = xf.view(torch.int16).cpu().numpy().view(np.uint16)
                b1h, s1h, b2h, s2h = (v.cpu().numpy() for v in (b1f, s1f, b2f, s2f))
                t0 = time.perf_counter()
                _, s2d_h, cnt_h = orc.moe_init_routing(idf.cpu().numpy(), ef)
                pk = orc.mx_quant_scatter_packed(xh, s2d_h, mf * topf, topf, orc.E4M3)
                _, c1 = orc.mx_gmm(pk[:, :K], pk[:, K:], b1h, s1h, N, K, orc.E4M3, 1, group_sizes=cnt_h, want_bf16=True, blocked=True)
                a2h, sa2h = orc.mx_quant_rows(orc.swiglu_bf16(c1), orc.E4M3)
                _, yh = orc.mx_gmm(a2h, sa2h, b2h, s2h, K, N // 2, orc.E4M3, 1, group_sizes=cnt_h, want_bf16=True, blocked=True)
                want = orc.bf16_to_f32(orc.moe_token_unpermute(yh, s2d_h, prf.cpu().numpy(), topf))
                dt = time.perf_counter() - t0
                ent["cpu_baseline"] = {"value": round(ffn_flop / dt / 1e12, 4), "unit": "TFLOP/s", "cores": orc.num_threads(), "kind": "port",
                                       "sample": "the whole chain on the same inputs, %.1f s, cache-blocked CPU GEMMs" % dt}
                rms = float(np.sqrt(np.mean(want ** 2)))
                # two implementations of this chain differ where a bf16 step of GMM1 moves a code of the quantised activation
                ent["parity"] = {"rms_err_over_rms": float(np.sqrt(np.mean((got - want) ** 2)) / rms), "max_err_over_rms": float(np.abs(got - want).max() / rms),
                                 "rows_checked": mf, "stagewise_bit_exact_checks": "tests/test_gpu_ffn_chain.py"}
            extra["mxfp8_ffn_chain_reference_shape"] = ent
            del b1f, s1f, b2f, s2f, gr, out_g
            # Yardstick, not part of this build: the vendor library's dense FP8 GEMM (per-tensor scales, E4M3,
            # bf16 out) on the headline's shape as one group, and this kernel on the same bytes with unit scales.
            try:
                ya = (torch.randn(T, K, device=dev) * 0.5).to(torch.float8_e4m3fn)
                yb = (torch.randn(N, K, device=dev) * 0.5).to(torch.float8_e4m3fn)
                one = torch.tensor(1.0, device=dev)
                t_lib = queue_time_ms(lambda: torch._scaled_mm(ya, yb.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16), 100, 150.0)
                ysa = torch.full((T, K // 32), 127, dtype=torch.uint8, device=dev)
                ysb = torch.full((N, K // 32), 127, dtype=torch.uint8, device=dev)
                t_own = queue_time_ms(lambda: cc.mx_matmul(ya.view(torch.uint8), ysa, yb.view(torch.uint8), ysb, "e4m3", 1), 100, 150.0)
                # The same two on constant operands (all ones): the matrix pipes then draw little and the clock stays up, so
                # this pair shows the cycles the kernels need, the pair above what the power limit leaves of them.
                ca = torch.ones(T, K, device=dev).to(torch.float8_e4m3fn)
                cb = torch.ones(N, K, device=dev).to(torch.float8_e4m3fn)
                t_lib1 = queue_time_ms(lambda: torch._scaled_mm(ca, cb.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16), 100, 150.0)
                t_own1 = queue_time_ms(lambda: cc.mx_matmul(ca.view(torch.uint8), ysa, cb.view(torch.uint8), ysb, "e4m3", 1), 100, 150.0)
                extra["yardstick_dense_fp8_16384x4096x7168"] = {
                    "library_scaled_mm_tflops": round(flop / (t_lib * 1e-3) / 1e12, 1), "this_kernel_same_data_tflops": round(flop / (t_own * 1e-3) / 1e12, 1),
                    "constant_operands": {"library_scaled_mm_tflops": round(flop / (t_lib1 * 1e-3) / 1e12, 1),
                                          "this_kernel_same_data_tflops": round(flop / (t_own1 * 1e-3) / 1e12, 1)},
                    "note": "library = torch._scaled_mm (per-tensor scales); both with B as [N,K]; random N(0,0.5) operands, then all ones"}
                del ca, cb
            except Exception as exc:   # the library call is optional: a box without it still reports everything else
                extra["yardstick_dense_fp8_16384x4096x7168"] = {"error": repr(exc)[:200]}
        result["extra"] = extra

    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
