"""CPU oracle (TEST INFRASTRUCTURE ONLY).

numpy-facing wrappers around ``oracle/liboracle.so`` (built from ``oracle.c`` by
``oracle/Makefile``).  Only the tests, the smoke check and the benchmark's
``cpu_baseline`` leg may import this package; the product never does.

Every function here is a thin marshalling layer: the arithmetic, and the
reference file:line each piece follows, live in ``oracle.c``.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

E4M3, E5M2, E2M1, E1M2 = 0, 1, 2, 3
FP4_FORMATS = (E2M1, E1M2)
RNE, LUT = 0, 1

_lib = None


def build(force=False):
    """Compile oracle.c with the Makefile next to it."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "liboracle.so"], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        c = ctypes
        L.orc_bf16_to_f32.restype = c.c_float
        L.orc_bf16_to_f32.argtypes = [c.c_uint16]
        L.orc_f32_to_bf16.restype = c.c_uint16
        L.orc_f32_to_bf16.argtypes = [c.c_float]
        for name in ("orc_e4m3_decode", "orc_e5m2_decode", "orc_e2m1_decode", "orc_e1m2_decode", "orc_e8m0_decode"):
            getattr(L, name).restype = c.c_float
            getattr(L, name).argtypes = [c.c_uint8]
        L.orc_encode.restype = c.c_uint8
        L.orc_encode.argtypes = [c.c_float, c.c_int, c.c_int]
        L.orc_decode.restype = c.c_float
        L.orc_decode.argtypes = [c.c_uint8, c.c_int]
        L.orc_round_through_f16.restype = c.c_float
        L.orc_round_through_f16.argtypes = [c.c_float]
        L.orc_trunc_through_f16.restype = c.c_float
        L.orc_trunc_through_f16.argtypes = [c.c_float]
        L.orc_shared_exp.restype = c.c_int
        L.orc_shared_exp.argtypes = [c.c_float, c.c_int, c.POINTER(c.c_int)]
        L.orc_sched_src_prev_sum.restype = c.c_int32
        L.orc_sched_src_prev_sum.argtypes = [c.c_void_p, c.c_int32, c.c_int32, c.c_int32, c.c_uint32]
        L.orc_sched_comm_loops.restype = c.c_uint32
        L.orc_sched_comm_loops.argtypes = [c.c_int32, c.c_uint32, c.c_uint32]
        L.orc_sched_block_offset_row.restype = c.c_uint32
        L.orc_sched_block_offset_row.argtypes = [c.c_uint32, c.c_uint32, c.c_uint32]
        L.orc_grouped_tile_order.restype = c.c_int64
        L.orc_num_threads.restype = c.c_int
        _lib = L
    return _lib


def _p(a):
    return None if a is None else ctypes.c_void_p(a.ctypes.data)


def _i64(v):
    return ctypes.c_int64(int(v))


def _rows(rows):
    if rows is None:
        return None, 0
    r = np.ascontiguousarray(rows, dtype=np.int64)
    return r, r.size


def num_threads():
    return int(lib().orc_num_threads())


# ------------------------------------------------------------------ formats

def f32_to_bf16(x):
    """fp32 array -> bf16 bit patterns (uint16), round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = ((u & 0x7F800000) == 0x7F800000) & ((u & 0x007FFFFF) != 0)
    r = ((u + (0x7FFF + ((u >> 16) & 1))) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_to_f32(h):
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def decode_table(fmt):
    n = 16 if fmt in FP4_FORMATS else 256
    return np.array([lib().orc_decode(i, fmt) for i in range(n)], dtype=np.float32)


def e8m0_table():
    return np.array([lib().orc_e8m0_decode(i) for i in range(256)], dtype=np.float32)


def encode(values, fmt, rounding=RNE):
    v = np.ascontiguousarray(values, dtype=np.float32).ravel()
    L = lib()
    return np.array([L.orc_encode(float(x), fmt, rounding) for x in v], dtype=np.uint8).reshape(np.shape(values))


def shared_exp(amax, emax):
    flag = ctypes.c_int(0)
    e = lib().orc_shared_exp(float(amax), emax, ctypes.byref(flag))
    return e, bool(flag.value)


# ------------------------------------------------------------- quantisation

def scale_cols(k):
    """Scale bytes per row for a K extent: even-padded block count."""
    return 2 * ((k + 63) // 64)


def mx_quant_rows(x_bf16, fmt=E4M3, rounding=RNE):
    """x_bf16 uint16 [M,K] -> (payload uint8 [M,K or ceil(K/2)], scales uint8 [M,scale_cols(K)])."""
    x = np.ascontiguousarray(x_bf16, dtype=np.uint16)
    m, k = x.shape
    pld = (k + 1) // 2 if fmt in FP4_FORMATS else k
    payload = np.empty((m, pld), dtype=np.uint8)
    scales = np.empty((m, scale_cols(k)), dtype=np.uint8)
    lib().orc_mx_quant_rows(_p(x), _i64(m), _i64(k), fmt, rounding, _p(payload), _p(scales))
    return payload, scales


def mx_quant_rows_f16(x_f16, fmt=E4M3, rounding=RNE):
    """IEEE half bits (uint16 [M,K], or a float16 array) -> (payload, scales) as mx_quant_rows."""
    x = np.asarray(x_f16)
    if x.dtype == np.float16:
        x = x.view(np.uint16)
    x = np.ascontiguousarray(x, dtype=np.uint16)
    m, k = x.shape
    pld = (k + 1) // 2 if fmt in FP4_FORMATS else k
    payload = np.empty((m, pld), dtype=np.uint8)
    scales = np.empty((m, scale_cols(k)), dtype=np.uint8)
    lib().orc_mx_quant_rows_f16(_p(x), _i64(m), _i64(k), fmt, rounding, _p(payload), _p(scales))
    return payload, scales


def packed_row_bytes(k, fmt=E4M3):
    """Bytes of one packed row: payload followed by the padded E8M0 scales."""
    return ((k + 1) // 2 if fmt in FP4_FORMATS else k) + scale_cols(k)


def mx_quant_scatter_packed(x_bf16, expanded_row_idx, out_rows, top_k, fmt=E4M3, rounding=RNE, fill=0):
    """Quantise each row of x once and write [payload | scales] to rows expanded_row_idx[t*top_k + r]
    of a uint8 [out_rows, packed_row_bytes] array (initialised to `fill`); negative entries are skipped."""
    x = np.ascontiguousarray(x_bf16, dtype=np.uint16)
    idx = np.ascontiguousarray(expanded_row_idx, dtype=np.int32).reshape(-1)
    tokens, k = x.shape
    assert idx.size == tokens * top_k
    out = np.full((out_rows, packed_row_bytes(k, fmt)), fill, dtype=np.uint8)
    rc = lib().orc_mx_quant_scatter_packed(_p(x), _p(idx), _i64(tokens), _i64(k), int(top_k), fmt, rounding, _p(out))
    assert rc == 0
    return out


def mx_quant_b(b_bf16, fmt=E4M3, rounding=RNE, trans_b=0):
    """b_bf16 uint16 [K,N] quantised along K; returns (payload, scales) in the boundary layouts."""
    b = np.ascontiguousarray(b_bf16, dtype=np.uint16)
    k, n = b.shape
    fp4 = fmt in FP4_FORMATS
    if trans_b:
        payload = np.empty((n, (k + 1) // 2 if fp4 else k), dtype=np.uint8)
        scales = np.empty((n, scale_cols(k)), dtype=np.uint8)
    else:
        payload = np.empty((k, (n + 1) // 2 if fp4 else n), dtype=np.uint8)
        scales = np.empty((scale_cols(k) // 2, n, 2), dtype=np.uint8)
    rc = lib().orc_mx_quant_b(_p(b), _i64(k), _i64(n), fmt, rounding, int(trans_b), _p(payload), _p(scales))
    assert rc == 0
    return payload, scales


def mx_dequant_rows(payload, scales, k, fmt=E4M3):
    payload = np.ascontiguousarray(payload, dtype=np.uint8)
    scales = np.ascontiguousarray(scales, dtype=np.uint8)
    m = payload.shape[0]
    out = np.empty((m, k), dtype=np.float32)
    lib().orc_mx_dequant_rows(_p(payload), _p(scales), _i64(m), _i64(k), fmt, _p(out))
    return out


# -------------------------------------------------------------------- GEMMs

DQ_DEVICE, DQ_GOLDEN = 0, 1


def dyn_quant_i8_rows(x_bf16, src=None, topk=1, mode=DQ_DEVICE, smooth=None, smooth_rows=None):
    """Per-token dynamic int8 quantisation: x uint16 [rows_in,K] -> (q int8 [T,K], scale float32 [T]).
    smooth float32 [S,K] (or [K]) multiplies every row first; smooth_rows int32 [T] picks its vector."""
    x = np.ascontiguousarray(x_bf16, dtype=np.uint16)
    rows_in, k = x.shape
    if src is not None:
        src = np.ascontiguousarray(src, dtype=np.int32)
        t = src.shape[0]
    else:
        t = rows_in
    ns = 0
    if smooth is not None:
        smooth = np.ascontiguousarray(smooth, dtype=np.float32).reshape(-1, k)
        ns = smooth.shape[0]
        if smooth_rows is not None:
            smooth_rows = np.ascontiguousarray(smooth_rows, dtype=np.int32)
            assert smooth_rows.shape == (t,)
    q = np.empty((t, k), dtype=np.int8)
    scale = np.empty(t, dtype=np.float32)
    lib().orc_dyn_quant_i8_rows(_p(x), _p(src) if src is not None else None, _i64(rows_in), _i64(t), _i64(k), int(topk),
                                int(mode), _p(smooth) if smooth is not None else None,
                                _p(smooth_rows) if smooth is not None and smooth_rows is not None else None, _i64(ns),
                                _p(q), _p(scale))
    return q, scale


def gemm_i8_dequant(a, b, per_tok, per_ch, trans_b=0, rows=None, want_bf16=False, blocked=False):
    """`blocked` picks the cache-blocked routine (the CPU baseline; same values), see oracle.c."""
    a = np.ascontiguousarray(a, dtype=np.int8)
    b = np.ascontiguousarray(b, dtype=np.int8)
    per_tok = np.ascontiguousarray(per_tok, dtype=np.float32)
    per_ch = np.ascontiguousarray(per_ch, dtype=np.float32)
    m, k = a.shape
    n = b.shape[0] if trans_b else b.shape[1]
    r, nr = _rows(rows)
    cnt = nr if rows is not None else m
    out = np.empty((cnt, n), dtype=np.float32)
    out16 = np.empty((cnt, n), dtype=np.uint16) if want_bf16 else None
    fn = lib().orc_gemm_i8_dequant_blocked if blocked else lib().orc_gemm_i8_dequant
    fn(_p(a), _p(b), _p(per_tok), _p(per_ch), _i64(m), _i64(n), _i64(k), int(trans_b), _p(r), _i64(nr), _p(out), _p(out16))
    return (out, out16) if want_bf16 else out


def gmm_i8_dequant_swiglu(x, w, group_sizes, per_tok, per_ch, fp16_step=False, rows=None, want_bf16=False, blocked=False):
    x = np.ascontiguousarray(x, dtype=np.int8)
    w = np.ascontiguousarray(w, dtype=np.int8)
    gs = np.ascontiguousarray(group_sizes, dtype=np.int32)
    per_tok = np.ascontiguousarray(per_tok, dtype=np.float32)
    per_ch = np.ascontiguousarray(per_ch, dtype=np.float32)
    t, k = x.shape
    e, k2, n = w.shape
    assert k2 == k and gs.size == e and per_ch.shape == (e, n)
    r, nr = _rows(rows)
    cnt = nr if rows is not None else t
    out = np.empty((cnt, n // 2), dtype=np.float32)
    out16 = np.empty((cnt, n // 2), dtype=np.uint16) if want_bf16 else None
    fn = lib().orc_gmm_i8_dequant_swiglu_blocked if blocked else lib().orc_gmm_i8_dequant_swiglu
    fn(_p(x), _p(w), _p(gs), _i64(e), _i64(t), _i64(k), _i64(n), _p(per_tok), _p(per_ch), int(fp16_step), _p(r), _i64(nr),
       _p(out), _p(out16))
    return (out, out16) if want_bf16 else out


def swiglu_bf16(c_bf16):
    """bf16 bits [T, N] (gate | up halves) -> bf16 bits [T, N/2] = silu(gate) * up, see oracle.c:orc_swiglu_bf16."""
    c = np.ascontiguousarray(c_bf16, dtype=np.uint16)
    t, n = c.shape
    assert n % 2 == 0
    out = np.empty((t, n // 2), dtype=np.uint16)
    lib().orc_swiglu_bf16(_p(c), _i64(t), _i64(n), _p(out))
    return out


def mx_gmm(a, sa, b, sb, n, k, fmt=E4M3, trans_b=0, group_sizes=None, rows=None, want_bf16=False, want_f64=False, blocked=False):
    """Dense (group_sizes None, b one expert) or grouped MX GEMM golden; see oracle.c:orc_mx_gmm.
    `blocked` picks the cache-blocked routine (the CPU baseline; same values, no fp64 copy)."""
    assert not (blocked and want_f64)
    a = np.ascontiguousarray(a, dtype=np.uint8)
    sa = np.ascontiguousarray(sa, dtype=np.uint8)
    b = np.ascontiguousarray(b, dtype=np.uint8)
    sb = np.ascontiguousarray(sb, dtype=np.uint8)
    t = a.shape[0]
    assert sa.shape == (t, scale_cols(k)), (sa.shape, t, scale_cols(k))
    if group_sizes is None:
        gs, e = None, 1
    else:
        gs = np.ascontiguousarray(group_sizes, dtype=np.int32)
        e = gs.size
    assert sb.size == e * scale_cols(k) * n, (sb.shape, e, k, n)
    r, nr = _rows(rows)
    cnt = nr if rows is not None else t
    out = np.empty((cnt, n), dtype=np.float32)
    out16 = np.empty((cnt, n), dtype=np.uint16) if want_bf16 else None
    out64 = np.empty((cnt, n), dtype=np.float64) if want_f64 else None
    if blocked:
        lib().orc_mx_gmm_blocked(_p(a), _p(sa), _p(b), _p(sb), _p(gs), _i64(e), _i64(t), _i64(n), _i64(k), fmt, int(trans_b),
                                 _p(r), _i64(nr), _p(out), _p(out16))
    else:
        lib().orc_mx_gmm(_p(a), _p(sa), _p(b), _p(sb), _p(gs), _i64(e), _i64(t), _i64(n), _i64(k), fmt, int(trans_b),
                         _p(r), _i64(nr), _p(out), _p(out16), _p(out64))
    res = [out]
    if want_bf16:
        res.append(out16)
    if want_f64:
        res.append(out64)
    return res[0] if len(res) == 1 else tuple(res)


# --------------------------------------------------------------- schedulers

def sched_src_prev_sum(token_per_expert, rank, ep, expert_per_rank, core_idx):
    t = np.ascontiguousarray(token_per_expert, dtype=np.int32)
    return int(lib().orc_sched_src_prev_sum(_p(t), rank, ep, expert_per_rank, core_idx))


def sched_comm_loops(ep, core_idx, core_num):
    return int(lib().orc_sched_comm_loops(ep, core_idx, core_num))


def sched_block_offset_row(core_idx, core_num, comm_idx):
    return int(lib().orc_sched_block_offset_row(core_idx, core_num, comm_idx))


def sched_cumsum_mm(token_per_expert, rank, ep, expert_per_rank):
    t = np.ascontiguousarray(token_per_expert, dtype=np.int32)
    out = np.zeros((ep, expert_per_rank), dtype=np.int32)
    lib().orc_sched_cumsum_mm(_p(t), rank, ep, expert_per_rank, _p(out))
    return out


def grouped_tile_order(group_sizes, n, bm, bn, nblocks):
    """Rows of {worker, group, row0, col0, rows, cols}, in global tile order."""
    gs = np.ascontiguousarray(group_sizes, dtype=np.int32)
    total = int(lib().orc_grouped_tile_order(_p(gs), _i64(gs.size), _i64(n), bm, bn, nblocks, _i64(0), None))
    rec = np.zeros((total, 6), dtype=np.int64)
    lib().orc_grouped_tile_order(_p(gs), _i64(gs.size), _i64(n), bm, bn, nblocks, _i64(total), _p(rec))
    return rec


def compare(d, g, rtol=2.0 ** -7):
    """Metrics dict; see oracle.c:orc_compare."""
    d = np.ascontiguousarray(d, dtype=np.float32).ravel()
    g = np.ascontiguousarray(g, dtype=np.float32).ravel()
    assert d.size == g.size
    m = np.zeros(5, dtype=np.float64)
    lib().orc_compare(_p(d), _p(g), _i64(d.size), ctypes.c_float(rtol), _p(m))
    return {"max_rel_floor1": m[0], "max_rel_floor_rms": m[1], "eb": m[2], "rms_golden": m[3], "frac_bad": m[4]}


def compare_double(d, g, g_low, err_threshold=2.0 ** -8, eb_threshold=2.0 ** -7):
    """The reference's double-golden acceptance metric (oracle.c:orc_compare_double): ratios of the result's max / mean
    relative error and RMSE against the high-precision golden to those of a low-precision golden, the eb percentage,
    and `ok` = the reference's verdict (ratios < 10, 2, 2 and eb <= 100)."""
    d = np.ascontiguousarray(d, dtype=np.float32).ravel()
    g = np.ascontiguousarray(g, dtype=np.float32).ravel()
    gl = np.ascontiguousarray(g_low, dtype=np.float32).ravel()
    assert d.size == g.size == gl.size
    m = np.zeros(10, dtype=np.float64)
    lib().orc_compare_double(_p(d), _p(g), _p(gl), _i64(d.size), ctypes.c_float(err_threshold), ctypes.c_float(eb_threshold), _p(m))
    names = ["max_rel_ratio", "mean_rel_ratio", "rmse_ratio", "eb_percent", "max_rel", "mean_rel", "rmse", "max_rel_low", "mean_rel_low", "rmse_low"]
    out = dict(zip(names, (float(x) for x in m)))
    out["ok"] = bool(m[0] < 10 and m[1] < 2 and m[2] < 2 and m[3] <= 100)
    return out


def moe_token_unpermute(permuted_bf16, sorted_indices, probs, top_k):
    """permuted uint16 [rows, hidden] (bf16 bits), sorted_indices int32 [tokens*top_k], probs float32
    [tokens*top_k] or None -> uint16 [tokens, hidden]."""
    x = np.ascontiguousarray(permuted_bf16, dtype=np.uint16)
    idx = np.ascontiguousarray(sorted_indices, dtype=np.int32).reshape(-1)
    rows, hidden = x.shape
    tokens = idx.size // top_k
    pr = None if probs is None else np.ascontiguousarray(probs, dtype=np.float32).reshape(-1)
    out = np.empty((tokens, hidden), dtype=np.uint16)
    rc = lib().orc_moe_token_unpermute(_p(x), _p(idx), _p(pr) if pr is not None else None, _i64(rows), _i64(tokens),
                                       _i64(hidden), int(top_k), _p(out))
    assert rc == 0
    return out


def send_buffer_row_map(global_tokens_per_local_expert, rank_rows=None):
    """Destination row of every result row of the down-projection grouped matmul.

    Tokens arrive grouped by local expert and, inside an expert, by the rank they came from
    (chunk (e, r) holds global_tokens_per_local_expert[r, e] rows); results leave grouped by
    destination rank and, inside a rank, by expert (the reference's RemapperC,
    include/catccos/dgemm/block/block_scheduler_reducescatter_alltoallv.hpp:237-256, and the golden's
    simulate_all_to_all_v_with_unpermute, examples/utils/gen_data_gmm_alltoallv_fp8_mx.py:720-737).
    Rank r's region starts at row r * rank_rows (default: directly after rank r-1's rows).
    Pure index arithmetic, pinned by a brute-force rebuild in the tests."""
    g = np.asarray(global_tokens_per_local_expert, dtype=np.int64)
    ranks, experts = g.shape
    per_rank = g.sum(axis=1)
    starts = np.arange(ranks) * rank_rows if rank_rows is not None else np.concatenate([[0], np.cumsum(per_rank)[:-1]])
    out = np.empty(int(g.sum()), dtype=np.int32)
    src = 0
    for e in range(experts):
        for r in range(ranks):
            n = int(g[r, e])
            dst = starts[r] + int(g[r, :e].sum())
            out[src:src + n] = np.arange(dst, dst + n)
            src += n
    return out


def scatter_rows(values, row_map, out_rows, fill=0):
    """out[row_map[i]] = values[i] for row_map[i] >= 0; other rows hold `fill`."""
    values = np.asarray(values)
    out = np.full((out_rows,) + values.shape[1:], fill, dtype=values.dtype)
    m = np.asarray(row_map)
    keep = m >= 0
    out[m[keep]] = values[: m.size][keep]
    return out


def moe_init_routing(expert_idx, num_experts, cumsum=False):
    """Stable sort of the flat (token, route) list by expert, as the reference's CPU stand-in does it
    (examples/utils/gen_data_moe.py:48-57: argsort(stable=True) of the flat expert indices and a
    bincount); entries outside [0, num_experts) are dropped (-1 in both maps).  Returns
    (dst_to_src, src_to_dst, expert_tokens).  Pinned in the tests by torch.argsort / torch.bincount."""
    flat = np.asarray(expert_idx, dtype=np.int64).reshape(-1)
    ok = (flat >= 0) & (flat < num_experts)
    order = np.argsort(np.where(ok, flat, num_experts), kind="stable")
    n_ok = int(ok.sum())
    dst_to_src = np.full(flat.size, -1, np.int32)
    dst_to_src[:n_ok] = order[:n_ok]
    src_to_dst = np.full(flat.size, -1, np.int32)
    src_to_dst[order[:n_ok]] = np.arange(n_ok, dtype=np.int32)
    counts = np.bincount(flat[ok], minlength=num_experts).astype(np.int32)
    return dst_to_src, src_to_dst, (np.cumsum(counts).astype(np.int32) if cumsum else counts)
