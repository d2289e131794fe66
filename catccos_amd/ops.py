"""Tensor-level entry points, shaped like the reference's torch binding
(examples/torch_binding/src/torch_bindings.cpp:123-200): check dtype / device / shape,
make inputs contiguous, allocate the output, take the current stream, call the C ABI.

torch is used for device memory and streams only; all arithmetic happens in the HIP library.
"""
import torch

from . import _abi
from ._abi import FMT_E1M2, FMT_E2M1, FMT_E4M3, FMT_E5M2, ROUND_LUT, ROUND_RNE, check

_FMT_NAMES = {"e4m3": FMT_E4M3, "e5m2": FMT_E5M2, "e2m1": FMT_E2M1, "e1m2": FMT_E1M2, "fp8": FMT_E4M3, "fp4": FMT_E2M1}
_FP4 = (FMT_E2M1, FMT_E1M2)   # two codes per byte; E1M2 exists for the quantiser only


def _fmt(fmt):
    if isinstance(fmt, str):
        if fmt.lower() not in _FMT_NAMES:
            raise ValueError("unknown MX payload format %r" % fmt)
        return _FMT_NAMES[fmt.lower()]
    if fmt not in (FMT_E4M3, FMT_E5M2, FMT_E2M1, FMT_E1M2):
        raise ValueError("unknown MX payload format %r" % (fmt,))
    return fmt


def _require_gpu(*tensors):
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError("catccos_amd ops take GPU tensors only (got %s)" % t.device)


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


def scale_cols(k):
    """E8M0 bytes per row for a K extent: block count padded to even."""
    return 2 * ((k + 63) // 64)


def mx_quant(x, fmt="e4m3", rounding=ROUND_RNE):
    """MX block quantisation along the last axis of a 2-D bf16 (or IEEE half) tensor.

    Returns (payload uint8 [M, K] or [M, ceil(K/2)] for FP4, scales uint8 [M, scale_cols(K)]).
    """
    fmt = _fmt(fmt)
    _require_gpu(x)
    if x.dim() != 2 or x.dtype not in (torch.bfloat16, torch.float16):
        raise ValueError("mx_quant expects a 2-D bfloat16 (or float16) tensor")
    x = x.contiguous()
    m, k = x.shape
    pld = (k + 1) // 2 if fmt in _FP4 else k
    payload = torch.empty((m, pld), dtype=torch.uint8, device=x.device)
    scales = torch.empty((m, scale_cols(k)), dtype=torch.uint8, device=x.device)
    fn = _abi.lib().cch_mx_quant_rows_f16 if x.dtype == torch.float16 else _abi.lib().cch_mx_quant_rows
    check(fn(_ptr(x), _ptr(payload), _ptr(scales), m, k, fmt, rounding, _stream()))
    return payload, scales


def packed_row_bytes(k, fmt="e4m3"):
    """Bytes of one packed row of mx_quant_scatter_packed: payload followed by the padded scales."""
    return ((k + 1) // 2 if _fmt(fmt) in _FP4 else k) + scale_cols(k)


def mx_quant_scatter_packed(x, expanded_row_idx, packed_out, top_k, fmt="e4m3", rounding=ROUND_RNE, check_routes=False):
    """Quantises every row of x (bf16 [tokens, K]) once and writes [payload | scales] to rows
    expanded_row_idx[t * top_k + r] of packed_out (uint8 [rows, packed_row_bytes(K)]), skipping
    negative entries and entries at or past `rows`.  Rows that no route names keep their contents.  Returns packed_out.

    An entry at or past `rows` is a caller's error that the kernel turns into a dropped token (it cannot report from the
    device, and the reference treats it as the caller's error too).  check_routes=True looks at the whole table first and
    raises ValueError for such an entry: a debugging aid, it waits for the stream."""
    fmt = _fmt(fmt)
    _require_gpu(x, expanded_row_idx, packed_out)
    if x.dim() != 2 or x.dtype != torch.bfloat16:
        raise ValueError("mx_quant_scatter_packed expects a 2-D bfloat16 tensor")
    tokens, k = x.shape
    if expanded_row_idx.dtype != torch.int32 or expanded_row_idx.numel() != tokens * top_k:
        raise ValueError("expanded_row_idx must hold tokens * top_k int32 entries")
    row_bytes = ((k + 1) // 2 if fmt in _FP4 else k) + scale_cols(k)
    if packed_out.dim() != 2 or packed_out.dtype != torch.uint8 or packed_out.shape[1] != row_bytes or not packed_out.is_contiguous():
        raise ValueError("packed_out must be a contiguous uint8 [rows, %d] tensor" % row_bytes)
    # the kernel skips entries at or past packed_out's rows (like negative ones): no pass over the table
    # here, which would stall the stream, unless the caller asks for it
    if check_routes and expanded_row_idx.numel() and int(expanded_row_idx.max()) >= packed_out.shape[0]:
        raise ValueError("expanded_row_idx names row %d but packed_out has %d rows" % (int(expanded_row_idx.max()), packed_out.shape[0]))
    x = x.contiguous()
    idx = expanded_row_idx.contiguous()
    check(_abi.lib().cch_mx_quant_scatter_packed_rows(_ptr(x), _ptr(idx), _ptr(packed_out), packed_out.shape[0], tokens, k, int(top_k),
                                                      fmt, rounding, _stream()))
    return packed_out


def mx_quant_b(b, fmt="e4m3", rounding=ROUND_RNE, trans_b=0):
    """MX quantisation of a right-hand operand b [K,N] (bf16) with blocks running down K.

    trans_b=0: payload [K,N] (FP4 [K,N/2]), scales [K/64, N, 2];
    trans_b=1: payload [N,K] (FP4 [N,K/2]), scales [N, K/32].
    """
    fmt = _fmt(fmt)
    _require_gpu(b)
    if b.dim() != 2 or b.dtype != torch.bfloat16:
        raise ValueError("mx_quant_b expects a 2-D bfloat16 tensor [K,N]")
    b = b.contiguous()
    k, n = b.shape
    fp4 = fmt in _FP4
    if trans_b:
        payload = torch.empty((n, k // 2 if fp4 else k), dtype=torch.uint8, device=b.device)
        scales = torch.empty((n, k // 32), dtype=torch.uint8, device=b.device)
    else:
        payload = torch.empty((k, n // 2 if fp4 else n), dtype=torch.uint8, device=b.device)
        scales = torch.empty((k // 64, n, 2), dtype=torch.uint8, device=b.device)
    check(_abi.lib().cch_mx_quant_b(_ptr(b), _ptr(payload), _ptr(scales), k, n, fmt, rounding, int(trans_b), _stream()))
    return payload, scales


DQ_DEVICE, DQ_GOLDEN = 0, 1


def dynamic_quant_i8(x, src_rows=None, topk=1, mode=DQ_DEVICE, smooth=None, smooth_rows=None):
    """Per-token dynamic int8 quantisation of a 2-D bf16 tensor, optionally gathering rows.

    Output row i quantises x[src_rows[i] // topk] (x[i] without a row map).  With `smooth`
    (float32 [S, K] or [K]) every element is first multiplied by its column's entry of vector
    smooth_rows[i] (vector 0 without `smooth_rows`).  Returns (q int8 [T, K], scale float32 [T])
    with scale = amax(row) / 127.
    """
    _require_gpu(x)
    if x.dim() != 2 or x.dtype != torch.bfloat16:
        raise ValueError("dynamic_quant_i8 expects a 2-D bfloat16 tensor")
    x = x.contiguous()
    rows_in, k = x.shape
    if src_rows is not None:
        if src_rows.dim() != 1 or src_rows.dtype != torch.int32:
            raise ValueError("src_rows must be a 1-D int32 tensor")
        _require_gpu(src_rows)
        src_rows = src_rows.contiguous()
        t = src_rows.shape[0]
    else:
        t = rows_in
    if smooth is None and smooth_rows is not None:
        raise ValueError("smooth_rows needs smooth")
    if smooth is not None:
        _require_gpu(smooth)
        if smooth.dtype != torch.float32 or smooth.dim() not in (1, 2) or smooth.shape[-1] != k:
            raise ValueError("smooth must be float32 [S, K] or [K]")
        smooth = smooth.contiguous().view(-1, k)
        if smooth_rows is not None:
            _require_gpu(smooth_rows)
            if smooth_rows.dtype != torch.int32 or smooth_rows.shape != (t,):
                raise ValueError("smooth_rows must be int32 [T]")
            smooth_rows = smooth_rows.contiguous()
    q = torch.empty((t, k), dtype=torch.int8, device=x.device)
    scale = torch.empty((t,), dtype=torch.float32, device=x.device)
    src_p = _ptr(src_rows) if src_rows is not None else None
    if smooth is None:
        check(_abi.lib().cch_dyn_quant_i8_rows(_ptr(x), src_p, _ptr(q), _ptr(scale), rows_in, t, k, int(topk), int(mode), _stream()))
    else:
        check(_abi.lib().cch_dyn_quant_i8_rows_smooth(_ptr(x), src_p, _ptr(smooth),
                                                      _ptr(smooth_rows) if smooth_rows is not None else None, smooth.shape[0],
                                                      _ptr(q), _ptr(scale), rows_in, t, k, int(topk), int(mode), _stream()))
    return q, scale


def moe_init_routing(expert_idx, num_experts, cumsum=False):
    """Stable sort of the flat (token, route) list by expert.

    expert_idx: int32 tensor (any shape, read flat); entries outside [0, num_experts) are dropped.
    Returns (dst_to_src, src_to_dst, expert_tokens): the flat entry at every sorted position (-1 past
    the routed entries), the sorted position of every flat entry (-1 if dropped), and the entries
    per expert (their running sum with cumsum=True)."""
    _require_gpu(expert_idx)
    if expert_idx.dtype != torch.int32:
        raise ValueError("expert_idx must be an int32 tensor")
    idx = expert_idx.contiguous().reshape(-1)
    rows = idx.numel()
    dst_to_src = torch.empty(rows, dtype=torch.int32, device=idx.device)
    src_to_dst = torch.empty(rows, dtype=torch.int32, device=idx.device)
    tokens = torch.empty(num_experts, dtype=torch.int32, device=idx.device)
    nbytes = _abi.lib().cch_moe_init_routing_workspace_bytes(rows, int(num_experts))
    ws = torch.empty(max(int(nbytes), 4), dtype=torch.uint8, device=idx.device)
    check(_abi.lib().cch_moe_init_routing(_ptr(idx), rows, int(num_experts), _ptr(dst_to_src), _ptr(src_to_dst), _ptr(tokens),
                                          1 if cumsum else 0, _ptr(ws), ws.numel(), _stream()))
    return dst_to_src, src_to_dst, tokens


def moe_token_unpermute(permuted_tokens, sorted_indices, probs=None, top_k=1):
    """out[t] = sum_j permuted_tokens[sorted_indices[t*top_k + j]] * probs[t*top_k + j] (bf16 [tokens, hidden]).

    permuted_tokens bf16 [rows, hidden]; sorted_indices int32 with tokens*top_k entries (entries outside
    [0, rows) contribute nothing); probs float32 with as many entries, or None for a plain sum."""
    _require_gpu(permuted_tokens, sorted_indices)
    if permuted_tokens.dim() != 2 or permuted_tokens.dtype != torch.bfloat16:
        raise ValueError("permuted_tokens must be a 2-D bfloat16 tensor")
    if sorted_indices.dtype != torch.int32 or sorted_indices.numel() % top_k != 0:
        raise ValueError("sorted_indices must hold tokens * top_k int32 entries")
    x = permuted_tokens.contiguous()
    idx = sorted_indices.contiguous().reshape(-1)
    rows, hidden = x.shape
    tokens = idx.numel() // top_k
    if probs is not None:
        _require_gpu(probs)
        if probs.dtype != torch.float32 or probs.numel() != idx.numel():
            raise ValueError("probs must hold tokens * top_k float32 entries")
        probs = probs.contiguous().reshape(-1)
    out = torch.empty((tokens, hidden), dtype=torch.bfloat16, device=x.device)
    check(_abi.lib().cch_moe_token_unpermute(_ptr(x), _ptr(idx), _ptr(probs) if probs is not None else None, _ptr(out), rows,
                                             tokens, hidden, int(top_k), _stream()))
    return out


def set_option(name, value):
    """Library switch (see cch_set_option in include/catccos_hip.h)."""
    check(_abi.lib().cch_set_option(name.encode(), int(value)))


def _out_code(out_dtype):
    if out_dtype not in (torch.bfloat16, torch.float16):
        raise ValueError("out_dtype must be torch.bfloat16 or torch.float16")
    return 1 if out_dtype == torch.float16 else 0


def _check_2d(name, t, dtype):
    if t.dim() != 2 or t.dtype != dtype:
        raise ValueError("%s must be a 2-D %s tensor" % (name, dtype))


def w8a8_matmul_dequant(a, b, per_tok, per_ch, trans_b=0, out_dtype=torch.bfloat16):
    """int8 [M,K] x int8 [K,N] (or [N,K] with trans_b=1) -> bf16 (or half) [M,N], scaled per token and per channel."""
    code = _out_code(out_dtype)
    _require_gpu(a, b, per_tok, per_ch)
    _check_2d("a", a, torch.int8)
    _check_2d("b", b, torch.int8)
    a, b = a.contiguous(), b.contiguous()
    m, k = a.shape
    n = b.shape[0] if trans_b else b.shape[1]
    if (b.shape[1] if trans_b else b.shape[0]) != k:
        raise ValueError("inner dimensions differ: a %s, b %s, trans_b=%d" % (tuple(a.shape), tuple(b.shape), trans_b))
    per_tok = per_tok.contiguous().float()
    per_ch = per_ch.contiguous().float()
    if per_tok.numel() != m or per_ch.numel() != n:
        raise ValueError("per_tok must have M entries and per_ch N entries")
    out = torch.empty((m, n), dtype=out_dtype, device=a.device)
    check(_abi.lib().cch_gemm_i8_dequant_out(_ptr(a), _ptr(b), _ptr(per_tok), _ptr(per_ch), _ptr(out), m, n, k,
                                             int(trans_b), code, _stream()))
    return out


def gmm_dequant(x, w, group_sizes, per_tok, per_ch, trans_b=0, out_dtype=torch.bfloat16):
    """Grouped int8 matmul + per-token x per-channel dequant (no activation); returns bf16 (or half) [T, N]."""
    return _gmm_i8(x, w, group_sizes, per_tok, per_ch, trans_b, False, out_dtype)


def gmm_dequant_swiglu(x, w, group_sizes, per_tok, per_ch, trans_b=0, out_dtype=torch.bfloat16):
    """Grouped int8 matmul + dequant + SwiGLU: x int8 [T,K] grouped by expert, w int8 [E,K,N]
    (or [E,N,K]), group_sizes int32 [E] on the device; returns bf16 (or half) [T, N/2]."""
    return _gmm_i8(x, w, group_sizes, per_tok, per_ch, trans_b, True, out_dtype)


def gmm_dequant_swiglu_mx(x, w, group_sizes, per_tok, per_ch, trans_b=0, fmt="e4m3"):
    """gmm_dequant_swiglu with the activation MX-quantised along its rows in the kernel's epilogue:
    returns (payload uint8 [T, N/2] (FP4: [T, N/4]), scales uint8 [T, scale_cols(N/2)]), the same bytes
    as mx_quant(gmm_dequant_swiglu(...), fmt)."""
    return _gmm_i8(x, w, group_sizes, per_tok, per_ch, trans_b, True, torch.bfloat16, mx_fmt=_fmt(fmt))


def _gmm_i8(x, w, group_sizes, per_tok, per_ch, trans_b, swiglu, out_dtype=torch.bfloat16, mx_fmt=None):
    code = _out_code(out_dtype)
    _require_gpu(x, w, group_sizes, per_tok, per_ch)
    _check_2d("x", x, torch.int8)
    if w.dim() != 3 or w.dtype != torch.int8:
        raise ValueError("w must be a 3-D int8 tensor")
    if group_sizes.dtype != torch.int32 or group_sizes.dim() != 1:
        raise ValueError("group_sizes must be a 1-D int32 tensor")
    x, w, group_sizes = x.contiguous(), w.contiguous(), group_sizes.contiguous()
    t, k = x.shape
    e = w.shape[0]
    n = w.shape[1] if trans_b else w.shape[2]
    if (w.shape[2] if trans_b else w.shape[1]) != k or group_sizes.numel() != e:
        raise ValueError("shape mismatch between x, w and group_sizes")
    per_tok = per_tok.contiguous().float()
    per_ch = per_ch.contiguous().float()
    if per_tok.numel() != t or tuple(per_ch.shape) != (e, n):
        raise ValueError("per_tok must be [T] and per_ch [E,N]")
    if mx_fmt is not None:
        if n % 2 or (mx_fmt == FMT_E2M1 and n % 4):
            raise ValueError("n must be even (a multiple of 4 for FP4 output)")
        h = n // 2
        payload = torch.empty((t, h // 2 if mx_fmt == FMT_E2M1 else h), dtype=torch.uint8, device=x.device)
        scales = torch.empty((t, scale_cols(h)), dtype=torch.uint8, device=x.device)
        check(_abi.lib().cch_gmm_i8_dequant_swiglu_mx(_ptr(x), _ptr(w), _ptr(group_sizes), _ptr(per_tok), _ptr(per_ch), _ptr(payload),
                                                      _ptr(scales), e, t, n, k, int(trans_b), mx_fmt, _stream()))
        return payload, scales
    out = torch.empty((t, n // 2 if swiglu else n), dtype=out_dtype, device=x.device)
    fn = _abi.lib().cch_gmm_i8_dequant_swiglu_out if swiglu else _abi.lib().cch_gmm_i8_dequant_out
    check(fn(_ptr(x), _ptr(w), _ptr(group_sizes), _ptr(per_tok), _ptr(per_ch), _ptr(out), e, t, n, k, int(trans_b), code,
             _stream()))
    return out


def _mx_shapes(a, sa, b, sb, fmt, trans_b, grouped):
    fmt = _fmt(fmt)
    if fmt == FMT_E1M2:
        raise ValueError("E1M2 is a quantiser format only: the matrix instructions have no such operand type")
    fp4 = fmt == FMT_E2M1
    _check_2d("a", a, torch.uint8)
    _check_2d("sa", sa, torch.uint8)
    t = a.shape[0]
    k = a.shape[1] * (2 if fp4 else 1)
    bs = b.shape[1:] if grouped else b.shape
    if len(bs) != 2 or b.dtype != torch.uint8 or sb.dtype != torch.uint8:
        raise ValueError("b / sb must be uint8 tensors of rank %d" % (3 if grouped else 2))
    if trans_b:
        n, kb = bs[0], bs[1] * (2 if fp4 else 1)
    else:
        kb, n = bs[0], bs[1] * (2 if fp4 else 1)
    if kb != k:
        raise ValueError("inner dimensions differ: a gives K=%d, b gives K=%d" % (k, kb))
    if tuple(sa.shape) != (t, scale_cols(k)):
        raise ValueError("sa must be [%d,%d]" % (t, scale_cols(k)))
    e = b.shape[0] if grouped else 1
    if sb.numel() != e * scale_cols(k) * n:
        raise ValueError("sb has %d entries, expected %d" % (sb.numel(), e * scale_cols(k) * n))
    return fmt, t, n, k, e


def mx_matmul(a, sa, b, sb, fmt="e4m3", trans_b=0, out_dtype=torch.bfloat16):
    """MX dense GEMM: payload/scales as produced by mx_quant (a) and mx_quant_b (b); bf16 (or half) [M,N]."""
    code = _out_code(out_dtype)
    _require_gpu(a, sa, b, sb)
    a, sa, b, sb = a.contiguous(), sa.contiguous(), b.contiguous(), sb.contiguous()
    fmt, m, n, k, _ = _mx_shapes(a, sa, b, sb, fmt, trans_b, False)
    out = torch.empty((m, n), dtype=out_dtype, device=a.device)
    check(_abi.lib().cch_mx_gemm_out(_ptr(a), _ptr(sa), _ptr(b), _ptr(sb), _ptr(out), m, n, k, fmt, int(trans_b), code, _stream()))
    return out


def mx_grouped_matmul(a, sa, b, sb, group_sizes, fmt="e4m3", trans_b=0, out_dtype=torch.bfloat16):
    """MX grouped GEMM: rows of a grouped by expert (group_sizes int32 [E] on the device),
    b [E,...] / sb [E,...] one operand per expert; bf16 (or, with out_dtype=torch.float16, half) [T,N]."""
    _require_gpu(a, sa, b, sb, group_sizes)
    if group_sizes.dtype != torch.int32 or group_sizes.dim() != 1:
        raise ValueError("group_sizes must be a 1-D int32 tensor")
    a, sa, b, sb, group_sizes = a.contiguous(), sa.contiguous(), b.contiguous(), sb.contiguous(), group_sizes.contiguous()
    fmt, t, n, k, e = _mx_shapes(a, sa, b, sb, fmt, trans_b, True)
    if group_sizes.numel() != e:
        raise ValueError("group_sizes must have one entry per expert")
    if out_dtype not in (torch.bfloat16, torch.float16):
        raise ValueError("out_dtype must be torch.bfloat16 or torch.float16")
    out = torch.empty((t, n), dtype=out_dtype, device=a.device)
    if out_dtype == torch.float16:
        check(_abi.lib().cch_mx_gmm_mapped(_ptr(a), _ptr(sa), _ptr(b), _ptr(sb), _ptr(group_sizes), None, _ptr(out), t, 1, e,
                                           t, n, k, fmt, int(trans_b), _stream()))
    else:
        check(_abi.lib().cch_mx_gmm(_ptr(a), _ptr(sa), _ptr(b), _ptr(sb), _ptr(group_sizes), _ptr(out), e, t, n, k, fmt,
                                    int(trans_b), _stream()))
    return out


def mx_grouped_matmul_swiglu(a, sa, b, sb, group_sizes, fmt="e4m3", trans_b=0, out_dtype=torch.bfloat16, out_fmt=None):
    """MX grouped GEMM + SwiGLU, the up projection of the MX FFN chain: the [T, N] product is rounded to
    bf16, columns [0, N/2) are the gate and [N/2, N) the up half, out = silu(gate) * up [T, N/2] in
    bf16 (or half).  With out_fmt ("e4m3", "e5m2", "e2m1") the activation leaves MX-quantised from the
    epilogue instead: returns (payload, scales), the bytes mx_quant makes of the bf16 result."""
    _require_gpu(a, sa, b, sb, group_sizes)
    if group_sizes.dtype != torch.int32 or group_sizes.dim() != 1:
        raise ValueError("group_sizes must be a 1-D int32 tensor")
    a, sa, b, sb, group_sizes = a.contiguous(), sa.contiguous(), b.contiguous(), sb.contiguous(), group_sizes.contiguous()
    fmt, t, n, k, e = _mx_shapes(a, sa, b, sb, fmt, trans_b, True)
    if group_sizes.numel() != e:
        raise ValueError("group_sizes must have one entry per expert")
    if n % 2:
        raise ValueError("n must be even (gate | up halves)")
    h = n // 2
    if out_fmt is not None:
        ofmt = _fmt(out_fmt)
        if ofmt == FMT_E2M1 and h % 2:
            raise ValueError("n must be a multiple of 4 for FP4 output")
        payload = torch.empty((t, h // 2 if ofmt == FMT_E2M1 else h), dtype=torch.uint8, device=a.device)
        scales = torch.empty((t, scale_cols(h)), dtype=torch.uint8, device=a.device)
        check(_abi.lib().cch_mx_gmm_swiglu_mx(_ptr(a), _ptr(sa), _ptr(b), _ptr(sb), _ptr(group_sizes), _ptr(payload), _ptr(scales), e, t, n, k,
                                              fmt, int(trans_b), ofmt, _stream()))
        return payload, scales
    out = torch.empty((t, h), dtype=out_dtype, device=a.device)
    check(_abi.lib().cch_mx_gmm_swiglu(_ptr(a), _ptr(sa), _ptr(b), _ptr(sb), _ptr(group_sizes), _ptr(out), e, t, n, k, fmt, int(trans_b),
                                       _out_code(out_dtype), _stream()))
    return out


def mx_grouped_matmul_swiglu_packed(packed_a, k, b, sb, group_sizes, fmt="e4m3", trans_b=0, out_fmt="e4m3"):
    """mx_grouped_matmul_swiglu(..., out_fmt=...) whose left-hand operand is the packed buffer that
    mx_quant_scatter_packed fills (uint8 [T, packed_row_bytes(k, fmt)]: payload then scales per row)."""
    _require_gpu(packed_a, b, sb, group_sizes)
    fmt, ofmt = _fmt(fmt), _fmt(out_fmt)
    if packed_a.dim() != 2 or packed_a.dtype != torch.uint8 or packed_a.shape[1] != packed_row_bytes(k, fmt) or not packed_a.is_contiguous():
        raise ValueError("packed_a must be a contiguous uint8 [T, %d] tensor" % packed_row_bytes(k, fmt))
    if group_sizes.dtype != torch.int32 or group_sizes.dim() != 1:
        raise ValueError("group_sizes must be a 1-D int32 tensor")
    b, sb, group_sizes = b.contiguous(), sb.contiguous(), group_sizes.contiguous()
    t, e = packed_a.shape[0], b.shape[0]
    epb = 2 if fmt in _FP4 else 1
    n = b.shape[1] if trans_b else b.shape[2] * epb
    if b.dim() != 3 or (b.shape[2] * epb if trans_b else b.shape[1]) != k or group_sizes.numel() != e or sb.numel() != e * scale_cols(k) * n:
        raise ValueError("shape mismatch between packed_a, b, sb and group_sizes")
    if n % 2 or (ofmt == FMT_E2M1 and n % 4):
        raise ValueError("n must be even (a multiple of 4 for FP4 output)")
    h = n // 2
    payload = torch.empty((t, h // 2 if ofmt == FMT_E2M1 else h), dtype=torch.uint8, device=packed_a.device)
    scales = torch.empty((t, scale_cols(h)), dtype=torch.uint8, device=packed_a.device)
    check(_abi.lib().cch_mx_gmm_swiglu_mx_packed(_ptr(packed_a), _ptr(b), _ptr(sb), _ptr(group_sizes), _ptr(payload), _ptr(scales), e, t, n, k,
                                                 fmt, int(trans_b), ofmt, _stream()))
    return payload, scales


def mx_grouped_matmul_mapped(a, sa, b, sb, group_sizes, out_row_map, out, fmt="e4m3", trans_b=0):
    """MX grouped GEMM whose result row i is written to out[out_row_map[i]] (entries that are negative
    or past the end of `out` are dropped; rows of `out` that the map does not name keep their contents).  `out` is a contiguous
    bfloat16 or float16 [rows, N] tensor supplied by the caller (its dtype selects the output type); returns it."""
    _require_gpu(a, sa, b, sb, group_sizes, out_row_map, out)
    if group_sizes.dtype != torch.int32 or group_sizes.dim() != 1:
        raise ValueError("group_sizes must be a 1-D int32 tensor")
    a, sa, b, sb, group_sizes = a.contiguous(), sa.contiguous(), b.contiguous(), sb.contiguous(), group_sizes.contiguous()
    fmt, t, n, k, e = _mx_shapes(a, sa, b, sb, fmt, trans_b, True)
    if group_sizes.numel() != e:
        raise ValueError("group_sizes must have one entry per expert")
    if out_row_map.dtype != torch.int32 or out_row_map.numel() != t:
        raise ValueError("out_row_map must hold one int32 entry per row of a")
    if out.dim() != 2 or out.dtype not in (torch.bfloat16, torch.float16) or out.shape[1] != n or not out.is_contiguous():
        raise ValueError("out must be a contiguous bfloat16 or float16 [rows, %d] tensor" % n)
    row_map = out_row_map.contiguous()   # held until the launch is queued (a strided map becomes a copy)
    check(_abi.lib().cch_mx_gmm_mapped(_ptr(a), _ptr(sa), _ptr(b), _ptr(sb), _ptr(group_sizes), _ptr(row_map),
                                       _ptr(out), out.shape[0], 1 if out.dtype == torch.float16 else 0, e, t, n, k, fmt,
                                       int(trans_b), _stream()))
    return out


def moe_ffn_mxfp8(x, expert_idx, probs, w1, sw1, w2, sw2, trans_b=1):
    """The MXFP8 MoE FFN of one rank that holds every expert, routing to combine, five launches on the current stream
    (the reference's Ascend950DispatchFFNCombine, examples/ascend950_dispatch_ffn_combine/ascend950_dispatch_ffn_combine_device.h:124-176):
    routing sort -> MXFP8 quantise-and-scatter -> GMM1 + SwiGLU + MXFP8 quantise -> GMM2 -> weighted un-permute.

    x bf16 [m, k]; expert_idx int32 [m, top_k]; probs float32 [m, top_k]; w1 / sw1 and w2 / sw2 E4M3 payload and E8M0 scales
    of the experts' up ([k, n], gate columns first) and down ([n/2, k]) projections in the layout `trans_b` names
    (1, as the reference's files hold them: [E, n, k] and [E, k, n/2]).  Returns bf16 [m, k]."""
    _require_gpu(x, expert_idx, probs, w1, sw1, w2, sw2)
    if x.dim() != 2 or x.dtype != torch.bfloat16:
        raise ValueError("x must be a 2-D bfloat16 tensor")
    if expert_idx.dim() != 2 or expert_idx.shape[0] != x.shape[0] or probs.shape != expert_idx.shape:
        raise ValueError("expert_idx and probs must be [m, top_k]")
    m, k = x.shape
    top_k, e = expert_idx.shape[1], w1.shape[0]
    _, s2d, cnt = moe_init_routing(expert_idx, e)
    packed = torch.empty((m * top_k, packed_row_bytes(k)), dtype=torch.uint8, device=x.device)
    mx_quant_scatter_packed(x, s2d, packed, top_k)
    act, act_scales = mx_grouped_matmul_swiglu_packed(packed, k, w1, sw1, cnt, "e4m3", trans_b, "e4m3")
    y = mx_grouped_matmul(act, act_scales, w2, sw2, cnt, "e4m3", trans_b)
    if y.shape[1] != k:
        raise ValueError("w2 must map back to the hidden size of x")
    return moe_token_unpermute(y, s2d, probs, top_k)

