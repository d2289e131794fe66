"""Tensor-level entry points, shaped like the reference's torch binding
(examples/torch_binding/src/torch_bindings.cpp:123-200): check dtype / device / shape,
make inputs contiguous, allocate the output, take the current stream, call the C ABI.

torch is used for device memory and streams only; all arithmetic happens in the HIP library.
"""
import torch

from . import _abi
from ._abi import FMT_E2M1, FMT_E4M3, FMT_E5M2, ROUND_LUT, ROUND_RNE, check

_FMT_NAMES = {"e4m3": FMT_E4M3, "e5m2": FMT_E5M2, "e2m1": FMT_E2M1, "fp8": FMT_E4M3, "fp4": FMT_E2M1}


def _fmt(fmt):
    if isinstance(fmt, str):
        if fmt.lower() not in _FMT_NAMES:
            raise ValueError("unknown MX payload format %r" % fmt)
        return _FMT_NAMES[fmt.lower()]
    if fmt not in (FMT_E4M3, FMT_E5M2, FMT_E2M1):
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
    """MX block quantisation along the last axis of a 2-D bf16 tensor.

    Returns (payload uint8 [M, K] or [M, ceil(K/2)] for FP4, scales uint8 [M, scale_cols(K)]).
    """
    fmt = _fmt(fmt)
    _require_gpu(x)
    if x.dim() != 2 or x.dtype != torch.bfloat16:
        raise ValueError("mx_quant expects a 2-D bfloat16 tensor")
    x = x.contiguous()
    m, k = x.shape
    pld = (k + 1) // 2 if fmt == FMT_E2M1 else k
    payload = torch.empty((m, pld), dtype=torch.uint8, device=x.device)
    scales = torch.empty((m, scale_cols(k)), dtype=torch.uint8, device=x.device)
    check(_abi.lib().cch_mx_quant_rows(_ptr(x), _ptr(payload), _ptr(scales), m, k, fmt, rounding, _stream()))
    return payload, scales


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
    fp4 = fmt == FMT_E2M1
    if trans_b:
        payload = torch.empty((n, k // 2 if fp4 else k), dtype=torch.uint8, device=b.device)
        scales = torch.empty((n, k // 32), dtype=torch.uint8, device=b.device)
    else:
        payload = torch.empty((k, n // 2 if fp4 else n), dtype=torch.uint8, device=b.device)
        scales = torch.empty((k // 64, n, 2), dtype=torch.uint8, device=b.device)
    check(_abi.lib().cch_mx_quant_b(_ptr(b), _ptr(payload), _ptr(scales), k, n, fmt, rounding, int(trans_b), _stream()))
    return payload, scales
