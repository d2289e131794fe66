"""`torch.ops.catccos.*`: the operator-library face of this package.

Mirrors the reference's torch binding (examples/torch_binding/src/torch_bindings.cpp:232-239
`TORCH_LIBRARY(catccos, m)` with `init` / `<op>` / `finalize`, device implementation registered for
the accelerator key only, and examples/torch_binding/src/torch_bindings_meta.cpp:18-35, a Meta
implementation that only builds the output shape), for the five compute halves this package holds
instead of `allgather_matmul`:

    torch.ops.catccos.init(rank_id, rank_size, local_mem_size, ip_port) -> int
    torch.ops.catccos.mx_quant(x, fmt, rounding) -> (payload, scales)
    torch.ops.catccos.w8a8_matmul_dequant(a, b, per_tok, per_ch, trans_b) -> Tensor
    torch.ops.catccos.mx_matmul(a, sa, b, sb, fmt, trans_b) -> Tensor
    torch.ops.catccos.gmm_dequant_swiglu(x, w, group_sizes, per_tok, per_ch, trans_b) -> Tensor
    torch.ops.catccos.mx_grouped_matmul(a, sa, b, sb, group_sizes, fmt, trans_b) -> Tensor
    torch.ops.catccos.finalize() -> int

Behaviour kept from the reference: an operator called before `init` fails with the reference's
message (torch_bindings.cpp:131-133); `init` checks its arguments like the reference and is a no-op the second
time (:88-95); `finalize` on an uninitialised library returns 0 (:205-207);
only the GPU key has kernels, so CPU tensors are refused by the dispatcher; the Meta kernels return
empty tensors of the result shape.  There is no communication here, so `init` accepts
`rank_size == 1` only and makes no use of `local_mem_size` / `ip_port` (the symmetric heap they size is the
part that was dropped).

Importing this module registers the library; `import catccos_amd` does not import it.
"""
import torch

from . import ops
from ._abi import FMT_E1M2, FMT_E2M1

_state = {"initialized": False, "rank_id": -1, "rank_size": 0}

_lib = torch.library.Library("catccos", "DEF")
_lib.define("init(int rank_id, int rank_size, int local_mem_size, str ip_port) -> int")
_lib.define("finalize() -> int")
_lib.define("mx_quant(Tensor x, str fmt, int rounding) -> (Tensor, Tensor)")
_lib.define("w8a8_matmul_dequant(Tensor a, Tensor b, Tensor per_tok, Tensor per_ch, int trans_b) -> Tensor")
_lib.define("mx_matmul(Tensor a, Tensor sa, Tensor b, Tensor sb, str fmt, int trans_b) -> Tensor")
_lib.define("gmm_dequant_swiglu(Tensor x, Tensor w, Tensor group_sizes, Tensor per_tok, Tensor per_ch, int trans_b) -> Tensor")
_lib.define("mx_grouped_matmul(Tensor a, Tensor sa, Tensor b, Tensor sb, Tensor group_sizes, str fmt, int trans_b) -> Tensor")
_lib.define("mx_grouped_matmul_swiglu_mx(Tensor a, Tensor sa, Tensor b, Tensor sb, Tensor group_sizes, str fmt, int trans_b, str out_fmt) -> (Tensor, Tensor)")
_lib.define("gmm_dequant_swiglu_mx(Tensor x, Tensor w, Tensor group_sizes, Tensor per_tok, Tensor per_ch, int trans_b, str fmt) -> (Tensor, Tensor)")
_lib.define("moe_ffn_mxfp8(Tensor x, Tensor expert_idx, Tensor probs, Tensor w1, Tensor sw1, Tensor w2, Tensor sw2, int trans_b) -> Tensor")


def _init(rank_id, rank_size, local_mem_size, ip_port):
    if _state["initialized"]:
        return 0   # torch_bindings.cpp:88-90: a second init is a no-op
    # the reference's argument checks and messages (torch_bindings.cpp:92-95)
    torch._check(rank_id >= 0, lambda: "invalid rank_id: %d" % rank_id)
    torch._check(rank_size > 0, lambda: "invalid rank_size: %d" % rank_size)
    torch._check(local_mem_size > 0, lambda: "invalid local_mem_size: %d" % local_mem_size)
    torch._check(len(ip_port) > 0, lambda: "ip_port is empty")
    torch._check(rank_size == 1 and rank_id == 0,
                 lambda: "catccos on one GPU has no peers: rank_size must be 1 and rank_id 0, got %d of %d" % (rank_id, rank_size))
    _state.update(initialized=True, rank_id=rank_id, rank_size=rank_size)
    return 0


def _finalize():
    if not _state["initialized"]:
        return 0
    if torch.cuda.is_available() and torch.cuda.is_initialized():
        torch.cuda.current_stream().synchronize()   # the reference drains the stream before it lets go of its buffers
    _state.update(initialized=False, rank_id=-1, rank_size=0)
    return 0


def _need_init():
    torch._check(_state["initialized"], lambda: "catccos TORCH_LIBRARY not initialized, call torch.ops.catccos.init(...) first")


def _guarded(fn):
    def run(*args):
        _need_init()
        with torch.cuda.device(args[0].device):
            return fn(*args)
    return run


# init / finalize take no tensors: one kernel for every backend, as in the reference
_lib.impl("init", _init, "CompositeExplicitAutograd")
_lib.impl("finalize", _finalize, "CompositeExplicitAutograd")
_lib.impl("mx_quant", _guarded(ops.mx_quant), "CUDA")
_lib.impl("w8a8_matmul_dequant", _guarded(ops.w8a8_matmul_dequant), "CUDA")
_lib.impl("mx_matmul", _guarded(ops.mx_matmul), "CUDA")
_lib.impl("gmm_dequant_swiglu", _guarded(ops.gmm_dequant_swiglu), "CUDA")
_lib.impl("mx_grouped_matmul", _guarded(ops.mx_grouped_matmul), "CUDA")
_lib.impl("gmm_dequant_swiglu_mx", _guarded(ops.gmm_dequant_swiglu_mx), "CUDA")
_lib.impl("moe_ffn_mxfp8", _guarded(ops.moe_ffn_mxfp8), "CUDA")
_lib.impl("mx_grouped_matmul_swiglu_mx", _guarded(lambda a, sa, b, sb, gs, fmt, tb, ofmt: ops.mx_grouped_matmul_swiglu(a, sa, b, sb, gs, fmt, tb, out_fmt=ofmt)),
          "CUDA")


# ---- Meta kernels: output shapes only (symbolic sizes pass through the arithmetic untouched)

def _fp4(fmt):
    return ops._fmt(fmt) in (FMT_E2M1, FMT_E1M2)


def _mx_quant_meta(x, fmt, rounding):
    m, k = x.shape
    payload = x.new_empty((m, (k + 1) // 2 if _fp4(fmt) else k), dtype=torch.uint8)
    return payload, x.new_empty((m, 2 * ((k + 63) // 64)), dtype=torch.uint8)


def _w8a8_meta(a, b, per_tok, per_ch, trans_b):
    return a.new_empty((a.shape[0], b.shape[0] if trans_b else b.shape[1]), dtype=torch.bfloat16)


def _mx_n(b_shape, fmt, trans_b):
    return b_shape[0] if trans_b else b_shape[1] * (2 if _fp4(fmt) else 1)


def _mx_matmul_meta(a, sa, b, sb, fmt, trans_b):
    return a.new_empty((a.shape[0], _mx_n(b.shape, fmt, trans_b)), dtype=torch.bfloat16)


def _gmm_swiglu_meta(x, w, group_sizes, per_tok, per_ch, trans_b):
    n = w.shape[1] if trans_b else w.shape[2]
    return x.new_empty((x.shape[0], n // 2), dtype=torch.bfloat16)


def _gmm_swiglu_mx_meta(x, w, group_sizes, per_tok, per_ch, trans_b, fmt):
    h = (w.shape[1] if trans_b else w.shape[2]) // 2
    payload = x.new_empty((x.shape[0], h // 2 if _fp4(fmt) else h), dtype=torch.uint8)
    return payload, x.new_empty((x.shape[0], 2 * ((h + 63) // 64)), dtype=torch.uint8)


def _mx_gmm_swiglu_mx_meta(a, sa, b, sb, group_sizes, fmt, trans_b, out_fmt):
    h = _mx_n(b.shape[1:], fmt, trans_b) // 2
    payload = a.new_empty((a.shape[0], h // 2 if _fp4(out_fmt) else h), dtype=torch.uint8)
    return payload, a.new_empty((a.shape[0], 2 * ((h + 63) // 64)), dtype=torch.uint8)


def _mx_gmm_meta(a, sa, b, sb, group_sizes, fmt, trans_b):
    return a.new_empty((a.shape[0], _mx_n(b.shape[1:], fmt, trans_b)), dtype=torch.bfloat16)


_lib.impl("moe_ffn_mxfp8", lambda x, expert_idx, probs, w1, sw1, w2, sw2, trans_b: x.new_empty(x.shape), "Meta")
_lib.impl("mx_quant", _mx_quant_meta, "Meta")
_lib.impl("w8a8_matmul_dequant", _w8a8_meta, "Meta")
_lib.impl("mx_matmul", _mx_matmul_meta, "Meta")
_lib.impl("gmm_dequant_swiglu", _gmm_swiglu_meta, "Meta")
_lib.impl("mx_grouped_matmul", _mx_gmm_meta, "Meta")
_lib.impl("gmm_dequant_swiglu_mx", _gmm_swiglu_mx_meta, "Meta")
_lib.impl("mx_grouped_matmul_swiglu_mx", _mx_gmm_swiglu_mx_meta, "Meta")
