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

The operators are a C++ `TORCH_LIBRARY` (catccos_amd/csrc/torch/torch_bindings.cpp, built by
`python -m catccos_amd.build` into catccos_amd/libcatccos_torch.so): C++ programs linking libtorch load that
library directly; importing this module loads it into the Python process (`import catccos_amd` does not).
Also there: `mx_grouped_matmul_swiglu_mx`, `gmm_dequant_swiglu_mx` (up projections with MX-quantised output) and
`moe_ffn_mxfp8` (the MXFP8 MoE FFN of one rank, routing to combine).
"""
import os

import torch

from . import _abi

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libcatccos_torch.so")
if not os.path.exists(LIB_PATH):
    raise ImportError("%s is missing: build it with `python -m catccos_amd.build`" % LIB_PATH)
_abi.lib()                       # the HIP library first: a missing or unloadable one is reported by name
torch.ops.load_library(LIB_PATH)
