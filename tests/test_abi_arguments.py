"""Argument checks of the C ABI that return before any device work: they run without a GPU.
Every entry point rejects negative or oversized shapes, bad enums and missing pointers with
CCH_EINVAL and leaves a message for cch_last_error()."""
from catccos_amd import _abi

P = 0x1000   # a non-null pointer that is never dereferenced: every call below fails its checks first
BIG = 1 << 31


def rejected(rc, *needles):
    msg = _abi.lib().cch_last_error().decode()
    assert rc == _abi.EINVAL, (rc, msg)
    for n in needles:
        assert n in msg, msg


def test_quantiser_arguments():
    L = _abi.lib()
    rejected(L.cch_mx_quant_rows(P, P, P, -1, 64, 0, 0, None), "cch_mx_quant_rows")
    rejected(L.cch_mx_quant_rows(P, P, P, 4, 64, 9, 0, None))          # format
    rejected(L.cch_mx_quant_rows(P, P, P, 4, 64, 0, 5, None))          # rounding
    rejected(L.cch_mx_quant_rows(None, P, P, 4, 64, 0, 0, None))
    rejected(L.cch_mx_quant_rows_f16(P, P, P, -1, 64, 0, 0, None), "cch_mx_quant_rows_f16")
    rejected(L.cch_mx_quant_rows_f16(P, P, P, 4, 64, 9, 0, None), "format")
    rejected(L.cch_mx_quant_rows_f16(P, P, P, 4, 64, 0, 5, None), "rounding")
    rejected(L.cch_mx_quant_rows_f16(None, P, P, 4, 64, 0, 0, None), "null")
    assert L.cch_mx_quant_rows_f16(None, None, None, 0, 64, 0, 0, None) == _abi.OK
    rejected(L.cch_mx_quant_scatter_packed(P, P, P, 4, 64, -1, 0, 0, None), "top_k")
    assert L.cch_mx_quant_scatter_packed(P, P, P, 4, 64, 0, 0, 0, None) == _abi.OK   # no routes: nothing to do
    rejected(L.cch_mx_quant_scatter_packed(P, P, P, 4, 64, 9, 0, 0, None), "top_k")
    rejected(L.cch_mx_quant_scatter_packed_rows(P, P, P, -1, 4, 64, 2, 0, 0, None), "out_rows")
    rejected(L.cch_mx_quant_scatter_packed_rows(P, P, P, 8, 4, 64, 2, 9, 0, None), "format")
    assert L.cch_mx_quant_scatter_packed_rows(P, P, P, 8, 0, 64, 2, 0, 0, None) == _abi.OK   # no tokens


def test_dynamic_quantiser_arguments():
    L = _abi.lib()
    rejected(L.cch_dyn_quant_i8_rows(P, None, P, P, 4, 4, -8, 1, 0, None), "negative")
    rejected(L.cch_dyn_quant_i8_rows(P, None, P, P, 4, 4, 64, 0, 0, None), "topk")
    rejected(L.cch_dyn_quant_i8_rows(P, None, P, P, 4, 4, 64, 1, 2, None), "mode")
    rejected(L.cch_dyn_quant_i8_rows(P, None, P, P, 4, 8, 64, 1, 0, None), "row map")
    rejected(L.cch_dyn_quant_i8_rows(P, None, P, None, 4, 4, 64, 1, 0, None), "scale")
    rejected(L.cch_dyn_quant_i8_rows_smooth(P, None, None, None, 1, P, P, 4, 4, 64, 1, 0, None), "smooth")
    rejected(L.cch_dyn_quant_i8_rows_smooth(P, None, P, None, 0, P, P, 4, 4, 64, 1, 0, None), "num_smooth")


def test_gemm_arguments():
    L = _abi.lib()
    rejected(L.cch_gemm_i8_dequant(P, P, P, P, P, -1, 8, 8, 0, None), "negative")
    rejected(L.cch_gemm_i8_dequant(P, P, P, P, P, 8, BIG, 8, 0, None), "too large")
    rejected(L.cch_gemm_i8_dequant(P, P, P, P, P, 8, 8, 8, 2, None), "trans_b")
    rejected(L.cch_gemm_i8_dequant(P, P, None, P, P, 8, 8, 8, 0, None), "null")
    rejected(L.cch_gmm_i8_dequant_swiglu(P, P, P, P, P, P, 2, 8, 7, 8, 0, None), "even")
    rejected(L.cch_gmm_i8_dequant_swiglu(P, P, P, P, P, P, 0, 8, 8, 8, 0, None), "num_experts")
    rejected(L.cch_gmm_i8_dequant_swiglu(P, P, None, P, P, P, 2, 8, 8, 8, 0, None), "null")
    rejected(L.cch_gmm_i8_dequant(P, P, P, P, P, P, 70000, 8, 8, 8, 0, None), "num_experts")
    # the group table of the kernels holds 256 experts: 257 is an error, not an overrun
    rejected(L.cch_gmm_i8_dequant(P, P, P, P, P, P, 257, 8, 8, 8, 0, None), "num_experts", "256")
    rejected(L.cch_gmm_i8_dequant_swiglu(P, P, P, P, P, P, 257, 8, 8, 8, 0, None), "num_experts", "256")
    rejected(L.cch_mx_gmm(P, P, P, P, P, P, 257, 8, 8, 64, 0, 0, None), "num_experts", "256")
    rejected(L.cch_mx_gmm_swiglu(P, P, P, P, P, P, 2, 8, 7, 64, 0, 0, 0, None), "even")
    rejected(L.cch_mx_gmm_swiglu(P, P, P, P, P, P, 2, 8, 8, 64, 0, 0, 2, None), "out_dtype")
    rejected(L.cch_mx_gmm_swiglu(P, P, P, P, None, P, 2, 8, 8, 64, 0, 0, 0, None), "group_sizes")
    rejected(L.cch_mx_gmm_swiglu(P, P, P, P, P, P, 257, 8, 8, 64, 0, 0, 0, None), "num_experts", "256")
    rejected(L.cch_mx_gmm_swiglu_mx(P, P, P, P, P, P, P, 2, 8, 8, 64, 0, 0, 3, None), "out_fmt")
    rejected(L.cch_mx_gmm_swiglu_mx(P, P, P, P, P, P, P, 2, 8, 6, 64, 0, 0, 2, None), "FP4")
    rejected(L.cch_mx_gmm_swiglu_mx(P, P, P, P, P, P, None, 2, 8, 8, 64, 0, 0, 0, None), "null")
    # SwiGLU with MX-quantised output: payload formats E4M3, E5M2, E2M1; n even (FP4: a multiple of 4)
    rejected(L.cch_gmm_i8_dequant_swiglu_mx(P, P, P, P, P, P, P, 2, 8, 8, 8, 0, 3, None), "fmt")
    rejected(L.cch_gmm_i8_dequant_swiglu_mx(P, P, P, P, P, P, P, 2, 8, 7, 8, 0, 0, None), "even")
    rejected(L.cch_gmm_i8_dequant_swiglu_mx(P, P, P, P, P, P, P, 2, 8, 6, 8, 0, 2, None), "FP4")
    rejected(L.cch_gmm_i8_dequant_swiglu_mx(P, P, P, P, P, P, P, 257, 8, 8, 8, 0, 0, None), "num_experts", "256")
    rejected(L.cch_gmm_i8_dequant_swiglu_mx(P, P, P, P, P, P, None, 2, 8, 8, 8, 0, 0, None), "null")
    assert L.cch_gmm_i8_dequant_swiglu_mx(None, None, None, None, None, None, None, 2, 0, 8, 8, 0, 0, None) == _abi.OK   # no rows
    rejected(L.cch_mx_gmm_mapped(P, P, P, P, P, P, P, 8, 0, 257, 8, 8, 64, 0, 0, None), "num_experts", "256")
    rejected(L.cch_mx_gemm(P, P, P, P, P, 8, 8, 64, 7, 0, None))           # format
    rejected(L.cch_mx_gemm(P, P, P, P, P, 8, 7, 64, 2, 0, None), "FP4")   # FP4 packs two columns per byte
    rejected(L.cch_mx_gmm(P, P, P, P, None, P, 2, 8, 8, 64, 0, 0, None))   # group sizes missing
    rejected(L.cch_mx_gmm_mapped(P, P, P, P, P, None, P, 9, 0, 2, 8, 8, 64, 0, 0, None), "row map")
    rejected(L.cch_mx_gmm_mapped(P, P, P, P, P, P, P, 8, 3, 2, 8, 8, 64, 0, 0, None), "out_dtype")
    rejected(L.cch_gemm_i8_dequant_out(P, P, P, P, P, 8, 8, 8, 0, 2, None), "out_dtype")
    rejected(L.cch_gmm_i8_dequant_out(P, P, P, P, P, P, 2, 8, 8, 8, 0, -1, None), "out_dtype")
    rejected(L.cch_gmm_i8_dequant_swiglu_out(P, P, P, P, P, P, 2, 8, 8, 8, 0, 5, None), "out_dtype")
    rejected(L.cch_mx_gemm_out(P, P, P, P, P, 8, 8, 64, 0, 0, 2, None), "out_dtype")


def test_routing_and_unpermute_arguments():
    L = _abi.lib()
    rejected(L.cch_moe_init_routing(P, 8, 0, P, P, P, 0, P, 1 << 20, None), "num_experts")
    rejected(L.cch_moe_init_routing(P, 8, 2000, P, P, P, 0, P, 1 << 20, None), "num_experts")
    rejected(L.cch_moe_init_routing(P, 8, 4, P, P, P, 0, P, 1, None), "workspace")
    rejected(L.cch_moe_init_routing(P, 8, 4, P, P, None, 0, P, 1 << 20, None), "expert_tokens")
    assert L.cch_moe_init_routing_workspace_bytes(2048, 8) == 2 * 8 * 4
    rejected(L.cch_moe_token_unpermute(P, P, None, P, 8, 4, 64, 0, None), "top_k")
    rejected(L.cch_moe_token_unpermute(P, P, None, P, 8, 4, 64, 9, None), "top_k")
    rejected(L.cch_moe_token_unpermute(P, P, None, P, -1, 4, 64, 2, None), "negative")
    rejected(L.cch_set_option(b"no_such_option", 1), "unknown option")
    rejected(L.cch_set_option(b"gemm_balance_rounds", 1), "unknown option")   # a switch that no longer exists
    # the switches the header documents are all known (set to their defaults: nothing changes)
    for name, default in ((b"force_generic_gemm", 0), (b"require_tiled_gemm", 0), (b"gemm_tile_order", -1), (b"gemm_nt_output", -1),
                          (b"i8_epilogue_fp16_step", 0), (b"quant_integer_encoder", 0), (b"routing_three_launches", 0)):
        assert L.cch_set_option(name, default) == _abi.OK, name


def test_empty_problems_succeed_without_a_device():
    L = _abi.lib()
    assert L.cch_gemm_i8_dequant(None, None, None, None, None, 0, 8, 8, 0, None) == _abi.OK
    assert L.cch_mx_gmm(None, None, None, None, None, None, 2, 0, 8, 64, 0, 0, None) == _abi.OK
    assert L.cch_dyn_quant_i8_rows(None, None, None, None, 0, 0, 64, 1, 0, None) == _abi.OK
    assert L.cch_moe_token_unpermute(None, None, None, None, 0, 0, 64, 2, None) == _abi.OK
