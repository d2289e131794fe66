"""torch.ops.catccos.*: registration, init / finalize state, Meta shapes and dispatcher behaviour, as the
reference's binding has them (examples/torch_binding/src/torch_bindings.cpp:84-239,
torch_bindings_meta.cpp:18-35).  No GPU needed: Meta tensors carry shapes only."""
import pytest
import torch

import catccos_amd.torch_library  # (loads the library)

OPS = torch.ops.catccos


@pytest.fixture
def initialised():
    assert OPS.init(0, 1, 1 << 20, "tcp://127.0.0.1:8666") == 0
    yield
    assert OPS.finalize() == 0


def test_operators_come_from_the_cpp_library():
    """The operators are a C++ TORCH_LIBRARY translation unit (catccos_amd/csrc/torch/torch_bindings.cpp), as the reference's
    are (examples/torch_binding/src/torch_bindings.cpp:232-239): the Python module only loads the built library."""
    import os
    path = catccos_amd.torch_library.LIB_PATH
    assert os.path.basename(path) == "libcatccos_torch.so" and os.path.exists(path)
    assert any(os.path.samefile(path, p) for p in torch.ops.loaded_libraries)
    assert torch._C._dispatch_has_kernel_for_dispatch_key("catccos::mx_quant", "CUDA")
    assert torch._C._dispatch_has_kernel_for_dispatch_key("catccos::mx_quant", "Meta")
    assert not torch._C._dispatch_has_kernel_for_dispatch_key("catccos::mx_quant", "CPU")


def test_schemas_are_registered():
    for name in ("init", "finalize", "mx_quant", "w8a8_matmul_dequant", "mx_matmul", "gmm_dequant_swiglu", "mx_grouped_matmul", "gmm_dequant_swiglu_mx", "mx_grouped_matmul_swiglu_mx"):
        assert hasattr(OPS, name), name
    assert str(OPS.init.default._schema) == "catccos::init(int rank_id, int rank_size, int local_mem_size, str ip_port) -> int"
    assert str(OPS.finalize.default._schema) == "catccos::finalize() -> int"


def test_init_checks_and_state():
    assert OPS.finalize() == 0                     # not initialised: nothing to do
    for args, msg in (((-1, 1, 1, "x"), "invalid rank_id"), ((0, 0, 1, "x"), "invalid rank_size"),
                      ((0, 1, 0, "x"), "invalid local_mem_size"), ((0, 1, 1, ""), "ip_port is empty"),
                      ((1, 2, 1, "x"), "no peers")):
        with pytest.raises(RuntimeError, match=msg):
            OPS.init(*args)
    assert OPS.init(0, 1, 1024, "x") == 0
    assert OPS.init(5, 7, 0, "") == 0              # already initialised: no-op, arguments not looked at
    assert OPS.finalize() == 0
    assert OPS.finalize() == 0


def test_meta_shapes(initialised):
    m, k, n, e = 300, 1000, 512, 4
    x = torch.empty((m, k), dtype=torch.bfloat16, device="meta")
    p, s = OPS.mx_quant(x, "e4m3", 0)
    assert p.shape == (m, k) and s.shape == (m, 32) and p.dtype == s.dtype == torch.uint8 and p.device.type == "meta"
    p4, s4 = OPS.mx_quant(x, "e2m1", 0)
    assert p4.shape == (m, k // 2) and s4.shape == (m, 32)
    a = torch.empty((m, k), dtype=torch.int8, device="meta")
    for tb, bshape in ((0, (k, n)), (1, (n, k))):
        b = torch.empty(bshape, dtype=torch.int8, device="meta")
        out = OPS.w8a8_matmul_dequant(a, b, torch.empty(m, device="meta"), torch.empty(n, device="meta"), tb)
        assert out.shape == (m, n) and out.dtype == torch.bfloat16
        w = torch.empty((e,) + bshape, dtype=torch.int8, device="meta")
        out = OPS.gmm_dequant_swiglu(a, w, torch.empty(e, dtype=torch.int32, device="meta"), torch.empty(m, device="meta"),
                                     torch.empty((e, n), device="meta"), tb)
        assert out.shape == (m, n // 2) and out.dtype == torch.bfloat16
        pq, sq = OPS.gmm_dequant_swiglu_mx(a, w, torch.empty(e, dtype=torch.int32, device="meta"), torch.empty(m, device="meta"),
                                           torch.empty((e, n), device="meta"), tb, "e2m1")
        assert pq.shape == (m, n // 4) and sq.shape == (m, 2 * ((n // 2 + 63) // 64)) and pq.dtype == sq.dtype == torch.uint8
    k = 1024
    u8 = lambda *shape: torch.empty(shape, dtype=torch.uint8, device="meta")   # noqa: E731
    assert OPS.mx_matmul(u8(m, k), u8(m, 32), u8(k, n), u8(16, n, 2), "e4m3", 0).shape == (m, n)
    assert OPS.mx_matmul(u8(m, k // 2), u8(m, 32), u8(n, k // 2), u8(n, 32), "e2m1", 1).shape == (m, n)
    assert OPS.mx_matmul(u8(m, k // 2), u8(m, 32), u8(k, n // 2), u8(16, n, 2), "e2m1", 0).shape == (m, n)
    out = OPS.mx_grouped_matmul(u8(m, k // 2), u8(m, 32), u8(e, k, n // 2), u8(e, 16, n, 2),
                                torch.empty(e, dtype=torch.int32, device="meta"), "e2m1", 0)
    assert out.shape == (m, n) and out.dtype == torch.bfloat16
    pq, sq = OPS.mx_grouped_matmul_swiglu_mx(u8(m, k), u8(m, 32), u8(e, k, n), u8(e, 16, n, 2), torch.empty(e, dtype=torch.int32, device="meta"),
                                             "e4m3", 0, "e4m3")
    assert pq.shape == (m, n // 2) and sq.shape == (m, 2 * ((n // 2 + 63) // 64))
    out = OPS.moe_ffn_mxfp8(torch.empty((m, k), dtype=torch.bfloat16, device="meta"), torch.empty((m, 2), dtype=torch.int32, device="meta"), torch.empty((m, 2), device="meta"),
                            u8(e, n, k), u8(e, n, 32), u8(e, k, n // 2), u8(e, k, 2 * ((n // 2 + 63) // 64)), 1)
    assert out.shape == (m, k) and out.dtype == torch.bfloat16


def test_cpu_tensors_have_no_kernel(initialised):
    """Only the GPU key holds kernels (the reference registers its operator for the accelerator key
    alone): the dispatcher refuses CPU tensors instead of some slower path running."""
    x = torch.zeros((4, 64), dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError):
        OPS.mx_quant(x, "e4m3", 0)
