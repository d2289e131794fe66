"""Pins of the oracle's quantise-and-scatter (CPU only).

The oracle restates CommBlockMxQuant::QuantScatterPacked
(include/catccos/comm/block/comm_block_mx_quant.hpp:319-369).  Its quantiser is the row quantiser,
pinned elsewhere; what is new is the packed row layout and the routing, checked here by rebuilding
the result with numpy indexing from the row quantiser's outputs."""
import numpy as np
import pytest

import oracle as orc


def rand_rows(rng, rows, k, sigma=1.0):
    return orc.f32_to_bf16((rng.standard_normal((rows, k)) * sigma).astype(np.float32))


@pytest.mark.parametrize("fmt", [orc.E4M3, orc.E5M2, orc.E2M1])
@pytest.mark.parametrize("shape", [(9, 64, 2), (5, 100, 3), (16, 7168, 8), (4, 31, 1)])
def test_scatter_equals_rows_then_index(shape, fmt):
    tokens, k, topk = shape
    rng = np.random.default_rng(tokens * 7 + k + fmt)
    xb = rand_rows(rng, tokens, k, 3.0)
    out_rows = tokens * topk + 3
    idx = rng.permutation(out_rows)[: tokens * topk].astype(np.int32)
    idx[rng.integers(0, idx.size, 2)] = -1
    got = orc.mx_quant_scatter_packed(xb, idx, out_rows, topk, fmt, fill=0xA5)
    payload, scales = orc.mx_quant_rows(xb, fmt)
    assert got.shape[1] == payload.shape[1] + scales.shape[1] == orc.packed_row_bytes(k, fmt)
    want = np.full_like(got, 0xA5)
    for t in range(tokens):
        for r in range(topk):
            d = idx[t * topk + r]
            if d >= 0:
                want[d] = np.concatenate([payload[t], scales[t]])
    assert np.array_equal(got, want)


def test_packed_row_bytes_follow_the_reference_formula():
    # quantBytes + AlignUp(CeilDiv(N, 32), 2), comm_block_mx_quant.hpp:328-331
    for k in (1, 31, 32, 33, 64, 96, 7168):
        raw = (k + 31) // 32
        assert orc.packed_row_bytes(k, orc.E4M3) == k + ((raw + 1) // 2) * 2
        assert orc.packed_row_bytes(k, orc.E2M1) == (k + 1) // 2 + ((raw + 1) // 2) * 2


def test_no_routes_is_a_no_op():
    xb = rand_rows(np.random.default_rng(0), 3, 64)
    out = orc.mx_quant_scatter_packed(xb, np.full(6, -1, np.int32), 8, 2, fill=7)
    assert (out == 7).all()
