"""GPU parity of the quantise-and-scatter entry point against the oracle: bit-exact packed rows,
all formats and both rounding rules, vector and byte store paths, skipped routes, untouched rows."""
import numpy as np
import pytest
import torch

import oracle as orc
import catccos_amd as cc

pytestmark = pytest.mark.gpu

FMTS = {"e4m3": orc.E4M3, "e5m2": orc.E5M2, "e2m1": orc.E2M1, "e1m2": orc.E1M2}


def rand_rows(rng, rows, k, sigma=1.0):
    x = (rng.standard_normal((rows, k)) * sigma).astype(np.float32)
    x[rng.random((rows, k)) < 0.001] *= 100.0
    return orc.f32_to_bf16(x)


def dev_bf16(bits):
    return torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16)


def run_case(tokens, k, topk, fmt, rounding, seed, drop=2):
    rng = np.random.default_rng(seed)
    xb = rand_rows(rng, tokens, k, 2.0)
    out_rows = tokens * topk + 5
    idx = rng.permutation(out_rows)[: tokens * topk].astype(np.int32)
    if idx.size:
        idx[rng.integers(0, idx.size, min(drop, idx.size))] = -1
    packed = torch.full((out_rows, cc.packed_row_bytes(k, fmt)), 0xA5, dtype=torch.uint8, device="cuda")
    cc.mx_quant_scatter_packed(dev_bf16(xb), torch.from_numpy(idx).cuda(), packed, topk, fmt, rounding)
    torch.cuda.synchronize()
    want = orc.mx_quant_scatter_packed(xb, idx, out_rows, topk, FMTS[fmt], rounding, fill=0xA5)
    assert np.array_equal(packed.cpu().numpy(), want)


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e2m1", "e1m2"])
@pytest.mark.parametrize("shape", [(64, 7168, 2), (33, 1024, 8), (7, 256, 1), (19, 4096, 4)])
def test_scatter_vector_path(shape, fmt):
    tokens, k, topk = shape
    run_case(tokens, k, topk, fmt, cc.ROUND_RNE, tokens + k + topk)


@pytest.mark.parametrize("fmt", ["e4m3", "e2m1"])
@pytest.mark.parametrize("shape", [(11, 64, 2), (5, 100, 3), (9, 31, 2), (6, 1000, 5), (3, 8200, 1)])
def test_scatter_byte_path_and_ragged_k(shape, fmt):
    # packed rows of these K are not multiples of 8 bytes (or K is ragged): byte stores
    tokens, k, topk = shape
    run_case(tokens, k, topk, fmt, cc.ROUND_RNE, tokens * 3 + k)


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e2m1", "e1m2"])
def test_scatter_lut_rounding(fmt):
    run_case(40, 2048, 2, fmt, cc.ROUND_LUT, 5)


def test_scatter_matches_row_quantiser_on_the_device():
    # the packed rows are the row quantiser's payload and scales, side by side
    rng = np.random.default_rng(3)
    tokens, k, topk = 128, 7168, 2
    xb = rand_rows(rng, tokens, k)
    x = dev_bf16(xb)
    idx = torch.arange(tokens * topk, dtype=torch.int32, device="cuda")
    packed = torch.zeros((tokens * topk, cc.packed_row_bytes(k)), dtype=torch.uint8, device="cuda")
    cc.mx_quant_scatter_packed(x, idx, packed, topk)
    payload, scales = cc.mx_quant(x)
    torch.cuda.synchronize()
    want = torch.cat([payload, scales], dim=1).repeat_interleave(topk, dim=0)
    assert torch.equal(packed, want)


def test_scatter_empty_and_errors():
    x = torch.zeros((0, 64), dtype=torch.bfloat16, device="cuda")
    packed = torch.full((4, cc.packed_row_bytes(64)), 9, dtype=torch.uint8, device="cuda")
    cc.mx_quant_scatter_packed(x, torch.zeros(0, dtype=torch.int32, device="cuda"), packed, 2)
    torch.cuda.synchronize()
    assert (packed == 9).all()
    x = torch.zeros((2, 64), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(cc.CatccosError):
        cc.mx_quant_scatter_packed(x, torch.zeros(18, dtype=torch.int32, device="cuda"), packed, 9)
    # entries at or past the rows of packed_out are skipped like negative ones (both kernels), nothing is written outside
    cc.mx_quant_scatter_packed(x, torch.full((4,), 7, dtype=torch.int32, device="cuda"), packed, 2)
    torch.cuda.synchronize()
    assert (packed == 9).all()


@pytest.mark.parametrize("shape", [(40, 2048, 2), (9, 96, 3)], ids=["streaming-kernel", "general-kernel"])
def test_scatter_skips_rows_past_the_output(shape):
    tokens, k, topk = shape
    rng = np.random.default_rng(tokens)
    xb = rand_rows(rng, tokens, k, 2.0)
    out_rows = tokens * topk - 7            # seven routes name rows that do not exist
    idx = rng.permutation(tokens * topk).astype(np.int32)
    # guard rows behind the buffer that the call is told about
    whole = torch.full((out_rows + 8, cc.packed_row_bytes(k)), 0x5A, dtype=torch.uint8, device="cuda")
    cc.mx_quant_scatter_packed(dev_bf16(xb), torch.from_numpy(idx).cuda(), whole[:out_rows], topk)
    torch.cuda.synchronize()
    want = orc.mx_quant_scatter_packed(xb, np.where(idx >= out_rows, -1, idx), out_rows, topk, orc.E4M3, orc.RNE, fill=0x5A)
    assert np.array_equal(whole[:out_rows].cpu().numpy(), want)
    assert (whole[out_rows:] == 0x5A).all()
    # the opt-in check names the caller's error instead of dropping the tokens
    with pytest.raises(ValueError, match="packed_out has"):
        cc.mx_quant_scatter_packed(dev_bf16(xb), torch.from_numpy(idx).cuda(), whole[:out_rows], topk, check_routes=True)
