"""GPU parity of the MX block quantiser against the CPU oracle: bytes and scales bit-exact."""
import numpy as np
import pytest
import torch

import oracle as orc
import catccos_amd as cc
from catccos_amd import _abi

pytestmark = pytest.mark.gpu

FMTS = [(orc.E4M3, cc.FMT_E4M3), (orc.E5M2, cc.FMT_E5M2), (orc.E2M1, cc.FMT_E2M1), (orc.E1M2, cc.FMT_E1M2)]


def to_dev(bits_u16):
    return torch.from_numpy(bits_u16.view(np.int16)).cuda().view(torch.bfloat16)


def gpu_quant(bits_u16, fmt, rounding):
    p, s = cc.mx_quant(to_dev(bits_u16), fmt, rounding)
    torch.cuda.synchronize()
    return p.cpu().numpy(), s.cpu().numpy()


def cfg1_input(m, k, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, k), dtype=np.float32)
    x = np.where(rng.random((m, k)) < 0.001, x * 100, x).astype(np.float32)
    return orc.f32_to_bf16(x)


@pytest.mark.parametrize("ofmt,gfmt", FMTS)
@pytest.mark.parametrize("rounding", [orc.RNE, orc.LUT])
@pytest.mark.parametrize("shape", [(256, 7168), (130, 1024), (3, 32), (1, 4096), (64, 96), (17, 8 * 37)])
def test_rows_bit_exact(ofmt, gfmt, rounding, shape):
    x = cfg1_input(*shape, seed=sum(shape) + ofmt)
    p, s = gpu_quant(x, gfmt, rounding)
    po, so = orc.mx_quant_rows(x, ofmt, rounding)
    assert np.array_equal(s, so)
    assert np.array_equal(p, po)


@pytest.mark.parametrize("ofmt,gfmt", FMTS)
@pytest.mark.parametrize("shape", [(5, 70), (9, 33), (4, 1), (7, 1001), (2, 31)])
def test_ragged_k_bit_exact(ofmt, gfmt, shape):
    """K not a multiple of 32 / 8 / 2: zero padded last block, even-padded scale row."""
    x = cfg1_input(*shape, seed=7)
    p, s = gpu_quant(x, gfmt, orc.RNE)
    po, so = orc.mx_quant_rows(x, ofmt, orc.RNE)
    assert np.array_equal(s, so)
    assert np.array_equal(p, po)


@pytest.mark.parametrize("ofmt,gfmt", FMTS)
@pytest.mark.parametrize("rounding", [orc.RNE, orc.LUT])
def test_every_bf16_value_under_every_block_maximum_class(ofmt, gfmt, rounding):
    """All 65536 bf16 patterns as block members, each row led by a block maximum chosen so that
    ties, zero results, subnormal codes and saturation all occur."""
    allbits = np.arange(65536, dtype=np.uint16)
    finite = allbits[(allbits & 0x7F80) != 0x7F80]
    rows = []
    for lead in (0x3F80, 0x43FA, 0x4400, 0x3F00 | 0x55, 0x7F7F, 0x0080, 0x2000, 0x3FC0):
        leadv = orc.bf16_to_f32(np.array([lead], np.uint16))[0]
        vals = orc.bf16_to_f32(finite)
        members = finite[np.abs(vals) <= leadv]
        n = (members.size + 30) // 31
        blk = np.zeros((n, 32), np.uint16)
        blk[:, 0] = lead
        flat = np.zeros(n * 31, np.uint16)
        flat[:members.size] = members
        blk[:, 1:] = flat.reshape(n, 31)
        rows.append(blk.reshape(-1))
    k = 2048
    flat = np.concatenate(rows)
    pad = (-flat.size) % k
    x = np.concatenate([flat, np.zeros(pad, np.uint16)]).reshape(-1, k)
    p, s = gpu_quant(x, gfmt, rounding)
    po, so = orc.mx_quant_rows(x, ofmt, rounding)
    assert np.array_equal(s, so)
    assert np.array_equal(p, po)


def test_special_blocks_match_oracle():
    f = np.zeros((2, 160), np.float32)
    f[0, 32:64] = 500.0
    f[0, 64] = -1e-30
    f[0, 96] = np.inf
    f[0, 128] = 1.0
    f[0, 130] = -2.0 ** -20
    f[1, 5] = np.nan
    f[1, 40] = -np.inf
    x = orc.f32_to_bf16(f)
    for ofmt, gfmt in FMTS:
        for rounding in (orc.RNE, orc.LUT):
            p, s = gpu_quant(x, gfmt, rounding)
            po, so = orc.mx_quant_rows(x, ofmt, rounding)
            assert np.array_equal(s, so), (ofmt, rounding)
            assert np.array_equal(p, po), (ofmt, rounding)


def test_hardware_cast_equals_integer_encoder():
    x = cfg1_input(512, 7168, seed=11)
    xd = to_dev(x)
    p1, s1 = cc.mx_quant(xd, "e4m3")
    L = _abi.lib()
    assert L.cch_set_option(b"quant_integer_encoder", 1) == 0
    try:
        p2, s2 = cc.mx_quant(xd, "e4m3")
    finally:
        assert L.cch_set_option(b"quant_integer_encoder", 0) == 0
    torch.cuda.synchronize()
    assert torch.equal(p1, p2) and torch.equal(s1, s2)


def test_full_size_config1_whole_tensor_and_properties():
    """[4096,7168] N(0,1) with 0.1% x100 outliers: every byte of the whole tensor bit-exact, and the
    size-independent properties: re-quantising the dequantised tensor is the identity,
    doubling the input shifts every scale byte by one and leaves the payload unchanged."""
    m, k = 4096, 7168
    x = cfg1_input(m, k, seed=1)
    xd = to_dev(x)
    p, s = cc.mx_quant(xd, "e4m3")
    torch.cuda.synchronize()
    po, so = orc.mx_quant_rows(x, orc.E4M3, orc.RNE)   # the whole tensor (the oracle takes well under a second)
    assert np.array_equal(p.cpu().numpy(), po) and np.array_equal(s.cpu().numpy(), so)
    deq = p.view(torch.float8_e4m3fn).to(torch.float32) * torch.exp2(s.to(torch.float32) - 127).repeat_interleave(32, 1)
    p2, s2 = cc.mx_quant(deq.to(torch.bfloat16), "e4m3")
    assert torch.equal(p2, p) and torch.equal(s2, s)
    p3, s3 = cc.mx_quant((xd.float() * 2).to(torch.bfloat16), "e4m3")
    assert torch.equal(p3, p) and torch.equal(s3, s + 1)
    # ties, signed zeros and clamped values are present in this input (they must be, for the test to bite)
    assert int((p == 0x80).sum()) > 0 and int(((p & 0x7F) == 0x7E).sum()) > 0


def test_empty_and_bad_arguments():
    e = torch.empty((0, 64), dtype=torch.bfloat16, device="cuda")
    p, s = cc.mx_quant(e)
    assert p.shape == (0, 64) and s.shape == (0, 2)
    with pytest.raises(ValueError):
        cc.mx_quant(torch.zeros(4, 64, device="cuda"))
    with pytest.raises(ValueError):
        cc.mx_quant(torch.zeros(4, 64, dtype=torch.bfloat16))
    with pytest.raises(cc.CatccosError):
        cc.mx_quant(torch.zeros(4, 64, dtype=torch.bfloat16, device="cuda"), "e4m3", rounding=7)


@pytest.mark.parametrize("ofmt,gfmt", FMTS)
@pytest.mark.parametrize("trans_b", [0, 1])
@pytest.mark.parametrize("rounding", [orc.RNE, orc.LUT])
def test_quant_b_bit_exact(ofmt, gfmt, trans_b, rounding):
    k, n = 256, 1030
    b = cfg1_input(k, n, seed=5)
    p, s = cc.mx_quant_b(to_dev(b), gfmt, rounding, trans_b)
    torch.cuda.synchronize()
    po, so = orc.mx_quant_b(b, ofmt, rounding, trans_b)
    assert np.array_equal(s.cpu().numpy(), so)
    assert np.array_equal(p.cpu().numpy(), po)
