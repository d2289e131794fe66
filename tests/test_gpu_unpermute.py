"""GPU parity of the MoE token un-permute against the oracle: bit-exact bf16 rows, with and
without probabilities, vector and element-wise paths, dropped routes."""
import numpy as np
import pytest
import torch

import oracle as orc
import catccos_amd as cc

pytestmark = pytest.mark.gpu


def bf16_rows(rng, rows, hidden, sigma=1.0):
    return orc.f32_to_bf16((rng.standard_normal((rows, hidden)) * sigma).astype(np.float32))


def dev_bf16(bits):
    return torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16)


def host_bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("with_probs", [True, False])
@pytest.mark.parametrize("shape", [(512, 7168, 2), (4096, 4096, 8), (100, 1000, 4), (33, 7, 3), (64, 520, 1), (5, 8200, 5)])
def test_unpermute_bit_exact(shape, with_probs):
    rows, hidden, top_k = shape
    rng = np.random.default_rng(rows + hidden + top_k)
    tokens = rows // top_k
    xb = bf16_rows(rng, rows, hidden, 2.0)
    idx = rng.permutation(rows)[: tokens * top_k].astype(np.int32)
    idx[rng.integers(0, idx.size, 3)] = rows + 7
    idx[rng.integers(0, idx.size, 2)] = -1
    idx[0] = rows                                   # route 0 of token 0 dropped: the sum starts at zero
    probs = rng.random(tokens * top_k).astype(np.float32) if with_probs else None
    out = cc.moe_token_unpermute(dev_bf16(xb), torch.from_numpy(idx).cuda(),
                                 torch.from_numpy(probs).cuda() if with_probs else None, top_k)
    torch.cuda.synchronize()
    want = orc.moe_token_unpermute(xb, idx, probs, top_k)
    assert np.array_equal(host_bits(out), want)


def test_unpermute_products_rounded_before_the_sum():
    x = np.array([[1.0 + 2.0 ** -7] * 8, [-1.0] * 8], np.float32)
    p0 = np.float32(1.0 + 2.0 ** -20)
    prod = np.float32(x[0, 0]) * p0
    probs = torch.tensor([p0, prod], dtype=torch.float32, device="cuda")
    out = cc.moe_token_unpermute(dev_bf16(orc.f32_to_bf16(x)), torch.tensor([0, 1], dtype=torch.int32, device="cuda"), probs, 2)
    torch.cuda.synchronize()
    assert (out.float() == 0).all()


def test_unpermute_inverts_the_routing_gather():
    # tokens gathered into expert order by the dynamic quantiser's row map come back in token order
    rng = np.random.default_rng(3)
    tokens, hidden, top_k = 256, 2048, 2
    xb = bf16_rows(rng, tokens, hidden)
    expert = rng.integers(0, 8, tokens * top_k)
    order = np.argsort(expert, kind="stable").astype(np.int32)        # sorted position -> expanded row
    inverse = np.empty_like(order)
    inverse[order] = np.arange(order.size, dtype=np.int32)            # expanded row -> sorted position
    x = dev_bf16(xb)
    permuted = x[torch.from_numpy(order // top_k).cuda().long()]      # [tokens*top_k, hidden] in expert order
    out = cc.moe_token_unpermute(permuted, torch.from_numpy(inverse).cuda(), None, top_k)
    torch.cuda.synchronize()
    want = orc.f32_to_bf16(orc.bf16_to_f32(xb) * 2.0)                 # each token summed with itself
    assert np.array_equal(host_bits(out), want)


def test_unpermute_empty_and_errors():
    x = torch.zeros((4, 64), dtype=torch.bfloat16, device="cuda")
    out = cc.moe_token_unpermute(x, torch.zeros(0, dtype=torch.int32, device="cuda"), None, 2)
    assert out.shape == (0, 64)
    with pytest.raises(cc.CatccosError):
        cc.moe_token_unpermute(x, torch.zeros(18, dtype=torch.int32, device="cuda"), None, 9)
