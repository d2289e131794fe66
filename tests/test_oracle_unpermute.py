"""Pins of the oracle's MoE token un-permute (CPU only).

The oracle restates KernelMoeTokenUnpermute (examples/aux_ops/moe_token_unpermute/
moe_token_unpermute.h:235-355).  It is checked against a torch restatement in which every step is
one separately rounded fp32 tensor operation (torch never fuses a multiply into an add), and through
special cases that fix the index convention and the rounding."""
import numpy as np
import torch

import oracle as orc


def bf16_rows(rng, rows, hidden, sigma=1.0):
    return orc.f32_to_bf16((rng.standard_normal((rows, hidden)) * sigma).astype(np.float32))


def torch_unpermute(xb, idx, probs, top_k):
    x = torch.from_numpy(orc.bf16_to_f32(xb))
    rows = x.shape[0]
    tokens = idx.size // top_k
    idx = idx.reshape(tokens, top_k)
    acc = torch.zeros((tokens, x.shape[1]), dtype=torch.float32)
    for j in range(top_k):
        col = torch.from_numpy(idx[:, j].astype(np.int64))
        ok = (col >= 0) & (col < rows)
        v = x[col.clamp(0, rows - 1)]
        if probs is not None:
            v = v * torch.from_numpy(probs.reshape(tokens, top_k)[:, j]).unsqueeze(1)
        if j == 0:
            acc = torch.where(ok.unsqueeze(1), v, acc)
        else:
            acc = torch.where(ok.unsqueeze(1), acc + v, acc)
    return acc.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def test_against_torch_stepwise():
    rng = np.random.default_rng(0)
    for rows, hidden, top_k in [(64, 128, 2), (300, 1000, 8), (40, 7168, 4), (9, 7, 3)]:
        tokens = rows // top_k
        xb = bf16_rows(rng, rows, hidden, 2.0)
        idx = rng.permutation(rows)[: tokens * top_k].astype(np.int32)
        idx[rng.integers(0, idx.size, 3)] = rows + 5          # dropped routes
        idx[rng.integers(0, idx.size, 2)] = -1
        probs = rng.random(tokens * top_k).astype(np.float32)
        got = orc.moe_token_unpermute(xb, idx, probs, top_k)
        assert np.array_equal(got, torch_unpermute(xb, idx, probs, top_k))
        got = orc.moe_token_unpermute(xb, idx, None, top_k)
        assert np.array_equal(got, torch_unpermute(xb, idx, None, top_k))


def test_top1_unit_probs_is_a_gather():
    rng = np.random.default_rng(1)
    xb = bf16_rows(rng, 50, 96)
    idx = rng.permutation(50).astype(np.int32)
    got = orc.moe_token_unpermute(xb, idx, np.ones(50, np.float32), 1)
    assert np.array_equal(got, xb[idx])


def test_scaling_probs_by_a_power_of_two_scales_the_result():
    rng = np.random.default_rng(2)
    xb = bf16_rows(rng, 32, 64)
    idx = rng.permutation(32).astype(np.int32)
    probs = rng.random(32).astype(np.float32)
    a = orc.bf16_to_f32(orc.moe_token_unpermute(xb, idx, probs, 4))
    b = orc.bf16_to_f32(orc.moe_token_unpermute(xb, idx, probs * 4.0, 4))
    assert np.array_equal(a * 4.0, b)


def test_products_are_rounded_before_the_sum():
    # x*p is inexact in fp32 and cancels against the second route: a fused multiply-add would keep
    # the low bits of the product and give a different (non-zero) answer.
    x = np.array([[1.0 + 2.0 ** -7], [-1.0]], np.float32)        # both exact in bf16
    p0 = np.float32(1.0 + 2.0 ** -20)
    prod = np.float32(x[0, 0]) * p0                               # rounded fp32 product
    xb = orc.f32_to_bf16(x)
    probs = np.array([p0, prod], np.float32)                      # second route contributes -prod exactly
    got = orc.bf16_to_f32(orc.moe_token_unpermute(xb, np.array([0, 1], np.int32), probs, 2))
    assert got[0, 0] == 0.0
