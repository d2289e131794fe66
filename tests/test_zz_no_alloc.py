"""cch_moe_init_routing_noalloc (built-in histogram area, no device allocation in the call) against
cch_moe_init_routing (caller's workspace): same integers, on two calls in a row of which the second
is smaller, and the size limit is an error."""
import numpy as np
import pytest
import torch

from catccos_amd import _abi

pytestmark = pytest.mark.gpu


def _ptr(t):
    return t.data_ptr()


def _route(idx, experts, cumsum, noalloc, outs=None):
    L = _abi.lib()
    rows = idx.numel()
    d2s, s2d, cnt = outs if outs is not None else (torch.full((rows,), -7, dtype=torch.int32, device="cuda"),
                                                   torch.full((rows,), -7, dtype=torch.int32, device="cuda"),
                                                   torch.full((experts,), -7, dtype=torch.int32, device="cuda"))
    stream = torch.cuda.current_stream().cuda_stream
    if noalloc:
        rc = L.cch_moe_init_routing_noalloc(_ptr(idx), rows, experts, _ptr(d2s), _ptr(s2d), _ptr(cnt), cumsum, stream)
    else:
        nbytes = L.cch_moe_init_routing_workspace_bytes(rows, experts)
        ws = torch.empty(max(int(nbytes), 4), dtype=torch.uint8, device="cuda")
        rc = L.cch_moe_init_routing(_ptr(idx), rows, experts, _ptr(d2s), _ptr(s2d), _ptr(cnt), cumsum, _ptr(ws), ws.numel(), stream)
    _abi.check(rc)
    torch.cuda.synchronize()
    return d2s.cpu().numpy(), s2d.cpu().numpy(), cnt.cpu().numpy()


def _case(rows, experts, seed):
    rng = np.random.default_rng(seed)
    idx = rng.integers(0, experts, rows).astype(np.int32)
    idx[rng.integers(0, rows, 3)] = -1
    idx[rng.integers(0, rows, 2)] = experts
    return torch.from_numpy(idx).cuda()


def test_noalloc_routing_matches_workspace_routing_on_two_calls():
    assert _abi.lib().cch_init(0) == 0
    # the second call is smaller in rows and in experts, so it reuses a part of what the first one left behind
    # (up to 8192 rows and 256 experts the sort is one workgroup that needs no histogram area: the second call stays above that)
    for (rows, experts, cumsum, seed) in ((70000, 256, 0, 1), (20000, 16, 1, 2), (5000, 16, 1, 4), (1, 1, 0, 3)):
        idx = _case(rows, experts, seed) if rows > 10 else torch.zeros(rows, dtype=torch.int32, device="cuda")
        # outputs allocated before the call under test; the call itself must not allocate
        outs = (torch.full((rows,), -7, dtype=torch.int32, device="cuda"), torch.full((rows,), -7, dtype=torch.int32, device="cuda"),
                torch.full((experts,), -7, dtype=torch.int32, device="cuda"))
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        got = _route(idx, experts, cumsum, True, outs)
        assert torch.cuda.memory_allocated() == before
        want = _route(idx, experts, cumsum, False)
        for g, w in zip(got, want):
            assert np.array_equal(g, w)


def test_noalloc_routing_empty_input():
    idx = torch.zeros(0, dtype=torch.int32, device="cuda")
    got = _route(idx, 4, 0, True)
    assert list(got[2]) == [0, 0, 0, 0]


def test_noalloc_routing_rejects_sizes_beyond_its_area():
    L = _abi.lib()
    rows, experts = 300 * 1024, 1024     # 300 chunks x 1024 experts > 262144 entries
    idx = torch.zeros(rows, dtype=torch.int32, device="cuda")
    out = torch.empty(rows, dtype=torch.int32, device="cuda")
    cnt = torch.empty(experts, dtype=torch.int32, device="cuda")
    rc = L.cch_moe_init_routing_noalloc(_ptr(idx), rows, experts, _ptr(out), _ptr(out), _ptr(cnt), 0, None)
    assert rc == _abi.EINVAL and b"exceeds the built-in area" in L.cch_last_error()
