"""Pins of the oracle's MoE routing sort (CPU only): torch's own stable argsort and bincount, which is
what the reference's CPU stand-in calls (examples/utils/gen_data_moe.py:48-57)."""
import numpy as np
import torch

import oracle as orc


def test_against_torch_argsort_and_bincount():
    rng = np.random.default_rng(0)
    for rows, e in [(64, 4), (1000, 16), (5000, 256), (7, 1)]:
        idx = rng.integers(0, e, rows).astype(np.int32)
        d2s, s2d, cnt = orc.moe_init_routing(idx, e)
        t = torch.from_numpy(idx).to(torch.int64)
        order = torch.argsort(t, stable=True).to(torch.int32).numpy()
        assert np.array_equal(d2s, order)
        assert np.array_equal(cnt, torch.bincount(t, minlength=e).to(torch.int32).numpy())
        assert np.array_equal(d2s[s2d], np.arange(rows))
        _, _, cs = orc.moe_init_routing(idx, e, cumsum=True)
        assert np.array_equal(cs, np.cumsum(cnt))


def test_dropped_entries():
    idx = np.array([2, -1, 0, 9, 2, 0], np.int32)
    d2s, s2d, cnt = orc.moe_init_routing(idx, 3)
    assert list(d2s) == [2, 5, 0, 4, -1, -1]
    assert list(s2d) == [2, -1, 0, -1, 3, 1]
    assert list(cnt) == [2, 0, 2]
