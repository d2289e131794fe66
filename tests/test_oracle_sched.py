"""Scheduler arithmetic: the reference's only numeric known-answer test, plus partition invariants."""
import json
import os

import numpy as np

import oracle as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_reference_unit_test_vector():
    """tests/comm_block_scheduler_alltoallv_gmm/test_comm_block_scheduler_alltoallv_gmm.cpp:37-102:
    rank=2, EP=4, expertPerRank=2, tokenData[i]=i+1; expected 16 ints (entries 2,3 are the
    freshly reset context).  The expected vector is the committed fixture golden/scheduler_kat.json."""
    kat = json.load(open(os.path.join(GOLDEN, "scheduler_kat.json")))
    tok = np.arange(1, 33, dtype=np.int32)
    rank, ep, epr = kat["rank"], kat["ep"], kat["expert_per_rank"]
    assert [(q["core"], q["num"]) for q in kat["queries"]] == [(1, 3), (4, 6), (0, 3)]
    got = []
    core, num = 1, 3
    got += [core, num, 0, 0, orc.sched_src_prev_sum(tok, rank, ep, epr, core), orc.sched_comm_loops(ep, core, num),
            orc.sched_block_offset_row(core, num, 0), orc.sched_block_offset_row(core, num, 1)]
    core, num = 4, 6
    got += [core, orc.sched_src_prev_sum(tok, rank, ep, epr, core), orc.sched_comm_loops(ep, core, num),
            orc.sched_block_offset_row(core, num, 0)]
    core, num = 0, 3
    got += [core, orc.sched_src_prev_sum(tok, rank, ep, epr, core), orc.sched_comm_loops(ep, core, num),
            orc.sched_block_offset_row(core, num, 1)]
    assert got == kat["expected"] == [1, 3, 0, 0, 42, 1, 1, 4, 4, 0, 0, 4, 0, 10, 2, 3]


def test_cumsum_mm_is_column_cumsum():
    rng = np.random.default_rng(0)
    ep, epr, rank = 4, 3, 1
    tok = rng.integers(0, 50, ep * ep * epr).astype(np.int32)
    got = orc.sched_cumsum_mm(tok, rank, ep, epr)
    want = np.cumsum(tok.reshape(ep, ep * epr)[:, rank * epr:(rank + 1) * epr], axis=0)
    assert np.array_equal(got, want)


def test_tile_order_partitions_output_once():
    gs = np.array([300, 0, 1, 128, 129, 0, 77], np.int32)
    n, bm, bn, nb = 600, 128, 256, 5
    rec = orc.grouped_tile_order(gs, n, bm, bn, nb)
    cover = np.zeros((int(gs.sum()), n), np.int32)
    starts = np.concatenate([[0], np.cumsum(gs)])
    for i, (w, g, r0, c0, rows, cols) in enumerate(rec):
        assert w == i % nb
        assert starts[g] <= r0 and r0 + rows <= starts[g + 1] and rows > 0 and cols > 0
        cover[r0:r0 + rows, c0:c0 + cols] += 1
    assert np.all(cover == 1)
    assert len(rec) == sum(-(-int(m) // bm) * -(-n // bn) for m in gs)
    assert not np.any(np.isin(rec[:, 1], [1, 5]))  # empty groups yield no tile


def test_tile_order_serpentine_small_case():
    rec = orc.grouped_tile_order(np.array([3, 2], np.int32), 3, 1, 1, 2)
    # group 0: 3x3 tiles, odd tile-rows reversed; group 1: 2x3
    want_cols = [0, 1, 2, 2, 1, 0, 0, 1, 2, 0, 1, 2, 2, 1, 0]
    want_rows = [0, 0, 0, 1, 1, 1, 2, 2, 2, 3, 3, 3, 4, 4, 4]
    assert list(rec[:, 3]) == want_cols and list(rec[:, 2]) == want_rows
    assert list(rec[:, 0]) == [i % 2 for i in range(15)]


def test_send_buffer_row_map_against_brute_force():
    # rebuild the golden's reordering literally: split the expert-major rows into (expert, rank)
    # chunks, then concatenate per destination rank in expert order
    # (gen_data_gmm_alltoallv_fp8_mx.py:720-737 with one expert-parallel rank)
    rng = np.random.default_rng(0)
    for ranks, experts in [(1, 4), (2, 3), (4, 8), (3, 1)]:
        g = rng.integers(0, 6, (ranks, experts))
        g[rng.integers(0, ranks), rng.integers(0, experts)] = 0
        total = int(g.sum())
        rows = np.arange(total)
        chunks = np.split(rows, np.cumsum(g.T.reshape(-1))[:-1])            # [expert][rank]
        want_order = np.concatenate([np.concatenate([chunks[e * ranks + r] for e in range(experts)] or [rows[:0]])
                                     for r in range(ranks)] or [rows[:0]])
        m = orc.send_buffer_row_map(g)
        assert sorted(m.tolist()) == list(range(total))
        assert np.array_equal(want_order[m], rows)                           # row i lands where the golden puts it
        padded = orc.send_buffer_row_map(g, rank_rows=total + 3)
        per_rank = g.sum(axis=1)
        for r in range(ranks):
            sel = (padded >= r * (total + 3)) & (padded < (r + 1) * (total + 3))
            assert sel.sum() == per_rank[r]


def test_scatter_rows_places_and_drops():
    vals = np.arange(12, dtype=np.float32).reshape(4, 3)
    out = orc.scatter_rows(vals, np.array([2, -1, 0, 5], np.int32), 6, fill=-7)
    assert np.array_equal(out[2], vals[0]) and np.array_equal(out[0], vals[2]) and np.array_equal(out[5], vals[3])
    assert (out[[1, 3, 4]] == -7).all()
