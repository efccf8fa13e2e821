"""Pins the oracle's count / scan / pos / capacity rules against torch library
routines (bincount, cumsum, stable sort), invariants, and the reference's own
input vectors."""
import os

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _ids(n, E, seed, drop=0.1):
    g = torch.Generator().manual_seed(seed)
    idx = torch.randint(0, E, (n,), generator=g)
    idx[torch.rand(n, generator=g) < drop] = -1
    return idx


@pytest.mark.parametrize("n,E,seed", [(0, 3, 0), (1, 1, 1), (500, 7, 2), (4096, 64, 3)])
def test_count_and_pos_match_library(n, E, seed):
    idx = _ids(n, E, seed)
    cnt = O.expert_count(idx, E)
    keep = idx >= 0
    assert torch.equal(cnt.long(), torch.bincount(idx[keep], minlength=E))
    pos, off = O.assign_pos(idx, E)
    # offsets: exclusive scan; the reference's inclusive cumsum is offsets[1:]
    assert torch.equal(off[1:].long(), torch.cumsum(cnt.long(), 0))
    assert off[0] == 0
    # closed form: a stable sort by expert id with the dropped entries removed
    key = torch.where(keep, idx, torch.full_like(idx, E))
    order = torch.sort(key, stable=True).indices[: int(keep.sum())]
    assert torch.equal(pos, order)
    # admissible for the reference's atomic fill (local_exchange.cu:6-17): a permutation of
    # the kept flat indices, each segment holding exactly its expert's indices
    assert sorted(pos.tolist()) == torch.nonzero(keep).view(-1).tolist()
    for e in range(E):
        seg = pos[off[e]:off[e + 1]]
        assert (idx[seg] == e).all()
    inv = O.inverse_pos(pos, n)
    assert (inv[pos] == torch.arange(pos.numel())).all() and (inv[~keep] == -1).all()


def test_capacity_rule():
    idx = torch.tensor([[0, 1], [0, 1], [0, 2], [0, 1], [1, 0]])
    kept = O.limit_by_capacity(idx, 3, 2)
    assert kept.tolist() == [[0, 1], [0, 1], [-1, 2], [-1, -1], [-1, -1]]
    assert torch.equal(O.limit_by_capacity(idx, 3, -1), idx)
    assert (O.limit_by_capacity(idx, 3, 0) == -1).all()
    # counts after limiting are min(count, capacity)
    big = _ids(3000, 5, 7, drop=0.0)
    lim = O.limit_by_capacity(big, 5, 400)
    assert torch.equal(O.expert_count(lim, 5).long(), torch.bincount(big, minlength=5).clamp(max=400))
    # the kept ones are the earliest in flat order
    for e in range(5):
        where = torch.nonzero(big == e).view(-1)
        assert (lim[where[:400]] == e).all() and (lim[where[400:]] == -1).all()


def test_reference_pos_vector_is_a_valid_top2_scatter_index():
    """csrc/pos.pt is pos // 2 for 4096 tokens with top-2: every token twice.  Used as the
    scatter index exactly as the reference's check does (csrc/test.cpp:405-449)."""
    p = torch.from_numpy(np.load(os.path.join(GOLDEN, "ref_pos_div2.npy")))
    assert p.shape == (8192,) and p.dtype == torch.int64
    assert torch.equal(torch.bincount(p, minlength=4096), torch.full((4096,), 2))
    x = torch.arange(4096 * 4, dtype=torch.float32).view(4096, 4)
    # local_scatter(x, pos, k) gathers rows pos // k: feed it 2 * p so that pos // 2 == p
    assert torch.equal(O.local_scatter(x, 2 * p, 2), torch.index_select(x, 0, p))


def test_planner_on_reference_count_table():
    """divide_into_block on the skewed 4x64 table the reference ships (rows sum to 8192)."""
    table = np.load(os.path.join(GOLDEN, "ref_all_expert_count.npy"))
    assert table.shape == (4, 64) and (table.sum(1) == 8192).all()
    for row in table:
        plan = O.divide_into_block(row.tolist(), 64)
        starts = np.concatenate([[0], np.cumsum(row)[:-1]])
        nb = plan["total_block_num"]
        assert nb == sum(-(-c // 64) for c in row)
        assert plan["remote_block_num"] == int((row % 64 != 0).sum())
        # blocks tile each expert's segment exactly, none longer than 64
        for e in range(64):
            blocks = sorted((plan["start_addrs"][b], plan["lens"][b]) for b in range(nb)
                            if plan["expert_ids"][b] == e)
            at = starts[e]
            for s, l in blocks:
                assert s == at and 0 < l <= 64
                at += l
            assert at == starts[e] + row[e]
        # CSR is consistent
        idxs, ids = plan["expert_block_id_idxs"], plan["expert_block_ids"]
        assert idxs[0] == 0 and idxs[-1] == nb and sorted(ids) == list(range(nb))
        for e in range(64):
            assert all(plan["expert_ids"][b] == e for b in ids[idxs[e]:idxs[e + 1]])
        # interleave: full blocks and tails alternate while both lists last
        lens = plan["lens"]
        n_tail = plan["remote_block_num"]
        n_full = nb - n_tail
        m = min(n_full, n_tail)
        assert all(lens[2 * i] == 64 for i in range(m)) and all(lens[2 * i + 1] < 64 for i in range(m))
