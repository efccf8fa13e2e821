"""GPU parity of each stage of the hot path against the CPU oracle, through the C ABI.

Integer results (expert choice, counts, offsets, pos) must be bit-exact; floating
point results must be within max-abs 2e-2 and mean-rel 1e-3 of the fp32 oracle.
"""
import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_REL = 2e-2, 1e-3


def _say(msg):
    print(msg, flush=True)


def dev(t):
    return t.cuda()


# ------------------------------------------------------------------ gate
@pytest.mark.parametrize("T,d,E,k,dtype,seed", [
    (64, 256, 4, 1, torch.float16, 0),
    (333, 768, 32, 1, torch.float16, 1),
    (512, 1024, 8, 2, torch.float16, 2),
    (129, 4096, 8, 2, torch.float16, 3),
    (100, 2048, 64, 2, torch.float16, 4),
    (77, 512, 70, 4, torch.float16, 5),
    (512, 256, 4, 1, torch.float32, 6),
    (300, 1032, 70, 3, torch.float32, 8),
    (64, 8, 2, 2, torch.float16, 7),
    (1, 8, 1, 1, torch.float16, 9),
    (3, 64, 1024, 8, torch.float16, 10),
    (70, 16384, 4, 2, torch.float16, 11),
    (5, 136, 17, 8, torch.float16, 12),
])
def test_gate_bit_exact(T, d, E, k, dtype, seed):
    from ccfuser_amd import ops
    _say(f"gate T={T} d={d} E={E} k={k} {dtype} seed={seed}")
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, d, generator=g).to(dtype)
    wg = (torch.randn(E, d, generator=g) * 0.02).to(dtype)
    bg = (torch.randn(E, generator=g) * 0.02).to(dtype)
    idx_ref, score_ref, logits_ref = O.naive_gate(x, wg, bg, k)
    idx, score, logits = ops.gate_topk_softmax(dev(x), dev(wg), dev(bg), k, return_logits=True)
    torch.cuda.synchronize()
    assert torch.equal(logits.cpu(), logits_ref), "logits differ bitwise"
    assert torch.equal(idx.cpu(), idx_ref), "expert choice differs"
    assert (score.cpu().float() - score_ref.float()).abs().max() <= 1e-3
    assert torch.allclose(score.float().sum(-1).cpu(), torch.ones(T), atol=2e-3)


_GATE_CASES = {}


def _gate_case(T, d, E, k):
    key = (T, d, E, k)
    if key not in _GATE_CASES:
        g = torch.Generator().manual_seed(T + E)
        x = torch.randn(T, d, generator=g).half()
        wg = (torch.randn(E, d, generator=g) * 0.05).half()
        bg = (torch.randn(E, generator=g) * 0.05).half()
        _GATE_CASES[key] = (x, wg, bg) + tuple(O.naive_gate(x, wg, bg, k))
    return _GATE_CASES[key]


@pytest.mark.parametrize("slots,waves,stream", [(0, 8, -1), (0, 8, 0), (1, 2, 0), (2, 1, 0), (4, 8, 0), (1, 8, 0),
                                                (0, 8, 1), (1, 8, 1), (2, 8, 1), (4, 8, 1)])
@pytest.mark.parametrize("T,d,E,k", [(5000, 512, 8, 2), (9000, 256, 32, 1), (40001, 128, 16, 2),
                                     (33000, 768, 32, 1), (300, 4096, 12, 2), (2100, 2048, 70, 4),
                                     (77, 8192, 8, 2), (130, 520, 40, 3)])
def test_gate_launch_shapes(slots, waves, stream, T, d, E, k):
    """Every way the gate spreads a problem over the machine gives the oracle's bits: 1, 2
    or 4 parts of K per wavefront (fewer tokens per workgroup), 1 to 8 wavefronts per
    workgroup (several rounds of parts when K is long) or every wavefront alone through all
    of K, both tile widths (16 and 32 experts, 1 to 3 tiles), a ragged last token group, a
    short last part."""
    from ccfuser_amd import ops
    _say(f"gate slots={slots} waves={waves} stream={stream} T={T} d={d} E={E} k={k}")
    x, wg, bg, idx_ref, score_ref, logits_ref = _gate_case(T, d, E, k)
    ops.set_option("gate_slots", slots)
    ops.set_option("gate_waves", waves)
    ops.set_option("gate_stream", stream)
    try:
        idx, score, logits = ops.gate_topk_softmax(dev(x), dev(wg), dev(bg), k, return_logits=True)
        torch.cuda.synchronize()
    finally:
        ops.set_option("gate_slots", 0)
        ops.set_option("gate_waves", 8)
        ops.set_option("gate_stream", -1)
    assert torch.equal(logits.cpu(), logits_ref), "logits differ bitwise"
    assert torch.equal(idx.cpu(), idx_ref), "expert choice differs"
    assert (score.cpu().float() - score_ref.float()).abs().max() <= 1e-3


@pytest.mark.parametrize("stream", [0, 1])
@pytest.mark.parametrize("E,k", [(32, 2), (8, 1), (70, 3)])
def test_gate_logits_that_are_nothing_but_rounding_error(E, k, stream):
    """Inputs whose exact logits are zero: inside every part of 128 the second half of the
    products repeats the first half, permuted and negated (weights are powers of two, so
    every product is exact).  What is left is the rounding error of the fp32 chain, which
    depends on the order of the additions and on every rounding being to nearest even;
    scaled into fp16's range it must equal the oracle's bit for bit."""
    from ccfuser_amd import ops
    _say(f"gate rounding residue E={E} k={k} stream={stream}")
    g = torch.Generator().manual_seed(E)
    T, d = 300, 512
    x = torch.empty(T, d)
    w = torch.empty(E, d)
    for p0 in range(0, d, 128):
        perm = torch.randperm(64, generator=g)
        xa = torch.randn(T, 64, generator=g) * 2.0 ** torch.randint(0, 7, (T, 64), generator=g)
        wa = 2.0 ** torch.randint(2, 8, (E, 64), generator=g) * (torch.randint(0, 2, (E, 64), generator=g) * 2 - 1)
        x[:, p0:p0 + 64] = xa
        w[:, p0:p0 + 64] = wa
        x[:, p0 + 64:p0 + 128] = -xa[:, perm]
        w[:, p0 + 64:p0 + 128] = wa[:, perm]
    x, w = x.half(), w.half()
    assert torch.equal((x.double() @ w.double().t()), torch.zeros(T, E, dtype=torch.float64))
    idx_ref, score_ref, logits_ref = O.naive_gate(x, w, None, k)
    assert (logits_ref != 0).float().mean() > 0.5          # the residue is there
    ops.set_option("gate_stream", stream)
    try:
        idx, score, logits = ops.gate_topk_softmax(dev(x), dev(w), None, k, return_logits=True)
        torch.cuda.synchronize()
    finally:
        ops.set_option("gate_stream", -1)
    assert torch.equal(logits.cpu(), logits_ref), "rounding residue differs"
    assert torch.equal(idx.cpu(), idx_ref)


def test_gate_random_shapes():
    """Thirty seeded random shapes (1..2500 tokens, K a multiple of 8 up to 3000, 1..140
    experts, any top-k the shape allows) under random launch shapes, all bitwise."""
    from ccfuser_amd import ops
    import random
    rng = random.Random(20240607)
    try:
        for case in range(30):
            T = rng.choice([1, 2, 15, 16, 17, 63, 64, 65, rng.randint(66, 2500)])
            d = 8 * rng.randint(1, 375)
            E = rng.choice([1, 2, 3, 8, 15, 16, 17, 31, 32, 33, 64, rng.randint(65, 140)])
            k = rng.randint(1, min(E, 8))
            slots, waves = rng.choice([0, 1, 2, 4]), rng.randint(1, 8)
            stream = (case * 7 + 1) % 3 - 1
            _say(f"gate random case {case}: T={T} d={d} E={E} k={k} slots={slots} waves={waves} stream={stream}")
            g = torch.Generator().manual_seed(case)
            x = (torch.randn(T, d, generator=g) * 2.0 ** rng.randint(-3, 3)).half()
            wg = (torch.randn(E, d, generator=g) * 0.05).half()
            bg = (torch.randn(E, generator=g) * 0.05).half() if case % 3 else None
            idx_ref, score_ref, logits_ref = O.naive_gate(x, wg, bg, k)
            ops.set_option("gate_slots", slots)
            ops.set_option("gate_waves", waves)
            ops.set_option("gate_stream", stream)
            idx, score, logits = ops.gate_topk_softmax(dev(x), dev(wg), None if bg is None else dev(bg), k,
                                                       return_logits=True)
            torch.cuda.synchronize()
            assert torch.equal(logits.cpu(), logits_ref), f"case {case}: logits differ bitwise"
            assert torch.equal(idx.cpu(), idx_ref), f"case {case}: expert choice differs"
            assert (score.cpu().float() - score_ref.float()).abs().max() <= 1e-3
    finally:
        ops.set_option("gate_slots", 0)
        ops.set_option("gate_waves", 8)
        ops.set_option("gate_stream", -1)


@pytest.mark.parametrize("tile", [32, 16])
def test_mfma_chain_equals_a_chain_of_fused_multiply_adds(tile):
    """What the fp16 gate rests on: a chain of K = 1 fp32 MFMAs gives, per output element,
    the bits of acc = fma(a, b, acc) step by step (round to nearest even), on operands that
    fp16 can hold with exponents spread over 16 binades, so that sums cancel and every
    rounding matters.  Products of such operands are exact in fp32, which lets numpy replay
    the chain with a multiply and an add.  Also pins which accumulator register of which lane
    holds which element, as the gate kernel assumes it."""
    import numpy as np
    from ccfuser_amd import _lib
    _say(f"mfma chain probe tile={tile}")
    steps, blocks, regs = 768, 64 // tile, 32 if tile == 32 else 16
    g = torch.Generator().manual_seed(tile)

    def operands():
        v = torch.randn(steps, 64, generator=g) * 2.0 ** torch.randint(-8, 9, (steps, 64), generator=g).float()
        return v.half().float()                                      # representable in fp16

    for trial in range(6):
        a, b = operands(), operands()
        out = torch.full((regs, 64), float("nan"), dtype=torch.float32, device="cuda")
        a_dev, b_dev = a.cuda(), b.cuda()
        assert _lib.probe_lib().ccf_probe_mfma_chain(a_dev.data_ptr(), b_dev.data_ptr(), steps, tile,
                                                     out.data_ptr(), None) == 0
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        an, bn = a.numpy(), b.numpy()
        for blk in range(blocks):
            ab, bb = an[:, blk * tile:(blk + 1) * tile], bn[:, blk * tile:(blk + 1) * tile]
            acc = np.zeros((tile, tile), np.float32)
            for s_ in range(steps):
                acc = acc + ab[s_][:, None] * bb[s_][None, :]
            for v in range(regs):
                if (v >> 4 if tile == 32 else v >> 2) != blk:
                    continue
                for lane in range(64):
                    if tile == 32:
                        row, col = 8 * ((v & 15) >> 2) + 4 * (lane >> 5) + (v & 3), lane & 31
                    else:
                        row, col = 4 * (lane >> 4) + (v & 3), lane & 15
                    assert got[v, lane] == acc[row, col], (trial, blk, v, lane)


def test_gate_ties_go_to_lower_expert():
    from ccfuser_amd import ops
    x = torch.ones(8, 64, dtype=torch.float16)
    wg = torch.zeros(6, 64, dtype=torch.float16)
    wg[1] = 0.5
    wg[4] = 0.5          # experts 1 and 4 tie for first, 0,2,3,5 tie for the rest
    idx, score = ops.gate_topk_softmax(dev(x), dev(wg), None, 3)
    assert idx.cpu().tolist() == [[1, 4, 0]] * 8
    ref_idx, ref_score, _ = O.naive_gate(x, wg, None, 3)
    assert torch.equal(idx.cpu(), ref_idx)
    assert (score.cpu().float() - ref_score.float()).abs().max() <= 1e-3


# --------------------------------------------------------------- routing
@pytest.mark.parametrize("n,E,k,cap,seed", [
    (1, 4, 1, -1, 0), (63, 4, 1, -1, 1), (1024, 8, 2, -1, 2), (1025, 8, 1, -1, 3),
    (16384, 8, 2, 2560, 4), (32768, 32, 1, -1, 5), (5000, 70, 2, 40, 6), (4096, 1000, 2, -1, 7),
    (3000, 3, 1, 0, 8),
    (70000, 600, 2, -1, 9),        # a table of counts too large for the pos launch to sum: the scan launch runs
    (40000, 900, 1, 30, 10),       # the same with a capacity
])
def test_route_bit_exact(n, E, k, cap, seed):
    from ccfuser_amd import ops
    _say(f"route n={n} E={E} k={k} cap={cap} seed={seed}")
    g = torch.Generator().manual_seed(seed)
    # skewed ids with some already-dropped entries
    p = torch.rand(E, generator=g) ** 3 + 1e-3
    idx = torch.multinomial(p / p.sum(), n, replacement=True, generator=g)
    idx[torch.rand(n, generator=g) < 0.05] = -1
    kept_ref = O.limit_by_capacity(idx, E, cap)
    counts_ref = O.expert_count(kept_ref, E)
    pos_ref, off_ref = O.assign_pos(kept_ref, E)
    r = ops.route(dev(idx), E, k, cap)
    torch.cuda.synchronize()
    R = int(off_ref[-1])
    assert torch.equal(r["counts"].cpu(), counts_ref)
    assert torch.equal(r["offsets"].cpu(), off_ref)
    assert torch.equal(r["idx_kept"].cpu(), kept_ref)
    assert torch.equal(r["pos"].cpu()[:R], pos_ref)
    assert torch.equal(r["src_row"].cpu()[:R].long(), pos_ref // k)
    assert torch.equal(r["dst_row"].cpu()[:R].long(), pos_ref)
    assert torch.equal(r["inv_pos"].cpu(), O.inverse_pos(pos_ref, n))


def test_expert_count_and_assign_pos_mirror_the_reference_calls():
    """functions.py:85-103 call sequence through the mirrored extension functions."""
    from ccfuser_amd import mix_moe_hip
    g = torch.Generator().manual_seed(11)
    E, n = 16, 8192
    gate = torch.randint(0, E, (n // 2, 2), generator=g)
    gate[torch.rand(n // 2, 2, generator=g) < 0.1] = -1
    cnt = torch.zeros(E, dtype=torch.int32, device="cuda")
    mix_moe_hip.expert_count(dev(gate), cnt)
    mix_moe_hip.expert_count(dev(gate), cnt)            # accumulates
    ref = O.expert_count(gate, E)
    assert torch.equal(cnt.cpu(), 2 * ref)
    lec_cum = torch.cumsum(ref.long(), 0).int().cuda()
    pos = torch.empty(int(lec_cum[-1]), dtype=torch.long, device="cuda")
    mix_moe_hip.assign_pos(lec_cum, dev(gate), pos)
    pos_ref, off_ref = O.assign_pos(gate, E)
    assert torch.equal(pos.cpu(), pos_ref)
    assert torch.equal(lec_cum.cpu(), off_ref[:-1])      # cum_count ends at the segment starts


def _count_cases():
    import os
    import numpy as np
    g = torch.Generator().manual_seed(5)
    table = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_all_expert_count.npy"))
    cases = [row.tolist() for row in table]                       # the reference's skewed 4x64 table
    cases += [[0, 0, 0], [63], [64], [65], [1, 64, 0, 128, 130, 5], [64] * 7, [3] * 9,
              [700, 0, 1, 0, 64, 63, 1000],                       # more full blocks than tails
              [1] * 40 + [128],                                   # more tails than full blocks
              torch.randint(0, 300, (1000,), generator=g).tolist(),
              torch.randint(0, 3, (1024,), generator=g).tolist()]
    return cases


@pytest.mark.parametrize("case", range(15))
def test_plan_blocks_matches_divide_into_block(case):
    """Device block planner against the oracle's divide_into_block, every array bit-exact."""
    from ccfuser_amd import ops
    counts = _count_cases()[case]
    _say(f"plan_blocks case={case} E={len(counts)} rows={sum(counts)}")
    ref = O.divide_into_block(counts, 64)
    got = ops.plan_blocks(torch.tensor(counts, dtype=torch.int32, device="cuda"), sum(counts), 64)
    total, remote = got["block_nums"].tolist()
    assert (total, remote) == (ref["total_block_num"], ref["remote_block_num"])
    for k in ("expert_ids", "ranks", "lens", "start_addrs", "expert_block_ids"):
        assert got[k][:total].tolist() == ref[k], k
        assert got[k].numel() >= total
    assert got["expert_block_id_idxs"].tolist() == ref["expert_block_id_idxs"]
    got32 = ops.plan_blocks(torch.tensor(counts, dtype=torch.int32, device="cuda"), sum(counts), 32, rank=3)
    ref32 = O.divide_into_block(counts, 32)
    t32 = int(got32["block_nums"][0])
    assert t32 == ref32["total_block_num"]
    assert got32["start_addrs"][:t32].tolist() == ref32["start_addrs"]
    assert got32["ranks"][:t32].tolist() == [3] * t32


@pytest.mark.parametrize("n_seg,E,seed", [(64, 8, 0), (1, 1, 1), (700, 37, 2), (3000, 200, 3), (5, 1024, 4)])
def test_segments_to_rows(n_seg, E, seed):
    """(start, len, expert) triples -> counts, offsets and the row list grouped by expert, rows of
    an expert in the order of the triple list and then row order (what the reference's kernels do
    per block through start_addrs / lens / expert_ids, mix_gemm.cu:296-301).  Triples with no
    rows or with an expert outside 0..E-1 are skipped.  Many triples, empty experts, bit for bit."""
    from ccfuser_amd import ops
    import numpy as np
    _say(f"segments_to_rows n_seg={n_seg} E={E} seed={seed}")
    rng = np.random.default_rng(seed)
    seg_len = rng.integers(0, 40, n_seg).astype(np.int32)
    seg_len[rng.random(n_seg) < 0.1] = 0
    seg_expert = rng.integers(0, E, n_seg).astype(np.int32)
    bad = rng.random(n_seg) < 0.05
    seg_expert[bad] = rng.choice([-1, E, E + 5], bad.sum())
    total = int(seg_len.sum())
    seg_start = (np.cumsum(seg_len) - seg_len).astype(np.int32)
    order = rng.permutation(n_seg)                       # the list is in no particular order
    seg_start, seg_len, seg_expert = seg_start[order], seg_len[order], seg_expert[order]
    counts_ref = np.zeros(E, dtype=np.int32)
    per = [[] for _ in range(E)]
    for st, ln, e in zip(seg_start, seg_len, seg_expert):
        if 0 <= e < E and ln > 0:
            counts_ref[e] += ln
            per[e].extend(range(st, st + ln))
    offsets_ref = np.concatenate([[0], np.cumsum(counts_ref)]).astype(np.int32)
    rows_ref = np.array([r for e in range(E) for r in per[e]], dtype=np.int32)
    counts, offsets, rows = ops.segments_to_rows(dev(torch.from_numpy(seg_start)), dev(torch.from_numpy(seg_len)),
                                                 dev(torch.from_numpy(seg_expert)), E, max(total, 1))
    torch.cuda.synchronize()
    assert np.array_equal(counts.cpu().numpy(), counts_ref)
    assert np.array_equal(offsets.cpu().numpy(), offsets_ref)
    assert np.array_equal(rows.cpu().numpy()[:len(rows_ref)], rows_ref)


# ------------------------------------------------- row moves and combine
def test_local_scatter_gather_with_reference_pos_vector():
    """The reference's own scatter check: index_select(input, 0, pos) with its
    pos.pt (csrc/test.cpp:405-449), M=4096 rows, N=1024."""
    import numpy as np, os
    from ccfuser_amd import ops
    pos = torch.from_numpy(np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_pos_div2.npy")))
    g = torch.Generator().manual_seed(0)
    x = torch.randn(4096, 1024, generator=g).half()
    out = ops.local_scatter(dev(x), dev(pos.int()))
    assert torch.equal(out.cpu(), torch.index_select(x, 0, pos))
    # gather is the inverse move on a permutation
    perm = torch.randperm(4096, generator=g)
    back = ops.local_gather(dev(x), dev(perm.int()), 4096)
    ref = torch.zeros_like(x)
    ref.index_copy_(0, perm, x)
    assert torch.equal(back.cpu(), ref)


@pytest.mark.parametrize("T,k,d", [(100, 1, 64), (257, 2, 1024), (64, 4, 256)])
def test_combine(T, k, d):
    from ccfuser_amd import ops
    g = torch.Generator().manual_seed(T)
    y = torch.randn(T * k, d, generator=g).half()
    s = torch.softmax(torch.randn(T, k, generator=g), -1).half()
    inv = torch.arange(T * k, dtype=torch.int32)
    inv[torch.rand(T * k, generator=g) < 0.2] = -1
    y_masked = y.clone()
    y_masked[inv < 0] = 0
    ref = O.combine(y_masked.float(), s.float(), k)
    out = ops.combine(dev(y), dev(s), k, dev(inv))
    assert (out.cpu().float() - ref).abs().max() <= 2e-3 * max(1.0, float(ref.abs().max()))
    if k == 1:      # closed form: out = score * y
        assert torch.equal(ops.combine(dev(y), dev(torch.ones(T, 1).half()), 1).cpu(), y)


# ------------------------------------------------------------ expert FFN
def _ffn_case(R, d, f, E, seed, skew=False):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(R, d, generator=g).half()
    w1 = (torch.randn(E, f, d, generator=g) * 0.02).half()
    b1 = (torch.randn(E, f, generator=g) * 0.02).half()
    w2 = (torch.randn(E, d, f, generator=g) * 0.02).half()
    b2 = (torch.randn(E, d, generator=g) * 0.02).half()
    if skew:
        p = torch.rand(E, generator=g) ** 4 + 1e-4
    else:
        p = torch.ones(E)
    e_of_row = torch.multinomial(p / p.sum(), R, replacement=True, generator=g)
    return x, w1, b1, w2, b2, e_of_row


@pytest.mark.parametrize("variant", [0, 1, 2, 3])
@pytest.mark.parametrize("R,d,f,E,skew,seed", [
    (512, 256, 1024, 4, False, 0),
    (700, 768, 3072, 32, True, 1),
    (1000, 1024, 512, 3, True, 2),
    (64, 64, 64, 1, False, 3),
    (1, 128, 192, 2, False, 4),
])
def test_ffn_stages(variant, R, d, f, E, skew, seed):
    from ccfuser_amd import ops
    _say(f"ffn variant={variant} R={R} d={d} f={f} E={E} skew={skew}")
    ops.set_option("gemm_variant", variant)
    try:
        x, w1, b1, w2, b2, e_of_row = _ffn_case(R, d, f, E, seed, skew)
        # rows arrive in token order; route them as a top-1 layer would
        pos_ref, off_ref = O.assign_pos(e_of_row, E)
        buf = O.local_scatter(x, pos_ref, 1)
        r = ops.route(dev(e_of_row), E, 1)
        h = ops.ffn1(dev(x), r["src_row"], r["offsets"], R, dev(w1), dev(b1), gelu=True)
        torch.cuda.synchronize()
        # FFN1 + GELU against fp32
        off = off_ref.tolist()
        h_ref = torch.zeros(R, f)
        for e in range(E):
            lo, hi = off[e], off[e + 1]
            if hi > lo:
                h_ref[lo:hi] = O.gelu_exact(buf[lo:hi].float() @ w1[e].float().t() + b1[e].float())
        assert O.max_abs_err(h.cpu(), h_ref) <= MAX_ABS
        assert O.mean_rel_err(h.cpu(), h_ref) <= MEAN_REL
        # FFN2 with the un-permute fused
        y = torch.zeros(R, d, dtype=torch.float16, device="cuda")
        ops.ffn2(h, r["dst_row"], r["offsets"], R, dev(w2), dev(b2), y)
        torch.cuda.synchronize()
        y_sorted = O.expert_ffn(buf, off_ref, w1, b1, w2, b2)
        y_ref = O.unpermute(y_sorted, pos_ref, R)
        assert O.max_abs_err(y.cpu(), y_ref) <= MAX_ABS
        assert O.mean_rel_err(y.cpu(), y_ref) <= MEAN_REL
    finally:
        ops.set_option("gemm_variant", -1)


@pytest.mark.parametrize("R,d,f,E,skew,seed", [
    (9000, 1024, 2048, 8, False, 50),          # several rounds of tiles per workgroup, ragged last tiles
    (3000, 768, 1536, 32, True, 51),           # many partly filled tiles (the eight-wavefront form computes their padding)
    (700, 256, 320, 5, False, 52),             # four K tiles, N no multiple of 256
])
def test_eight_wavefront_kernel_gives_the_four_wavefront_bits(R, d, f, E, skew, seed):
    """The persistent kernel with eight wavefronts per workgroup (one register buffer of token
    fragments, refilled row block by row block) adds over K in the same order with the same
    instruction as the four-wavefront form: both GEMMs must agree bit for bit."""
    from ccfuser_amd import ops
    x, w1, b1, w2, b2, e_of_row = _ffn_case(R, d, f, E, seed, skew)
    r = ops.route(dev(e_of_row), E, 1)
    _say(f"8 vs 4 wavefronts R={R} d={d} f={f} E={E} counts={r['counts'].tolist()[:10]}")
    res = {}
    ops.set_option("split_tail", 0)
    try:
        for variant in (2, 3):
            ops.set_option("gemm_variant", variant)
            h = ops.ffn1(dev(x), r["src_row"], r["offsets"], R, dev(w1), dev(b1), gelu=True)
            y = torch.zeros(R, d, dtype=torch.float16, device="cuda")
            ops.ffn2(h, r["dst_row"], r["offsets"], R, dev(w2), dev(b2), y)
            torch.cuda.synchronize()
            res[variant] = (h.cpu(), y.cpu())
    finally:
        ops.set_option("gemm_variant", -1)
        ops.set_option("split_tail", 1)
    assert torch.isfinite(res[3][0].float()).all() and res[3][0].abs().sum() > 0
    assert torch.equal(res[2][0], res[3][0]), "first GEMM"
    assert torch.equal(res[2][1], res[3][1]), "second GEMM"


def test_ffn_special_cases():
    """Closed forms: zero weights give the bias path; a single expert is a dense MLP."""
    from ccfuser_amd import ops
    R, d, f = 300, 128, 256
    g = torch.Generator().manual_seed(5)
    x = torch.randn(R, d, generator=g).half()
    b1 = (torch.randn(1, f, generator=g)).half()
    b2 = (torch.randn(1, d, generator=g)).half()
    w1 = torch.zeros(1, f, d).half()
    w2 = torch.zeros(1, d, f).half()
    off = torch.tensor([0, R], dtype=torch.int32).cuda()
    h = ops.ffn1(dev(x), None, off, R, dev(w1), dev(b1), gelu=True)
    ref_h = O.gelu_exact(b1.float()).half().expand(R, f)
    assert (h.cpu().float() - ref_h.float()).abs().max() <= 2e-3
    y = torch.zeros(R, d, dtype=torch.float16, device="cuda")
    ops.ffn2(h, None, off, R, dev(w2), dev(b2), y)
    assert torch.equal(y.cpu(), b2.expand(R, d))
    # the GELU itself over [-8, 8] (zero weights: h = gelu(b1)); every fp16 value of the
    # sweep within one fp16 rounding step of the exact erf form
    f2 = 4096
    sweep = torch.linspace(-8.0, 8.0, f2).half().reshape(1, f2)
    h2 = ops.ffn1(dev(x), None, off, R, dev(torch.zeros(1, f2, d).half()), dev(sweep), gelu=True)
    exact = O.gelu_exact(sweep.float()).reshape(-1)
    got = h2[0].cpu().float()
    step = torch.maximum(exact.abs() * 2.0 ** -10, torch.tensor(6.2e-5))
    assert bool(((got - exact).abs() <= step).all()), float(((got - exact).abs() / step).max())
    assert torch.equal(h2[0], h2[R - 1])
    # pre-activation output
    w1 = (torch.randn(1, f, d, generator=g) * 0.05).half()
    pre = ops.ffn1(dev(x), None, off, R, dev(w1), dev(b1), gelu=False)
    ref = x.float() @ w1[0].float().t() + b1.float()
    assert O.max_abs_err(pre.cpu(), ref) <= MAX_ABS


@pytest.mark.parametrize("inside", [1, 0])
def test_split_k_tail_at_its_default_threshold(inside):
    """K = 4096 is where the split of the last round switches on by itself: 36 M tiles x 16 N
    tiles = 2.25 rounds of 256 workgroups, in both GEMMs, whole outputs against fp32.  The parts
    run inside the persistent launch (each workgroup one, behind its tiles) or as a launch of
    their own."""
    from ccfuser_amd import ops
    ops.set_option("split_inside", inside)
    g = torch.Generator().manual_seed(22)
    R, d, f, E = 8192, 4096, 4096, 6
    x = torch.randn(R, d, generator=g).half()
    w1 = (torch.randn(E, f, d, generator=g) * 0.02).half()
    b1 = (torch.randn(E, f, generator=g) * 0.05).half()
    w2 = (torch.randn(E, d, f, generator=g) * 0.02).half()
    b2 = (torch.randn(E, d, generator=g) * 0.05).half()
    idx = torch.randint(0, E, (R,), generator=g)
    r = ops.route(dev(idx), E, 1, -1)
    off, pos = r["offsets"].cpu(), r["pos"].cpu()
    _say(f"split-K tail by default R={R} d={d} f={f} E={E} counts={r['counts'].tolist()}")
    out = {}
    ops.set_option("skinny", 0)               # every row in 256-row tiles: the tile count this test is built on
    for mode in (1, 0):
        ops.set_option("split_tail", mode)
        try:
            h = ops.ffn1(dev(x), r["src_row"], r["offsets"], R, dev(w1), dev(b1), gelu=True)
            y = torch.zeros(R, d, dtype=torch.float16, device="cuda")
            ops.ffn2(h, r["dst_row"], r["offsets"], R, dev(w2), dev(b2), y)
            out[mode] = (h.cpu(), y.cpu())
        finally:
            ops.set_option("split_tail", 1)
    ops.set_option("skinny", 1)
    buf = x[pos].float()
    h_ref = torch.zeros(R, f)
    y_ref = torch.zeros(R, d)
    hq = out[1][0].float()
    for e in range(E):
        lo, hi = int(off[e]), int(off[e + 1])
        h_ref[lo:hi] = O.gelu_exact(buf[lo:hi] @ w1[e].float().t() + b1[e].float())
        y_ref[pos[lo:hi]] = hq[lo:hi] @ w2[e].float().t() + b2[e].float()
    assert O.max_abs_err(out[1][0], h_ref) <= MAX_ABS and O.mean_rel_err(out[1][0], h_ref) <= MEAN_REL
    assert O.max_abs_err(out[1][1], y_ref) <= MAX_ABS and O.mean_rel_err(out[1][1], y_ref) <= MEAN_REL
    # the split did run: bits differ from the unsplit kernels
    assert not torch.equal(out[1][0], out[0][0]) and not torch.equal(out[1][1], out[0][1])
    ops.set_option("split_inside", 1)


def test_split_k_tail_all_epilogues():
    """The last, partly filled round of tiles is cut along K and reduced by a separate kernel.
    By default that happens for K >= 4096 only; here it is forced on a small K so that the
    reduction's three epilogues (plain with row index and scale, GELU, GELU keeping the
    pre-activation) are compared with the oracle and with the unsplit kernels."""
    from ccfuser_amd import ops
    g = torch.Generator().manual_seed(21)
    R, d, f, E = 8192, 2048, 2048, 6           # 16+ M tiles x 8 N tiles: more tiles than workgroups, a ragged last round
    x = (torch.randn(R, d, generator=g)).half()
    w1 = (torch.randn(E, f, d, generator=g) * 0.05).half()
    b1 = (torch.randn(E, f, generator=g) * 0.05).half()
    w2 = (torch.randn(E, d, f, generator=g) * 0.02).half()
    b2 = (torch.randn(E, d, generator=g) * 0.05).half()
    idx = torch.randint(0, E, (R,), generator=g)
    r = ops.route(dev(idx), E, 1, -1)
    off = r["offsets"].cpu()
    pos = r["pos"].cpu()
    scale = (torch.rand(R, generator=g) + 0.5).half()
    _say(f"split-K tail R={R} d={d} f={f} E={E} counts={r['counts'].tolist()}")
    results = {}
    ops.set_option("skinny", 0)               # every row in 256-row tiles: the tile count this test is built on
    for mode in (0, 4, -4):                   # -4: as 4, the parts as a launch of their own
        ops.set_option("split_tail", abs(mode))
        ops.set_option("split_inside", 0 if mode < 0 else 1)
        try:
            h = ops.ffn1(dev(x), r["src_row"], r["offsets"], R, dev(w1), dev(b1), gelu=True)
            act, pre = ops.ffn1_keep(dev(x), r["src_row"], r["offsets"], R, dev(w1), dev(b1))
            y = torch.zeros(R, d, dtype=torch.float16, device="cuda")
            ops.ffn2(h, r["dst_row"], r["offsets"], R, dev(w2), dev(b2), y, row_scale=dev(scale))
            results[mode] = [t.cpu() for t in (h, act, pre, y)]
        finally:
            ops.set_option("split_tail", 1)
            ops.set_option("split_inside", 1)
    ops.set_option("skinny", 1)
    # the same parts and the same order of summation wherever they run
    assert all(torch.equal(a, b) for a, b in zip(results[4], results[-4]))
    buf = x[torch.div(pos, 1, rounding_mode="floor")].float()
    h_ref = torch.zeros(R, f)
    pre_ref = torch.zeros(R, f)
    for e in range(E):
        lo, hi = int(off[e]), int(off[e + 1])
        pre_ref[lo:hi] = buf[lo:hi] @ w1[e].float().t() + b1[e].float()
    h_ref = O.gelu_exact(pre_ref)
    for mode, (h, act, pre, y) in results.items():
        assert O.max_abs_err(h, h_ref) <= MAX_ABS and O.mean_rel_err(h, h_ref) <= MEAN_REL, mode
        assert torch.equal(h, act), mode
        assert O.max_abs_err(pre, pre_ref) <= MAX_ABS, mode
    y_ref = torch.zeros(R, d)
    hq = results[4][0].float()
    for e in range(E):
        lo, hi = int(off[e]), int(off[e + 1])
        y_ref[pos[lo:hi]] = (hq[lo:hi] @ w2[e].float().t() + b2[e].float()) * scale[lo:hi].float()[:, None]
    assert O.max_abs_err(results[4][3], y_ref) <= MAX_ABS and O.mean_rel_err(results[4][3], y_ref) <= MEAN_REL
    # split and unsplit differ only in summation order (and do differ: the split path ran)
    assert O.max_abs_err(results[4][3], results[0][3].float()) <= MAX_ABS
    assert O.max_abs_err(results[4][0], results[0][0].float()) <= MAX_ABS
    assert not torch.equal(results[4][3], results[0][3]) and not torch.equal(results[4][0], results[0][0])


# Forced cases are sized so that both GEMMs have at least as many worst-case tiles as the chip has
# CUs ((ceil(R / 256) + E) * ceil(N / 256) >= 256): only then does the persistent launch set
# workgroups aside for skinny tiles.  `expect`: which GEMMs must report skinny tiles actually run.
@pytest.mark.parametrize("R,d,f,E,skew,seed,mode,expect", [
    (8192, 4096, 4096, 6, False, 31, 1, ""),          # remainders of 56..122 rows: one or two skinny tiles each, if the plan wants them
    (8192 + 6 * 200, 4096, 4096, 6, False, 35, 1, ""),   # remainders of ~25 rows, long K: the plan's own choice
    (0, 256, 1024, 60, False, 32, -2, "1"),           # first GEMM with K = 256: four K tiles, the shortest the loop takes
    (2100, 1024, 2048, 70, True, 33, -1, "12"),       # most experts are nothing but a skinny tile, some are empty
    (1150, 512, 768, 3, False, 34, -3, ""),           # remainders of 127, 130 and 125 rows: none is skinny, nothing to do
    (15360, 1088, 832, 60, False, 36, -4, "12"),      # N no multiple of 256 in either GEMM (832, 1088)
    (8192, 4096, 4096, 6, False, 37, -5, "12"),       # as a launch of their own, cut along K: a workgroup's range inside one tile
    (0, 1536, 4160, 40, False, 38, -5, "12"),         # experts of 17..64 rows only: ranges of four tiles, N = 4160
    (8192, 4096, 4096, 6, False, 39, -6, "12"),       # cut along K inside the persistent launch, before / behind the 256-row tiles
    (0, 1536, 4160, 40, False, 40, -6, "12"),         # the same where most workgroups have no 256-row tile at all
    (20000, 2048, 2048, 12, False, 41, -6, "12"),     # several 256-row tiles per workgroup in front of / behind the ranges
])
def test_skinny_tiles(R, d, f, E, skew, seed, mode, expect):
    """Rows beyond an expert's full 256-row tiles (at most 64) run as 64-row tiles: in workgroups
    the plan sets aside beside the 256-row tiles (mode -n: forced, n workgroups per XCD) or as a
    launch of their own cut along K (mode -5: forced) or cut along K inside the persistent launch
    (mode -6: forced); mode 1 leaves the choice to the plan's cost model.  All three forward epilogues with that path on and off, each against fp32.
    Beside the 256-row tiles the path adds over K in the same order as they do and must agree
    bit for bit; cut along K it agrees within rounding.  The plan must report that skinny tiles
    really ran where the case is built for them."""
    from ccfuser_amd import ops
    counts = None
    if expect and not skew:
        # every expert: whole 256-row tiles (R / E rounded down to them) plus a remainder of 17..64 rows
        counts = torch.tensor([(R // E) // 256 * 256 + 17 + (e * 11) % 48 for e in range(E)])
        R = int(counts.sum())
    x, w1, b1, w2, b2, e_of_row = _ffn_case(R, d, f, E, seed, skew)
    g = torch.Generator().manual_seed(seed)
    if counts is not None:
        e_of_row = torch.repeat_interleave(torch.arange(E), counts)[torch.randperm(R, generator=g)]
    scale = (torch.rand(R, generator=g) + 0.5).half()
    r = ops.route(dev(e_of_row), E, 1)
    off, pos = r["offsets"].cpu().tolist(), r["pos"].cpu()
    rem = r["counts"].cpu() % 256
    _say(f"skinny mode={mode} R={R} d={d} f={f} E={E} remainders={rem.tolist()[:12]}")
    ws = ops.ffn_workspace(R, E, d, f, dev(x))
    res, info = {}, {}
    for m in (mode, 0):
        ops.set_option("skinny", m)
        # beside the 256-row tiles: keep those unsplit, the comparison is about the skinny path;
        # a launch of their own needs the split kernels launched (every K tile count allowed)
        ops.set_option("split_tail", 2 if mode <= -5 else 0)
        ops.set_option("skinny_tail", 1 if mode == -5 else 0)   # the launch of their own is off by default
        try:
            h = ops.ffn1(dev(x), r["src_row"], r["offsets"], R, dev(w1), dev(b1), gelu=True, workspace=ws)
            info[m, 1] = ops.ffn_plan_info(ws, R, E, d, f, 1)
            act, pre = ops.ffn1_keep(dev(x), r["src_row"], r["offsets"], R, dev(w1), dev(b1))
            y = torch.zeros(R, d, dtype=torch.float16, device="cuda")
            ops.ffn2(h, r["dst_row"], r["offsets"], R, dev(w2), dev(b2), y, row_scale=dev(scale), workspace=ws)
            info[m, 2] = ops.ffn_plan_info(ws, R, E, d, f, 2)
            torch.cuda.synchronize()
            res[m] = [t.cpu() for t in (h, act, pre, y)]
        finally:
            ops.set_option("skinny", 1)
            ops.set_option("split_tail", 1)
            ops.set_option("skinny_tail", 0)
    _say(f"  plan, first GEMM: {info[mode, 1]}")
    _say(f"  plan, second GEMM: {info[mode, 2]}")
    for which in (1, 2):
        i = info[mode, which]
        ran = i["skinny_tiles"] > 0 and (i["skinny_wgs_per_xcd"] > 0 or i["skinny_tail_steps"] != 0)
        if str(which) in expect:
            assert ran, (which, i)
            # steps > 0: as a launch of their own; < 0: inside the persistent launch
            assert (i["skinny_tail_steps"] > 0) == (mode == -5) and (i["skinny_tail_steps"] < 0) == (mode == -6), i
            assert i["skinny_wgs_per_xcd"] == (-mode if mode > -5 else 0), i
        if mode < 0:
            assert info[0, which]["skinny_tiles"] == 0
    buf = x[pos].float()
    pre_ref = torch.zeros(R, f)
    for e in range(E):
        lo, hi = off[e], off[e + 1]
        if hi > lo:
            pre_ref[lo:hi] = buf[lo:hi] @ w1[e].float().t() + b1[e].float()
    h_ref = O.gelu_exact(pre_ref)
    for m, (h, act, pre, y) in res.items():
        assert O.max_abs_err(h, h_ref) <= MAX_ABS and O.mean_rel_err(h, h_ref) <= MEAN_REL, m
        assert torch.equal(h, act), m
        assert O.max_abs_err(pre, pre_ref) <= MAX_ABS, m
        y_ref = torch.zeros(R, d)
        hq = h.float()
        for e in range(E):
            lo, hi = off[e], off[e + 1]
            if hi > lo:
                y_ref[pos[lo:hi]] = (hq[lo:hi] @ w2[e].float().t() + b2[e].float()) * scale[lo:hi].float()[:, None]
        assert O.max_abs_err(y, y_ref) <= MAX_ABS and O.mean_rel_err(y, y_ref) <= MEAN_REL, m
    same = [torch.equal(a, b) for a, b in zip(res[mode], res[0])]
    _say(f"  skinny on/off bitwise equal (h, act, pre, y): {same}")
    cut = any(info[mode, which]["skinny_tail_steps"] != 0 for which in (1, 2))   # the plan's own choice may be a K cut too
    if mode <= -5 or cut:
        # another summation order: close, and not identical where skinny tiles ran
        for a, b in zip(res[mode], res[0]):
            assert O.max_abs_err(a, b.float()) <= MAX_ABS
        assert not all(same)
    else:
        assert all(same)


def test_mfma_probe_runs_and_counts_its_flop():
    """ccf_probe_mfma: the MFMA-only loop bench.py times for its measured ceiling.  With zero
    operands every sum it leaves is zero; the flop count is the closed form."""
    import ctypes as C
    from ccfuser_amd import _lib
    probe = _lib.probe_lib()
    wgs, iters = 16, 10
    out = torch.full((wgs * 256,), 7.0, dtype=torch.float32, device="cuda")
    flop = C.c_double()
    for const in (1, 0):
        assert probe.ccf_probe_mfma(wgs, iters, const, out.data_ptr(), C.byref(flop), None) == 0
        torch.cuda.synchronize()
        assert flop.value == wgs * 4 * iters * 64 * 16 * 16 * 32 * 2
        assert bool(torch.isfinite(out).all())
        if const:
            assert not out.any()
    assert probe.ccf_probe_mfma(0, iters, 1, out.data_ptr(), C.byref(flop), None) == 1
