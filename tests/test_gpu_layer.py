"""GPU parity of the whole layer (fused C-ABI call and the mirrored Python API)
against the CPU oracle, on the named workloads at reduced row counts, plus
size-independent properties at full size."""
import os

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_REL = 2e-2, 1e-3
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _say(msg):
    print(msg, flush=True)


def _cuda(wl, *names):
    return [wl.tensors[n].cuda() for n in names]


def _check_layer(wl, out, routing, ref):
    R = int(ref["offsets"][-1])
    assert torch.equal(routing["idx"].cpu().view(-1), ref["idx_kept"].view(-1)), "expert choice"
    assert torch.equal(routing["counts"].cpu(), ref["counts"])
    assert torch.equal(routing["offsets"].cpu(), ref["offsets"])
    assert torch.equal(routing["pos"].cpu()[:R], ref["pos"])
    assert (routing["score"].cpu().float() - ref["score"].float()).abs().max() <= 1e-3
    ma, mr = O.max_abs_err(out.cpu(), ref["out"]), O.mean_rel_err(out.cpu(), ref["out"])
    _say(f"  {wl.name}: R={R} max_abs={ma:.3e} mean_rel={mr:.3e}")
    assert ma <= MAX_ABS and mr <= MEAN_REL


@pytest.mark.parametrize("name,rows", [
    ("c1_tiny", None),          # 512 tokens, run in fp16 on the GPU (the reference's GPU path is fp16 only)
    ("c2_gshard", 1024),        # capacity 1.25 with drops
    ("c3_mixtral", 256),        # d=4096, f=14336
    ("c5_skewed", 2048),        # 32 experts, Zipf loads, tiny experts
])
def test_fused_layer_matches_oracle(workloads, name, rows):
    from ccfuser_amd import ops
    wl = workloads(name, rows)
    _say(f"layer {name} rows={wl.tokens}")
    t = {k: (v.half() if v.is_floating_point() else v) for k, v in wl.tensors.items()}
    ref = O.moe_layer_forward(t["x"], t["wg"], t["bg"], t["w1"], t["b1"], t["w2"], t["b2"],
                              wl.top_k, capacity=wl.capacity)
    args = [t[n].cuda() for n in ("x", "wg", "bg", "w1", "b1", "w2", "b2")]
    out, routing = ops.moe_forward(*args, wl.top_k, wl.capacity, return_routing=True)
    torch.cuda.synchronize()
    _check_layer(wl, out, routing, ref)
    # determinism: a second call gives the same bits
    out2 = ops.moe_forward(*args, wl.top_k, wl.capacity)
    assert torch.equal(out, out2)


def test_golden_layer_fixture():
    """The committed small case: routing bit-exact, output within tolerance."""
    from ccfuser_amd import ops
    z = np.load(os.path.join(GOLDEN, "layer_small.npz"))
    t = {k: torch.from_numpy(z[k]) for k in ("x", "wg", "bg", "w1", "b1", "w2", "b2")}
    k, cap = int(z["top_k"]), int(z["capacity"])
    out, r = ops.moe_forward(*[t[n].cuda() for n in ("x", "wg", "bg", "w1", "b1", "w2", "b2")],
                             k, cap, return_routing=True)
    R = int(z["offsets"][-1])
    assert np.array_equal(r["idx"].cpu().numpy().reshape(-1), z["idx_kept"].reshape(-1))
    assert np.array_equal(r["counts"].cpu().numpy(), z["counts"])
    assert np.array_equal(r["offsets"].cpu().numpy(), z["offsets"])
    assert np.array_equal(r["pos"].cpu().numpy()[:R], z["pos"])
    ref = torch.from_numpy(z["out"])
    assert O.max_abs_err(out.cpu(), ref) <= MAX_ABS and O.mean_rel_err(out.cpu(), ref) <= MEAN_REL


def test_mirrored_module_staged_equals_fused(workloads):
    """MixMOETransformerMLP through process_data + MixMOE.forward (the reference's
    call sequence) gives the same bits as the single fused call, and the async
    assignment path does too."""
    from ccfuser_amd.mix_moe import MixMOETransformerMLP
    wl = workloads("c2_gshard", 512)
    E, d, f, k = wl.num_expert, wl.d_model, wl.d_ffn, wl.top_k
    mlp = MixMOETransformerMLP("naive", {"num_local_expert": E, "hidden_size": f}, d, 0, 1,
                               total_batch_size=wl.tokens, top_k=k, capacity_factor=1.25).half().cuda()
    t = wl.tensors
    with torch.no_grad():
        mlp.gate.gate.weight.copy_(t["wg"]); mlp.gate.gate.bias.copy_(t["bg"])
        mlp.experts.htoh4.weight[:E].copy_(t["w1"]); mlp.experts.htoh4.bias[:E].copy_(t["b1"])
        mlp.experts.h4toh.weight[:E].copy_(t["w2"]); mlp.experts.h4toh.bias[:E].copy_(t["b2"])
    x = t["x"].cuda().view(4, -1, d)                       # [B, L, d] like a transformer block
    with torch.no_grad():                                  # with gradients wanted the staged path runs anyway
        fused = mlp(x)
        assert fused.shape == x.shape
        mlp.fused = False
        staged = mlp(x)
        assert torch.equal(fused, staged)
        mlp.async_expert_assignment(x)
        overlapped = mlp(x)
        assert torch.equal(fused, overlapped)
    ref = O.moe_layer_forward(t["x"], t["wg"], t["bg"], t["w1"], t["b1"], t["w2"], t["b2"], k,
                              capacity=mlp._capacity(wl.tokens))
    assert O.max_abs_err(fused.view(-1, d).cpu(), ref["out"]) <= MAX_ABS
    assert O.mean_rel_err(fused.view(-1, d).cpu(), ref["out"]) <= MEAN_REL
    # the reference's block arrays, produced on demand, tile every segment
    pos, score, infos = mlp.async_expert_assign.process_data(mlp.gate, x.view(-1, d), E, 1)
    # the gate leaves the reference's dummy loss (naive_gate.py:41): a zero on the input's device that takes a gradient
    assert mlp.gate.has_loss
    loss = mlp.gate.get_loss()
    assert loss.is_cuda and loss.requires_grad and loss.is_leaf and float(loss.detach()) == 0.0 and not mlp.gate.has_loss
    lens, starts, ids = (infos[n].cpu().tolist() for n in ("lens", "start_addrs", "expert_ids"))
    off = infos["offsets"].cpu().tolist()
    covered = sorted((s, s + l) for s, l in zip(starts, lens))
    assert covered[0][0] == 0 and covered[-1][1] == off[-1]
    assert all(a[1] == b[0] for a, b in zip(covered, covered[1:]))
    assert all(off[e] <= s and s + l <= off[e + 1] and l <= 64 for s, l, e in zip(starts, lens, ids))
    mlp.close()


def test_extension_class_with_reference_block_arrays(workloads):
    """mix_moe_cuda.MixMOE.first_gemm_forward / second_gemm_forward / forward called
    with the reference's argument lists (pybind.cpp:39-58): [E,K,N] weights and the
    64-row block arrays."""
    from ccfuser_amd import mix_moe_hip, ops
    from ccfuser_amd.mix_moe.transformer import plan_blocks
    wl = workloads("c2_gshard", 512)
    t = wl.tensors
    E, d, f, k = wl.num_expert, wl.d_model, wl.d_ffn, wl.top_k
    idx, score, _ = O.naive_gate(t["x"], t["wg"], t["bg"], k)
    pos_ref, off_ref = O.assign_pos(idx, E)
    plan = plan_blocks(O.expert_count(idx, E).numpy())
    dev_i32 = lambda l: torch.tensor(l, dtype=torch.int32, device="cuda")
    blocks = (dev_i32(plan["expert_ids"]), dev_i32(plan["ranks"]), dev_i32(plan["lens"]),
              dev_i32(plan["start_addrs"]), plan["total_block_num"], plan["remote_block_num"])
    m = mix_moe_hip.MixMOE(1, wl.tokens, E, k, d, f, 64)
    w1_kn = t["w1"].cuda().transpose(-2, -1).contiguous()       # what linear.py:74 passes
    w2_kn = t["w2"].cuda().transpose(-2, -1).contiguous()
    x, pos = t["x"].cuda(), pos_ref.cuda()
    merged, h_pre = m.first_gemm_forward(x, pos, *blocks, w1_kn, t["b1"].cuda())
    h = torch.nn.functional.gelu(h_pre)
    _, y_flat = m.second_gemm_forward(h, pos, *blocks, w2_kn, t["b2"].cuda())
    buf = O.local_scatter(t["x"], pos_ref, k)
    y_ref = O.unpermute(O.expert_ffn(buf, off_ref, t["w1"], t["b1"], t["w2"], t["b2"]), pos_ref,
                        wl.tokens * k)
    assert O.max_abs_err(y_flat.cpu(), y_ref) <= MAX_ABS
    assert O.mean_rel_err(y_flat.cpu(), y_ref) <= MEAN_REL
    # merged_input rows are the scattered tokens, block by block
    b0 = plan["start_addrs"][0]
    assert torch.equal(merged[: plan["lens"][0]].cpu(), buf[b0: b0 + plan["lens"][0]])
    m2 = mix_moe_hip.MixMOE(1, wl.tokens, E, k, d, f, 64, w1_kn, w2_kn, t["b1"].cuda(), t["b2"].cuda())
    y2 = m2.forward(x, pos, *blocks, None)
    assert O.max_abs_err(y2.cpu(), y_ref) <= MAX_ABS


def test_extension_class_backward_with_reference_block_arrays(workloads):
    """mix_moe_cuda.MixMOE.first_gemm_backward / second_gemm_backward called the way
    MixMOELinear1/2.backward call them (linear.py:103, 162; pybind.cpp:56-57): stored
    [E, out, in] weights, gradients and saved inputs in the padded 64-row block layout,
    the block arrays and the CSR arrays.  Against the oracle's closed-form backward."""
    from ccfuser_amd import mix_moe_hip
    from ccfuser_amd.mix_moe.transformer import plan_blocks
    wl = workloads("c2_gshard", 512)
    t = wl.tensors
    E, d, f, k = wl.num_expert, wl.d_model, wl.d_ffn, wl.top_k
    idx, score, _ = O.naive_gate(t["x"], t["wg"], t["bg"], k)
    pos_ref, off_ref = O.assign_pos(idx, E)
    R, n_flat = pos_ref.numel(), wl.tokens * k
    plan = plan_blocks(O.expert_count(idx, E).numpy())
    dev_i32 = lambda l: torch.tensor(l, dtype=torch.int32, device="cuda")
    blocks = (dev_i32(plan["expert_ids"]), dev_i32(plan["ranks"]), dev_i32(plan["lens"]),
              dev_i32(plan["start_addrs"]), plan["total_block_num"], plan["remote_block_num"])
    csr = (dev_i32(plan["expert_block_ids"]), dev_i32(plan["expert_block_id_idxs"]))
    nb, bs = plan["total_block_num"], 64
    # expert-order row of every padded row (-1 = padding of a short block)
    sorted_of_padded = torch.full((nb * bs,), -1, dtype=torch.long)
    for b in range(nb):
        n, st = plan["lens"][b], plan["start_addrs"][b]
        sorted_of_padded[b * bs: b * bs + n] = torch.arange(st, st + n)
    valid = sorted_of_padded >= 0

    def to_padded(rows_sorted):
        out = torch.zeros(nb * bs, rows_sorted.shape[1], dtype=rows_sorted.dtype)
        out[valid] = rows_sorted[sorted_of_padded[valid]]
        return out

    g = torch.Generator().manual_seed(5)
    m = mix_moe_hip.MixMOE(1, wl.tokens, E, k, d, f, bs)
    x, pos = t["x"].cuda(), pos_ref.cuda()
    w1, w2 = t["w1"].cuda(), t["w2"].cuda()                      # stored layout, as linear.py:103, 162 pass it
    merged, _ = m.first_gemm_forward(x, pos, *blocks, w1.transpose(-2, -1).contiguous(), t["b1"].cuda())
    # ---- first_gemm_backward
    g_h = torch.randn(R, f, generator=g).half()
    _say(f"first_gemm_backward blocks={nb} rows={R}")
    grad_in, g_w1, g_b1 = m.first_gemm_backward(to_padded(g_h).cuda(), w1, t["b1"].cuda(), merged, *csr, pos,
                                                *blocks)
    ref_in, ref_w1, ref_b1 = O.ffn1_backward(g_h, t["x"], pos_ref, k, off_ref, t["w1"])
    assert tuple(grad_in.shape) == (n_flat // k, d)
    for got, ref, what in ((grad_in, ref_in, "grad_in"), (g_w1, ref_w1, "grad_w1"), (g_b1, ref_b1, "grad_b1")):
        got, ref = got.float().cpu(), ref.float()
        assert O.max_abs_err(got, ref) <= MAX_ABS * max(1.0, float(ref.abs().max())), what
        assert O.mean_rel_err(got, ref) <= MEAN_REL, what
    # ---- second_gemm_backward
    act = torch.randn(R, f, generator=g).half()
    g_y = torch.randn(n_flat, d, generator=g).half()
    _say("second_gemm_backward")
    g_buf, g_w2, g_b2 = m.second_gemm_backward(g_y.cuda(), to_padded(act).cuda(), *csr, w2, t["b2"].cuda(), pos,
                                               *blocks)
    ref_act, ref_w2, ref_b2 = O.ffn2_backward(g_y, act, pos_ref, off_ref, t["w2"])
    assert tuple(g_buf.shape) == (nb * bs, f)
    g_buf = g_buf.cpu()
    assert not g_buf[~valid].any(), "padding rows of grad_inp_buf must be zero"
    for got, ref, what in ((g_buf[valid], ref_act[sorted_of_padded[valid]], "grad_inp_buf"),
                           (g_w2, ref_w2, "grad_w2"), (g_b2, ref_b2, "grad_b2")):
        got, ref = got.float().cpu(), ref.float()
        assert O.max_abs_err(got, ref) <= MAX_ABS * max(1.0, float(ref.abs().max())), what
        assert O.mean_rel_err(got, ref) <= MEAN_REL, what
    with pytest.raises(ValueError):                              # the backward takes the stored layout only
        m.second_gemm_backward(g_y.cuda(), to_padded(act).cuda(), *csr, w2.transpose(-2, -1).contiguous(),
                               t["b2"].cuda(), pos, *blocks)


def test_ep_share_segments(workloads):
    """One GPU's expert-parallel share at reduced rows: (start, len, expert) triples."""
    from ccfuser_amd import ops
    wl = workloads("c4_ep_share", 1536)
    t = wl.tensors
    _say(f"segments rows={wl.tokens} n_seg={t['seg_start'].numel()}")
    y = ops.moe_ffn_segments(*[t[n].cuda() for n in ("x", "seg_start", "seg_len", "seg_expert",
                                                      "w1", "b1", "w2", "b2")])
    ref = O.ffn_segments(t["x"], t["seg_start"], t["seg_len"], t["seg_expert"], t["w1"], t["b1"],
                         t["w2"], t["b2"])
    assert O.max_abs_err(y.cpu(), ref) <= MAX_ABS and O.mean_rel_err(y.cpu(), ref) <= MEAN_REL


def test_error_paths_raise():
    from ccfuser_amd import ops, _lib
    x = torch.randn(8, 64, device="cuda")                       # fp32
    w = torch.randn(2, 64, 64, device="cuda").half()
    b = torch.randn(2, 64, device="cuda").half()
    off = torch.tensor([0, 4, 8], dtype=torch.int32, device="cuda")
    with pytest.raises(TypeError):
        ops.ffn1(x, None, off, 8, w, b)
    with pytest.raises(ValueError):
        ops.ffn1(x.half().cpu(), None, off, 8, w, b)            # CPU tensor: no fallback
    with pytest.raises(_lib.CcfError):
        ops.ffn1(torch.randn(8, 72, device="cuda").half(), None, off, 8,
                 torch.randn(2, 64, 72, device="cuda").half(), b)   # K not a multiple of 64
    with pytest.raises(_lib.CcfError):
        ops.gate_topk_softmax(x.half(), torch.randn(4, 64, device="cuda").half(), None, 9)


def _dense_token(t, tok, experts, scores):
    """The layer's output row of one token by the dense per-token formula in fp32; a
    dropped slot (expert -1) contributes zero."""
    acc = torch.zeros(t["x"].shape[1])
    for e, sc in zip(experts, scores):
        if e < 0:
            continue
        h = O.gelu_exact(t["w1"][e].float() @ t["x"][tok].float() + t["b1"][e].float())
        acc += float(sc) * (t["w2"][e].float() @ h + t["b2"][e].float())
    return acc


def _full_size_check(wl, t, n_sample=48, must_drop=False):
    """The fused call at full size, with every tile-plan feature at its default (skinny tiles,
    the split last round and the routing-built plans only engage at these sizes): routing
    bit-exact against the oracle, the WHOLE output against the oracle's layer by both error
    measures, sampled tokens against the dense per-token formula as a second pin, and exact
    linearity in the second layer's parameters."""
    from ccfuser_amd import ops
    E, k = wl.num_expert, wl.top_k
    args = [t[n].cuda() for n in ("x", "wg", "bg", "w1", "b1", "w2", "b2")]
    out, r = ops.moe_forward(*args, k, wl.capacity, return_routing=True)
    torch.cuda.synchronize()
    idx_ref, score_ref, _ = O.naive_gate(t["x"], t["wg"], t["bg"], k)
    kept_ref = O.limit_by_capacity(idx_ref, E, wl.capacity)
    dropped = int((kept_ref < 0).sum())
    _say(f"  routed {int((kept_ref >= 0).sum())} rows, {dropped} slots dropped by capacity {wl.capacity}")
    assert not must_drop or dropped > 0
    assert torch.equal(r["idx"].cpu(), kept_ref)
    pos_ref, off_ref = O.assign_pos(kept_ref, E)
    R = int(off_ref[-1])
    assert torch.equal(r["offsets"].cpu(), off_ref)
    assert torch.equal(r["counts"].cpu().long(), O.expert_count(kept_ref, E).long())
    assert torch.equal(r["pos"].cpu()[:R], pos_ref)
    assert torch.isfinite(out.float()).all()
    # whole output: the oracle's layer on the same tensors (seconds on the host's cores)
    ref = O.moe_layer_forward(*[t[n] for n in ("x", "wg", "bg", "w1", "b1", "w2", "b2")], k, capacity=wl.capacity)
    assert torch.equal(ref["idx_kept"], kept_ref)
    ma, mr = O.max_abs_err(out.cpu(), ref["out"]), O.mean_rel_err(out.cpu(), ref["out"])
    _say(f"  whole output [{out.shape[0]}, {out.shape[1]}]: max_abs={ma:.3e} mean_rel={mr:.3e}")
    assert ma <= MAX_ABS and mr <= MEAN_REL
    del ref
    g = torch.Generator().manual_seed(0)
    sample = torch.randperm(wl.tokens, generator=g)[:n_sample].tolist()
    if dropped:                                       # make sure tokens that lost a slot are among the sample
        lost = torch.nonzero((kept_ref < 0).any(-1)).view(-1)
        sample += lost[torch.randperm(lost.numel(), generator=g)[:8]].tolist()
    for tok in sample:
        ref_row = _dense_token(t, tok, kept_ref[tok].tolist(), score_ref[tok].tolist())
        assert (out[tok].cpu().float() - ref_row).abs().max() <= MAX_ABS, tok
    # Linearity: the output is linear in (w2, b2), and doubling is exact in fp16 and in the
    # fp32 accumulators, so doubling both doubles every output bit for bit, except where an
    # expert output falls into fp16's subnormal range (below 2^-14 the rounding step is
    # absolute, so rounding does not commute with doubling there): such an element may move the
    # token's sum by one rounding step.
    out2 = ops.moe_forward(args[0], args[1], args[2], args[3], args[4], args[5] * 2, args[6] * 2, k, wl.capacity)
    want = out.float() * 2
    diff = (out2.float() - want).abs()
    assert bool((diff <= want.abs() * 2.0 ** -10 + 2.0 ** -22).all()), "doubling w2 and b2 did not double the output"
    mism = float((diff > 0).float().mean())
    _say(f"  linearity: {mism:.2e} of the elements off by one rounding step")
    assert mism < 1e-2


@pytest.mark.parametrize("name", ["c2_gshard", "c3_mixtral", "c5_skewed"])
def test_full_size_properties(workloads, name):
    """The named workloads at their full sizes: whole output against the oracle, plus what
    does not depend on size (see _full_size_check)."""
    wl = workloads(name)
    _say(f"full size {name}")
    _full_size_check(wl, wl.tensors)


def test_full_size_gshard_shape_with_binding_capacity(workloads):
    """The capacity-limited workload's own seed routes almost uniformly, so its capacity of
    2560 rows per expert drops nothing.  Same shapes and tensors with a gate bias that sends
    most tokens to experts 2 and 5: both overflow, their late slots are dropped (expert -1,
    score kept, zero contribution) and every other check of the full-size test must hold."""
    wl = workloads("c2_gshard")
    t = dict(wl.tensors)
    bg = t["bg"].clone().float()
    bg[2] += 0.6
    bg[5] += 0.5
    t["bg"] = bg.half()
    _say("full size c2_gshard shapes, biased gate")
    _full_size_check(wl, t, must_drop=True)


def test_full_size_ep_share_segments(workloads):
    """One GPU's expert-parallel share at its full 16384 inbound rows (K = 8192 in the second
    GEMM, so the last round of tiles is cut along K): the whole output against the oracle by both
    error measures, sampled rows against the dense formula, a second call bit-identical."""
    from ccfuser_amd import ops
    wl = workloads("c4_ep_share")
    t = wl.tensors
    names = ("x", "seg_start", "seg_len", "seg_expert", "w1", "b1", "w2", "b2")
    _say(f"full size c4_ep_share rows={wl.tokens} n_seg={t['seg_start'].numel()}")
    args = [t[n].cuda() for n in names]
    y = ops.moe_ffn_segments(*args)
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all()
    ref = O.ffn_segments(t["x"], t["seg_start"], t["seg_len"], t["seg_expert"], t["w1"], t["b1"], t["w2"], t["b2"])
    ma, mr = O.max_abs_err(y.cpu(), ref), O.mean_rel_err(y.cpu(), ref)
    _say(f"  whole output [{y.shape[0]}, {y.shape[1]}]: max_abs={ma:.3e} mean_rel={mr:.3e}")
    assert ma <= MAX_ABS and mr <= MEAN_REL
    del ref
    expert_of_row = torch.full((wl.tokens,), -1, dtype=torch.long)
    for st, ln, e in zip(t["seg_start"].tolist(), t["seg_len"].tolist(), t["seg_expert"].tolist()):
        expert_of_row[st:st + ln] = e
    assert (expert_of_row >= 0).all()                     # the segments tile the inbound buffer
    g = torch.Generator().manual_seed(1)
    rows = torch.randperm(wl.tokens, generator=g)[:48].tolist()
    rows += [0, wl.tokens - 1] + t["seg_start"].tolist()[:8]      # buffer ends and segment heads
    for r_ in rows:
        ref_row = _dense_token(t, r_, [int(expert_of_row[r_])], [1.0])
        assert (y[r_].cpu().float() - ref_row).abs().max() <= MAX_ABS, r_
    assert torch.equal(y, ops.moe_ffn_segments(*args))


def test_combine_in_the_second_gemm_epilogue(workloads):
    """Option "fused_combine": for top-2 the second GEMM's epilogue adds score * y into the
    zero-filled output with packed fp16 atomic adds instead of writing y_flat for a combine
    pass (off by default: measured slower).  Two addends onto zero commute, so the result is
    deterministic; it must meet the oracle's tolerance, with capacity drops too."""
    from ccfuser_amd import ops
    wl = workloads("c2_gshard", 1024)
    t = dict(wl.tensors)
    bg = t["bg"].clone().float()
    bg[2] += 0.6                                   # expert 2 overflows its capacity: dropped slots add nothing
    t["bg"] = bg.half()
    names = ("x", "wg", "bg", "w1", "b1", "w2", "b2")
    ref = O.moe_layer_forward(*[t[n] for n in names], wl.top_k, capacity=wl.capacity)
    assert int((ref["idx_kept"] < 0).sum()) > 0
    args = [t[n].cuda() for n in names]
    _say(f"fused combine T={wl.tokens}")
    ops.set_option("fused_combine", 1)
    try:
        a = ops.moe_forward(*args, wl.top_k, wl.capacity)
        b = ops.moe_forward(*args, wl.top_k, wl.capacity)
    finally:
        ops.set_option("fused_combine", 0)
    assert torch.equal(a, b)
    assert O.max_abs_err(a.cpu(), ref["out"]) <= MAX_ABS and O.mean_rel_err(a.cpu(), ref["out"]) <= MEAN_REL
    plain = ops.moe_forward(*args, wl.top_k, wl.capacity)
    assert O.max_abs_err(a.cpu(), plain.float().cpu()) <= 4e-3


def test_forward_replays_from_a_hip_graph(workloads):
    """The whole-layer call allocates nothing and never synchronises, so it can be captured
    into a HIP graph.  Replayed several times with fresh inputs, with eager work and
    synchronisations between the replays, every replay must equal the eager result bit for bit
    (routing changes with the input, so the graph's kernels must pick the new tile plan up)."""
    from ccfuser_amd import ops
    wl = workloads("c2_gshard", 1024)
    t = wl.tensors
    T, d, f, E, k = wl.tokens, wl.d_model, wl.d_ffn, wl.num_expert, wl.top_k
    params = [t[n].cuda() for n in ("wg", "bg", "w1", "b1", "w2", "b2")]
    x_static = t["x"].cuda().clone()
    ws = ops.moe_workspace(T, d, f, E, k, "cuda")
    _say(f"graph replay T={T} d={d} f={f} E={E} k={k}")
    side = torch.cuda.Stream()                               # default priority
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):                                   # warm-up outside the capture
            ops.moe_forward(x_static, *params, k, wl.capacity, workspace=ws)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out_static = ops.moe_forward(x_static, *params, k, wl.capacity, workspace=ws)
    g = torch.Generator().manual_seed(99)
    for rep in range(4):
        x_new = torch.randn(T, d, generator=g).half().cuda()
        eager = ops.moe_forward(x_new, *params, k, wl.capacity)      # own workspace, eager
        torch.cuda.synchronize()
        x_static.copy_(x_new)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_static, eager), f"replay {rep} differs from the eager call"


def test_top1_output_written_by_ffn2_equals_the_staged_path(workloads):
    """With top-1 and no capacity limit the fused call lets FFN2 write the layer output (the
    score is exactly 1); the staged path, which runs the combine kernel, must give the same bits."""
    from ccfuser_amd import ops
    wl = workloads("c5_skewed", 2048)
    t = wl.tensors
    assert wl.top_k == 1 and wl.capacity < 0
    args = [t[n].cuda() for n in ("x", "wg", "bg", "w1", "b1", "w2", "b2")]
    _say(f"top-1 direct output T={wl.tokens}")
    fused, r = ops.moe_forward(*args, 1, -1, return_routing=True)
    assert bool((r["score"] == 1.0).all())
    x, wg, bg, w1, b1, w2, b2 = args
    idx, score = ops.gate_topk_softmax(x, wg, bg, 1)
    rt = ops.route(idx.reshape(-1), wl.num_expert, 1, -1)
    n = wl.tokens
    h = ops.ffn1(x, rt["src_row"], rt["offsets"], n, w1, b1, gelu=True)
    y = torch.empty(n, wl.d_model, dtype=torch.float16, device="cuda")
    ops.ffn2(h, rt["dst_row"], rt["offsets"], n, w2, b2, y)
    staged = ops.combine(y, score.reshape(-1), 1, rt["inv_pos"])
    assert torch.equal(fused, staged)


def _staged_forward(ops, args, E, k, capacity):
    x, wg, bg, w1, b1, w2, b2 = args
    idx, score = ops.gate_topk_softmax(x, wg, bg, k)
    rt = ops.route(idx.reshape(-1), E, k, capacity)
    n = x.shape[0] * k
    h = ops.ffn1(x, rt["src_row"], rt["offsets"], n, w1, b1, gelu=True)
    y = torch.zeros(n, x.shape[1], dtype=torch.float16, device="cuda")
    ops.ffn2(h, rt["dst_row"], rt["offsets"], n, w2, b2, y)
    return ops.combine(y, score.reshape(-1), k, rt["inv_pos"])


@pytest.mark.parametrize("name,rows,variant", [("c3_mixtral", None, -1)] +
                         [("c2_gshard", 1024, v) for v in (0, 1, 2, 3)] + [("c5_skewed", None, 3), ("c3_mixtral", None, 3)])
def test_fused_call_equals_stage_by_stage_calls(workloads, name, rows, variant):
    """In the fused call the routing stage builds the tile plans of both GEMMs; stand-alone
    GEMM calls build their own.  Same plans, same kernels, so the same bits: at full size on the
    benchmark shape (last round of tiles split along K in both GEMMs) and, on a small batch, for
    every launch form (chosen by K, one workgroup per tile, persistent with four and with eight
    wavefronts), the eight-wavefront form also at full size."""
    from ccfuser_amd import ops
    wl = workloads(name, rows) if rows else workloads(name)
    t = wl.tensors
    args = [t[n].cuda() for n in ("x", "wg", "bg", "w1", "b1", "w2", "b2")]
    _say(f"fused against staged {name} T={wl.tokens} variant={variant}")
    ops.set_option("gemm_variant", variant)
    try:
        fused = ops.moe_forward(*args, wl.top_k, wl.capacity)
        staged = _staged_forward(ops, args, wl.num_expert, wl.top_k, wl.capacity)
        assert torch.equal(fused, staged)
    finally:
        ops.set_option("gemm_variant", -1)


@pytest.mark.parametrize("T,d,f,E,k", [(2048, 64, 128, 600, 2), (4096, 128, 64, 1024, 1), (300, 64, 64, 37, 4),
                                       (1000, 128, 64, 20, 3), (5000, 256, 64, 8, 8)])
def test_fused_layer_with_many_experts(T, d, f, E, k):
    """Most experts get a handful of rows or none; the routing launch builds the tile plans with
    eight workgroups per plan and needs more than 64 KB of LDS past 512 experts.  The cases also
    cover the ways the routing stage gets its counts: from the gate kernel's workgroups (top-k
    a power of two, small table), from its own histogram launch (1024 experts; top-3)."""
    from ccfuser_amd import ops
    g = torch.Generator().manual_seed(E)
    r = lambda *s, sc=1.0: (torch.randn(*s, generator=g) * sc).half()
    x, wg, bg = r(T, d), r(E, d, sc=0.3), r(E, sc=0.3)
    w1, b1, w2, b2 = r(E, f, d, sc=0.1), r(E, f, sc=0.1), r(E, d, f, sc=0.1), r(E, d, sc=0.1)
    _say(f"many experts T={T} d={d} f={f} E={E} k={k}")
    args = [a.cuda() for a in (x, wg, bg, w1, b1, w2, b2)]
    fused, rt = ops.moe_forward(*args, k, -1, return_routing=True)
    ref = O.moe_layer_forward(x, wg, bg, w1, b1, w2, b2, k)
    assert torch.equal(rt["idx"].cpu(), ref["idx"])
    assert torch.equal(rt["offsets"].cpu().long(), ref["offsets"].long())
    assert O.max_abs_err(fused.cpu(), ref["out"]) <= MAX_ABS
    assert O.mean_rel_err(fused.cpu(), ref["out"]) <= MEAN_REL
    assert torch.equal(fused, _staged_forward(ops, args, E, k, -1))


def _random_layer_shapes(count, seed):
    g = torch.Generator().manual_seed(seed)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    shapes = []
    for i in range(count):
        E = ri(1, 40)
        k = ri(1, min(4, E))
        T = ri(1, 3000)
        d, f = 64 * ri(1, 12), 64 * ri(1, 16)
        cap = -1 if i % 3 else max(1, (T * k) // (2 * E))       # every third case drops about half of the busier experts' slots
        shapes.append((T, d, f, E, k, cap, 9000 + i))
    return shapes + [(1, 64, 64, 1, 1, -1, 9100), (257, 832, 320, 3, 3, 100, 9101)]


@pytest.mark.parametrize("T,d,f,E,k,cap,seed", _random_layer_shapes(12, 777))
def test_fused_layer_random_shapes(T, d, f, E, k, cap, seed):
    """Shapes drawn at random (1-3000 tokens, widths any multiple of 64 up to 768 x 1024, 1-40
    experts, top-1..4, every third with a binding capacity) plus a single token and widths that
    are no multiple of 256: routing bit-exact, output within the tolerance, fused call = staged
    calls bit for bit."""
    from ccfuser_amd import ops
    g = torch.Generator().manual_seed(seed)
    r = lambda *s, sc=1.0: (torch.randn(*s, generator=g) * sc).half()
    x, wg, bg = r(T, d), r(E, d, sc=0.3), r(E, sc=0.3)
    w1, b1, w2, b2 = r(E, f, d, sc=0.1), r(E, f, sc=0.1), r(E, d, f, sc=0.1), r(E, d, sc=0.1)
    _say(f"random layer T={T} d={d} f={f} E={E} k={k} cap={cap}")
    args = [a.cuda() for a in (x, wg, bg, w1, b1, w2, b2)]
    fused, rt = ops.moe_forward(*args, k, cap, return_routing=True)
    ref = O.moe_layer_forward(x, wg, bg, w1, b1, w2, b2, k, capacity=cap)
    R = int(ref["offsets"][-1])
    assert torch.equal(rt["idx"].cpu().view(-1), ref["idx_kept"].view(-1))      # after the capacity limit
    assert torch.equal(rt["offsets"].cpu().long(), ref["offsets"].long())
    assert torch.equal(rt["pos"].cpu()[:R], ref["pos"])
    assert O.max_abs_err(fused.cpu(), ref["out"]) <= MAX_ABS
    if float(ref["out"].abs().mean()) > 1e-6:
        assert O.mean_rel_err(fused.cpu(), ref["out"]) <= MEAN_REL
    assert torch.equal(fused, _staged_forward(ops, args, E, k, cap))


def _forced_plan_cases(count, seed):
    g = torch.Generator().manual_seed(seed)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    modes = [(-6, 0), (-5, 1), (-1, 0), (-3, 0), (-6, 0), (1, 0), (-4, 0), (-6, 0)]
    cases = []
    for i in range(count):
        E = ri(4, 24)
        k = ri(1, 2)
        T = ri(9000, 20000) // k
        d, f = 256 * ri(2, 4), 256 * ri(2, 5)
        skinny, sk_tail = modes[i % len(modes)]
        cases.append((T, d, f, E, k, skinny, sk_tail, 9500 + i))
    return cases


@pytest.mark.parametrize("T,d,f,E,k,skinny,sk_tail,seed", _forced_plan_cases(8, 4321))
def test_fused_layer_random_shapes_with_forced_plans(T, d, f, E, k, skinny, sk_tail, seed):
    """Shapes large enough for the persistent launch (more worst-case tiles than CUs), drawn at
    random, with the tile plan's choices forced in turn: skinny tiles beside the 256-row tiles,
    cut along K inside the persistent launch or as a launch of their own, and the last round of
    tiles cut along K (its parts inside the persistent launch) at every K.  Routing bit-exact,
    whole output within the tolerance, a second call the same bits."""
    from ccfuser_amd import ops
    g = torch.Generator().manual_seed(seed)
    r = lambda *s, sc=1.0: (torch.randn(*s, generator=g) * sc).half()
    x, wg, bg = r(T, d), r(E, d, sc=0.1), r(E, sc=0.1)
    w1, b1, w2, b2 = r(E, f, d, sc=0.05), r(E, f, sc=0.1), r(E, d, f, sc=0.05), r(E, d, sc=0.1)
    _say(f"forced plans T={T} d={d} f={f} E={E} k={k} skinny={skinny} skinny_tail={sk_tail}")
    args = [a.cuda() for a in (x, wg, bg, w1, b1, w2, b2)]
    ops.set_option("skinny", skinny)
    ops.set_option("skinny_tail", sk_tail)
    ops.set_option("split_tail", 2)
    try:
        fused, rt = ops.moe_forward(*args, k, -1, return_routing=True)
        again = ops.moe_forward(*args, k, -1)
        torch.cuda.synchronize()
    finally:
        ops.set_option("skinny", 1)
        ops.set_option("skinny_tail", 0)
        ops.set_option("split_tail", 1)
    ref = O.moe_layer_forward(x, wg, bg, w1, b1, w2, b2, k)
    assert torch.equal(rt["idx"].cpu().view(-1), ref["idx_kept"].view(-1))
    assert torch.equal(rt["offsets"].cpu().long(), ref["offsets"].long())
    ma, mr = O.max_abs_err(fused.cpu(), ref["out"]), O.mean_rel_err(fused.cpu(), ref["out"])
    _say(f"  counts={ref['counts'].tolist()} max_abs={ma:.3e} mean_rel={mr:.3e}")
    assert ma <= MAX_ABS and mr <= MEAN_REL
    assert torch.equal(fused, again)
