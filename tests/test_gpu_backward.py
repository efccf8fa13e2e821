"""GPU parity of the backward stages against the CPU oracle, through the C ABI.

Gradients are fp16 with fp32 accumulation.  Tolerance: max-abs error at most
2e-2 times max(1, largest reference magnitude) (weight gradients sum over an
expert's rows and exceed 1), and mean-rel (mean |err| / mean |ref|) at most 1e-3.
"""
import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_REL = 2e-2, 1e-3


def _say(msg):
    print(msg, flush=True)


def _close(got, ref, what):
    got, ref = got.float().cpu(), ref.float()
    bound = MAX_ABS * max(1.0, float(ref.abs().max()))
    err = O.max_abs_err(got, ref)
    assert err <= bound, (what, err, bound)
    if float(ref.abs().mean()) > 1e-6:
        assert O.mean_rel_err(got, ref) <= MEAN_REL, (what, O.mean_rel_err(got, ref))


def _case(T, d, f, E, k, seed, skew=False):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s, sc=1.0: (torch.randn(*s, generator=g) * sc).half()
    p = {"x": r(T, d), "wg": r(E, d, sc=0.05), "bg": r(E, sc=0.05), "w1": r(E, f, d, sc=0.05),
         "b1": r(E, f, sc=0.05), "w2": r(E, d, f, sc=0.05), "b2": r(E, d, sc=0.05)}
    if skew:                                   # most tokens to expert 0, expert 1 empty
        p["bg"][0] += 3.0
        p["bg"][1] -= 50.0
    return p


@pytest.mark.parametrize("T,d,f,E,k,cap,skew,seed", [
    (300, 256, 512, 4, 2, -1, False, 0),
    (512, 512, 256, 8, 2, 100, False, 1),     # capacity drops slots
    (257, 256, 1024, 3, 1, -1, False, 2),
    (64, 256, 256, 16, 2, -1, False, 3),      # every expert far below one K tile of rows
    (700, 256, 512, 4, 2, -1, True, 4),       # one large expert, one empty
])
def test_ffn_backward_stages(T, d, f, E, k, cap, skew, seed):
    from ccfuser_amd import ops
    _say(f"ffn backward T={T} d={d} f={f} E={E} k={k} cap={cap} skew={skew}")
    p = _case(T, d, f, E, k, seed, skew)
    g = torch.Generator().manual_seed(1000 + seed)
    grad_out = torch.randn(T, d, generator=g).half()
    ref = O.moe_layer_backward(p["x"], p["wg"], p["bg"], p["w1"], p["b1"], p["w2"], p["b2"], k,
                               grad_out, capacity=cap)
    pos, offsets = ref["pos"], ref["offsets"]
    n = T * k
    idx_kept = O.limit_by_capacity(ref["idx"], E, cap)
    rt = ops.route(idx_kept.reshape(-1).cuda(), E, k, -1)
    assert torch.equal(rt["offsets"].cpu().long(), offsets.long())

    # combine backward on the fp16-rounded forward values
    y16, s16 = ref["y_flat_fwd"].half(), ref["score_fwd"].half()
    gy_ref, gs_ref = O.combine_backward(grad_out, y16, s16, k)
    kept = (O.inverse_pos(pos, n) >= 0)
    gy_ref = gy_ref * kept[:, None]
    gs_ref = gs_ref.reshape(-1) * kept
    gy, gs = ops.combine_backward(grad_out.cuda(), y16.cuda(), s16.reshape(-1).cuda(), k, rt["inv_pos"])
    _close(gy, gy_ref, "grad_y_flat")
    _close(gs, gs_ref, "grad_score")

    # second GEMM backward
    act16, gy16 = ref["act_fwd"].half(), gy_ref.half()
    a_pad = torch.zeros(n, f, dtype=torch.float16)
    a_pad[: act16.shape[0]] = act16
    ga_ref, gw2_ref, gb2_ref = O.ffn2_backward(gy16, act16, pos, offsets, p["w2"])
    ga, gw2, gb2 = ops.ffn2_backward(gy16.cuda(), a_pad.cuda(), rt["dst_row"], rt["offsets"], n, p["w2"].cuda())
    R = pos.numel()
    _close(ga[:R], ga_ref, "grad_act")
    assert float(ga[R:].abs().max()) == 0.0 if R < n else True
    _close(gw2, gw2_ref, "grad_w2")
    _close(gb2, gb2_ref, "grad_b2")

    # first GEMM backward
    gh16 = ref["h"].half()
    gh_pad = torch.zeros(n, f, dtype=torch.float16)
    gh_pad[:R] = gh16
    gin_ref, gw1_ref, gb1_ref = O.ffn1_backward(gh16, p["x"], pos, k, offsets, p["w1"])
    gx_flat, gw1, gb1 = ops.ffn1_backward(gh_pad.cuda(), p["x"].cuda(), rt["src_row"], rt["dst_row"],
                                          rt["offsets"], n, p["w1"].cuda(), n)
    ones = torch.ones(n, dtype=torch.float16, device="cuda")
    gin = ops.combine(gx_flat, ones, k, rt["inv_pos"])
    _close(gin, gin_ref, "grad_in")
    _close(gw1, gw1_ref, "grad_w1")
    _close(gb1, gb1_ref, "grad_b1")


@pytest.mark.parametrize("T,d,f,E,k,cf,seed", [
    (384, 256, 512, 4, 2, None, 10),
    (512, 256, 512, 8, 2, 1.0, 11),          # capacity factor 1.0 drops slots
    (200, 512, 256, 4, 1, None, 12),
])
def test_module_backward_matches_oracle(T, d, f, E, k, cf, seed):
    """loss = <out, grad_out> through MixMOETransformerMLP (gate, two expert GEMMs with
    torch's GELU between them, combine) against the oracle's closed-form gradients."""
    from ccfuser_amd.mix_moe import MixMOETransformerMLP
    _say(f"module backward T={T} d={d} f={f} E={E} k={k} cf={cf}")
    p = _case(T, d, f, E, k, seed)
    g = torch.Generator().manual_seed(2000 + seed)
    grad_out = torch.randn(T, d, generator=g).half()
    mlp = MixMOETransformerMLP("naive", {"num_local_expert": E, "hidden_size": f}, d, 0, 1,
                               total_batch_size=T, top_k=k, capacity_factor=cf).half().cuda()
    with torch.no_grad():
        mlp.gate.gate.weight.copy_(p["wg"]); mlp.gate.gate.bias.copy_(p["bg"])
        mlp.experts.htoh4.weight[:E].copy_(p["w1"]); mlp.experts.htoh4.bias[:E].copy_(p["b1"])
        mlp.experts.h4toh.weight[:E].copy_(p["w2"]); mlp.experts.h4toh.bias[:E].copy_(p["b2"])
    x = p["x"].cuda().requires_grad_(True)
    out = mlp(x)
    out.backward(grad_out.cuda())
    cap = mlp._capacity(T)
    ref = O.moe_layer_backward(p["x"], p["wg"], p["bg"], p["w1"], p["b1"], p["w2"], p["b2"], k,
                               grad_out, capacity=cap)
    fwd = O.moe_layer_forward(p["x"], p["wg"], p["bg"], p["w1"], p["b1"], p["w2"], p["b2"], k, capacity=cap)
    assert O.max_abs_err(out.detach().cpu(), fwd["out"]) <= MAX_ABS
    _close(x.grad, ref["x"], "grad_x")
    _close(mlp.gate.gate.weight.grad, ref["wg"], "grad_wg")
    _close(mlp.gate.gate.bias.grad, ref["bg"], "grad_bg")
    _close(mlp.experts.htoh4.weight.grad[:E], ref["w1"], "grad_w1")
    _close(mlp.experts.htoh4.bias.grad[:E], ref["b1"], "grad_b1")
    _close(mlp.experts.h4toh.weight.grad[:E], ref["w2"], "grad_w2")
    _close(mlp.experts.h4toh.bias.grad[:E], ref["b2"], "grad_b2")
    assert float(mlp.experts.htoh4.weight.grad[E:].abs().max()) == 0.0     # slots of no expert
    # the path overlapped with a side stream differentiates the same way
    mlp.zero_grad()
    x2 = p["x"].cuda().requires_grad_(True)
    mlp.async_expert_assignment(x2)
    mlp(x2).backward(grad_out.cuda())
    _close(x2.grad, ref["x"], "grad_x (async)")
    _close(mlp.experts.h4toh.weight.grad[:E], ref["w2"], "grad_w2 (async)")
    mlp.close()
