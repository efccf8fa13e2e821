"""Pins the oracle's closed-form backward against torch autograd through library
operations and against finite differences (none of them restates its formulas)."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O


def _params(T, d, f, E, seed, dtype=torch.float32, scale=0.3):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: (torch.randn(*s, generator=g) * scale).to(dtype)
    return {"x": r(T, d) / scale, "wg": r(E, d), "bg": r(E), "w1": r(E, f, d), "b1": r(E, f),
            "w2": r(E, d, f), "b2": r(E, d)}


def _library_layer(p, k, idx_kept, idx=None):
    """The layer from torch library ops only, routing given (it is piecewise constant).
    ``idx`` is the gate's choice before capacity limiting (scores come from it)."""
    T = p["x"].shape[0]
    E = p["w1"].shape[0]
    logits = F.linear(p["x"], p["wg"], p["bg"])
    idx = idx_kept if idx is None else idx
    score = torch.softmax(torch.gather(logits, 1, idx), dim=-1)
    flat = idx_kept.reshape(-1)
    y_flat = torch.zeros(T * k, p["x"].shape[1], dtype=p["x"].dtype)
    for e in range(E):
        sel = torch.nonzero(flat == e).reshape(-1)
        if sel.numel() == 0:
            continue
        rows = torch.index_select(p["x"], 0, sel // k)
        h = F.gelu(F.linear(rows, p["w1"][e], p["b1"][e]))
        y_flat = y_flat.index_copy(0, sel, F.linear(h, p["w2"][e], p["b2"][e]))
    return torch.bmm(score.view(T, 1, k), y_flat.view(T, k, -1)).reshape(T, -1)


@pytest.mark.parametrize("T,d,f,E,k,cap,seed", [
    (24, 16, 32, 4, 2, -1, 0),
    (40, 8, 16, 3, 1, -1, 1),
    (33, 16, 24, 5, 2, 10, 2),      # capacity drops some slots
    (16, 8, 8, 1, 1, -1, 3),        # one expert: a dense MLP
    (20, 8, 16, 6, 3, -1, 4),
])
def test_layer_backward_against_autograd(T, d, f, E, k, cap, seed):
    p = _params(T, d, f, E, seed)
    g = torch.Generator().manual_seed(100 + seed)
    grad_out = torch.randn(T, d, generator=g)
    ref = O.moe_layer_forward(p["x"], p["wg"], p["bg"], p["w1"], p["b1"], p["w2"], p["b2"], k, capacity=cap)
    q = {n: v.clone().requires_grad_(True) for n, v in p.items()}
    out = _library_layer(q, k, ref["idx_kept"].reshape(T, k), ref["idx"])
    assert torch.allclose(out.detach(), ref["out"], atol=1e-5)
    out.backward(grad_out)
    got = O.moe_layer_backward(p["x"], p["wg"], p["bg"], p["w1"], p["b1"], p["w2"], p["b2"], k,
                               grad_out, capacity=cap)
    for n in ("x", "wg", "bg", "w1", "b1", "w2", "b2"):
        assert torch.allclose(got[n], q[n].grad, atol=2e-5, rtol=1e-4), n


def test_stage_backwards_against_finite_differences():
    """Central differences in float64 on a tiny layer, one scalar loss."""
    T, d, f, E, k = 6, 8, 6, 3, 2
    p = {n: v.double() for n, v in _params(T, d, f, E, 7).items()}
    g = torch.Generator().manual_seed(9)
    grad_out = torch.randn(T, d, generator=g).double()
    p32 = {n: v.float() for n, v in p.items()}
    idx_kept = O.moe_layer_forward(*[p32[n] for n in ("x", "wg", "bg", "w1", "b1", "w2", "b2")], k)["idx_kept"].reshape(T, k)
    got = O.moe_layer_backward(*[p32[n] for n in ("x", "wg", "bg", "w1", "b1", "w2", "b2")], k, grad_out.float())

    def loss(q):
        return float((_library_layer(q, k, idx_kept) * grad_out).sum())

    eps = 1e-5
    gen = torch.Generator().manual_seed(3)
    for n in ("x", "wg", "bg", "w1", "b1", "w2", "b2"):
        flat = p[n].reshape(-1)
        for i in torch.randperm(flat.numel(), generator=gen)[:6].tolist():
            old = float(flat[i])
            flat[i] = old + eps
            up = loss(p)
            flat[i] = old - eps
            down = loss(p)
            flat[i] = old
            fd = (up - down) / (2 * eps)
            assert abs(fd - float(got[n].reshape(-1)[i])) <= 2e-4 * max(1.0, abs(fd)), (n, i)


def test_backward_special_cases():
    """k = 1: score is 1 and carries no gradient to the gate.  Zero incoming gradient
    gives zero everywhere.  An expert without rows has zero weight gradients."""
    T, d, f, E = 12, 8, 16, 4
    p = _params(T, d, f, E, 5)
    args = [p[n] for n in ("x", "wg", "bg", "w1", "b1", "w2", "b2")]
    g = torch.Generator().manual_seed(1)
    go = torch.randn(T, d, generator=g)
    r = O.moe_layer_backward(*args, 1, go)
    assert float(r["wg"].abs().max()) < 1e-6 and float(r["x_gate"].abs().max()) < 1e-6
    z = O.moe_layer_backward(*args, 2, torch.zeros(T, d))
    assert all(float(z[n].abs().max()) == 0.0 for n in ("x", "wg", "w1", "b1", "w2", "b2"))
    counts = O.expert_count(r["idx"], E)
    for e in torch.nonzero(counts == 0).reshape(-1).tolist():
        assert float(r["w1"][e].abs().max()) == 0.0 and float(r["b2"][e].abs().max()) == 0.0
    # bias gradients are the per-expert column sums of what reaches the bias
    off = r["offsets"].tolist()
    for e in range(E):
        assert torch.allclose(r["b1"][e], r["h"][off[e]:off[e + 1]].sum(0), atol=1e-6)


def test_gelu_backward_against_library():
    h = torch.linspace(-6, 6, 241, requires_grad=True)
    F.gelu(h).backward(torch.ones_like(h))
    assert torch.allclose(O.gelu_backward(torch.ones(241), h.detach()), h.grad, atol=1e-6)
