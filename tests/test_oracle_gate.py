"""Pins the oracle's gate against torch library routines, brute force and closed forms.

None of these checks retypes the oracle's formula: the logits are compared with
``F.linear`` (fp32 and fp64), the selection with ``torch.topk`` / ``argmax`` and
a Python brute force, the scores with ``F.softmax``.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O


@pytest.mark.parametrize("T,d,E,dtype", [(37, 64, 4, torch.float16), (16, 768, 32, torch.float16),
                                         (9, 4096, 8, torch.float16), (33, 256, 4, torch.float32),
                                         (5, 8, 3, torch.float16), (7, 520, 5, torch.float16)])
def test_logits_match_linear(T, d, E, dtype):
    g = torch.Generator().manual_seed(T * d)
    x = torch.randn(T, d, generator=g).to(dtype)
    w = (torch.randn(E, d, generator=g) * 0.05).to(dtype)
    b = (torch.randn(E, generator=g) * 0.05).to(dtype)
    got = O.gate_logits(x, w, b)
    ref64 = F.linear(x.double(), w.double(), b.double())
    # fp32 accumulation error bound: a few ulp times sqrt(d) of the running magnitude
    scale = (x.double().abs() @ w.double().abs().t()).max().item()
    assert (got.double() - ref64).abs().max().item() <= 4e-7 * scale * np.sqrt(d) + 1e-7
    assert got.dtype == torch.float32
    # without the bias the result is the plain dot product, e.g. exact on small integers
    xi = torch.randint(-4, 5, (T, d), generator=g).to(dtype)
    wi = torch.randint(-4, 5, (E, d), generator=g).to(dtype)
    assert torch.equal(O.gate_logits(xi, wi, None), (xi.double() @ wi.double().t()).float())


def test_logits_order_is_the_documented_one():
    """Brute-force replay of the documented order with Python floats rounded to fp32
    at every step, on a case with two full parts and a short third one."""
    g = torch.Generator().manual_seed(3)
    d = 128 * 2 + 8 * 3
    x = torch.randn(2, d, generator=g).half()
    w = torch.randn(3, d, generator=g).half()
    b = torch.randn(3, generator=g).half()
    got = O.gate_logits(x, w, b)
    f32 = np.float32
    for t in range(2):
        for e in range(3):
            parts = []
            for p0 in range(0, d, 128):
                acc = f32(0)
                for k in range(p0, min(p0 + 128, d)):
                    acc = f32(acc + f32(f32(x[t, k].item()) * f32(w[e, k].item())))
                parts.append(acc)
            total = parts[0]
            for p in parts[1:]:
                total = f32(total + p)
            assert f32(total + f32(b[e].item())) == got[t, e].item()


def test_logits_chain_is_a_chain_of_fused_multiply_adds():
    """For fp16 inputs every product is exact in fp32, so each step of a part's chain is
    one rounding of the exact acc + x*w: replayed here with exact rational arithmetic."""
    from fractions import Fraction
    g = torch.Generator().manual_seed(11)
    d = 128 + 16
    x = (torch.randn(1, d, generator=g) * 8).half()
    w = (torch.randn(2, d, generator=g) * 0.01).half()
    got = O.gate_logits(x, w, None)
    for e in range(2):
        parts = []
        for p0 in range(0, d, 128):
            acc = np.float32(0)
            for k in range(p0, min(p0 + 128, d)):
                exact = Fraction(float(acc)) + Fraction(x[0, k].item()) * Fraction(w[e, k].item())
                acc = np.float32(float(exact))          # exact sums here fit a double: one rounding to fp32
                assert Fraction(float(np.float64(float(exact)))) == exact
            parts.append(acc)
        assert np.float32(parts[0] + parts[1]) == got[0, e].item()


@pytest.mark.parametrize("k", [1, 2, 4])
def test_topk_matches_torch_when_no_ties(k):
    g = torch.Generator().manual_seed(k)
    logits = torch.randn(500, 16, generator=g)          # fp32: ties have probability ~0
    val, idx = O.gate_topk(logits, k)
    tv, ti = torch.topk(logits, k, dim=-1, largest=True, sorted=True)
    assert torch.equal(idx, ti) and torch.equal(val, tv)
    # sorted=False may permute the slots: as sets they agree as well
    _, tu = torch.topk(logits, k, dim=-1, largest=True, sorted=False)
    assert torch.equal(torch.sort(tu, -1).values, torch.sort(idx, -1).values)
    if k == 1:
        assert torch.equal(idx[:, 0], logits.argmax(-1))


def test_topk_tie_rule_brute_force():
    g = torch.Generator().manual_seed(9)
    logits = torch.randint(0, 3, (200, 7), generator=g).half()      # many ties
    val, idx = O.gate_topk(logits, 3)
    for t in range(200):
        row = logits[t].tolist()
        taken = []
        for _ in range(3):
            best = None
            for e in range(7):
                if e in taken:
                    continue
                if best is None or row[e] > row[best]:
                    best = e                                     # first (lowest id) maximum wins
            taken.append(best)
        assert idx[t].tolist() == taken
        assert val[t].tolist() == [row[e] for e in taken]


def test_scores_match_softmax():
    g = torch.Generator().manual_seed(4)
    val = torch.randn(300, 2, generator=g).half()
    got = O.gate_scores(val, torch.float16)
    ref = F.softmax(val.float(), dim=-1)
    assert (got.float() - ref).abs().max() <= 5e-4               # one fp16 rounding
    assert torch.equal(O.gate_scores(val[:, :1], torch.float16), torch.ones(300, 1).half())  # k=1
    # fp32 in, fp32 out: equal to the library softmax to rounding
    assert torch.allclose(O.gate_scores(val.float(), torch.float32), ref, atol=1e-7)


def test_naive_gate_agrees_with_the_reference_recipe():
    """linear -> topk -> softmax with torch calls (naive_gate.py:31-38): same experts
    wherever the top-k margin exceeds the accumulation noise."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(400, 128, generator=g).half()
    w = (torch.randn(8, 128, generator=g) * 0.1).half()
    b = (torch.randn(8, generator=g) * 0.1).half()
    idx, score, logits = O.naive_gate(x, w, b, 2)
    ref_logits = F.linear(x.float(), w.float(), b.float())
    tv, ti = torch.topk(ref_logits, 3, dim=-1)
    clear = (tv[:, 1] - tv[:, 2]) > 2e-3                           # 3rd place clearly below 2nd
    clear &= (tv[:, 0] - tv[:, 1]) > 2e-3
    assert clear.sum() > 300
    assert torch.equal(idx[clear], ti[clear][:, :2])
    assert (score.float()[clear] - F.softmax(tv[clear][:, :2], -1)).abs().max() < 2e-3
    assert (logits.float() - ref_logits).abs().max() < 2e-3
