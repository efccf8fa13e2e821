"""Pins the oracle's scatter / FFN / un-permute / combine against brute force,
library routines and closed forms, and the golden fixture."""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _case(T, d, f, E, k, seed, dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s, std=1.0: (torch.randn(*s, generator=g) * std).to(dtype)
    return dict(x=mk(T, d), wg=mk(E, d, std=0.1), bg=mk(E, std=0.1), w1=mk(E, f, d, std=0.1),
                b1=mk(E, f, std=0.1), w2=mk(E, d, f, std=0.1), b2=mk(E, d, std=0.1))


def test_gelu_is_the_erf_form():
    h = torch.linspace(-6, 6, 1001)
    assert torch.allclose(O.gelu_exact(h), F.gelu(h, approximate="none"), atol=1e-6)
    assert abs(O.gelu_exact(torch.tensor(1.0)).item() - 0.5 * (1 + math.erf(1 / math.sqrt(2)))) < 1e-7
    # not the tanh approximation
    assert (O.gelu_exact(h) - F.gelu(h, approximate="tanh")).abs().max() > 1e-4


@pytest.mark.parametrize("k", [1, 2, 3])
def test_layer_equals_per_token_brute_force(k):
    """Textbook triple loops, token by token (the form of cpuF16F16Gemm, csrc/test.cpp:215-226)."""
    c = _case(10, 8, 12, 4, k, seed=k)
    r = O.moe_layer_forward(**c, top_k=k)
    x, w1, b1, w2, b2 = (c[n].double() for n in ("x", "w1", "b1", "w2", "b2"))
    for t in range(10):
        acc = [0.0] * 8
        for s in range(k):
            e = int(r["idx"][t, s])
            h = []
            for n in range(12):
                v = sum(float(x[t, q]) * float(w1[e, n, q]) for q in range(8)) + float(b1[e, n])
                h.append(0.5 * v * (1 + math.erf(v / math.sqrt(2))))
            for m in range(8):
                y = sum(h[n] * float(w2[e, m, n]) for n in range(12)) + float(b2[e, m])
                acc[m] += float(r["score"][t, s]) * y
        assert np.allclose(r["out"][t].numpy(), acc, atol=2e-5)


def test_special_cases():
    c = _case(64, 16, 32, 5, 1, seed=11)
    # k = 1: score == 1, out[t] is exactly the expert output of the chosen expert
    r = O.moe_layer_forward(**c, top_k=1)
    assert torch.equal(r["score"], torch.ones(64, 1).half())
    assert torch.equal(r["out"], r["y_flat"])
    # single expert: a dense MLP
    c1 = _case(20, 16, 32, 1, 1, seed=12)
    r1 = O.moe_layer_forward(**c1, top_k=1)
    dense = F.linear(F.gelu(F.linear(c1["x"].float(), c1["w1"][0].float(), c1["b1"][0].float())),
                     c1["w2"][0].float(), c1["b2"][0].float())
    assert torch.allclose(r1["out"], dense, atol=1e-5)
    # zero weights: out = sum_s score * b2[e]   (+ gelu(b1) has no path to the output)
    z = dict(c)
    z["w1"] = torch.zeros_like(c["w1"]); z["w2"] = torch.zeros_like(c["w2"])
    rz = O.moe_layer_forward(**z, top_k=1)
    assert torch.allclose(rz["out"], c["b2"].float()[rz["idx"][:, 0]], atol=1e-6)
    # dropped slots contribute nothing
    rd = O.moe_layer_forward(**c, top_k=1, capacity=3)
    dropped = rd["idx_kept"].view(-1) < 0
    assert dropped.any() and (rd["out"][dropped] == 0).all()
    assert torch.equal(rd["out"][~dropped], r["out"][~dropped])


def test_stages_match_library_forms():
    c = _case(50, 16, 24, 3, 2, seed=13)
    r = O.moe_layer_forward(**c, top_k=2)
    pos = r["pos"]
    # scatter == index_select(x, pos // k)  (layers.py:19-21 / 389)
    buf = O.local_scatter(c["x"], pos, 2)
    assert torch.equal(buf, c["x"][pos // 2])
    # un-permute == index_copy_, and it inverts the scatter on a permutation
    assert torch.equal(O.unpermute(r["y_sorted"], pos, 100)[pos], r["y_sorted"])
    # combine == bmm == explicit weighted sum
    y = r["y_flat"].view(50, 2, 16)
    s = r["score"].float()
    assert torch.allclose(r["out"], s[:, 0:1] * y[:, 0] + s[:, 1:2] * y[:, 1], atol=1e-6)
    # the torch-only layer (the timed baseline) agrees with the staged oracle
    ref = O.reference_layer_torch(*[c[n].float() for n in ("x", "wg", "bg", "w1", "b1", "w2", "b2")], 2)
    same = torch.equal(torch.sort(r["idx"], -1).values,
                       torch.sort(torch.topk(F.linear(c["x"].float(), c["wg"].float(), c["bg"].float()), 2).indices, -1).values)
    if same:
        assert O.max_abs_err(ref, r["out"]) < 2e-3      # fp16 score rounding only


def test_round_intermediate_models_fp16_storage():
    c = _case(40, 32, 64, 2, 1, seed=14)
    a = O.moe_layer_forward(**c, top_k=1)
    b = O.moe_layer_forward(**c, top_k=1, round_intermediate=torch.float16)
    assert torch.equal(b["y_sorted"], b["y_sorted"].half().float())
    assert 0 < O.max_abs_err(a["out"], b["out"]) < 2e-2


def test_segments_equal_sorted_ffn():
    c = _case(30, 16, 24, 3, 1, seed=15)
    seg_start = torch.tensor([0, 5, 12, 20, 26], dtype=torch.int32)
    seg_len = torch.tensor([5, 7, 8, 6, 4], dtype=torch.int32)
    seg_expert = torch.tensor([2, 0, 2, 1, 0], dtype=torch.int32)
    y = O.ffn_segments(c["x"], seg_start, seg_len, seg_expert, c["w1"], c["b1"], c["w2"], c["b2"])
    for s, n, e in zip(seg_start.tolist(), seg_len.tolist(), seg_expert.tolist()):
        dense = F.linear(F.gelu(F.linear(c["x"][s:s + n].float(), c["w1"][e].float(), c["b1"][e].float())),
                         c["w2"][e].float(), c["b2"][e].float())
        assert torch.allclose(y[s:s + n], dense, atol=1e-5)


def test_golden_fixture_is_reproduced():
    z = np.load(os.path.join(GOLDEN, "layer_small.npz"))
    t = {n: torch.from_numpy(z[n]) for n in ("x", "wg", "bg", "w1", "b1", "w2", "b2")}
    r = O.moe_layer_forward(**t, top_k=int(z["top_k"]), capacity=int(z["capacity"]))
    for n in ("logits", "idx", "idx_kept", "score", "counts", "offsets", "pos"):
        assert np.array_equal(r[n].numpy(), z[n]), n
    assert np.allclose(r["out"].numpy(), z["out"], atol=1e-5)
    assert (z["idx_kept"] < 0).any()                      # the fixture exercises capacity drops
