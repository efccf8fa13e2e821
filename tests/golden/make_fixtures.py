"""Writes the fixtures under tests/golden/.  Run from the repository root:

    python tests/golden/make_fixtures.py

Two kinds of data:

* ``ref_pos_div2.npy`` and ``ref_all_expert_count.npy`` are the two input
  vectors the reference ships for its own checks (mix_moe/csrc/pos.pt, used by
  the scatter check in csrc/test.cpp:405-449, and mix_moe/mix_moe/all_expert_count.pt,
  used by mix_moe/mix_moe/t.py:143).  They are tensors saved with torch.save; they
  are read with ``torch.load(weights_only=True)`` (which executes nothing from
  the file) and re-saved as plain .npy so the tests need neither the reference
  tree nor a pickle loader.  They are inputs only: the reference holds no
  expected outputs for this path.
* ``layer_small.npz`` holds a small seeded layer case with every intermediate
  the oracle computes (logits, expert choice, scores, counts, offsets, pos,
  output), so that a change in the oracle's rules shows up as a diff here.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
REF = "/root/reference/mix_moe"


def reference_inputs():
    pos = torch.load(os.path.join(REF, "csrc", "pos.pt"), map_location="cpu", weights_only=True)
    assert pos.dtype == torch.int64 and pos.shape == (8192,)
    np.save(os.path.join(HERE, "ref_pos_div2.npy"), pos.numpy())
    cnt = torch.load(os.path.join(REF, "mix_moe", "all_expert_count.pt"), map_location="cpu",
                     weights_only=True)
    assert cnt.dtype == torch.int64 and cnt.shape == (4, 64)
    np.save(os.path.join(HERE, "ref_all_expert_count.npy"), cnt.numpy())


def layer_small():
    from oracle import moe_oracle as O
    g = torch.Generator().manual_seed(1234)
    T, d, f, E, k = 96, 64, 128, 6, 2
    x = torch.randn(T, d, generator=g).half()
    wg = (torch.randn(E, d, generator=g) * 0.1).half()
    bg = (torch.randn(E, generator=g) * 0.1).half()
    w1 = (torch.randn(E, f, d, generator=g) * 0.05).half()
    b1 = (torch.randn(E, f, generator=g) * 0.05).half()
    w2 = (torch.randn(E, d, f, generator=g) * 0.05).half()
    b2 = (torch.randn(E, d, generator=g) * 0.05).half()
    cap = 30
    r = O.moe_layer_forward(x, wg, bg, w1, b1, w2, b2, k, capacity=cap)
    np.savez_compressed(
        os.path.join(HERE, "layer_small.npz"),
        x=x.numpy(), wg=wg.numpy(), bg=bg.numpy(), w1=w1.numpy(), b1=b1.numpy(), w2=w2.numpy(),
        b2=b2.numpy(), top_k=np.int64(k), capacity=np.int64(cap),
        logits=r["logits"].numpy(), idx=r["idx"].numpy(), idx_kept=r["idx_kept"].numpy(),
        score=r["score"].numpy(), counts=r["counts"].numpy(), offsets=r["offsets"].numpy(),
        pos=r["pos"].numpy(), out=r["out"].numpy())


if __name__ == "__main__":
    if os.path.isdir(REF):
        reference_inputs()
    else:
        print("reference tree not present: keeping the committed reference input vectors")
    layer_small()
    print("fixtures written to", HERE)
