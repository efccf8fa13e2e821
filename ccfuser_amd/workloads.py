"""Seeded synthetic workloads for the per-GPU MoE layer forward.

Five named workloads cover the shapes the layer is measured and checked on.
Everything is generated on the CPU from ``torch.Generator().manual_seed(seed)``
in fp32 and then rounded to the workload's storage dtype, so the same call
produces the same bytes on every machine.  Nothing here touches the GPU; the
callers move tensors where they need them.

Weight layout follows the reference's parameter containers
(reference mix_moe/mix_moe/linear.py:198-202): ``w1 [E, f, d]``, ``b1 [E, f]``,
``w2 [E, d, f]``, ``b2 [E, d]``; the gate is ``wg [E_tot, d]``, ``bg [E_tot]``
(reference mix_moe/mix_moe/gates/naive_gate.py:22).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch


@dataclass
class Workload:
    name: str
    seed: int
    tokens: int            # T (for the expert-parallel share: inbound rows R)
    d_model: int
    d_ffn: int
    num_expert: int        # experts held by this GPU
    tot_expert: int        # experts the gate scores (== num_expert unless EP share)
    top_k: int
    dtype: torch.dtype
    capacity_factor: Optional[float] = None
    description: str = ""
    tensors: Dict[str, torch.Tensor] = field(default_factory=dict)

    @property
    def capacity(self) -> int:
        """Rows an expert may keep; -1 means unlimited."""
        if self.capacity_factor is None:
            return -1
        return int(math.ceil(self.capacity_factor * self.tokens * self.top_k / self.num_expert))

    def flops(self, routed_rows: int) -> float:
        """Expert-FFN flop for ``routed_rows`` rows: two GEMMs of 2*R*d*f each."""
        return 4.0 * routed_rows * self.d_model * self.d_ffn


_SPECS = {
    # name: (seed, T, d, f, E_local, E_tot, k, dtype, capacity_factor, zipf_s)
    "c1_tiny": (0, 512, 256, 1024, 4, 4, 1, torch.float32, None, None),
    "c2_gshard": (1, 8192, 1024, 4096, 8, 8, 2, torch.float16, 1.25, None),
    "c3_mixtral": (2, 4096, 4096, 14336, 8, 8, 2, torch.float16, None, None),
    "c4_ep_share": (3, 16384, 2048, 8192, 8, 64, 2, torch.float16, None, 1.2),
    "c5_skewed": (4, 32768, 768, 3072, 32, 32, 1, torch.float16, None, 1.5),
}

WORKLOAD_NAMES = tuple(_SPECS)


def _randn(gen: torch.Generator, *shape, std: float = 1.0) -> torch.Tensor:
    return torch.randn(*shape, generator=gen, dtype=torch.float32) * std


def _zipf_bias(gen: torch.Generator, n_expert: int, s: float) -> torch.Tensor:
    """Additive logit bias ``-s*log(rank_e)`` over a seeded expert permutation."""
    perm = torch.randperm(n_expert, generator=gen)
    rank = torch.empty(n_expert, dtype=torch.float32)
    rank[perm] = torch.arange(1, n_expert + 1, dtype=torch.float32)
    return -s * torch.log(rank)


def make_workload(name: str, *, scale_rows: Optional[int] = None) -> Workload:
    """Build one workload.

    ``scale_rows`` replaces the token count (same seed, same shapes otherwise)
    so CPU-side tests can run a small slice of a large workload.
    """
    if name not in _SPECS:
        raise KeyError(f"unknown workload {name!r}; choose from {WORKLOAD_NAMES}")
    seed, T, d, f, E, E_tot, k, dtype, cap, zipf_s = _SPECS[name]
    if scale_rows is not None:
        T = int(scale_rows)
    gen = torch.Generator().manual_seed(seed)
    wl = Workload(name=name, seed=seed, tokens=T, d_model=d, d_ffn=f, num_expert=E,
                  tot_expert=E_tot, top_k=k, dtype=dtype, capacity_factor=cap)
    t = wl.tensors
    # Expert weights first so they do not depend on the token count.
    t["w1"] = _randn(gen, E, f, d, std=0.02).to(dtype)
    t["b1"] = _randn(gen, E, f, std=0.02).to(dtype)
    t["w2"] = _randn(gen, E, d, f, std=0.02).to(dtype)
    t["b2"] = _randn(gen, E, d, std=0.02).to(dtype)
    t["wg"] = _randn(gen, E_tot, d, std=0.02).to(dtype)
    bg = _randn(gen, E_tot, std=0.02)
    if name == "c5_skewed":
        # Zipf(1.5) expert loads: the bias is part of the gate's bias vector.
        # argmax(logit + b) samples expert e with probability softmax(b) when the
        # logit noise is Gumbel(0,1) (std pi/sqrt(6)); here the noise is Gaussian
        # with std 0.02*sqrt(d), so the bias is scaled by the ratio of the two
        # standard deviations.  The head of the load curve then follows
        # r^-1.5 and about a dozen experts end up with 0-16 tokens.
        noise_ratio = 0.02 * math.sqrt(d) / (math.pi / math.sqrt(6.0))
        bg = bg + noise_ratio * _zipf_bias(gen, E_tot, zipf_s)
        wl.description = ("32768 tokens, top-1, 32 experts, gate bias ~ -1.5*log(rank) so loads "
                          "follow Zipf(1.5); several experts receive 0-16 tokens")
    t["bg"] = bg.to(dtype)
    if name == "c4_ep_share":
        _fill_ep_share(wl, gen, zipf_s)
    else:
        t["x"] = _randn(gen, T, d).to(dtype)
    if not wl.description:
        wl.description = {
            "c1_tiny": "512 tokens, top-1, 4 experts, fp32",
            "c2_gshard": "8192 tokens, top-2, 8 experts, capacity 1.25 with overflow dropped",
            "c3_mixtral": "4096 tokens, top-2, 8 experts, d=4096, ffn=14336, no capacity limit",
        }.get(name, wl.description)
    return wl


def _fill_ep_share(wl: Workload, gen: torch.Generator, zipf_s: float) -> None:
    """One GPU's expert-parallel share.

    The GPU holds ``num_expert`` of ``tot_expert`` experts.  Its inbound buffer
    holds ``tokens`` rows that 8 simulated source ranks routed to those local
    experts.  Each source contributes one contiguous span of random length; the
    rows inside a span are grouped by local expert, as a sender that has sorted
    its tokens by expert would lay them out.  The result is a list of
    ``(start, len, expert)`` segments, the same triple the reference's planner
    emits per block (reference mix_moe/mix_moe/transformer.py:242-250:
    ``start_addrs``, ``lens``, ``expert_ids``).
    """
    R, E, E_tot, d = wl.tokens, wl.num_expert, wl.tot_expert, wl.d_model
    n_src = 8
    # Expert popularity: Zipf over all experts under a seeded permutation; the
    # local experts are ids 0..E-1 and inherit whatever ranks they drew.
    logit_bias = _zipf_bias(gen, E_tot, zipf_s)
    p_local = torch.softmax(logit_bias[:E], dim=0)
    # Span lengths: a random composition of R into n_src positive parts.
    cuts = torch.sort(torch.randperm(R - 1, generator=gen)[: n_src - 1] + 1).values
    bounds = torch.cat([torch.tensor([0]), cuts, torch.tensor([R])])
    seg_start: List[int] = []
    seg_len: List[int] = []
    seg_expert: List[int] = []
    seg_source: List[int] = []
    for s in range(n_src):
        lo, hi = int(bounds[s]), int(bounds[s + 1])
        draws = torch.multinomial(p_local, hi - lo, replacement=True, generator=gen)
        cnt = torch.bincount(draws, minlength=E)
        at = lo
        for e in range(E):
            c = int(cnt[e])
            if c:
                seg_start.append(at)
                seg_len.append(c)
                seg_expert.append(e)
                seg_source.append(s)
                at += c
    t = wl.tensors
    t["x"] = _randn(gen, R, d).to(wl.dtype)
    t["seg_start"] = torch.tensor(seg_start, dtype=torch.int32)
    t["seg_len"] = torch.tensor(seg_len, dtype=torch.int32)
    t["seg_expert"] = torch.tensor(seg_expert, dtype=torch.int32)
    t["seg_source"] = torch.tensor(seg_source, dtype=torch.int32)
    t["zipf_bias"] = logit_bias
    wl.description = ("16384 inbound rows for 8 local of 64 experts, laid out as 8 contiguous "
                      "per-source spans each grouped by local expert; Zipf(1.2) expert loads")
