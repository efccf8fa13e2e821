"""CPU oracle for the per-GPU MoE layer forward and backward.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU with numpy and torch's CPU kernels, the
arithmetic of the reference's MoE layer forward, and the gradients of it that
the reference's backward pair computes:

    gate (linear -> top-k -> softmax)      mix_moe/mix_moe/gates/naive_gate.py:26-45
    expert count, cumulative sum, pos      mix_moe/mix_moe/functions.py:83-105
                                           mix_moe/csrc/cuda/local_exchange.cu:6-17,37-70
    token scatter into expert order        mix_moe/mix_moe/layers.py:19-21, 389
                                           mix_moe/csrc/cuda/mix_moe_kernel.cu:18-33
    expert FFN (mm+bias, GELU, mm+bias)    mix_moe/mix_moe/layers.py:401-429
                                           mix_moe/csrc/cuda/mix_gemm.cu:282-345, 439-490
    un-permute to flat token*k order       mix_moe/csrc/mix_moe.h:431-433
    gate-weighted combine                  mix_moe/mix_moe/layers.py:550-559
    64-row block planner (one GPU)         mix_moe/mix_moe/transformer.py:150-250
    backward of the two expert GEMMs       mix_moe/csrc/mix_moe.h:300-388, 439-505
                                           mix_moe/mix_moe/linear.py:91-113, 148-173

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import it.  The product (``ccfuser_amd``) never does; its
device path fails loudly when the HIP library is missing.

Where the reference leaves a result unspecified this file fixes a rule, and
the HIP kernels implement the same rule:

* gate logits are accumulated in fp32 in a fixed order (``gate_logits``), so
  that the top-k selection is reproducible bit for bit;
* ``torch.topk(sorted=False)`` leaves slot order and ties open: here slot 0
  holds the largest logit and equal logits go to the lower expert id;
* ``assign_pos`` fills each expert's segment through an atomic race: here the
  flat indices inside a segment ascend (a stable sort by expert id), which is
  one of the orders the reference can produce;
* capacity limiting is absent from the reference (only the ``-1`` plumbing
  exists, local_exchange.cu:12,48): here an expert keeps its first ``capacity``
  slots in flat-index order and the rest become ``-1``.

Pinning.  Every function below is checked in ``tests/test_oracle_*.py`` against
something other than its own formula: torch library routines (``F.linear``,
``topk``, ``softmax``, ``bincount``, ``cumsum``, stable ``sort``,
``index_select``, ``F.gelu``, ``bmm``), brute-force Python loops on tiny
inputs, closed forms (k=1, single expert, zero weights), and the two input
vectors the reference ships (csrc/pos.pt, mix_moe/all_expert_count.pt).  The
backward functions are closed-form chain rules and use no autograd; they are
pinned against torch's autograd through library operations (``F.linear``,
``topk``, ``softmax``, ``index_select``, ``F.gelu``, ``index_copy``, ``bmm``)
and against central finite differences in float64 on tiny inputs.  The
reference holds no expected-output vectors for this path and its Python cannot
be imported without its CUDA extension, so the third-party arithmetic it
delegates to torch (README pins torch 2.0.1) is pinned by the textbook
definitions as computed by the torch build installed here; at that boundary
parity is unpinned.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn.functional as F

PART = 128         # consecutive K elements whose products are summed as one chain


# --------------------------------------------------------------------------
# gate
# --------------------------------------------------------------------------
def gate_logits(x: torch.Tensor, wg: torch.Tensor, bg: Optional[torch.Tensor]) -> torch.Tensor:
    """``x @ wg.T + bg`` accumulated in fp32 in a fixed order; returns fp32 [T, E].

    Follows ``self.gate(inp)`` (naive_gate.py:31).  The order: K is cut into
    parts of 128 consecutive elements (the last may be shorter); a part's sum
    starts at zero and takes its products one at a time in ascending K; the
    part sums are added one after the other in ascending order, starting from
    the first; the bias is added last.  Products of two fp16 values are exact
    in fp32, so for fp16 inputs ``acc + x*w`` with the product rounded first is
    the same number as a fused multiply-add; for fp32 inputs the multiply is
    rounded before the add (no fused multiply-add).
    """
    T, d = x.shape
    E = wg.shape[0]
    if d % 8:
        raise ValueError("d_model must be a multiple of 8")
    x32 = np.ascontiguousarray(x.detach().to(torch.float32).numpy().T)     # [d, T]
    w32 = np.ascontiguousarray(wg.detach().to(torch.float32).numpy().T)    # [d, E]
    out = np.empty((T, E), np.float32)
    step = max(1, (1 << 22) // max(1, E))              # bound the temporaries
    for t0 in range(0, T, step):
        xs = x32[:, t0:t0 + step]
        total = None
        for p0 in range(0, d, PART):
            acc = np.zeros((xs.shape[1], E), np.float32)
            for k in range(p0, min(p0 + PART, d)):
                acc = acc + xs[k][:, None] * w32[k][None, :]
            total = acc if total is None else total + acc
        out[t0:t0 + step] = total
    if bg is not None:
        out = out + bg.detach().to(torch.float32).numpy()[None, :]
    return torch.from_numpy(out)


def round_logits(logits32: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """The reference's gate is an ``nn.Linear`` in the model dtype, so its logits
    are rounded to that dtype once (naive_gate.py:31 under ``model.half()``)."""
    return logits32.to(dtype)


def gate_topk(logits: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Top-k of each row: values descending, ties to the lower expert id.

    Follows ``torch.topk(gate, k, dim=-1, largest=True, sorted=False)``
    (naive_gate.py:32-34), whose slot order and tie handling are unspecified.
    Returns ``(val [T,k] in logits' dtype, idx [T,k] int64)``.
    """
    T, E = logits.shape
    if k > E:
        raise ValueError("top_k exceeds the number of experts")
    v = logits.to(torch.float32).numpy()
    # lexsort: last key is primary.  primary = -value (descending), secondary = expert id.
    ids = np.broadcast_to(np.arange(E), (T, E))
    order = np.lexsort((ids, -v), axis=1)[:, :k]
    idx = torch.from_numpy(np.ascontiguousarray(order)).to(torch.int64)
    val = torch.gather(logits, 1, idx)
    return val, idx


def gate_scores(val: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Softmax over the k selected logits (naive_gate.py:35-38), fp32 inside,
    rounded once to ``dtype``."""
    v = val.to(torch.float32)
    m = v.max(dim=-1, keepdim=True).values
    e = torch.exp(v - m)
    return (e / e.sum(dim=-1, keepdim=True)).to(dtype)


def naive_gate(x, wg, bg, k: int):
    """(idx int64 [T,k], score [T,k] in x.dtype, logits [T,E] in x.dtype)."""
    logits = round_logits(gate_logits(x, wg, bg), x.dtype)
    val, idx = gate_topk(logits, k)
    return idx, gate_scores(val, x.dtype), logits


# --------------------------------------------------------------------------
# count / scan / pos
# --------------------------------------------------------------------------
def limit_by_capacity(idx: torch.Tensor, num_expert: int, capacity: int) -> torch.Tensor:
    """Drop overflow: expert ``e`` keeps its first ``capacity`` slots in flat
    index (t*k+s) order, later ones become -1.  ``capacity < 0`` keeps all."""
    flat = idx.reshape(-1).clone()
    if capacity < 0:
        return flat.view_as(idx)
    seen = [0] * num_expert
    fl = flat.tolist()
    for i, e in enumerate(fl):
        if e < 0:
            continue
        if seen[e] >= capacity:
            fl[i] = -1
        else:
            seen[e] += 1
    return torch.tensor(fl, dtype=torch.int64).view_as(idx)


def expert_count(idx: torch.Tensor, num_expert: int) -> torch.Tensor:
    """int32 [E] histogram of the non-negative entries (local_exchange.cu:37-70)."""
    flat = idx.reshape(-1)
    cnt = np.zeros(num_expert, np.int32)
    for e in flat.tolist():
        if e == -1:
            continue
        cnt[e] += 1
    return torch.from_numpy(cnt)


def assign_pos(idx: torch.Tensor, num_expert: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """(pos int64 [R], offsets int32 [E+1]).

    ``pos`` lists the flat indices grouped by expert (functions.py:100-103,
    local_exchange.cu:6-17: ``pos[--cum[e]] = i``); inside a segment the flat
    indices ascend.  ``offsets`` is the exclusive scan of the counts, so
    segment ``e`` is ``pos[offsets[e]:offsets[e+1]]``.
    """
    flat = idx.reshape(-1).tolist()
    buckets: List[List[int]] = [[] for _ in range(num_expert)]
    for i, e in enumerate(flat):
        if e > -1:
            buckets[e].append(i)
    offsets = [0]
    for b in buckets:
        offsets.append(offsets[-1] + len(b))
    pos = [i for b in buckets for i in b]
    return (torch.tensor(pos, dtype=torch.int64),
            torch.tensor(offsets, dtype=torch.int32))


def inverse_pos(pos: torch.Tensor, n_flat: int) -> torch.Tensor:
    """int32 [n_flat]: row of flat slot i in expert order, -1 if dropped."""
    inv = torch.full((n_flat,), -1, dtype=torch.int32)
    inv[pos] = torch.arange(pos.numel(), dtype=torch.int32)
    return inv


# --------------------------------------------------------------------------
# scatter / FFN / un-permute / combine
# --------------------------------------------------------------------------
def local_scatter(x: torch.Tensor, pos: torch.Tensor, top_k: int) -> torch.Tensor:
    """``buf[j] = x[pos[j] // k]`` (layers.py:19-21 with 389; mix_moe.h:250-253)."""
    return torch.index_select(x, 0, torch.div(pos, top_k, rounding_mode="floor"))


def gelu_exact(h: torch.Tensor) -> torch.Tensor:
    """erf-form GELU, ``0.5*h*(1+erf(h/sqrt(2)))`` (transformer.py:88, 445)."""
    return 0.5 * h * (1.0 + torch.erf(h * (1.0 / math.sqrt(2.0))))


def expert_ffn(buf: torch.Tensor, offsets: torch.Tensor, w1, b1, w2, b2,
               *, round_intermediate: Optional[torch.dtype] = None) -> torch.Tensor:
    """Rows ``offsets[e]:offsets[e+1]`` go through expert ``e``:
    ``gelu(buf @ w1[e].T + b1[e]) @ w2[e].T + b2[e]`` (layers.py:410-419).

    Computed in fp32 from the stored values.  ``round_intermediate`` rounds the
    activation and the result to that dtype, as a kernel that stores them in
    fp16 does; None keeps pure fp32.
    """
    off = offsets.tolist()
    out = torch.zeros(buf.shape[0], w2.shape[1], dtype=torch.float32)
    b32 = buf.to(torch.float32)
    for e in range(len(off) - 1):
        lo, hi = off[e], off[e + 1]
        if hi == lo:
            continue
        h = torch.mm(b32[lo:hi], w1[e].to(torch.float32).t()) + b1[e].to(torch.float32)
        h = gelu_exact(h)
        if round_intermediate is not None:
            h = h.to(round_intermediate).to(torch.float32)
        y = torch.mm(h, w2[e].to(torch.float32).t()) + b2[e].to(torch.float32)
        out[lo:hi] = y
    if round_intermediate is not None:
        out = out.to(round_intermediate).to(torch.float32)
    return out


def unpermute(y_sorted: torch.Tensor, pos: torch.Tensor, n_flat: int) -> torch.Tensor:
    """``y_flat[pos[j]] = y_sorted[j]``, dropped slots stay zero (mix_moe.h:423-433)."""
    out = torch.zeros(n_flat, y_sorted.shape[1], dtype=y_sorted.dtype)
    out.index_copy_(0, pos, y_sorted)
    return out


def combine(y_flat: torch.Tensor, score: torch.Tensor, top_k: int) -> torch.Tensor:
    """``out[t] = sum_s score[t,s] * y_flat[t*k+s]`` via bmm (layers.py:550-559)."""
    d = y_flat.shape[-1]
    y = y_flat.view(-1, top_k, d)
    g = score.to(y.dtype).view(-1, 1, top_k)
    return torch.bmm(g, y).reshape(-1, d)


def moe_layer_forward(x, wg, bg, w1, b1, w2, b2, top_k: int, *, capacity: int = -1,
                      round_intermediate: Optional[torch.dtype] = None) -> Dict[str, torch.Tensor]:
    """The whole layer (transformer.py:475-497 -> layers.py:501-559) on the CPU.

    Returns every intermediate so tests can compare stage by stage.  ``out`` is
    fp32; with ``round_intermediate`` the activation, the expert output and the
    gate scores carry the rounding a fp16 pipeline applies.
    """
    T = x.shape[0]
    E = w1.shape[0]
    idx, score, logits = naive_gate(x, wg, bg, top_k)
    idx_kept = limit_by_capacity(idx, E, capacity)
    counts = expert_count(idx_kept, E)
    pos, offsets = assign_pos(idx_kept, E)
    buf = local_scatter(x, pos, top_k)
    y_sorted = expert_ffn(buf, offsets, w1, b1, w2, b2, round_intermediate=round_intermediate)
    y_flat = unpermute(y_sorted, pos, T * top_k)
    out = combine(y_flat, score.to(torch.float32), top_k)
    return {"logits": logits, "idx": idx, "idx_kept": idx_kept, "score": score,
            "counts": counts, "offsets": offsets, "pos": pos, "y_sorted": y_sorted,
            "y_flat": y_flat, "out": out}


def ffn_segments(x, seg_start, seg_len, seg_expert, w1, b1, w2, b2, *,
                 round_intermediate: Optional[torch.dtype] = None) -> torch.Tensor:
    """Expert FFN over rows addressed by (start, len, expert) triples, output in
    the input's row layout.  One triple is what the reference plans per block
    (transformer.py:242-250) and its kernels address with ``start_addrs``,
    ``lens``, ``expert_ids`` (mix_gemm.cu:296-301, 449-456)."""
    out = torch.zeros(x.shape[0], w2.shape[1], dtype=torch.float32)
    for s, n, e in zip(seg_start.tolist(), seg_len.tolist(), seg_expert.tolist()):
        if n == 0:
            continue
        off = torch.tensor([0, n], dtype=torch.int32)
        out[s:s + n] = expert_ffn(x[s:s + n], off, w1[e:e + 1], b1[e:e + 1], w2[e:e + 1],
                                  b2[e:e + 1], round_intermediate=round_intermediate)
    return out


# --------------------------------------------------------------------------
# backward of the same path (closed-form chain rule, fp32, no autograd)
# --------------------------------------------------------------------------
def combine_backward(grad_out: torch.Tensor, y_flat: torch.Tensor, score: torch.Tensor,
                     top_k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Backward of ``combine`` (the bmm at layers.py:556): ``grad_y_flat[t*k+s] =
    score[t,s] * grad_out[t]`` and ``grad_score[t,s] = <grad_out[t], y_flat[t*k+s]>``."""
    g = grad_out.to(torch.float32)
    sc = score.to(torch.float32).reshape(-1, top_k)
    gy = (sc[:, :, None] * g[:, None, :]).reshape(-1, g.shape[1])
    gs = (y_flat.to(torch.float32).view(-1, top_k, g.shape[1]) * g[:, None, :]).sum(-1)
    return gy, gs


def gelu_backward(grad_act: torch.Tensor, h_pre: torch.Tensor) -> torch.Tensor:
    """d/dh of the erf GELU: ``Phi(h) + h * phi(h)`` times the incoming gradient."""
    h = h_pre.to(torch.float32)
    cdf = 0.5 * (1.0 + torch.erf(h * (1.0 / math.sqrt(2.0))))
    pdf = torch.exp(-0.5 * h * h) * (1.0 / math.sqrt(2.0 * math.pi))
    return grad_act.to(torch.float32) * (cdf + h * pdf)


def ffn2_backward(grad_y_flat: torch.Tensor, act: torch.Tensor, pos: torch.Tensor,
                  offsets: torch.Tensor, w2: torch.Tensor):
    """``second_gemm_backward`` (mix_moe.h:439-505): the gradient rows are brought into
    expert order (``local_scatter`` at 453-454, the inverse of the index_copy_ at 433),
    ``grad_act = gy @ w2[e]`` (first_mix_gemm at 470-483 with the stored [E, d, f]
    weight as [E, K, N]), ``grad_w2[e] = gy^T @ act`` (launch_compute_weight_grad,
    497-503).  The reference returns ``grad_bias`` uninitialised (489); here it is the
    column sum of ``gy`` over the expert's rows, which is what the forward's
    ``+ b2[e]`` differentiates to.  Returns (grad_act [R, f], grad_w2, grad_b2)."""
    off = offsets.tolist()
    gy = grad_y_flat.to(torch.float32)[pos]
    a32 = act.to(torch.float32)
    E, d, f = w2.shape
    g_act = torch.zeros(gy.shape[0], f)
    g_w = torch.zeros(E, d, f)
    g_b = torch.zeros(E, d)
    for e in range(E):
        lo, hi = off[e], off[e + 1]
        if hi == lo:
            continue
        g_act[lo:hi] = torch.mm(gy[lo:hi], w2[e].to(torch.float32))
        g_w[e] = torch.mm(gy[lo:hi].t(), a32[lo:hi])
        g_b[e] = gy[lo:hi].sum(0)
    return g_act, g_w, g_b


def ffn1_backward(grad_h: torch.Tensor, x: torch.Tensor, pos: torch.Tensor, top_k: int,
                  offsets: torch.Tensor, w1: torch.Tensor):
    """``first_gemm_backward`` (mix_moe.h:300-388): ``grad_buf = grad_h @ w1[e]``
    (second_mix_gemm at 322-335 with the stored [E, f, d] weight as [E, K, N]),
    ``grad_w1[e] = grad_h^T @ buf`` (347-353), and the rows added back onto their
    tokens, ``grad_in.index_add_(0, pos // k, grad_buf)`` (359-365).  ``grad_bias``
    as in ``ffn2_backward``.  Returns (grad_in [T, d], grad_w1, grad_b1)."""
    off = offsets.tolist()
    gh = grad_h.to(torch.float32)
    src = torch.div(pos, top_k, rounding_mode="floor")
    buf = x.to(torch.float32)[src]
    E, f, d = w1.shape
    g_buf = torch.zeros(gh.shape[0], d)
    g_w = torch.zeros(E, f, d)
    g_b = torch.zeros(E, f)
    for e in range(E):
        lo, hi = off[e], off[e + 1]
        if hi == lo:
            continue
        g_buf[lo:hi] = torch.mm(gh[lo:hi], w1[e].to(torch.float32))
        g_w[e] = torch.mm(gh[lo:hi].t(), buf[lo:hi])
        g_b[e] = gh[lo:hi].sum(0)
    g_in = torch.zeros(x.shape[0], d)
    g_in.index_add_(0, src, g_buf)
    return g_in, g_w, g_b


def gate_backward(grad_score: torch.Tensor, score: torch.Tensor, idx: torch.Tensor,
                  x: torch.Tensor, wg: torch.Tensor):
    """Backward of ``NaiveGate.forward`` (naive_gate.py:31-38) for the gradient of the
    scores: softmax over the k selected logits, the selection as a scatter into
    [T, E], then the linear layer.  Returns (grad_x [T, d], grad_wg, grad_bg)."""
    T, k = idx.shape
    s = score.to(torch.float32).reshape(T, k)
    g = grad_score.to(torch.float32).reshape(T, k)
    g_val = s * (g - (s * g).sum(-1, keepdim=True))
    g_logits = torch.zeros(T, wg.shape[0])
    g_logits.scatter_add_(1, idx, g_val)
    return (torch.mm(g_logits, wg.to(torch.float32)), torch.mm(g_logits.t(), x.to(torch.float32)),
            g_logits.sum(0))


def moe_layer_backward(x, wg, bg, w1, b1, w2, b2, top_k: int, grad_out: torch.Tensor, *,
                       capacity: int = -1) -> Dict[str, torch.Tensor]:
    """Gradients of ``moe_layer_forward``'s ``out`` with respect to ``x`` and every
    parameter, for the incoming ``grad_out`` [T, d]: the forward is recomputed in fp32
    and the stages above are chained in reverse.  The routing is piecewise constant."""
    T = x.shape[0]
    E = w1.shape[0]
    idx, score, _ = naive_gate(x, wg, bg, top_k)
    idx_kept = limit_by_capacity(idx, E, capacity)
    pos, offsets = assign_pos(idx_kept, E)
    off = offsets.tolist()
    buf = local_scatter(x, pos, top_k).to(torch.float32)
    h_pre = torch.zeros(buf.shape[0], w1.shape[1])
    y_sorted = torch.zeros(buf.shape[0], w2.shape[1])
    for e in range(E):
        lo, hi = off[e], off[e + 1]
        if hi > lo:
            h_pre[lo:hi] = torch.mm(buf[lo:hi], w1[e].to(torch.float32).t()) + b1[e].to(torch.float32)
            y_sorted[lo:hi] = torch.mm(gelu_exact(h_pre[lo:hi]), w2[e].to(torch.float32).t()) \
                + b2[e].to(torch.float32)
    act = gelu_exact(h_pre)
    y_flat = unpermute(y_sorted, pos, T * top_k)
    g_y_flat, g_score = combine_backward(grad_out, y_flat, score, top_k)
    g_act, g_w2, g_b2 = ffn2_backward(g_y_flat, act, pos, offsets, w2)
    g_h = gelu_backward(g_act, h_pre)
    g_x, g_w1, g_b1 = ffn1_backward(g_h, x, pos, top_k, offsets, w1)
    gx_gate, g_wg, g_bg = gate_backward(g_score, score, idx, x, wg)
    return {"x": g_x + gx_gate, "x_experts": g_x, "x_gate": gx_gate, "wg": g_wg, "bg": g_bg,
            "w1": g_w1, "b1": g_b1, "w2": g_w2, "b2": g_b2, "score": g_score, "act": g_act,
            "h": g_h, "y_flat": g_y_flat, "h_pre": h_pre, "act_fwd": act, "y_flat_fwd": y_flat,
            "pos": pos, "offsets": offsets, "idx": idx, "score_fwd": score}


# --------------------------------------------------------------------------
# block planner (one GPU)
# --------------------------------------------------------------------------
def divide_into_block(counts: Sequence[int], block_size: int = 64) -> Dict[str, List[int]]:
    """Block plan of ``AsyncExpertAssignment.divide_into_block`` at world_size 1
    with the identity expert plan (transformer.py:150-250).

    Per expert, in id order: full ``block_size``-row blocks go to the "local"
    list and a shorter tail to the "remote" list (191-193); the two lists are
    interleaved l0, r0, l1, r1, ... (199); ``expert_block_ids`` /
    ``expert_block_id_idxs`` form a CSR from expert to its blocks (213-219).

    One departure: the reference only emits a tail when the expert also has a
    full block (the tail test sits inside ``if count >= block_size``, 184-193),
    which loses experts with fewer than ``block_size`` rows; here every
    non-empty tail is planned so the blocks tile every segment exactly.
    """
    local, remote = [], []
    start = 0
    for e, c in enumerate(counts):
        c = int(c)
        nfull = c // block_size
        for b in range(nfull):
            local.append((e, block_size, start + b * block_size))
        if c % block_size:
            remote.append((e, c % block_size, start + nfull * block_size))
        start += c
    plan = []
    for i in range(max(len(local), len(remote))):
        if i < len(local):
            plan.append(local[i])
        if i < len(remote):
            plan.append(remote[i])
    expert_ids = [p[0] for p in plan]
    by_expert: List[List[int]] = [[] for _ in counts]
    for b, e in enumerate(expert_ids):
        by_expert[e].append(b)
    ids, idxs = [], [0]
    for lst in by_expert:
        ids.extend(lst)
        idxs.append(len(ids))
    return {"expert_ids": expert_ids, "local_expert_id_indexs": list(expert_ids),
            "ranks": [0] * len(plan), "lens": [p[1] for p in plan],
            "start_addrs": [p[2] for p in plan], "total_block_num": len(plan),
            "remote_block_num": len(remote), "expert_block_ids": ids,
            "expert_block_id_idxs": idxs}


# --------------------------------------------------------------------------
# tolerance metrics used by the parity tests and the smoke check
# --------------------------------------------------------------------------
def max_abs_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    return float((got.to(torch.float32) - ref.to(torch.float32)).abs().max())


def mean_rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    """mean|got-ref| / mean|ref| (a ratio of means: elementwise ratios blow up
    at the zeros every activation tensor has)."""
    g, r = got.to(torch.float32), ref.to(torch.float32)
    return float((g - r).abs().mean() / r.abs().mean().clamp_min(1e-30))


# --------------------------------------------------------------------------
# the layer through torch library calls only (the timed CPU baseline)
# --------------------------------------------------------------------------
def reference_layer_torch(x, wg, bg, w1, b1, w2, b2, top_k: int, *, capacity: int = -1) -> torch.Tensor:
    """The layer written the way the reference writes it, one torch call per
    step, computing in fp32 on whatever CPU threads torch has: ``F.linear`` ->
    ``topk`` -> ``softmax`` (naive_gate.py:31-38); ``bincount``/``cumsum`` and a
    stable sort for ``pos`` (functions.py:83-105); ``index_select``
    (layers.py:19-21); per-expert ``mm``+bias, GELU, ``mm``+bias
    (layers.py:410-419); ``index_copy_`` (mix_moe.h:433); ``bmm``
    (layers.py:556).  Inputs are expected in fp32 already (fp16 workloads are
    upcast once by the caller, outside the timed region).  This is what
    ``bench.py`` times as ``cpu_baseline``; the selection here uses torch's own
    accumulation order, so it is a speed baseline, not the parity checker.
    """
    T, d = x.shape
    E = w1.shape[0]
    logits = F.linear(x, wg, bg)
    val, idx = torch.topk(logits, k=top_k, dim=-1, largest=True, sorted=False)
    score = F.softmax(val.view(-1, top_k), dim=-1)
    flat = idx.reshape(-1)
    if capacity >= 0:
        order = torch.sort(flat, stable=True).indices
        cnt_all = torch.bincount(flat, minlength=E)
        start = torch.cumsum(cnt_all, 0) - cnt_all
        rank = torch.empty_like(flat)
        rank[order] = torch.arange(flat.numel()) - start[flat[order]]
        flat = torch.where(rank < capacity, flat, torch.full_like(flat, -1))
    keep = flat > -1
    cnt = torch.bincount(flat[keep], minlength=E)
    cum = torch.cumsum(cnt, 0)
    order = torch.sort(torch.where(keep, flat, torch.full_like(flat, E)), stable=True).indices
    pos = order[: int(cum[-1])]
    buf = torch.index_select(x, 0, torch.div(pos, top_k, rounding_mode="floor"))
    outs = []
    base = 0
    for e in range(E):
        n = int(cnt[e])
        sl = buf[base:base + n]
        h = torch.mm(sl, w1[e].t()) + b1[e]
        h = F.gelu(h)
        outs.append(torch.mm(h, w2[e].t()) + b2[e])
        base += n
    y_sorted = torch.cat(outs, 0)
    y_flat = torch.zeros(T * top_k, d, dtype=x.dtype)
    y_flat.index_copy_(0, pos, y_sorted)
    return torch.bmm(score.view(-1, 1, top_k), y_flat.view(-1, top_k, d)).reshape(-1, d)
