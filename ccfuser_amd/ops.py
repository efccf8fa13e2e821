"""Torch-tensor front end of the C ABI: argument checks, workspaces, streams.

Every function takes CUDA (ROCm) tensors, launches on torch's current stream
for the tensors' device and returns without a host synchronisation unless its
docstring says otherwise.  Wrong dtypes, shapes or devices raise Python
exceptions (the reference prints and returns an empty tensor,
mix_moe/csrc/mix_moe.h:242-245, or asserts, mix_moe/csrc/cuda/utils.h:4-6).
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from . import _lib

CCF_F16, CCF_F32 = 0, 1


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _check(t: torch.Tensor, name: str, dtype=None, ndim=None) -> None:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a tensor")
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got {t.device}); there is no CPU path")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if ndim is not None and t.dim() != ndim:
        raise ValueError(f"{name} must have {ndim} dimensions, got {tuple(t.shape)}")


def _workspace(nbytes: int, like: torch.Tensor) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=like.device)


def set_option(name: str, value: int) -> None:
    _lib.call("ccf_set_option", name.encode(), int(value))


# ------------------------------------------------------------------ gate
def gate_topk_softmax(x: torch.Tensor, wg: torch.Tensor, bg: Optional[torch.Tensor], top_k: int,
                      return_logits: bool = False):
    """(idx int64 [T,k], score [T,k]) and optionally logits [T,E], all on x's device."""
    _check(x, "x", ndim=2)
    if x.dtype not in (torch.float16, torch.float32):
        raise TypeError(f"gate input must be float16 or float32, got {x.dtype}")
    _check(wg, "gate weight", dtype=x.dtype, ndim=2)
    if bg is not None:
        _check(bg, "gate bias", dtype=x.dtype, ndim=1)
    T, d = x.shape
    E = wg.shape[0]
    if wg.shape[1] != d or (bg is not None and bg.shape[0] != E):
        raise ValueError("gate weight/bias shapes do not match the input")
    idx = torch.empty(T, top_k, dtype=torch.int64, device=x.device)
    score = torch.empty(T, top_k, dtype=x.dtype, device=x.device)
    logits = torch.empty(T, E, dtype=x.dtype, device=x.device) if return_logits else None
    with torch.cuda.device(x.device):
        _lib.call("ccf_gate_topk_softmax", _ptr(x), _ptr(wg), _ptr(bg), T, d, E, int(top_k),
                  CCF_F16 if x.dtype == torch.float16 else CCF_F32, _ptr(idx), _ptr(score),
                  _ptr(logits), _stream(x))
    return (idx, score, logits) if return_logits else (idx, score)


def gate_backward(score: torch.Tensor, grad_score: torch.Tensor, idx: torch.Tensor, tot_expert: int,
                  want_bias: bool = True):
    """(grad_logits fp16 [T, E], grad_bias fp16 [E] or None): the gate's top-k softmax and
    selection, backwards."""
    _check(score, "score", dtype=torch.float16, ndim=2)
    _check(grad_score, "grad_score", dtype=torch.float16, ndim=2)
    _check(idx, "idx", dtype=torch.int64, ndim=2)
    if grad_score.shape != score.shape or idx.shape != score.shape:
        raise ValueError("score, grad_score and idx must have one shape")
    T, k = score.shape
    E = int(tot_expert)
    g_logits = torch.empty(T, E, dtype=torch.float16, device=score.device)
    g_bias = torch.empty(E, dtype=torch.float16, device=score.device) if want_bias else None
    with torch.cuda.device(score.device):
        nbytes = _lib.lib().ccf_gate_backward_workspace_bytes(T, E) if want_bias else 0
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=score.device) if want_bias else None
        _lib.call("ccf_gate_backward", _ptr(score), _ptr(grad_score), _ptr(idx), T, k, E, _ptr(g_logits),
                  _ptr(g_bias), _ptr(ws), nbytes, _stream(score))
    return g_logits, g_bias


# --------------------------------------------------------------- routing
def expert_count(gate_idx: torch.Tensor, expert_count_out: torch.Tensor) -> None:
    """Accumulate the histogram of ``gate_idx`` into ``expert_count_out`` (int32)."""
    _check(gate_idx, "gate_idx", dtype=torch.int64)
    _check(expert_count_out, "expert_count", dtype=torch.int32, ndim=1)
    with torch.cuda.device(gate_idx.device):
        _lib.call("ccf_expert_count", _ptr(gate_idx), gate_idx.numel(), _ptr(expert_count_out),
                  expert_count_out.numel(), _stream(gate_idx))


def assign_pos(cum_count: torch.Tensor, gate: torch.Tensor, pos: torch.Tensor) -> None:
    """Fill ``pos`` from the inclusive cumulative count; ``cum_count`` is consumed."""
    _check(cum_count, "cum_count", dtype=torch.int32, ndim=1)
    _check(gate, "gate", dtype=torch.int64)
    _check(pos, "pos", dtype=torch.int64, ndim=1)
    n, E = gate.numel(), cum_count.numel()
    if pos.numel() > n:
        raise ValueError("pos is longer than the gate index list")
    with torch.cuda.device(gate.device):
        nbytes = _lib.lib().ccf_route_workspace_bytes(n, E)
        ws = _workspace(nbytes, gate)
        # pos may be shorter than n (dropped entries); the kernel bounds writes by n, so hand it
        # a full-length buffer when the caller's is shorter
        full = pos if pos.numel() == n else torch.empty(n, dtype=torch.int64, device=gate.device)
        _lib.call("ccf_assign_pos", _ptr(cum_count), _ptr(gate), n, E, _ptr(full), _ptr(ws),
                  ws.numel(), _stream(gate))
        if full is not pos:
            pos.copy_(full[: pos.numel()])


def route(gate_idx: torch.Tensor, num_expert: int, top_k: int, capacity: int = -1) -> Dict[str, torch.Tensor]:
    """Counts, offsets, deterministic pos and the row maps, all on the device.

    ``pos``/``src_row``/``dst_row`` have ``n_flat`` entries of which the first
    ``offsets[num_expert]`` are valid; nothing is synchronised to find that count.
    """
    _check(gate_idx, "gate_idx", dtype=torch.int64)
    n = gate_idx.numel()
    dev = gate_idx.device
    out = {
        "counts": torch.empty(num_expert, dtype=torch.int32, device=dev),
        "offsets": torch.empty(num_expert + 1, dtype=torch.int32, device=dev),
        "pos": torch.empty(n, dtype=torch.int64, device=dev),
        "src_row": torch.empty(n, dtype=torch.int32, device=dev),
        "dst_row": torch.empty(n, dtype=torch.int32, device=dev),
        "inv_pos": torch.empty(n, dtype=torch.int32, device=dev),
        "idx_kept": torch.empty(n, dtype=torch.int64, device=dev),
    }
    with torch.cuda.device(dev):
        ws = _workspace(_lib.lib().ccf_route_workspace_bytes(n, num_expert), gate_idx)
        _lib.call("ccf_route", _ptr(gate_idx), n, int(num_expert), int(top_k), int(capacity),
                  _ptr(out["counts"]), _ptr(out["offsets"]), _ptr(out["pos"]), _ptr(out["src_row"]),
                  _ptr(out["dst_row"]), _ptr(out["inv_pos"]), _ptr(out["idx_kept"]), _ptr(ws),
                  ws.numel(), _stream(gate_idx))
    return out


def route_static(gate_idx: torch.Tensor, num_expert: int, top_k: int, capacity: int = -1,
                 out: Optional[Dict[str, torch.Tensor]] = None) -> Dict[str, torch.Tensor]:
    """``route`` through the entry point that allocates nothing: its scratch is a device
    array inside the library.  ``out`` takes preallocated result tensors (the keys ``route``
    returns); without it they are allocated here, before the call.  Raises ``CcfError`` when
    ``ceil(n / 1024) * num_expert`` exceeds the built-in scratch."""
    _check(gate_idx, "gate_idx", dtype=torch.int64)
    n = gate_idx.numel()
    dev = gate_idx.device
    if out is None:
        out = {
            "counts": torch.empty(num_expert, dtype=torch.int32, device=dev),
            "offsets": torch.empty(num_expert + 1, dtype=torch.int32, device=dev),
            "pos": torch.empty(n, dtype=torch.int64, device=dev),
            "src_row": torch.empty(n, dtype=torch.int32, device=dev),
            "dst_row": torch.empty(n, dtype=torch.int32, device=dev),
            "inv_pos": torch.empty(n, dtype=torch.int32, device=dev),
            "idx_kept": torch.empty(n, dtype=torch.int64, device=dev),
        }
    with torch.cuda.device(dev):
        _lib.call("ccf_route_static", _ptr(gate_idx), n, int(num_expert), int(top_k), int(capacity),
                  _ptr(out["counts"]), _ptr(out["offsets"]), _ptr(out["pos"]), _ptr(out["src_row"]),
                  _ptr(out["dst_row"]), _ptr(out["inv_pos"]), _ptr(out["idx_kept"]), _stream(gate_idx))
    return out


def plan_blocks(counts: torch.Tensor, max_rows: int, block_size: int = 64, rank: int = 0) -> Dict[str, torch.Tensor]:
    """The reference's block arrays (transformer.py:242-250) from per-expert counts,
    on the device and without a host synchronisation.

    Arrays have ``max_rows // block_size + E`` entries (an upper bound for any
    counts summing to at most ``max_rows``); ``block_nums`` holds
    ``{total_block_num, remote_block_num}`` and says how many are valid.
    """
    _check(counts, "counts", dtype=torch.int32, ndim=1)
    E = counts.numel()
    dev = counts.device
    cap = int(max_rows) // int(block_size) + E
    names = ("expert_ids", "ranks", "lens", "start_addrs", "expert_block_ids")
    out = {k: torch.zeros(cap, dtype=torch.int32, device=dev) for k in names}
    out["expert_block_id_idxs"] = torch.empty(E + 1, dtype=torch.int32, device=dev)
    out["block_nums"] = torch.empty(2, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        _lib.call("ccf_plan_blocks", _ptr(counts), E, int(block_size), int(rank), cap,
                  *[_ptr(out[k]) for k in names], _ptr(out["expert_block_id_idxs"]),
                  _ptr(out["block_nums"]), _stream(counts))
    return out


def segments_to_rows(seg_start, seg_len, seg_expert, num_expert: int, total_rows: int):
    for t, nm in ((seg_start, "seg_start"), (seg_len, "seg_len"), (seg_expert, "seg_expert")):
        _check(t, nm, dtype=torch.int32, ndim=1)
    dev = seg_start.device
    counts = torch.empty(num_expert, dtype=torch.int32, device=dev)
    offsets = torch.empty(num_expert + 1, dtype=torch.int32, device=dev)
    rows = torch.zeros(total_rows, dtype=torch.int32, device=dev)   # entries past offsets[-1] stay 0
    with torch.cuda.device(dev):
        _lib.call("ccf_segments_to_rows", _ptr(seg_start), _ptr(seg_len), _ptr(seg_expert),
                  seg_start.numel(), int(num_expert), int(total_rows), _ptr(counts), _ptr(offsets),
                  _ptr(rows), _stream(seg_start))
    return counts, offsets, rows


# ------------------------------------------------- row moves and combine
def local_scatter(inp: torch.Tensor, pos: torch.Tensor) -> torch.Tensor:
    """``out[j] = inp[pos[j]]``; pos int32."""
    _check(inp, "inp", dtype=torch.float16, ndim=2)
    _check(pos, "pos", dtype=torch.int32, ndim=1)
    out = torch.empty(pos.numel(), inp.shape[1], dtype=inp.dtype, device=inp.device)
    with torch.cuda.device(inp.device):
        _lib.call("ccf_local_scatter", _ptr(inp), _ptr(out), _ptr(pos), pos.numel(), inp.shape[1],
                  _stream(inp))
    return out


def local_gather(inp: torch.Tensor, pos: torch.Tensor, out_rows: int) -> torch.Tensor:
    """``out[pos[j]] = inp[j]``; rows nothing maps to are zero."""
    _check(inp, "inp", dtype=torch.float16, ndim=2)
    _check(pos, "pos", dtype=torch.int32, ndim=1)
    if pos.numel() != inp.shape[0]:
        raise ValueError("pos and inp disagree on the number of rows")
    out = torch.zeros(out_rows, inp.shape[1], dtype=inp.dtype, device=inp.device)
    with torch.cuda.device(inp.device):
        _lib.call("ccf_local_gather", _ptr(inp), _ptr(out), _ptr(pos), pos.numel(), inp.shape[1],
                  _stream(inp))
    return out


def combine(y_flat: torch.Tensor, score: torch.Tensor, top_k: int,
            inv_pos: Optional[torch.Tensor] = None) -> torch.Tensor:
    _check(y_flat, "y_flat", dtype=torch.float16, ndim=2)
    _check(score, "score", dtype=torch.float16)
    if inv_pos is not None:
        _check(inv_pos, "inv_pos", dtype=torch.int32, ndim=1)
    n, d = y_flat.shape
    if n % top_k or score.numel() != n or (inv_pos is not None and inv_pos.numel() != n):
        raise ValueError("combine: sizes do not match tokens*top_k")
    out = torch.empty(n // top_k, d, dtype=y_flat.dtype, device=y_flat.device)
    with torch.cuda.device(y_flat.device):
        _lib.call("ccf_combine", _ptr(y_flat), _ptr(score), _ptr(inv_pos), _ptr(out), n // top_k,
                  int(top_k), d, _stream(y_flat))
    return out


# ------------------------------------------------------------ expert FFN
def ffn_workspace(max_rows: int, E: int, d: int, f: int, like: torch.Tensor) -> torch.Tensor:
    """A workspace for ``ffn1`` / ``ffn2`` (one call at a time per workspace)."""
    return _workspace(_lib.lib().ccf_ffn_workspace_bytes(int(max_rows), E, d, f), like)


def ffn_plan_info(workspace: torch.Tensor, max_rows: int, E: int, d: int, f: int, which: int) -> Dict[str, int]:
    """What the tile plan left in ``workspace`` by the last ``ffn1`` (which=1) or ``ffn2`` (which=2)
    call decided (diagnostic; synchronises)."""
    import ctypes as C
    info = (C.c_int32 * 8)()
    with torch.cuda.device(workspace.device):
        _lib.call("ccf_ffn_plan_info", _ptr(workspace), int(max_rows), E, d, f, int(which), info, _stream(workspace))
    names = ("split_tiles", "split_parts", "skinny_tiles", "skinny_wgs_per_xcd", "skinny_per_xcd", "skinny_tail_steps",
             "persistent_wgs", "worst_case_tiles")
    return dict(zip(names, list(info)))


def _check_expert(w: torch.Tensor, b: torch.Tensor, name: str) -> None:
    _check(w, f"{name} weight", dtype=torch.float16, ndim=3)
    _check(b, f"{name} bias", dtype=torch.float16, ndim=2)
    if b.shape[0] != w.shape[0] or b.shape[1] != w.shape[1]:
        raise ValueError(f"{name}: bias {tuple(b.shape)} does not match weight {tuple(w.shape)}")


def ffn1(x: torch.Tensor, src_row: Optional[torch.Tensor], offsets: torch.Tensor, max_rows: int,
         w1: torch.Tensor, b1: torch.Tensor, gelu: bool = True,
         out: Optional[torch.Tensor] = None, dst_row: Optional[torch.Tensor] = None,
         workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """h [max_rows, f] (or ``out``); rows nothing maps to are left as they were."""
    if x.dtype != torch.float16:
        raise TypeError("moe input data type must be float 16")
    _check(x, "x", dtype=torch.float16, ndim=2)
    _check_expert(w1, b1, "ffn1")
    _check(offsets, "offsets", dtype=torch.int32, ndim=1)
    E, f, d = w1.shape
    if x.shape[1] != d or offsets.numel() != E + 1:
        raise ValueError("ffn1: x/offsets do not match the weight shape")
    if src_row is not None:
        _check(src_row, "src_row", dtype=torch.int32, ndim=1)
        if src_row.numel() < max_rows:
            raise ValueError("ffn1: src_row shorter than max_rows")
    elif x.shape[0] < max_rows:
        raise ValueError("ffn1: x has fewer rows than max_rows")
    if dst_row is not None:
        _check(dst_row, "dst_row", dtype=torch.int32, ndim=1)
        if out is None or dst_row.numel() < max_rows:
            raise ValueError("ffn1: dst_row needs an explicit `out` and max_rows entries")
    h = out if out is not None else torch.empty(max_rows, f, dtype=x.dtype, device=x.device)
    _check(h, "h", dtype=torch.float16, ndim=2)
    if h.shape[1] != f or (dst_row is None and h.shape[0] < max_rows):
        raise ValueError("ffn1: output buffer too small")
    with torch.cuda.device(x.device):
        ws = workspace if workspace is not None else ffn_workspace(max_rows, E, d, f, x)
        _lib.call("ccf_ffn1_forward", _ptr(x), _ptr(src_row), _ptr(dst_row), _ptr(offsets), int(max_rows), E, d, f,
                  _ptr(w1), _ptr(b1), int(bool(gelu)), _ptr(h), _ptr(ws), ws.numel(), _stream(x))
    return h


def ffn1_keep(x: torch.Tensor, src_row: Optional[torch.Tensor], offsets: torch.Tensor, max_rows: int,
              w1: torch.Tensor, b1: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """(act, h_pre), both [max_rows, f]: ``ffn1`` with the GELU, keeping the pre-activation
    for the backward."""
    _check(x, "x", dtype=torch.float16, ndim=2)
    _check_expert(w1, b1, "ffn1")
    _check(offsets, "offsets", dtype=torch.int32, ndim=1)
    E, f, d = w1.shape
    if x.shape[1] != d or offsets.numel() != E + 1:
        raise ValueError("ffn1_keep: x/offsets do not match the weight shape")
    if src_row is not None:
        _check(src_row, "src_row", dtype=torch.int32, ndim=1)
        if src_row.numel() < max_rows:
            raise ValueError("ffn1_keep: src_row shorter than max_rows")
    elif x.shape[0] < max_rows:
        raise ValueError("ffn1_keep: x has fewer rows than max_rows")
    act = torch.empty(max_rows, f, dtype=x.dtype, device=x.device)
    h_pre = torch.empty_like(act)
    with torch.cuda.device(x.device):
        ws = _workspace(_lib.lib().ccf_ffn_workspace_bytes(max_rows, E, d, f), x)
        _lib.call("ccf_ffn1_forward_keep", _ptr(x), _ptr(src_row), _ptr(offsets), int(max_rows), E, d, f,
                  _ptr(w1), _ptr(b1), _ptr(h_pre), _ptr(act), _ptr(ws), ws.numel(), _stream(x))
    return act, h_pre


def ffn2(h: torch.Tensor, dst_row: Optional[torch.Tensor], offsets: torch.Tensor, max_rows: int,
         w2: torch.Tensor, b2: torch.Tensor, y: torch.Tensor,
         row_scale: Optional[torch.Tensor] = None,
         src_row: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Writes ``y[dst_row[j]]`` for the routed rows and returns ``y``."""
    _check(h, "h", dtype=torch.float16, ndim=2)
    _check_expert(w2, b2, "ffn2")
    _check(offsets, "offsets", dtype=torch.int32, ndim=1)
    _check(y, "y", dtype=torch.float16, ndim=2)
    E, d, f = w2.shape
    if h.shape[1] != f or offsets.numel() != E + 1 or y.shape[1] != d:
        raise ValueError("ffn2: h/offsets/y do not match the weight shape")
    if src_row is not None:
        _check(src_row, "src_row", dtype=torch.int32, ndim=1)
        if src_row.numel() < max_rows:
            raise ValueError("ffn2: src_row shorter than max_rows")
    elif h.shape[0] < max_rows:
        raise ValueError("ffn2: h has fewer rows than max_rows")
    if dst_row is not None:
        _check(dst_row, "dst_row", dtype=torch.int32, ndim=1)
        if dst_row.numel() < max_rows:
            raise ValueError("ffn2: dst_row shorter than max_rows")
    elif y.shape[0] < max_rows:
        raise ValueError("ffn2: y has fewer rows than max_rows")
    if row_scale is not None:
        _check(row_scale, "row_scale", dtype=torch.float16, ndim=1)
    with torch.cuda.device(h.device):
        ws = workspace if workspace is not None else ffn_workspace(max_rows, E, d, f, h)
        _lib.call("ccf_ffn2_forward", _ptr(h), _ptr(src_row), _ptr(dst_row), _ptr(offsets), int(max_rows), E, d, f,
                  _ptr(w2), _ptr(b2), _ptr(row_scale), _ptr(y), _ptr(ws), ws.numel(), _stream(h))
    return y


# -------------------------------------------------------------- backward
def combine_backward(grad_out: torch.Tensor, y_flat: torch.Tensor, score: torch.Tensor, top_k: int,
                     inv_pos: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """(grad_y_flat [T*k, d], grad_score [T*k]) of ``combine``; zero for dropped slots."""
    _check(grad_out, "grad_out", dtype=torch.float16, ndim=2)
    _check(y_flat, "y_flat", dtype=torch.float16, ndim=2)
    _check(score, "score", dtype=torch.float16)
    if inv_pos is not None:
        _check(inv_pos, "inv_pos", dtype=torch.int32, ndim=1)
    n, d = y_flat.shape
    T = grad_out.shape[0]
    if T * top_k != n or grad_out.shape[1] != d or score.numel() != n or \
            (inv_pos is not None and inv_pos.numel() != n):
        raise ValueError("combine_backward: sizes do not match tokens*top_k")
    g_y = torch.empty_like(y_flat)
    g_s = torch.empty(n, dtype=torch.float16, device=y_flat.device)
    with torch.cuda.device(y_flat.device):
        _lib.call("ccf_combine_backward", _ptr(grad_out), _ptr(y_flat), _ptr(score), _ptr(inv_pos), T,
                  int(top_k), d, _ptr(g_y), _ptr(g_s), _stream(y_flat))
    return g_y, g_s


def _backward_ws(max_rows: int, E: int, d: int, f: int, like: torch.Tensor) -> torch.Tensor:
    return _workspace(_lib.lib().ccf_ffn_backward_workspace_bytes(int(max_rows), E, d, f), like)


def _grad_outputs(w: torch.Tensor, grad_w: Optional[torch.Tensor], grad_b: Optional[torch.Tensor]):
    E, n_out, _ = w.shape
    if grad_w is None:
        grad_w = torch.empty_like(w)
    if grad_b is None:
        grad_b = torch.empty(E, n_out, dtype=torch.float16, device=w.device)
    _check(grad_w, "grad_w", dtype=torch.float16, ndim=3)
    _check(grad_b, "grad_b", dtype=torch.float16, ndim=2)
    if grad_w.shape != w.shape or tuple(grad_b.shape) != (E, n_out):
        raise ValueError("gradient buffers do not match the weight shape")
    return grad_w, grad_b


def ffn2_backward(grad_y_flat: torch.Tensor, act: torch.Tensor, dst_row: Optional[torch.Tensor],
                  offsets: torch.Tensor, max_rows: int, w2: torch.Tensor,
                  grad_w: Optional[torch.Tensor] = None, grad_b: Optional[torch.Tensor] = None,
                  may_drop: bool = True, h_pre: Optional[torch.Tensor] = None):
    """(grad_act [max_rows, f], grad_w2 [E, d, f], grad_b2 [E, d]) of ``ffn2``.
    Rows of ``grad_act`` past ``offsets[-1]`` are zero (``may_drop=False`` promises there
    are none and skips the zero fill).  With ``h_pre`` (``act = gelu(h_pre)``, from
    ``ffn1_keep``) the first result is the gradient of ``h_pre`` instead."""
    _check(grad_y_flat, "grad_y_flat", dtype=torch.float16, ndim=2)
    if h_pre is not None:
        _check(h_pre, "h_pre", dtype=torch.float16, ndim=2)
        if h_pre.shape != act.shape:
            raise ValueError("ffn2_backward: h_pre and act differ in shape")
    _check(act, "act", dtype=torch.float16, ndim=2)
    _check(w2, "ffn2 weight", dtype=torch.float16, ndim=3)
    _check(offsets, "offsets", dtype=torch.int32, ndim=1)
    E, d, f = w2.shape
    if grad_y_flat.shape[1] != d or act.shape[1] != f or offsets.numel() != E + 1 or act.shape[0] < max_rows:
        raise ValueError("ffn2_backward: shapes do not match the weight")
    if dst_row is not None:
        _check(dst_row, "dst_row", dtype=torch.int32, ndim=1)
        if dst_row.numel() < max_rows:
            raise ValueError("ffn2_backward: dst_row shorter than max_rows")
    elif grad_y_flat.shape[0] < max_rows:
        raise ValueError("ffn2_backward: grad_y_flat has fewer rows than max_rows")
    dev = act.device
    g_act = (torch.zeros if may_drop else torch.empty)(max_rows, f, dtype=torch.float16, device=dev)
    g_w, g_b = _grad_outputs(w2, grad_w, grad_b)
    with torch.cuda.device(dev):
        ws = _backward_ws(max_rows, E, d, f, act)
        _lib.call("ccf_ffn2_backward", _ptr(grad_y_flat), _ptr(act), _ptr(h_pre), _ptr(dst_row), _ptr(offsets),
                  int(max_rows), E, d, f, _ptr(w2), _ptr(g_act), _ptr(g_w), _ptr(g_b), _ptr(ws),
                  ws.numel(), _stream(act))
    return g_act, g_w, g_b


def ffn1_backward(grad_h: torch.Tensor, x: torch.Tensor, src_row: Optional[torch.Tensor],
                  dst_row: Optional[torch.Tensor], offsets: torch.Tensor, max_rows: int,
                  w1: torch.Tensor, n_flat: int,
                  grad_w: Optional[torch.Tensor] = None, grad_b: Optional[torch.Tensor] = None,
                  may_drop: bool = True, h_pre: Optional[torch.Tensor] = None):
    """(grad_x_flat [n_flat, d], grad_w1 [E, f, d], grad_b1 [E, f]) of ``ffn1`` without the
    fused GELU.  ``grad_x_flat[dst_row[j]]`` is the gradient of sorted row j; rows nothing
    maps to are zero (``may_drop=False`` promises every row is written).  With ``h_pre`` (from
    ``ffn1_keep``) ``grad_h`` is the gradient of ``gelu(h_pre)`` on entry and is overwritten
    with the gradient of ``h_pre``: the backward through the GELU and the linear layer."""
    _check(grad_h, "grad_h", dtype=torch.float16, ndim=2)
    if h_pre is not None:
        _check(h_pre, "h_pre", dtype=torch.float16, ndim=2)
        if h_pre.shape != grad_h.shape:
            raise ValueError("ffn1_backward: h_pre and grad_h differ in shape")
    _check(x, "x", dtype=torch.float16, ndim=2)
    _check(w1, "ffn1 weight", dtype=torch.float16, ndim=3)
    _check(offsets, "offsets", dtype=torch.int32, ndim=1)
    E, f, d = w1.shape
    if grad_h.shape[1] != f or x.shape[1] != d or offsets.numel() != E + 1 or grad_h.shape[0] < max_rows:
        raise ValueError("ffn1_backward: shapes do not match the weight")
    for t, nm in ((src_row, "src_row"), (dst_row, "dst_row")):
        if t is not None:
            _check(t, nm, dtype=torch.int32, ndim=1)
            if t.numel() < max_rows:
                raise ValueError(f"ffn1_backward: {nm} shorter than max_rows")
    if src_row is None and x.shape[0] < max_rows:
        raise ValueError("ffn1_backward: x has fewer rows than max_rows")
    if n_flat < max_rows:
        raise ValueError("ffn1_backward: n_flat smaller than max_rows")
    dev = x.device
    g_x = (torch.zeros if may_drop else torch.empty)(n_flat, d, dtype=torch.float16, device=dev)
    g_w, g_b = _grad_outputs(w1, grad_w, grad_b)
    with torch.cuda.device(dev):
        ws = _backward_ws(max_rows, E, d, f, x)
        if h_pre is not None:
            _lib.call("ccf_ffn1_backward_gelu", _ptr(grad_h), _ptr(h_pre), _ptr(x), _ptr(src_row), _ptr(dst_row),
                      _ptr(offsets), int(max_rows), E, d, f, _ptr(w1), _ptr(g_x), _ptr(g_w), _ptr(g_b), _ptr(ws),
                      ws.numel(), _stream(x))
        else:
            _lib.call("ccf_ffn1_backward", _ptr(grad_h), _ptr(x), _ptr(src_row), _ptr(dst_row), _ptr(offsets),
                      int(max_rows), E, d, f, _ptr(w1), _ptr(g_x), _ptr(g_w), _ptr(g_b), _ptr(ws),
                      ws.numel(), _stream(x))
    return g_x, g_w, g_b


# ------------------------------------------------------- the whole layer
def moe_forward(x, wg, bg, w1, b1, w2, b2, top_k: int, capacity: int = -1,
                return_routing: bool = False, workspace: Optional[torch.Tensor] = None):
    """The fused layer forward: out [T, d] fp16 (and the routing tensors on request)."""
    if x.dtype != torch.float16:
        raise TypeError("moe input data type must be float 16")
    _check(x, "x", dtype=torch.float16, ndim=2)
    _check(wg, "gate weight", dtype=torch.float16, ndim=2)
    if bg is not None:
        _check(bg, "gate bias", dtype=torch.float16, ndim=1)
    _check_expert(w1, b1, "ffn1")
    _check_expert(w2, b2, "ffn2")
    T, d = x.shape
    E, f, d1 = w1.shape
    if d1 != d or tuple(w2.shape) != (E, d, f) or tuple(wg.shape) != (E, d):
        raise ValueError("moe_forward: weight shapes do not match (one GPU: the gate scores the local experts)")
    dev = x.device
    out = torch.empty(T, d, dtype=x.dtype, device=dev)
    n = T * top_k
    extra = {}
    if return_routing:
        extra = {"idx": torch.empty(T, top_k, dtype=torch.int64, device=dev),
                 "score": torch.empty(T, top_k, dtype=x.dtype, device=dev),
                 "pos": torch.empty(n, dtype=torch.int64, device=dev),
                 "counts": torch.empty(E, dtype=torch.int32, device=dev),
                 "offsets": torch.empty(E + 1, dtype=torch.int32, device=dev)}
    with torch.cuda.device(dev):
        need = _lib.lib().ccf_moe_workspace_bytes(T, d, f, E, int(top_k))
        ws = workspace if workspace is not None else _workspace(need, x)
        _lib.call("ccf_moe_forward", _ptr(x), _ptr(wg), _ptr(bg), _ptr(w1), _ptr(b1), _ptr(w2),
                  _ptr(b2), T, d, f, E, int(top_k), int(capacity), _ptr(out), _ptr(extra.get("idx")),
                  _ptr(extra.get("score")), _ptr(extra.get("pos")), _ptr(extra.get("counts")),
                  _ptr(extra.get("offsets")), _ptr(ws), ws.numel(), _stream(x))
    return (out, extra) if return_routing else out


def moe_workspace(tokens: int, d_model: int, d_ffn: int, num_expert: int, top_k: int,
                  device) -> torch.Tensor:
    """A reusable workspace for ``moe_forward`` (one layer call at a time per workspace)."""
    need = _lib.lib().ccf_moe_workspace_bytes(tokens, d_model, d_ffn, num_expert, top_k)
    return torch.empty(max(need, 256), dtype=torch.uint8, device=device)


def moe_ffn_segments(x, seg_start, seg_len, seg_expert, w1, b1, w2, b2,
                     y: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Expert FFN over an inbound buffer addressed by (start, len, expert) triples."""
    if x.dtype != torch.float16:
        raise TypeError("moe input data type must be float 16")
    _check(x, "x", dtype=torch.float16, ndim=2)
    for t, nm in ((seg_start, "seg_start"), (seg_len, "seg_len"), (seg_expert, "seg_expert")):
        _check(t, nm, dtype=torch.int32, ndim=1)
    _check_expert(w1, b1, "ffn1")
    _check_expert(w2, b2, "ffn2")
    R, d = x.shape
    E, f, _ = w1.shape
    if y is None:
        y = torch.zeros(R, d, dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        need = _lib.lib().ccf_segments_workspace_bytes(R, seg_start.numel(), E, d, f)
        ws = _workspace(need, x)
        _lib.call("ccf_moe_ffn_segments", _ptr(x), _ptr(seg_start), _ptr(seg_len), _ptr(seg_expert),
                  seg_start.numel(), R, d, f, E, _ptr(w1), _ptr(b1), _ptr(w2), _ptr(b2), _ptr(y),
                  _ptr(ws), ws.numel(), _stream(x))
    return y
