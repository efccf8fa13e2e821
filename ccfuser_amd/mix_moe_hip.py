"""Mirror of the reference's extension module ``mix_moe_cuda``
(mix_moe/csrc/pybind.cpp:23-60) on top of the HIP C ABI.

Free functions ``expert_count``, ``assign_pos`` and ``cpy_data2tensor`` and the
class ``MixMOE`` with ``forward``, ``first_gemm_forward``, ``second_gemm_forward``,
``first_gemm_backward`` and ``second_gemm_backward``, called with the reference's
argument lists.  The block
arrays the reference plans on the host (``expert_ids``, ``expert_lens``,
``start_addrs``; 64-row blocks over the expert-sorted buffer) are accepted as
they are: each block is a (start, len, expert) segment, the segments are
regrouped by expert on the device and both GEMMs run over that row list, so no
staging copy of the tokens is made.  NVSHMEM, MPI and the private stream of
the reference's class (mix_moe/csrc/mix_moe.h:56-79, 118) have no counterpart:
everything runs on torch's current stream.  The AG/GA test hooks (bare kernel
timing loops, pybind.cpp:57-58) are not provided.

Weight layouts: the forward calls receive ``weight.transpose(-2, -1).contiguous()``,
i.e. [E, K, N] (mix_moe/mix_moe/linear.py:74, 129), the backward calls the stored
``weight.contiguous()``, [E, out, in] (linear.py:103, 162).  A square weight
(d_model == d_ffn) cannot be told apart by shape: the forward calls always take it
as the reference's [E, K, N] and transpose it back.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from . import ops


def expert_count(gate_idx: torch.Tensor, expert_count_out: torch.Tensor) -> None:
    """Accumulates the histogram of ``gate_idx`` (int64) into ``expert_count_out``
    (int32); reference mix_moe/csrc/cuda/local_exchange.cu:98-108."""
    ops.expert_count(gate_idx.contiguous(), expert_count_out)


def assign_pos(cum_count: torch.Tensor, gate: torch.Tensor, pos: torch.Tensor) -> None:
    """Fills ``pos`` from the inclusive cumulative counts; ``cum_count`` ends at
    the segment starts, as after the reference's atomicSub loop
    (mix_moe/csrc/cuda/local_exchange.cu:6-17, 81-96).  Inside a segment the
    flat indices ascend."""
    ops.assign_pos(cum_count, gate.contiguous(), pos)


def cpy_data2tensor(data: List[int], tensor: torch.Tensor) -> None:
    """Host list -> the head of an int32 device tensor
    (reference mix_moe/csrc/cuda/global_exchange.cpp:41-48, a blocking cudaMemcpy)."""
    if tensor.dtype != torch.int32:
        raise TypeError("cpy_data2tensor expects an int32 tensor")
    n = len(data)
    if n > tensor.numel():
        raise ValueError("cpy_data2tensor: list longer than the tensor")
    if n:
        tensor.view(-1)[:n].copy_(torch.tensor(data, dtype=torch.int32))


def _stored_layout(weight: torch.Tensor, n_out: int, k_in: int) -> torch.Tensor:
    """The reference passes ``weight.transpose(-2, -1).contiguous()``, i.e. [E, K, N]
    (mix_moe/mix_moe/linear.py:74); the kernels here read [E, N, K].  A tensor
    already in [E, N, K] is used as is; a [E, K, N] one is transposed back."""
    if weight.dim() != 3:
        raise ValueError("expert weight must be 3-D")
    if tuple(weight.shape[1:]) == (n_out, k_in) and n_out != k_in:
        return weight.contiguous()
    if tuple(weight.shape[1:]) == (k_in, n_out):
        return weight.transpose(-2, -1).contiguous()
    raise ValueError(f"expert weight {tuple(weight.shape)} matches neither [E,{k_in},{n_out}] nor [E,{n_out},{k_in}]")


class MixMOE:
    """``mix_moe_cuda.MixMOE(batch_size, seq_len, local_expert_num, top_k, hidden,
    ffn_hidden, block_size[, w1, w2, b1, b2])`` (pybind.cpp:39-58)."""

    def __init__(self, batch_size, seq_len, local_expert_num, top_k, hidden_size, ffn_hidden_size,
                 block_size, expert_weight_ffn1: Optional[torch.Tensor] = None,
                 expert_weight_ffn2: Optional[torch.Tensor] = None,
                 expert_bias_ffn1: Optional[torch.Tensor] = None,
                 expert_bias_ffn2: Optional[torch.Tensor] = None):
        self._batch_size, self._seq_len = batch_size, seq_len
        self._local_expert_num, self._top_k = local_expert_num, top_k
        self._hidden_size, self._ffn_hidden_size = hidden_size, ffn_hidden_size
        self._block_size = block_size
        self._w1, self._w2 = expert_weight_ffn1, expert_weight_ffn2
        self._b1, self._b2 = expert_bias_ffn1, expert_bias_ffn2

    # -- block arrays -> rows grouped by expert, in the padded block layout ----
    def _plan(self, pos, expert_ids, expert_lens, start_addrs, total_block_num, num_expert):
        nb, bs = int(total_block_num), self._block_size
        dev = pos.device
        lens = expert_lens[:nb].to(torch.int32).contiguous()
        starts = start_addrs[:nb].to(torch.int64)
        r = torch.arange(bs, device=dev)
        sorted_idx = (starts[:, None] + r[None, :]).clamp_(max=max(pos.numel() - 1, 0))
        valid = r[None, :] < lens[:, None]
        flat_of_padded = pos.to(torch.int64)[sorted_idx].reshape(-1)         # flat index per padded row
        seg_start = (torch.arange(nb, device=dev, dtype=torch.int32) * bs).contiguous()
        eids = expert_ids[:nb].to(torch.int32).contiguous()
        counts, offsets, rows = ops.segments_to_rows(seg_start, lens, eids, num_expert, nb * bs)
        return flat_of_padded, valid.reshape(-1), offsets, rows

    def _plan_full(self, pos, expert_ids, expert_lens, start_addrs, total_block_num, num_expert):
        """``_plan`` with the row list completed to a permutation of all padded rows: the
        rows of the blocks grouped by expert first (what ``_plan`` returns), then the padding
        rows of short blocks.  Moving rows between the padded block layout and expert order
        through it touches every padded row exactly once."""
        flat_of_padded, valid, offsets, _ = self._plan(pos, expert_ids, expert_lens, start_addrs,
                                                       total_block_num, num_expert)
        nb, bs = int(total_block_num), self._block_size
        key = expert_ids[:nb].to(torch.int64)[:, None].expand(nb, bs).reshape(-1)
        key = torch.where(valid, key, torch.full_like(key, num_expert))
        rows = torch.sort(key, stable=True).indices.to(torch.int32)
        return flat_of_padded, valid, offsets, rows

    def first_gemm_forward(self, inp, pos, expert_ids, ranks, expert_lens, start_addrs,
                           total_block_num, remote_block_num, weight, bias, _gelu=False):
        if inp.dtype != torch.float16:
            raise TypeError("moe input data type must be float 16")
        E = weight.shape[0]
        w = _stored_layout(weight, self._ffn_hidden_size, self._hidden_size)
        flat_of_padded, valid, offsets, rows = self._plan(pos, expert_ids, expert_lens, start_addrs,
                                                          total_block_num, E)
        src_of_padded = torch.div(flat_of_padded, self._top_k, rounding_mode="floor")
        a_rows = src_of_padded[rows.long()].to(torch.int32)
        M = int(total_block_num) * self._block_size
        ffn1_out = torch.zeros(M, self._ffn_hidden_size, dtype=inp.dtype, device=inp.device)
        ops.ffn1(inp.contiguous(), a_rows, offsets, M, w, bias.contiguous(), gelu=_gelu,
                 out=ffn1_out, dst_row=rows)
        merged_input = inp[src_of_padded] * valid[:, None].to(inp.dtype)
        return [merged_input, ffn1_out]

    def second_gemm_forward(self, ffn1_out, pos, expert_ids, ranks, expert_lens, start_addrs,
                            total_block_num, remote_block_num, weight, bias):
        E = weight.shape[0]
        w = _stored_layout(weight, self._hidden_size, self._ffn_hidden_size)
        flat_of_padded, valid, offsets, rows = self._plan(pos, expert_ids, expert_lens, start_addrs,
                                                          total_block_num, E)
        c_rows = flat_of_padded[rows.long()].to(torch.int32)
        M = int(total_block_num) * self._block_size
        output = torch.zeros(pos.numel(), self._hidden_size, dtype=ffn1_out.dtype, device=ffn1_out.device)
        ops.ffn2(ffn1_out.contiguous(), c_rows, offsets, M, w, bias.contiguous(), output, src_row=rows)
        return [ffn1_out, output]

    def forward(self, inp, pos, expert_ids, ranks, expert_lens, start_addrs, total_block_num,
                remote_block_num, test_out=None):
        """Scatter, FFN1, GELU, FFN2 and gather with the weights given at
        construction; returns [pos.numel(), hidden] in flat token order
        (mix_moe/csrc/mix_moe.h:507-598)."""
        if self._w1 is None:
            raise RuntimeError("MixMOE.forward needs the expert weights passed to the constructor")
        _, h = self.first_gemm_forward(inp, pos, expert_ids, ranks, expert_lens, start_addrs,
                                       total_block_num, remote_block_num, self._w1, self._b1, _gelu=True)
        return self.second_gemm_forward(h, pos, expert_ids, ranks, expert_lens, start_addrs,
                                        total_block_num, remote_block_num, self._w2, self._b2)[1]

    @staticmethod
    def _stored(weight: torch.Tensor, n_out: int, k_in: int) -> torch.Tensor:
        if weight.dim() != 3 or tuple(weight.shape[1:]) != (n_out, k_in):
            raise ValueError(f"backward expects the stored weight [E,{n_out},{k_in}], got {tuple(weight.shape)}")
        return weight.contiguous()

    def first_gemm_backward(self, grad_out, weight, bias, merged_input, expert_block_ids, expert_id_idxs,
                            pos, expert_ids, ranks, expert_lens, start_addrs, total_block_num,
                            remote_block_num):
        """Backward of ``first_gemm_forward`` (mix_moe/csrc/mix_moe.h:300-388, called from
        MixMOELinear1.backward, mix_moe/mix_moe/linear.py:91-113).  ``grad_out`` and
        ``merged_input`` are in the padded block layout the forward returned, ``weight`` is the
        stored [E, ffn_hidden, hidden].  Returns ``[grad_in, grad_weight, grad_bias]`` with
        ``grad_in`` [pos.numel() / top_k, hidden]: the gradient rows added back onto their
        tokens (the ``index_add_`` at 359-365).  ``grad_bias`` is the column sum of the
        gradient rows (the reference returns it uninitialised, 342).  The CSR arrays
        ``expert_block_ids`` / ``expert_id_idxs`` are accepted and not needed: the rows are
        regrouped by expert from the block arrays."""
        if grad_out.dtype != torch.float16:
            raise TypeError("moe input data type must be float 16")
        w = self._stored(weight, self._ffn_hidden_size, self._hidden_size)
        E = w.shape[0]
        flat_of_padded, _, offsets, rows = self._plan_full(pos, expert_ids, expert_lens, start_addrs,
                                                           total_block_num, E)
        M = int(total_block_num) * self._block_size
        k = self._top_k
        tokens = pos.numel() // k
        n_flat = max(tokens, (M + k - 1) // k) * k       # the padded layout may hold more rows than pos has entries
        g_sorted = ops.local_scatter(grad_out.contiguous(), rows)              # padded layout -> expert order
        dst_row = flat_of_padded[rows.long()].to(torch.int32)
        g_x_flat, g_w, g_b = ops.ffn1_backward(g_sorted, merged_input.contiguous(), rows, dst_row, offsets, M, w,
                                               n_flat)
        ones = torch.ones(n_flat, dtype=torch.float16, device=grad_out.device)
        grad_in = ops.combine(g_x_flat, ones, k)[:tokens]                      # sum of a token's slots
        return [grad_in, g_w, g_b]

    def second_gemm_backward(self, grad_out, input_buf, expert_block_ids, expert_id_idxs, weight, bias,
                             pos, expert_ids, ranks, expert_lens, start_addrs, total_block_num,
                             remote_block_num):
        """Backward of ``second_gemm_forward`` (mix_moe/csrc/mix_moe.h:439-505, called from
        MixMOELinear2.backward, mix_moe/mix_moe/linear.py:148-173).  ``grad_out`` is
        [pos.numel(), hidden] in flat token order, ``input_buf`` the forward's input in the
        padded block layout, ``weight`` the stored [E, hidden, ffn_hidden].  Returns
        ``[grad_inp_buf, grad_weight, grad_bias]`` with ``grad_inp_buf`` in the padded block
        layout (padding rows zero); ``grad_bias`` as in ``first_gemm_backward`` (489)."""
        if grad_out.dtype != torch.float16:
            raise TypeError("moe input data type must be float 16")
        w = self._stored(weight, self._hidden_size, self._ffn_hidden_size)
        E = w.shape[0]
        flat_of_padded, _, offsets, rows = self._plan_full(pos, expert_ids, expert_lens, start_addrs,
                                                           total_block_num, E)
        M = int(total_block_num) * self._block_size
        act_sorted = ops.local_scatter(input_buf.contiguous(), rows)           # padded layout -> expert order
        dst_row = flat_of_padded[rows.long()].to(torch.int32)
        g_act, g_w, g_b = ops.ffn2_backward(grad_out.contiguous(), act_sorted, dst_row, offsets, M, w)
        grad_inp_buf = ops.local_gather(g_act, rows, M)                        # expert order -> padded layout
        return [grad_inp_buf, g_w, g_b]

    def AG_test(self, *args, **kwargs):
        raise NotImplementedError("AG_test / GA_test are the reference's kernel timing loops "
                                  "(mix_moe/csrc/pybind.cpp:57-58); use bench.py")

    GA_test = AG_test
