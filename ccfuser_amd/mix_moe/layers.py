"""MoE layer base (reference mix_moe/mix_moe/layers.py)."""
import torch
import torch.nn as nn

from .. import ops
from .gates import NaiveGate
from .linear import MixMOEInstance


def mark_module_parallel_comm(module, comm):
    """Tag every parameter with the data-parallel group it belongs to
    (reference layers.py:10-16)."""
    for p in module.parameters():
        setattr(p, "dp_comm", comm)


def _local_scatter(inp, pos):
    """``inp[pos]`` row gather (reference layers.py:19-21) through the HIP row kernel."""
    return ops.local_scatter(inp.contiguous(), pos.to(torch.int32))


def _local_gather(inp, pos, out_batch_size, maybe_overlap=True):
    """Rows back to their slots (reference layers.py:24-31) by the HIP row kernel; every
    slot is written at most once.  The reference's accumulating form
    (``maybe_overlap=True``, an ``index_add_``) is never used on this path (its one call,
    layers.py:453, passes ``False``) and has no kernel here: asking for it raises instead
    of falling back to a torch op."""
    if maybe_overlap:
        raise NotImplementedError("_local_gather(maybe_overlap=True) has no HIP kernel: rows that share a slot "
                                  "are summed by ops.combine; pass maybe_overlap=False for a pure row move")
    return ops.local_gather(inp.contiguous(), pos.to(torch.int32), out_batch_size)


class _Combine(torch.autograd.Function):
    """Gate-weighted sum over a token's k expert outputs and its backward (the bmm of
    the reference, layers.py:550-559, and what autograd derives from it)."""

    @staticmethod
    def forward(ctx, y_flat, score, top_k, inv_pos):
        flat_score = score.contiguous().view(-1)
        ctx.save_for_backward(y_flat, flat_score, inv_pos)
        ctx.top_k = top_k
        ctx.score_shape = score.shape
        return ops.combine(y_flat, flat_score, top_k, inv_pos)

    @staticmethod
    def backward(ctx, grad_out):
        y_flat, flat_score, inv_pos = ctx.saved_tensors
        g_y, g_s = ops.combine_backward(grad_out.contiguous(), y_flat, flat_score, ctx.top_k, inv_pos)
        return g_y, g_s.view(ctx.score_shape), None, None


class MixMOE(nn.Module):
    """Gate + experts + gate-weighted combine (reference layers.py:34-83, 496-568)."""

    def __init__(self, num_expert=16, d_model=1024, ffn_hidden_size=1024, world_size=1, top_k=2,
                 gate=NaiveGate, my_rank=0, expert=None, gate_hook=None, mask=None, mask_dict=None,
                 mix_moe=None) -> None:
        super().__init__()
        if world_size != 1:
            raise NotImplementedError("single-GPU build: world_size must be 1")
        self.num_expert = num_expert
        self.d_model = d_model
        self.ffn_hidden_size = ffn_hidden_size
        self.world_size = world_size
        self.my_rank = my_rank
        self.top_k = top_k
        self.gate = gate(d_model, num_expert, world_size, top_k)
        self.mix_moe = mix_moe
        self.experts = expert
        self.expert_partition = [[j + i * num_expert for j in range(num_expert)]
                                 for i in range(world_size)]

    def init_mix_moe(self, total_batch_size):
        if self.mix_moe is None:
            self.mix_moe = MixMOEInstance.instance(total_batch_size, self.num_expert, self.top_k,
                                                   self.d_model, self.ffn_hidden_size, 64)

    def mark_parallel_comm(self, expert_dp_comm="none"):
        if self.experts is not None:
            if isinstance(self.experts, list):
                for e in self.experts:
                    mark_module_parallel_comm(e, expert_dp_comm)
            else:
                mark_module_parallel_comm(self.experts, expert_dp_comm)
        mark_module_parallel_comm(self.gate, "gate")

    def moe_forward(self, moe_inp, pos, moe_inp_block_infos):
        if self.experts is not None:
            return self.experts.forward(moe_inp, pos, moe_inp_block_infos)
        raise RuntimeError("MixMOE has no experts")

    def forward(self, moe_inp, pos, gate_score, moe_inp_block_infos):
        """``out[t] = sum_s gate_score[t, s] * y[t*k + s]`` over the expert outputs
        in flat token order.  The reference does this with a bmm
        (layers.py:550-559); here one HIP kernel accumulates in fp32 and rounds
        once, skipping dropped slots."""
        moe_output = self.moe_forward(moe_inp, pos, moe_inp_block_infos)
        inv_pos = moe_inp_block_infos.get("inv_pos") if hasattr(moe_inp_block_infos, "get") else None
        return _Combine.apply(moe_output, gate_score, self.top_k, inv_pos)
