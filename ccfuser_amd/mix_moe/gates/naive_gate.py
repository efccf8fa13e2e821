"""Top-k softmax gate (reference mix_moe/mix_moe/gates/naive_gate.py:11-45)."""
import math

import torch
import torch.nn as nn

from ... import ops
from .base_gate import BaseGate


_ZEROS = {}


def _zero_on(device):
    z = _ZEROS.get(device)
    if z is None:
        z = _ZEROS[device] = torch.zeros(1, device=device)
    return z


class _GateFunction(torch.autograd.Function):
    """The fused gate kernel with the backward autograd derives for the reference's
    linear -> topk -> softmax (naive_gate.py:31-38): softmax over the k selected
    logits, the selection as a scatter into [T, E], then the linear layer.  For fp16 the
    first two are one HIP kernel (``ops.gate_backward``); the two products with the [T, E]
    gradient are small library GEMMs."""

    @staticmethod
    def forward(ctx, x, weight, bias, top_k, return_logits):
        res = ops.gate_topk_softmax(x, weight.detach().contiguous(),
                                    None if bias is None else bias.detach(), top_k,
                                    return_logits=return_logits)
        ctx.save_for_backward(x, weight, res[0], res[1])
        ctx.has_bias = bias is not None
        ctx.set_materialize_grads(False)                 # no zero-filled gradients for the index outputs
        ctx.mark_non_differentiable(res[0])
        if return_logits:
            ctx.mark_non_differentiable(res[2])
            return res[0], res[1], res[2]
        return res[0], res[1]

    @staticmethod
    def backward(ctx, grad_idx, grad_score, grad_logits=None):
        x, weight, idx, score = ctx.saved_tensors
        if grad_score is None:                           # the scores were not used
            return None, None, None, None, None
        want_bias = ctx.has_bias and ctx.needs_input_grad[2]
        if x.dtype == torch.float16:
            g16, grad_b = ops.gate_backward(score, grad_score.contiguous(), idx, weight.shape[0], want_bias)
        else:
            s = score.float()
            g = grad_score.float()
            g_val = s * (g - (s * g).sum(-1, keepdim=True))
            g_logits = torch.zeros(x.shape[0], weight.shape[0], dtype=torch.float32, device=x.device)
            g_logits.scatter_add_(1, idx, g_val)
            g16 = g_logits.to(x.dtype)
            grad_b = g_logits.sum(0).to(x.dtype) if want_bias else None
        grad_x = torch.mm(g16, weight) if ctx.needs_input_grad[0] else None
        grad_w = torch.mm(g16.t(), x) if ctx.needs_input_grad[1] else None
        return grad_x, grad_w, grad_b, None, None


class NaiveGate(BaseGate):
    """``nn.Linear(d_model, tot_expert)`` followed by top-k and a softmax over the
    k selected logits.  The three torch kernels of the reference (linear, topk,
    softmax; naive_gate.py:31-38) are one HIP kernel here, whose fp32
    accumulation order is fixed so the expert choice is reproducible; slot 0
    holds the largest logit and ties go to the lower expert id.
    """

    def __init__(self, d_model, num_expert, world_size, top_k=2):
        super().__init__(num_expert, world_size)
        self.gate = nn.Linear(d_model, self.tot_expert)
        torch.nn.init.kaiming_uniform_(self.gate.weight, a=math.sqrt(0.1))
        self.top_k = top_k

    def forward(self, inp, return_all_scores=False):
        lead = inp.shape[:-1]
        x = inp.reshape(-1, inp.shape[-1])
        if not x.is_contiguous():
            x = x.contiguous()
        res = _GateFunction.apply(x, self.gate.weight, self.gate.bias, self.top_k, bool(return_all_scores))
        idx = res[0].view(*lead, self.top_k)
        score = res[1]                                   # [(B*L), top_k], as the reference returns it
        # dummy loss, on the input's device (naive_gate.py:41): a fresh leaf over a zero made once per
        # device, so that the forward pays no fill kernel for it
        self.set_loss(_zero_on(inp.device).detach().requires_grad_(True))
        if return_all_scores:
            return idx, score, res[2].view(*lead, self.tot_expert)
        return idx, score
