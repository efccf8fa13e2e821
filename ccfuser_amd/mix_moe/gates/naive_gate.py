"""Top-k softmax gate (reference mix_moe/mix_moe/gates/naive_gate.py:11-45)."""
import math

import torch
import torch.nn as nn

from ... import ops
from .base_gate import BaseGate


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
        with torch.no_grad():
            res = ops.gate_topk_softmax(x, self.gate.weight.detach().contiguous(),
                                        None if self.gate.bias is None else self.gate.bias.detach(),
                                        self.top_k, return_logits=return_all_scores)
        idx = res[0].view(*lead, self.top_k)
        score = res[1]                                   # [(B*L), top_k], as the reference returns it
        # dummy loss, on the input's device (naive_gate.py:41)
        self.set_loss(torch.zeros(1, requires_grad=True, device=inp.device))
        if return_all_scores:
            return idx, score, res[2].view(*lead, self.tot_expert)
        return idx, score
