"""Expert linear layers (reference mix_moe/mix_moe/linear.py).

``MixMOELinear1`` / ``MixMOELinear2`` keep the reference's call shape
``apply(inp, pos, block_infos, weight, bias)`` (linear.py:60-86, 115-143) but
hand the stored ``[E, out, in]`` weight straight to the grouped GEMM: the
per-call ``weight.transpose(-2, -1).contiguous()`` of the reference
(linear.py:74, 129) is gone.  The backward halves (linear.py:91-113, 148-173)
return gradients for the input rows, the weight and the bias.
"""
import math
import threading

import torch
import torch.nn as nn
from torch.autograd import Function

from .. import mix_moe_hip, ops


class MixMOEInstance(object):
    """Process-wide holder of the extension object (reference linear.py:15-29)."""
    _instance_lock = threading.Lock()

    def __init__(self, total_batch_size, num_expert, top_k, d_model, ffn_hidden_size, block_size):
        self.mix_moe = mix_moe_hip.MixMOE(1, total_batch_size, num_expert, top_k, d_model,
                                          ffn_hidden_size, block_size)

    @classmethod
    def instance(cls, *args, **kwargs):
        if not hasattr(MixMOEInstance, "_instance"):
            with MixMOEInstance._instance_lock:
                if not hasattr(MixMOEInstance, "_instance"):
                    MixMOEInstance._instance = MixMOEInstance(*args, **kwargs)
        return MixMOEInstance._instance


def _param_grads(weight, E):
    """Gradient buffers shaped like the parameter; slots past E belong to no expert here."""
    grad_w = torch.empty_like(weight)
    grad_b = torch.empty(weight.shape[0], weight.shape[1], dtype=weight.dtype, device=weight.device)
    if weight.shape[0] > E:
        grad_w[E:].zero_()
        grad_b[E:].zero_()
    return grad_w, grad_b


def _routing(pos, block_infos, top_k_hint=None):
    """(src_row, dst_row, offsets, max_rows, n_flat) for the grouped GEMMs."""
    if "offsets" in block_infos:                      # planned by this package: all on device
        return (block_infos["src_row"], block_infos["dst_row"], block_infos["offsets"],
                block_infos["max_rows"], block_infos["n_flat"])
    raise KeyError("block_infos lacks 'offsets': plan it with AsyncExpertAssignment.process_data, or "
                   "use ccfuser_amd.mix_moe_hip.MixMOE for the reference's block arrays")


class MixMOELinear1(Function):
    """h = x[pos // k] @ W1[e]^T + b1[e] per expert segment, optionally with the
    erf GELU fused (``fuse_gelu``); h is in expert order, [max_rows, d_ffn]."""

    @staticmethod
    def forward(ctx, input_buf, pos, moe_inp_block_infos, weight, bias=None, fuse_gelu=False):
        src_row, dst_row, offsets, max_rows, n_flat = _routing(pos, moe_inp_block_infos)
        E = offsets.numel() - 1
        ctx.save_for_backward(input_buf, weight, src_row, dst_row, offsets,
                              moe_inp_block_infos.get("inv_pos"))
        ctx.sizes = (max_rows, n_flat, bool(fuse_gelu), bool(moe_inp_block_infos.get("may_drop", True)))
        return ops.ffn1(input_buf, src_row, offsets, max_rows, weight.detach()[:E],
                        bias.detach()[:E], gelu=bool(fuse_gelu))

    @staticmethod
    def backward(ctx, grad_out):
        """first_gemm_backward (mix_moe/csrc/mix_moe.h:300-388): rows of the input gradient
        come back in flat token order and are summed per token (the reference's
        index_add_ at 359-365)."""
        input_buf, weight, src_row, dst_row, offsets, inv_pos = ctx.saved_tensors
        max_rows, n_flat, fused, may_drop = ctx.sizes
        if fused:
            raise RuntimeError("MixMOELinear1 ran with the GELU fused into its epilogue, which keeps no "
                               "pre-activation: run the forward with fuse_gelu=False to differentiate it")
        E = offsets.numel() - 1
        grad_w, grad_b = _param_grads(weight, E)
        g_flat, _, _ = ops.ffn1_backward(grad_out.contiguous(), input_buf, src_row, dst_row, offsets,
                                         max_rows, weight.detach()[:E], n_flat, grad_w[:E], grad_b[:E],
                                         may_drop=may_drop)
        top_k = n_flat // input_buf.shape[0]
        ones = torch.ones(n_flat, dtype=g_flat.dtype, device=g_flat.device)
        grad_in = ops.combine(g_flat, ones, top_k, inv_pos)
        return grad_in, None, None, grad_w, grad_b, None


class MixMOELinear2(Function):
    """y_flat[pos[j]] = h[j] @ W2[e]^T + b2[e]; y_flat is [tokens*top_k, d_model]
    in flat token order (the reference's index_copy_ after the second GEMM,
    mix_moe/csrc/mix_moe.h:433, happens in the GEMM epilogue)."""

    @staticmethod
    def forward(ctx, input_buf, pos, moe_inp_block_infos, weight, bias=None):
        _, dst_row, offsets, max_rows, n_flat = _routing(pos, moe_inp_block_infos)
        E = offsets.numel() - 1
        d = weight.shape[1]
        alloc = torch.zeros if moe_inp_block_infos.get("may_drop", True) else torch.empty
        y = alloc(n_flat, d, dtype=input_buf.dtype, device=input_buf.device)
        ctx.save_for_backward(input_buf, weight, dst_row, offsets)
        ctx.sizes = (max_rows, bool(moe_inp_block_infos.get("may_drop", True)))
        return ops.ffn2(input_buf, dst_row, offsets, max_rows, weight.detach()[:E],
                        bias.detach()[:E], y)

    @staticmethod
    def backward(ctx, grad_out):
        """second_gemm_backward (mix_moe/csrc/mix_moe.h:439-505); the bias gradient, which
        the reference leaves uninitialised (489), is the column sum of the gradient rows."""
        input_buf, weight, dst_row, offsets = ctx.saved_tensors
        max_rows, may_drop = ctx.sizes
        E = offsets.numel() - 1
        grad_w, grad_b = _param_grads(weight, E)
        g_act, _, _ = ops.ffn2_backward(grad_out.contiguous(), input_buf, dst_row, offsets, max_rows,
                                        weight.detach()[:E], grad_w[:E], grad_b[:E], may_drop=may_drop)
        return g_act, None, None, grad_w, grad_b


_ONES = {}


def _ones(n, dtype, device):
    """A constant vector of ones (the scores of a plain sum over the k slots), made once per size."""
    key = (n, dtype, device)
    t = _ONES.get(key)
    if t is None:
        if len(_ONES) >= 8:
            _ONES.clear()
        t = _ONES[key] = torch.ones(n, dtype=dtype, device=device)
    return t


class MixMOEFusedFFN(Function):
    """Both expert linears with the erf GELU between them as one differentiable step:
    ``y_flat[pos[j]] = gelu(x[pos[j] // k] @ W1[e]^T + b1[e]) @ W2[e]^T + b2[e]``.

    The reference keeps the activation a separate torch op between its two functions
    (mix_moe/mix_moe/transformer.py:82-91) so that autograd differentiates it; here the
    first GEMM's epilogue applies the GELU and also stores the pre-activation, so the
    forward has no activation pass.  In the backward GELU' is applied by the pass that
    transposes the gradient rows for the first layer's weight gradient
    (``ops.ffn1_backward(h_pre=...)``), in place.  The input-gradient GEMM of the second
    layer can multiply by it in its epilogue too (``ops.ffn2_backward(h_pre=...)``), but
    that epilogue runs with the matrix pipe idle and measures slower (config 3: +0.21 ms)."""

    @staticmethod
    def forward(ctx, input_buf, pos, moe_inp_block_infos, w1, b1, w2, b2):
        src_row, dst_row, offsets, max_rows, n_flat = _routing(pos, moe_inp_block_infos)
        E = offsets.numel() - 1
        may_drop = bool(moe_inp_block_infos.get("may_drop", True))
        act, h_pre = ops.ffn1_keep(input_buf, src_row, offsets, max_rows, w1.detach()[:E], b1.detach()[:E])
        y = (torch.zeros if may_drop else torch.empty)(n_flat, w2.shape[1], dtype=input_buf.dtype,
                                                       device=input_buf.device)
        ops.ffn2(act, dst_row, offsets, max_rows, w2.detach()[:E], b2.detach()[:E], y)
        ctx.save_for_backward(input_buf, w1, w2, act, h_pre, src_row, dst_row, offsets,
                              moe_inp_block_infos.get("inv_pos"))
        ctx.sizes = (max_rows, n_flat, may_drop)
        return y

    @staticmethod
    def backward(ctx, grad_y):
        input_buf, w1, w2, act, h_pre, src_row, dst_row, offsets, inv_pos = ctx.saved_tensors
        max_rows, n_flat, may_drop = ctx.sizes
        E = offsets.numel() - 1
        grad_w2, grad_b2 = _param_grads(w2, E)
        grad_act, _, _ = ops.ffn2_backward(grad_y.contiguous(), act, dst_row, offsets, max_rows,
                                           w2.detach()[:E], grad_w2[:E], grad_b2[:E], may_drop=may_drop)
        grad_w1, grad_b1 = _param_grads(w1, E)
        g_flat, _, _ = ops.ffn1_backward(grad_act, input_buf, src_row, dst_row, offsets, max_rows,
                                         w1.detach()[:E], n_flat, grad_w1[:E], grad_b1[:E], may_drop=may_drop,
                                         h_pre=h_pre)
        top_k = n_flat // input_buf.shape[0]
        grad_in = ops.combine(g_flat, _ones(n_flat, g_flat.dtype, g_flat.device), top_k, inv_pos)
        return grad_in, None, None, grad_w1, grad_b1, grad_w2, grad_b2


class FMoELinear(nn.Module):
    """Parameter container for E experts: weight [E, out, in], bias [E, out]
    (reference linear.py:177-233)."""

    def __init__(self, num_expert: int, in_feat: int, out_feat: int, bias: bool = True, rank: int = 0):
        super().__init__()
        self.num_expert = num_expert
        self.in_feat = in_feat
        self.out_feat = out_feat
        self.rank = rank
        self.weight = nn.Parameter(torch.empty(num_expert, out_feat, in_feat))
        if bias:
            self.bias = nn.Parameter(torch.zeros(num_expert, out_feat))
        else:
            self.register_parameter("bias", None)
        self.reset_parameters()

    def extra_repr(self) -> str:
        return "num_expert={}, in_features={}, out_features={}, bias={}, rank={}".format(
            self.num_expert, self.in_feat, self.out_feat, self.bias is not None, self.rank)

    def reset_parameters(self):
        torch.nn.init.kaiming_uniform_(self.weight, a=math.sqrt(0.9))
        if self.bias is not None:
            torch.nn.init.kaiming_uniform_(self.bias, a=math.sqrt(0.9))
