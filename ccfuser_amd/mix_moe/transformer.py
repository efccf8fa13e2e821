"""The MoE MLP of a transformer block (reference mix_moe/mix_moe/transformer.py)."""
import numpy as np
import torch
import torch.nn as nn

from .. import ops
from .layers import MixMOE
from .linear import FMoELinear, MixMOEFusedFFN, MixMOEInstance, MixMOELinear1, MixMOELinear2

_COMPAT_KEYS = ("expert_ids", "local_expert_id_indexs", "ranks", "lens", "start_addrs",
                "remote_block_num", "total_block_num", "expert_block_ids", "expert_block_id_idxs")


def plan_blocks(counts, block_size=64):
    """Block plan in the reference's wire format for one GPU with the identity
    expert plan (``AsyncExpertAssignment.divide_into_block``, transformer.py:150-250).

    Per expert in id order: full ``block_size``-row blocks ("local" list), then
    a shorter tail ("remote" list, rank = self); the two lists are interleaved
    l0, r0, l1, r1, ...; ``expert_block_ids`` / ``expert_block_id_idxs`` are a
    CSR from expert to block.  Unlike the reference, an expert with fewer than
    ``block_size`` rows still gets its tail block (the reference only plans a
    tail next to a full block, transformer.py:184-193, and so loses such rows).
    Returns plain Python lists and ints.
    """
    counts = np.asarray(counts, dtype=np.int64).reshape(-1)
    starts = np.concatenate([[0], np.cumsum(counts)[:-1]])
    local, remote = [], []
    for e, (c, s) in enumerate(zip(counts.tolist(), starts.tolist())):
        nfull, tail = divmod(c, block_size)
        local.extend((e, block_size, s + b * block_size) for b in range(nfull))
        if tail:
            remote.append((e, tail, s + nfull * block_size))
    plan = []
    for i in range(max(len(local), len(remote))):
        plan.extend(lst[i] for lst in (local, remote) if i < len(lst))
    expert_ids = [p[0] for p in plan]
    order = sorted(range(len(plan)), key=lambda b: (expert_ids[b], b))
    per_expert = np.bincount(np.asarray(expert_ids, dtype=np.int64), minlength=len(counts))
    return {"expert_ids": expert_ids, "local_expert_id_indexs": list(expert_ids),
            "ranks": [0] * len(plan), "lens": [p[1] for p in plan],
            "start_addrs": [p[2] for p in plan], "total_block_num": len(plan),
            "remote_block_num": len(remote), "expert_block_ids": order,
            "expert_block_id_idxs": np.concatenate([[0], np.cumsum(per_expert)]).tolist()}


class BlockInfos(dict):
    """What the planner hands to the expert FFN.

    Device tensors ``offsets`` [E+1], ``counts`` [E], ``src_row`` / ``dst_row`` /
    ``inv_pos`` [tokens*top_k] and the ints ``max_rows`` / ``n_flat`` drive the
    grouped GEMMs, whose tile list is derived from ``offsets`` on the device.
    The reference's nine keys (transformer.py:242-250) are produced on first
    access by one small kernel from the counts; the arrays are then trimmed to
    ``total_block_num`` entries, which reads two ints back (the reference's
    ``total_block_num`` / ``remote_block_num`` are Python ints).
    """

    def __missing__(self, key):
        if key not in _COMPAT_KEYS:
            raise KeyError(key)
        plan = ops.plan_blocks(self["counts"], self["n_flat"])
        total, remote = plan.pop("block_nums").tolist()
        for k, v in plan.items():
            self[k] = v if k == "expert_block_id_idxs" else v[:total]
        self["local_expert_id_indexs"] = self["expert_ids"]
        self["total_block_num"], self["remote_block_num"] = total, remote
        return dict.__getitem__(self, key)


class _Expert(nn.Module):
    """Two grouped linear layers with an activation between them
    (reference transformer.py:70-91)."""

    def __init__(self, num_expert, d_model, d_hidden, activation, rank=0):
        super().__init__()
        self.htoh4 = FMoELinear(num_expert, d_model, d_hidden, bias=True, rank=rank)
        self.h4toh = FMoELinear(num_expert, d_hidden, d_model, bias=True, rank=rank)
        self.activation = activation
        self.fuse_training = True     # False: the reference's three steps (linear, torch activation, linear)

    def _gelu_is_fusable(self):
        return isinstance(self.activation, nn.GELU) and getattr(self.activation, "approximate", "none") == "none"

    def forward(self, inp, pos, moe_inp_block_infos):
        wants_grad = torch.is_grad_enabled() and (inp.requires_grad or self.htoh4.weight.requires_grad)
        fuse = self._gelu_is_fusable()
        if fuse and wants_grad and self.fuse_training:
            # one differentiable step: the GELU and its derivative live in GEMM epilogues
            return MixMOEFusedFFN.apply(inp, pos, moe_inp_block_infos, self.htoh4.weight, self.htoh4.bias,
                                        self.h4toh.weight, self.h4toh.bias)
        # the inference epilogue keeps no pre-activation, so it is used only when nothing is differentiated
        fuse = fuse and not wants_grad
        x = MixMOELinear1.apply(inp, pos, moe_inp_block_infos, self.htoh4.weight, self.htoh4.bias, fuse)
        if not fuse:
            x = self.activation(x)
        return MixMOELinear2.apply(x, pos, moe_inp_block_infos, self.h4toh.weight, self.h4toh.bias)


class AsyncExpertAssignment:
    """Gate + count/scan/pos, optionally ahead of time on a second HIP stream.

    The reference runs this on a Python thread so that its host-side planning
    (``divide_into_block``, seven blocking copies) hides under the attention
    kernels (transformer.py:102-145, 376-423).  Here the planning is three small
    kernels, so the "thread" is a side stream plus an event; ``close`` has
    nothing to join.
    """

    def __init__(self, rank_id, world_size, popular_expert_num, expert_num, total_batch_size):
        self.my_rank = rank_id
        self.world_size = world_size
        self.popular_expert_num = popular_expert_num
        self.local_expert_num = popular_expert_num + expert_num
        self.total_num_expert = expert_num * world_size
        self.total_batch_size = total_batch_size
        self.num_expert = expert_num
        self.block_size = 64
        self.capacity = -1
        self.result = None
        self._event = None
        self._side = None
        self.assignment_plan = {r: [i + r * expert_num for i in range(expert_num)]
                                for r in range(world_size)}

    def divide_into_block(self, expert_partition_plan, all_expert_count, topk_indices=None):
        """The reference's planner output for this rank's counts (see ``plan_blocks``)."""
        counts = torch.as_tensor(all_expert_count).reshape(self.world_size, -1)[self.my_rank]
        return plan_blocks(counts.cpu().numpy(), self.block_size)

    def generate_kernel_paras(self, all_expert_count, expert_partition_plan, topk_indices, device):
        return self.divide_into_block(expert_partition_plan, all_expert_count, topk_indices)

    def process_data(self, gate, attn_inp, num_expert, world_size):
        """(pos, gate_score, block_infos), nothing synchronised with the host.
        ``pos`` has tokens*top_k entries; the first ``offsets[-1]`` are valid."""
        if world_size != 1:
            raise NotImplementedError("single-GPU build: world_size must be 1")
        gate_top_k_idx, gate_score = gate(attn_inp)
        top_k = gate_top_k_idx.shape[-1]
        r = ops.route(gate_top_k_idx.reshape(-1), num_expert, top_k, self.capacity)
        infos = BlockInfos(offsets=r["offsets"], counts=r["counts"], src_row=r["src_row"],
                           dst_row=r["dst_row"], inv_pos=r["inv_pos"], idx_kept=r["idx_kept"],
                           max_rows=r["pos"].numel(), n_flat=r["pos"].numel(),
                           may_drop=self.capacity >= 0)
        return r["pos"], gate_score, infos

    def add_task(self, gate, attn_inp, num_expert, world_size):
        dev = attn_inp.device
        if self._side is None:
            self._side = torch.cuda.Stream(device=dev)      # default priority
        main = torch.cuda.current_stream(dev)
        self._side.wait_stream(main)
        with torch.cuda.stream(self._side):
            self.result = self.process_data(gate, attn_inp, num_expert, world_size)
            self._event = self._side.record_event()
        attn_inp.record_stream(self._side)

    def get_result(self):
        return self.result

    def wait_for_completion(self):
        if self._event is None:
            raise RuntimeError("no expert assignment has been queued")
        main = torch.cuda.current_stream()
        main.wait_event(self._event)
        pos, score, infos = self.result
        for t in [pos, score] + [v for v in infos.values() if isinstance(v, torch.Tensor)]:
            t.record_stream(main)

    def close(self):
        self.result = None
        self._event = None


class MixMOETransformerMLP(MixMOE):
    """A complete MoE MLP module of a transformer block
    (reference transformer.py:428-497).

    ``experts`` is ``{'num_local_expert': E, 'hidden_size': f, ...}``.  The
    expert containers hold ``E + popular_expert_num`` slots like the reference's
    (transformer.py:449-453) so state dicts line up; expert ``e`` uses slot ``e``.
    ``capacity_factor`` (not in the reference) drops overflow beyond
    ``ceil(factor * tokens * top_k / E)`` rows per expert.  ``fused=True`` runs
    the whole forward as one C-ABI call; ``fused=False`` goes stage by stage
    through ``process_data`` and ``MixMOE.forward`` like the reference.  When a
    gradient is wanted (grad mode on and the input or a parameter requires it)
    the staged path runs, whose stages carry their backward.
    """

    def __init__(self, gate_type, experts, model_dim: int, expert_rank, world_size,
                 scan_expert_func=None, total_batch_size=4096, expert_dp_comm="none",
                 activation=torch.nn.GELU(), mix_moe=None, capacity_factor=None, fused=True,
                 popular_expert_num=3, **kwargs):
        super().__init__(num_expert=experts["num_local_expert"], d_model=model_dim,
                         ffn_hidden_size=experts["hidden_size"], expert=None, my_rank=expert_rank,
                         world_size=world_size, **kwargs)
        self.experts = _Expert(experts["num_local_expert"] + popular_expert_num, model_dim,
                               experts["hidden_size"], activation, expert_rank)
        if scan_expert_func is not None:
            for n, p in self.experts.named_parameters():
                scan_expert_func(n, p)
        self.init_mix_moe(total_batch_size)
        self.mark_parallel_comm(expert_dp_comm)
        self.async_ = False
        self.capacity_factor = capacity_factor
        self.fused = fused
        self.async_expert_assign = AsyncExpertAssignment(expert_rank, world_size, popular_expert_num,
                                                         experts["num_local_expert"], total_batch_size)

    def _capacity(self, tokens):
        if self.capacity_factor is None:
            return -1
        return int(-(-self.capacity_factor * tokens * self.top_k // self.num_expert))

    def async_expert_assignment(self, attn_inp: torch.Tensor):
        inp = attn_inp.reshape(-1, self.d_model)
        self.async_expert_assign.capacity = self._capacity(inp.shape[0])
        self.async_expert_assign.add_task(self.gate, inp, self.num_expert, self.world_size)
        self.async_ = True

    def close(self):
        self.async_expert_assign.close()

    def forward(self, inp: torch.Tensor):
        original_shape = inp.shape
        inp = inp.reshape(-1, self.d_model)
        if inp.dtype != torch.float16:
            raise TypeError("moe input data type must be float 16")
        if not inp.is_contiguous():
            inp = inp.contiguous()
        E = self.num_expert
        if self.async_:
            self.async_expert_assign.wait_for_completion()
            pos, gate_score, infos = self.async_expert_assign.result
            self.async_ = False
            output = super().forward(inp, pos, gate_score, infos)
        elif self.fused and self.experts._gelu_is_fusable() and not (
                torch.is_grad_enabled() and (inp.requires_grad or
                                             any(p.requires_grad for p in self.parameters()))):
            ex = self.experts
            with torch.no_grad():
                output = ops.moe_forward(inp, self.gate.gate.weight.detach(),
                                         None if self.gate.gate.bias is None else self.gate.gate.bias.detach(),
                                         ex.htoh4.weight.detach()[:E], ex.htoh4.bias.detach()[:E],
                                         ex.h4toh.weight.detach()[:E], ex.h4toh.bias.detach()[:E],
                                         self.top_k, self._capacity(inp.shape[0]))
        else:
            self.async_expert_assign.capacity = self._capacity(inp.shape[0])
            pos, gate_score, infos = self.async_expert_assign.process_data(
                self.gate, inp, self.num_expert, self.world_size)
            output = super().forward(inp, pos, gate_score, infos)
        return output.reshape(original_shape)
