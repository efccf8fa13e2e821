"""Count / scan / pos host functions (reference mix_moe/mix_moe/functions.py).

The reference's versions call two CUDA kernels with a cumsum, an ``.item()``
and a ``.cpu()`` in between (functions.py:83-105).  Here one C-ABI call does
count, scan and a deterministic pos on the device; the host synchronises only
where the reference's return values demand it (the length of ``pos`` and the
CPU copy of the counts).
"""
import torch

from .. import ops

_moe_group = None


def ensure_comm(t, comm):
    """One GPU: nothing to initialise (reference functions.py:16-21 sets up NCCL)."""
    if comm is not None:
        raise RuntimeError("single-GPU build: no communicator can be attached")


def get_moe_group():
    return _moe_group


def _require_single(world_size):
    if world_size != 1:
        raise NotImplementedError(
            f"world_size={world_size}: this build covers one GPU's share; the expert-parallel "
            "exchange of the reference (expert_all_gather, global_scatter) is out of scope")


def _route(gate, num_expert, require_pos=True):
    flat = gate.reshape(-1).contiguous()
    top_k = gate.shape[-1] if gate.dim() == 2 else 1
    r = ops.route(flat, num_expert, top_k)
    local_expert_count = r["counts"].long()
    pos = None
    if require_pos:
        # the reference sizes pos by lec_cum[-1].item() (functions.py:101): one sync
        n_routed = int(r["offsets"][-1].item())
        pos = r["pos"][:n_routed]
    return pos, local_expert_count, r


def count_by_gate(gate, num_expert, world_size, my_rank, require_pos=True):
    """(pos, local_expert_count, global_expert_count, all_expert_count), all on the
    gate's device (reference functions.py:28-54)."""
    _require_single(world_size)
    with torch.no_grad():
        pos, local_expert_count, _ = _route(gate, num_expert * world_size, require_pos)
        all_expert_count = local_expert_count.reshape(world_size, num_expert * world_size)
        global_expert_count = all_expert_count[:, my_rank * num_expert:(my_rank + 1) * num_expert]
    return pos, local_expert_count, global_expert_count, all_expert_count


def prepare_forward(gate, num_expert, world_size, my_rank):
    """Reference functions.py:57-81: the same counts on the CPU plus the batch size."""
    pos, local_expert_count, global_expert_count, all_expert_count = count_by_gate(
        gate, num_expert, world_size, my_rank)
    with torch.no_grad():
        fwd_expert_count = global_expert_count.view(world_size, num_expert).sum(dim=0)
        fwd_batch_size = int(fwd_expert_count.sum().item())
    return (pos, local_expert_count.cpu(), global_expert_count.cpu(), fwd_expert_count.cpu(),
            all_expert_count.cpu(), fwd_batch_size)


def perpare_expert_assignment(gate, num_expert, world_size, require_pos=True):
    """(pos on the device, all_expert_count [world, E_tot] on the CPU); the name
    keeps the reference's spelling (functions.py:83-105)."""
    _require_single(world_size)
    with torch.no_grad():
        pos, local_expert_count, _ = _route(gate, num_expert * world_size, require_pos)
        all_expert_count = local_expert_count.reshape(world_size, num_expert * world_size)
    return pos, all_expert_count.cpu()
