"""Helpers kept for interface parity (reference mix_moe/mix_moe/utils.py)."""


def get_torch_default_comm():
    """The reference digs the NCCL communicator out of torch.distributed for its
    multi-GPU exchange (utils.py:7-37).  This build runs on one GPU and has no
    communicator to return."""
    raise RuntimeError("single-GPU build: there is no communicator (world_size must be 1)")
