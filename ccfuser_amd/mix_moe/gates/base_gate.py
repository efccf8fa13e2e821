"""Gate interface (reference mix_moe/mix_moe/gates/base_gate.py:7-29)."""
import torch.nn as nn


class BaseGate(nn.Module):
    """Holds the expert counts and an optional auxiliary loss, as the reference's
    BaseGate does; subclasses implement ``forward``."""

    def __init__(self, num_expert, world_size):
        super().__init__()
        self.world_size = world_size
        self.num_expert = num_expert
        self.tot_expert = world_size * num_expert
        self.loss = None

    def forward(self, x):
        raise NotImplementedError("Base gate cannot be directly used for fwd")

    def set_loss(self, loss):
        self.loss = loss

    def get_loss(self, clear=True):
        loss, self.loss = self.loss, (None if clear else self.loss)
        return loss

    @property
    def has_loss(self):
        return self.loss is not None
