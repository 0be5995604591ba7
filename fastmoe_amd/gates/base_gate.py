r"""Common interface of the gates (fmoe/gates/base_gate.py)."""
import torch.nn as nn


class BaseGate(nn.Module):
    r"""Holds the expert counts and an auxiliary loss slot that a training loop
    reads with `get_loss()`."""

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
