"""Token shift: a sublayer reads h + (h_prev - h) * mu, a per-channel blend of a token's input with the previous token's
(zero before the first token).  The last input of every sequence is state: one tensor [slots, layers, width] holds it for
every (state slot, layer); the row is written when the sublayer closes (hy_ops.sublayer_close ``carry``)."""
import torch
from torch import nn

from nanovllm import hy_ops, seq_ops


class TokenShift(nn.Module):
    def __init__(self, width: int):
        super().__init__()
        self.mu = nn.Parameter(torch.zeros(width), requires_grad=False)
        self.state = None          # [slots, layers, width], shared by all layers (set by the cache allocation)

    def forward(self, h, layer: int):
        return hy_ops.token_shift(h, self.mu, self.state, layer, seq_ops.get_step())
