"""Short causal convolution over time on every channel, added to its input ("canon" layer).  The last taps-1 inputs of
every sequence are state: the engine gives each sequence a state slot, and one tensor holds the state of every
(slot, layer run)."""
import torch
from torch import nn

from nanovllm import seq_ops


class CausalTaps(nn.Module):
    def __init__(self, width: int, taps: int):
        super().__init__()
        self.taps = taps
        self.weight = nn.Parameter(torch.zeros(width, taps), requires_grad=False)     # [channel, tap]; tap taps-1 = now
        self.state = None          # [slots, runs, taps-1, width], shared by all layer runs (set by the cache allocation)

    def forward(self, h, run: int):
        return seq_ops.canon_conv(h, self.weight, self.state, run, seq_ops.get_step())
