"""A sublayer's place on a float32 residual with norms on both sides and a learned gate on its result:
    h = rms_norm(x) * norm;   x <- x + mult * rms_norm(sublayer(h) * sigmoid(W_g h + b_g)) * post_norm
``GatedPort`` holds one sublayer's weights.  The gate's product may be merged into a product of the sublayer that reads
the same h (``own_gate_weight=False``: the owner of the merged weight keeps the rows)."""
import torch
from torch import nn


class GatedPort(nn.Module):
    def __init__(self, width: int, own_gate_weight: bool = True):
        super().__init__()
        self.norm = nn.Parameter(torch.ones(width), requires_grad=False)
        self.post_norm = nn.Parameter(torch.ones(width), requires_grad=False)
        self.gate_bias = nn.Parameter(torch.zeros(width), requires_grad=False)
        self.gate_weight = nn.Parameter(torch.empty(width, width), requires_grad=False) if own_gate_weight else None
