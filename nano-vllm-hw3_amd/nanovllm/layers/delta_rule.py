"""Generalized delta rule: a recurrent mixer whose per-head state S [dim, dim] decays per key channel, forgets along the
unit key direction at a learned per-channel rate, and learns the outer product of key and value:
    S <- diag(w) S - (a * u)(u^T S) + k v^T,   o = S^T r,   u = k / |k|
with w = exp(-decay_scale * sigmoid(W_w2 tanh(W_w1 h) + w0)) and a = sigmoid(W_a h + b_a).  Every head's o is divided by
its RMS, scaled by a weight, gated by sigmoid(W_g h) and projected.  The state is float32, one [heads, dim, dim] block per
state slot; r, k, v, g, a and the decay's inner projection come from ONE merged product."""
import math

import torch
import torch.nn.functional as F
from torch import nn

from nanovllm import hy_ops, seq_ops


class GeneralDelta(nn.Module):
    def __init__(self, width, heads, dim, decay_rank, eps, decay_scale=math.exp(-0.5), unit_eps=1e-6):
        super().__init__()
        self.heads, self.dim, self.rank, self.eps = heads, dim, decay_rank, eps
        self.decay_scale, self.unit_eps = decay_scale, unit_eps
        hd = heads * dim
        # rows: r | k | v | g | a | w1
        self.in_proj = nn.Parameter(torch.empty(5 * hd + decay_rank, width), requires_grad=False)
        self.w2 = nn.Parameter(torch.empty(hd, decay_rank), requires_grad=False)
        self.w0 = nn.Parameter(torch.zeros(hd), requires_grad=False)
        self.a_bias = nn.Parameter(torch.zeros(hd), requires_grad=False)
        self.out_norm = nn.Parameter(torch.ones(hd), requires_grad=False)
        self.o_proj = nn.Parameter(torch.empty(width, hd), requires_grad=False)
        self.state = None          # f32 [slots, heads, dim, dim]

    ROWS = ("r", "k", "v", "g", "a")

    def allocate(self, num_slots, device):
        self.state = torch.zeros(num_slots, self.heads, self.dim, self.dim, dtype=torch.float32, device=device)

    def state_bytes_per_slot(self):
        return self.heads * self.dim * self.dim * 4

    def forward(self, h):
        ctx = seq_ops.get_step()
        hd = self.heads * self.dim
        p = F.linear(h, self.in_proj)
        cols = ((0, hd), (hd, hd), (4 * hd, hd), (5 * hd, self.rank))                  # r, k, a, w1
        prep = hy_ops.delta_prepare(p, cols, self.w2, self.w0, self.a_bias, self.heads, self.dim, self.decay_scale,
                                    self.unit_eps)
        o = hy_ops.delta_recurrence(prep, p[:, 2 * hd:3 * hd], self.state, ctx)
        y = hy_ops.delta_gate_norm(o, p[:, 3 * hd:4 * hd], self.out_norm, self.eps, h.dtype)
        return F.linear(y, self.o_proj)
