"""Attention over a paged key/value cache with rotary positions on part of every head and the variations that differ
between designs as constructor arguments:
  proj_norm   RMS norm with a weight over the whole q and the whole k projection, before the rotation
  unit_norm   every rotated q and k head divided by its RMS (no weight)
  sink        "learned": a per-head score that joins the softmax denominator without a value; "zero": the same with score
              0 (one added to the denominator); None: plain softmax
  window, keep_first   window > 0: a query sees the last ``window`` positions and the first ``keep_first`` tokens
  v_mix       values blended with those of the first such layer of the model, (1 - lam) v + lam v_first, before caching
Grouped heads: query head h reads key/value head h // (heads / kv_heads).  q, k and v come from ONE merged product."""
import torch
import torch.nn.functional as F
from torch import nn

from nanovllm import hy_ops, seq_ops


class PagedRotaryAttention(nn.Module):
    def __init__(self, width, heads, kv_heads, dim, vdim, scale, eps, rot_dims, rot_base, proj_norm=False, unit_norm=False,
                 sink=None, window=0, keep_first=0, v_mix=False):
        super().__init__()
        assert heads % kv_heads == 0 and rot_dims % 2 == 0 and rot_dims <= dim and sink in (None, "learned", "zero")
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.eps, self.unit_norm = float(scale), eps, unit_norm
        self.window, self.keep_first, self.v_mix = int(window), int(keep_first), v_mix
        self.rot_dims, self.rot_base = rot_dims, rot_base
        self.qkv_proj = nn.Parameter(torch.empty(heads * dim + kv_heads * (dim + vdim), width), requires_grad=False)
        self.o_proj = nn.Parameter(torch.empty(width, heads * vdim), requires_grad=False)
        f32 = dict(dtype=torch.float32)
        self.q_norm = nn.Parameter(torch.ones(heads * dim), requires_grad=False) if proj_norm else None
        self.k_norm = nn.Parameter(torch.ones(kv_heads * dim), requires_grad=False) if proj_norm else None
        self.sink = nn.Parameter(torch.zeros(heads, **f32), requires_grad=False) if sink else None
        self.lam = nn.Parameter(torch.zeros(1, **f32), requires_grad=False) if v_mix else None
        self.inv_freq = None       # f32 [rot_dims / 2], made with the cache
        self.k_cache = self.v_cache = None

    def allocate(self, num_blocks, block_size, dtype, device):
        self.k_cache = torch.zeros(num_blocks, block_size, self.kv_heads, self.dim, dtype=dtype, device=device)
        self.v_cache = torch.zeros(num_blocks, block_size, self.kv_heads, self.vdim, dtype=dtype, device=device)
        self.inv_freq = hy_ops.rotary_inv_freq(self.rot_dims, self.rot_base, device)

    def cache_bytes_per_token(self, itemsize):
        return self.kv_heads * (self.dim + self.vdim) * itemsize

    def forward(self, h, v_first=None):
        """h [T, width] -> (output [T, width], this layer's own values [T, kv_heads * vdim] before any blending)."""
        ctx = seq_ops.get_step()
        qkv = F.linear(h, self.qkv_proj)
        q = hy_ops.qkv_prepare(qkv, self.heads, self.kv_heads, self.dim, self.vdim, self.q_norm, self.k_norm, self.eps,
                               self.inv_freq, self.unit_norm, ctx, self.k_cache, self.v_cache,
                               v_first if self.v_mix else None, self.lam)
        o = hy_ops.paged_attention(q, self.k_cache, self.v_cache, ctx, self.scale, self.sink, self.window, self.keep_first)
        return F.linear(o, self.o_proj), qkv[:, (self.heads + self.kv_heads) * self.dim:]
