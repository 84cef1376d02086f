"""Latent attention: keys and values are up-projections of one small per-token latent, and only the latent is cached.
No positional rotation.  The key up-projection is folded into the query ("absorbed": q'_h = W_uk,h^T q_h, so that
q_h . k_h = q'_h . c) and the value up-projection is applied after the attention sum, which makes the cached latent
both key and value of a multi-query attention with ``heads`` query heads of size ``kv_rank``."""
import torch
import torch.nn.functional as F
from torch import nn

from nanovllm import seq_ops


class LatentAttention(nn.Module):
    def __init__(self, width: int, heads: int, dim: int, vdim: int, kv_rank: int, scale: float, eps: float):
        super().__init__()
        self.heads, self.dim, self.vdim, self.kv_rank, self.scale, self.eps = heads, dim, vdim, kv_rank, float(scale), eps
        # query and latent down-projection share one product: rows [0, heads*dim) = W_q, then kv_rank rows of W_dkv
        self.qc_proj = nn.Parameter(torch.empty(heads * dim + kv_rank, width), requires_grad=False)
        self.latent_norm = nn.Parameter(torch.ones(kv_rank), requires_grad=False)
        self.uk = nn.Parameter(torch.empty(heads, dim, kv_rank), requires_grad=False)      # per head [dim, kv_rank]
        self.uv = nn.Parameter(torch.empty(heads, vdim, kv_rank), requires_grad=False)     # per head [vdim, kv_rank]
        self.o_proj = nn.Parameter(torch.empty(width, heads * vdim), requires_grad=False)
        self.cache = {}            # layer run -> [blocks, block_size, kv_rank]

    def forward(self, h, run: int):
        ctx = seq_ops.get_step()
        T = h.shape[0]
        H, D = self.heads, self.dim
        qc = F.linear(h, self.qc_proj)                                     # [T, H*D + R]
        cache = self.cache[run]
        seq_ops.latent_norm_store(qc[:, H * D:], self.latent_norm, self.eps, cache, ctx.slot_mapping)
        q = qc[:, :H * D].view(T, H, D).transpose(0, 1)                    # [H, T, D]
        qa = torch.bmm(q, self.uk).transpose(0, 1).contiguous()            # absorbed queries [T, H, R]
        ol = seq_ops.latent_attention(qa, cache, ctx, self.scale)          # [T, H, R]
        ov = torch.bmm(ol.transpose(0, 1), self.uv.transpose(1, 2))        # [H, T, V]
        return F.linear(ov.transpose(0, 1).reshape(T, H * self.vdim), self.o_proj)
