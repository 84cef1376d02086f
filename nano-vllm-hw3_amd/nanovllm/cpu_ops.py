"""Plain-torch counterparts of nanovllm/ops.py for tensors that live on the CPU.  PLUMBING ONLY: they let the
unquantized model run through the engine on a host without a GPU (Config(device="cpu")), following the formulas
of the reference's layers (layernorm.py:16-40, rotary_embedding.py:7-48, activation.py:11-14, attention.py:43-75,
sampler.py:10-12).  Nothing quantized goes through here and no HIP kernel falls back to this file: ops.py
dispatches on the device of its input and refuses CPU tensors for every quantized operator."""
import torch
import torch.nn.functional as F


def add_rmsnorm(x, residual, weight, eps):
    s = x.float() if residual is None else x.float() + residual.float()
    new_res = x if residual is None else s.to(x.dtype)
    out = (s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype) * weight
    return out, new_res


def silu_mul(x):
    a, b = x.chunk(2, -1)
    return F.silu(a) * b


def _rope(x, positions, cos_sin):
    cs = cos_sin[positions] if positions is not None else cos_sin      # [T, D] f32: cos | sin
    half = cs.shape[-1] // 2
    cos, sin = cs[:, None, :half], cs[:, None, half:]
    x1, x2 = x.float()[..., :half], x.float()[..., half:]
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), -1).to(x.dtype)


def _head_norm(x, w, eps):
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype) * w


def qknorm_rope_store(qkv, positions, cos_sin, q_norm_w, k_norm_w, eps, num_heads, num_kv_heads, head_dim,
                      k_cache=None, v_cache=None, slot_mapping=None, want_kv=True):
    T = qkv.shape[0]
    q, k, v = qkv.split([num_heads * head_dim, num_kv_heads * head_dim, num_kv_heads * head_dim], -1)
    q, k, v = q.view(T, num_heads, head_dim), k.view(T, num_kv_heads, head_dim), v.view(T, num_kv_heads, head_dim)
    if q_norm_w is not None:
        q, k = _head_norm(q, q_norm_w, eps), _head_norm(k, k_norm_w, eps)
    q, k = _rope(q, positions, cos_sin), _rope(k, positions, cos_sin)
    if slot_mapping is not None and k_cache is not None and k_cache.numel() > 0:
        slots = slot_mapping.long()
        keep = slots >= 0
        kc, vc = k_cache.view(-1, num_kv_heads, head_dim), v_cache.view(-1, num_kv_heads, head_dim)
        kc[slots[keep]] = k[keep]
        vc[slots[keep]] = v[keep]
    return q.contiguous(), (k.contiguous() if want_kv else None), (v.contiguous() if want_kv else None)


def _sdpa(q, k, v, scale, causal):
    # q [Tq, Hq, D], k/v [Tk, Hkv, D] -> [Tq, Hq, D]
    o = F.scaled_dot_product_attention(q.transpose(0, 1)[None].float(), k.transpose(0, 1)[None].float(),
                                       v.transpose(0, 1)[None].float(), is_causal=causal, scale=scale, enable_gqa=True)
    return o[0].transpose(0, 1).to(q.dtype)


def attn_prefill(q, k, v, cu_seqlens, max_seqlen, scale):
    cu = cu_seqlens.tolist()
    out = torch.empty_like(q)
    for a, b in zip(cu[:-1], cu[1:]):
        out[a:b] = _sdpa(q[a:b], k[a:b], v[a:b], scale, True)
    return out


def paged_attn_decode(q, k_cache, v_cache, block_tables, context_lens, scale):
    B = q.shape[0]
    block_size = k_cache.shape[1]
    out = torch.zeros_like(q)
    for b in range(B):
        n = int(context_lens[b])
        if n == 0:
            continue
        t = torch.arange(n)
        rows = block_tables[b, t // block_size].long() * block_size + t % block_size
        kk = k_cache.view(-1, *k_cache.shape[2:])[rows]
        vv = v_cache.view(-1, *v_cache.shape[2:])[rows]
        out[b:b + 1] = _sdpa(q[b:b + 1], kk, vv, scale, False)
    return out


def argmax_rows(logits):
    return logits.float().argmax(-1)


# ---- plumbing counterparts of nanovllm/seq_ops.py -------------------------------------------------------------------
def embed_streams(ids, positions, embed, pos_table, streams):
    x = embed[ids].float()
    if pos_table is not None:
        x = x + pos_table[positions.long()].float()
    return x[:, None, :].repeat(1, streams, 1).contiguous()


def stream_step(X, y, mix, out, w_in, norm_w, eps, dtype):
    if y is not None:
        X.copy_(torch.einsum("sr,tsw->trw", mix, X) + out[None, :, None] * y.float()[:, None, :])
    if w_in is None:
        return None
    u = torch.einsum("s,tsw->tw", w_in, X)
    return (u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()).to(dtype)


def canon_conv(h, w, state, run, ctx):
    taps = w.shape[1]
    out = torch.empty_like(h)
    qs = ctx.qstart.tolist()
    for b in range(ctx.num_seqs):
        a, e = qs[b], qs[b + 1]
        if e <= a:
            continue
        slot, pos0 = int(ctx.seq_slot[b]), int(ctx.seq_pos0[b])
        prev = state[slot, run][:taps - 1].float().clone()                     # [taps-1, W]: inputs at pos0-(taps-1) .. pos0-1
        for k in range(taps - 1):
            if pos0 - (taps - 1) + k < 0:
                prev[k] = 0
        hist = torch.cat([prev, h[a:e].float()], 0)
        acc = h[a:e].float().clone()
        for j in range(taps):
            acc += w[:, j].float() * hist[j:j + e - a]
        out[a:e] = acc.to(h.dtype)
        if taps > 1:
            state[slot, run] = hist[-(taps - 1):].to(state.dtype)
    return out


def latent_norm_store(x, w, eps, cache, slot_mapping):
    xf = x.float()
    c = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(cache.dtype)
    keep = slot_mapping >= 0
    cache.view(-1, cache.shape[-1])[slot_mapping[keep].long()] = c[keep]


def latent_attention(q, cache, ctx, scale):
    o = torch.empty_like(q)
    bs = cache.shape[1]
    rows = cache.view(-1, cache.shape[-1])
    qs = ctx.qstart.tolist()
    for b in range(ctx.num_seqs):
        a, e = qs[b], qs[b + 1]
        if e <= a:
            continue
        n = int(ctx.ctx_lens[b])
        t = torch.arange(n)
        c = rows[ctx.block_tables[b, t // bs].long() * bs + t % bs].float()          # [n, R]
        s = torch.einsum("thr,nr->thn", q[a:e].float(), c) * scale
        pos = ctx.tok_pos[a:e].long()
        s = s.masked_fill(t[None, None, :] > pos[:, None, None], float("-inf"))
        o[a:e] = torch.einsum("thn,nr->thr", torch.softmax(s, -1), c).to(q.dtype)
    return o


def poly_norm(z, coef, eps):
    zf = z.float()

    def unit(v):
        return v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    a, b, c, e = coef.tolist()
    return (a * unit(zf) + b * unit(zf * zf) + c * unit(zf * zf * zf) + e).to(z.dtype)


def clamped_glu(gu, limit, alpha):
    g, u = gu.float().chunk(2, -1)
    g = g.clamp(max=limit)
    u = u.clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1)).to(gu.dtype)


def moe_route(h, router_w, top, groups, keep):
    T, E = h.shape[0], router_w.shape[0]
    s = torch.softmax(h.float() @ router_w.t(), -1)
    masked = s
    if groups > 1:
        per = E // groups
        best = s.view(T, groups, per).amax(-1).topk(keep, -1).indices
        ok = torch.zeros(T, groups, dtype=torch.bool).scatter_(1, best, True)
        masked = s.masked_fill(~ok.repeat_interleave(per, 1), -1.0)
    idx = masked.topk(top, -1).indices
    w = s.gather(1, idx)
    return idx.int(), w / (w.sum(-1, keepdim=True) + 1e-20)


def moe_experts(h, idx, wts, w_gu, w_down, limit, alpha, shared):
    y = torch.zeros(h.shape, dtype=torch.float32)
    for e in idx.unique().tolist():
        tok, k = (idx == e).nonzero(as_tuple=True)
        act = clamped_glu(F.linear(h[tok], w_gu[e]), limit, alpha)
        y.index_add_(0, tok, wts[tok, k][:, None] * F.linear(act, w_down[e]).float())
    if shared is not None:
        y = y + shared.float()
    return y.to(h.dtype)
