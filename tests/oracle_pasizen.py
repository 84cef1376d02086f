"""A plain, slow restatement of the Pasizen decoder in fp32 torch on the CPU: one function per mechanism, whole
sequences at once, no cache, no batching.  Test infrastructure only; it shares no code with the package.

Notation.  T tokens, W model width, S residual streams.  Weights are a dict name -> tensor with the checkpoint's
names ('l3.mix.q', 'l3.mlp.e0.gate', ...); linear weights are [out, in].
"""
import torch


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return rms_unit(x, eps) * w


def causal_taps(h, w):
    """h [T, W], w [W, taps] -> [T, W]: out[t] = sum_j w[:, j] * h[t - (taps - 1) + j], zero before the start."""
    T, taps = h.shape[0], w.shape[1]
    out = torch.zeros_like(h)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                out[t] += w[:, j] * h[src]
    return out


def stream_read(xs, w_in):
    """xs [S, T, W], w_in [S] -> the sublayer's input [T, W]."""
    return torch.einsum("s,stw->tw", w_in, xs)


def stream_write(xs, y, w_mix, w_out):
    """new[t] = sum_s mix[s, t] * old[s] + out[t] * y, every stream from the OLD ones."""
    return torch.einsum("sr,stw->rtw", w_mix, xs) + w_out[:, None, None] * y[None]


def latent_attention(h, W, p, m, eps):
    """h [T, W]; m = the layer's mixer sizes (heads, dim, vdim, kv_rank, scale)."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).view(T, H, D)
    c = rms_norm(h @ W[p + "dkv"].T, W[p + "dkv.norm"], eps)          # the latent: all that a cache would hold
    k = (c @ W[p + "uk"].T).view(T, H, D)
    v = (c @ W[p + "uv"].T).view(T, H, V)
    out = torch.zeros(T, H, V)
    for i in range(T):
        for hh in range(H):
            s = (k[: i + 1, hh] @ q[i, hh]) * m["scale"]
            a = torch.softmax(s, 0)
            out[i, hh] = a @ v[: i + 1, hh]
    return out.reshape(T, H * V) @ W[p + "o"].T


def poly_norm(z, coef, eps):
    a, b, c, e = [float(v) for v in coef]
    return a * rms_unit(z, eps) + b * rms_unit(z * z, eps) + c * rms_unit(z * z * z, eps) + e


def dense_ff(h, W, p, eps):
    return poly_norm(h @ W[p + "up"].T, W[p + "act"], eps) @ W[p + "down"].T


def clamped_glu_expert(h, W, p, limit):
    g = torch.clamp(h @ W[p + "gate"].T, max=limit)
    u = torch.clamp(h @ W[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ W[p + "down"].T


def route(h, w_router, r):
    """Returns (chosen experts [T, top], their weights [T, top])."""
    T = h.shape[0]
    E, top = r["experts"], r["top"]
    s = torch.softmax(h @ w_router.T, -1)
    allowed = torch.ones(T, E, dtype=torch.bool)
    g = r.get("groups")
    if g:
        per = E // g["count"]
        gs = s.view(T, g["count"], per).max(-1).values
        best = gs.topk(g["keep"], -1).indices
        ok = torch.zeros(T, g["count"], dtype=torch.bool)
        ok.scatter_(1, best, True)
        allowed = ok[:, :, None].expand(T, g["count"], per).reshape(T, E)
    idx = s.masked_fill(~allowed, -1.0).topk(top, -1).indices
    w = s.gather(1, idx)
    return idx, w / (w.sum(-1, keepdim=True) + 1e-20)


def moe_ff(h, W, p, mlp):
    idx, w = route(h, W[p + "router"], mlp["router"])
    out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0])
    for t in range(h.shape[0]):
        for e, we in zip(idx[t].tolist(), w[t]):
            out[t] += we * clamped_glu_expert(h[t:t + 1], W, f"{p}e{e}.", mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        out = out + clamped_glu_expert(h, W, p + "shared.", mlp["shared"]["limit"])
    return out


def layer_runs(cfg):
    """The order in which layers run: layers start..stop-1 repeat 'times' times in a row."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    body = list(range(lp["start"], lp["stop"]))
    return list(range(lp["start"])) + body * lp["times"] + list(range(lp["stop"], n))


def forward(cfg, W, tokens, return_layers=False):
    """tokens: list of ids of ONE sequence -> logits [T, vocab] (and the summed streams after every layer run)."""
    W = {k: (v.float() if v.is_floating_point() else v) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    S = cfg.get("streams") or 0
    T = len(tokens)
    x = W["embed"][torch.tensor(tokens)] + W["pos"][:T]
    xs = x[None].repeat(max(S, 1), 1, 1)
    trace = []
    for li in layer_runs(cfg):
        L = cfg["layers"][li]
        p = f"l{li}."
        for q, kind in ((1, "mix"), (2, "mlp")):
            if kind == "mlp" and L.get("mlp") is None:
                continue
            u = stream_read(xs, W[f"{p}hc{q}.in"]) if S else xs[0]
            h = rms_norm(u, W[f"{p}norm{q}"], eps)
            if kind == "mix":
                if cfg.get("canon"):
                    h = h + causal_taps(h, W[p + "canon1"])
                assert L["type"] == "latent_attention"
                y = latent_attention(h, W, p + "mix.", L["mixer"], eps)
            elif L["mlp"]["kind"] == "dense":
                y = dense_ff(h, W, p + "mlp.", eps)
            else:
                y = moe_ff(h, W, p + "mlp.", L["mlp"])
            xs = stream_write(xs, y, W[f"{p}hc{q}.mix"], W[f"{p}hc{q}.out"]) if S else xs + y[None]
        trace.append(xs.sum(0))
    x = rms_norm(xs.sum(0), W["final.norm"], eps)
    logits = x @ W["head"].T
    return (logits, torch.stack(trace)) if return_layers else logits


def absorbed_attention(qa, c, positions, scale):
    """The attention sum with the key up-projection folded into the query: qa [T, H, R], latents c [N, R] (position j
    in row j), positions [T] -> o [T, H, R] with o[t, h] = sum_{j <= positions[t]} softmax_j(scale * qa[t, h] . c_j) c_j.
    (latent_attention above equals W_o applied to W_uv,h o[t, h] with qa[t, h] = W_uk,h^T q[t, h].)"""
    T, H, R = qa.shape
    o = torch.zeros(T, H, R)
    for t in range(T):
        n = int(positions[t]) + 1
        for h in range(H):
            a = torch.softmax((c[:n] @ qa[t, h]) * scale, 0)
            o[t, h] = a @ c[:n]
    return o
