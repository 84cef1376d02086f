"""A plain, slow restatement of the Lipelix decoder in float64 torch: one function per mechanism, whole sequences, no
cache, no state carried between calls, no code shared with the package.  Weights are a dict name -> tensor under the
checkpoint's names; ``cfg`` is the parsed config.json."""
import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def token_shift(h, mu):
    """h [T, W] -> h + (previous h - h) * mu, the row before the first being zero."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], 0)
    return h + (prev - h) * mu


def rotate(x, pos, dims, base):
    """x [T, heads, D]: the first ``dims`` channels of every head turn by pos * base^(-2i/dims), channel i paired with
    channel i + dims/2."""
    half = dims // 2
    f = base ** (-2.0 * torch.arange(half, dtype=F64) / dims)
    ang = pos.to(F64)[:, None] * f[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], -1)


def visible(T, window=None, keep_first=0):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window is not None:
        ok &= ((i - j) < window) | (j < keep_first)
    return ok


def softmax_with_sink(scores, ok, sink):
    """scores [H, T, T]; ``sink`` [H]: one more term exp(sink) in every row's denominator, with no value."""
    s = scores.masked_fill(~ok[None], -math.inf)
    m = torch.maximum(s.max(-1, keepdim=True).values, sink[:, None, None])
    e = torch.exp(s - m)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink[:, None, None] - m))


def attention(h, w, pre, m, eps, kind, v_first):
    """Both attention mixers.  kind "attention": RMS norm with a weight over the whole q / k projection before the
    rotation, a learned sink per head, full causal.  kind "attention_2": rotation, then every head of q and k divided
    by its RMS, a sink of score 0, a window that also keeps the first tokens.  Returns (output, the cached values)."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ w[pre + "q"].T, h @ w[pre + "k"].T, h @ w[pre + "v"].T
    if kind == "attention":
        q = rms(q, eps) * w[pre + "q.norm"]
        k = rms(k, eps) * w[pre + "k.norm"]
    q, k, v = q.view(T, H, D), k.view(T, G, D), v.view(T, G, V)
    pos = torch.arange(T)
    q, k = rotate(q, pos, m["rot"]["dims"], m["rot"]["base"]), rotate(k, pos, m["rot"]["dims"], m["rot"]["base"])
    if kind == "attention_2":
        q, k = rms(q, eps), rms(k, eps)
    if m.get("v_mix"):
        if v_first is not None:
            lam = w[pre + "vmix"]
            v = (1 - lam) * v + lam * v_first
    rep = H // G
    kh, vh = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)
    scores = torch.einsum("ihd,jhd->hij", q, kh) * m["scale"]
    if kind == "attention":
        ok, sink = visible(T), w[pre + "sink"].to(F64)
    else:
        ok, sink = visible(T, m["mask"]["size"], m["mask"]["keep_first"]), torch.zeros(H, dtype=F64)
    p = softmax_with_sink(scores, ok, sink)
    o = torch.einsum("hij,jhv->ihv", p, vh).reshape(T, H * V)
    return o @ w[pre + "o"].T, v


def general_delta(h, w, pre, m, eps):
    """S <- diag(decay) S - (a u)(u^T S) + k v^T per head, both terms reading the old S; o = S^T r."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    r, k, v = (h @ w[pre + n].T for n in ("r", "k", "v"))
    decay = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(h @ w[pre + "w1"].T) @ w[pre + "w2"].T + w[pre + "w0"]))
    a = torch.sigmoid(h @ w[pre + "a"].T + w[pre + "a.b"])
    r, k, v, decay, a = (x.view(T, H, D) for x in (r, k, v, decay, a))
    u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    S = torch.zeros(H, D, D, dtype=F64)
    out = []
    for t in range(T):
        uS = torch.einsum("hi,hij->hj", u[t], S)
        S = decay[t][:, :, None] * S - (a[t] * u[t])[:, :, None] * uS[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hij,hi->hj", S, r[t]))
    o = rms(torch.stack(out), eps).reshape(T, H * D) * w[pre + "norm"]
    o = o * torch.sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T


def relu2_mlp(h, w, pre):
    return torch.relu(h @ w[pre + "up"].T) ** 2 @ w[pre + "down"].T


def forward(cfg, weights, tokens, layers_out=None):
    """Logits [T, vocab] of one whole sequence; ``layers_out`` receives the residual after every layer."""
    w = {k: v.to(F64) for k, v in weights.items()}
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = w["embed"][torch.as_tensor(tokens)] * cfg["embedding"]["scale"]
    v_first = None
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms(x, eps) * w[p + "norm1"]
        gate = torch.sigmoid(h @ w[p + "rg1"].T + w[p + "rg1.b"])
        hs = token_shift(h, w[p + "shift"])
        if spec["type"] in ("attention", "attention_2"):
            y, v = attention(hs, w, p + "mix.", spec["mixer"], eps, spec["type"], v_first)
            if spec["mixer"].get("v_mix") and v_first is None:
                v_first = v
        elif spec["type"] == "general_delta":
            y = general_delta(hs, w, p + "mix.", spec["mixer"], eps)
        else:
            raise ValueError(spec["type"])
        x = x + mult * rms(y * gate, eps) * w[p + "norm1b"]
        if spec.get("mlp") is not None:
            h = rms(x, eps) * w[p + "norm2"]
            gate = torch.sigmoid(h @ w[p + "rg2"].T + w[p + "rg2.b"])
            x = x + mult * rms(relu2_mlp(h, w, p + "mlp.") * gate, eps) * w[p + "norm2b"]
        if layers_out is not None:
            layers_out.append(x.clone())
    return (rms(x, eps) * w["final.norm"]) @ w["head"].T
