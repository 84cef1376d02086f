"""Each mechanism of nanovllm.seq_ops alone against its restatement in tests/oracle_pasizen.py: on the CPU the
engine's plumbing operators, on the GPU (marked gpu) the HIP kernels of libseqmix in float32 and bfloat16, the
matrix-core attention kernels against the portable one and the oracle.  Inputs are shaped so that a fault shows: one
key's score stands far out (a dropped or leaked key changes the output by O(1)), placed at the first keys, at cache
block and tile borders, far back, and just inside / just outside a query's causal edge."""
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "nano-vllm-hw3_amd"))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import oracle_pasizen as O  # noqa: E402
from nanovllm import seq_ops  # noqa: E402

CASES = [("cpu", torch.float32), pytest.param("cuda", torch.float32, marks=pytest.mark.gpu),
         pytest.param("cuda", torch.bfloat16, marks=pytest.mark.gpu)]


def gen(seed):
    return torch.Generator().manual_seed(seed)


def rnd(g, *shape, s=1.0):
    return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16).float()      # bf16-representable in every format


def tol(dtype, scale=1.0):
    return dict(atol=(2e-5 if dtype == torch.float32 else 2e-2) * scale, rtol=1e-5 if dtype == torch.float32 else 2e-2)


def step_context(portions, block_size, tables, slots, device):
    """portions [(pos0, n)] -> StepContext with the packed layout the engine builds."""
    B = len(portions)
    tok_seq, tok_pos, slot_map, qstart = [], [], [], [0]
    for b, (p0, n) in enumerate(portions):
        for p in range(p0, p0 + n):
            tok_seq.append(b)
            tok_pos.append(p)
            slot_map.append(tables[b][p // block_size] * block_size + p % block_size)
        qstart.append(qstart[-1] + n)
    mb = max(len(t) for t in tables)
    bt = torch.zeros(B, mb, dtype=torch.int32)
    for b, t in enumerate(tables):
        bt[b, :len(t)] = torch.tensor(t, dtype=torch.int32)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)  # noqa: E731
    return seq_ops.StepContext(tok_seq=i32(tok_seq), tok_pos=i32(tok_pos), qstart=i32(qstart), seq_pos0=i32([p for p, _ in portions]),
                               ctx_lens=i32([p + n for p, n in portions]), seq_slot=i32(slots), slot_mapping=i32(slot_map),
                               block_tables=bt.to(device), num_seqs=B, num_tokens=len(tok_seq), max_q=max(n for _, n in portions),
                               block_size=block_size, qstart_host=qstart)


# ------------------------------------------------------------------------------------------ streams + norm
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("S,W", [(1, 40), (4, 200), (3, 1000)])
def test_stream_step(device, dtype, S, W):
    g = gen(S * W)
    T = 5
    X0, y = rnd(g, T, S, W), rnd(g, T, W)
    mix, out, w_in, nw = rnd(g, S, S, s=0.5), rnd(g, S), rnd(g, S), 1 + rnd(g, W, s=0.1)
    xs = X0.permute(1, 0, 2)                                           # oracle layout [S, T, W]
    new = O.stream_write(xs, y, mix, out)
    h_ref = O.rms_norm(O.stream_read(new, w_in), nw, 1e-5)
    X = X0.clone().to(device)
    h = seq_ops.stream_step(X, y.to(device, dtype), mix.to(device), out.to(device), w_in.to(device), nw.to(device, dtype), 1e-5, dtype)
    assert torch.allclose(X.cpu(), new.permute(1, 0, 2), atol=1e-5, rtol=1e-5)          # the streams are float32 always
    assert torch.allclose(h.float().cpu(), h_ref, **tol(dtype, 4))
    # read only (the first sublayer) and write only
    X = X0.clone().to(device)
    h = seq_ops.stream_step(X, None, None, None, w_in.to(device), nw.to(device, dtype), 1e-5, dtype)
    assert torch.equal(X.cpu(), X0) and torch.allclose(h.float().cpu(), O.rms_norm(O.stream_read(xs, w_in), nw, 1e-5), **tol(dtype, 4))
    assert seq_ops.stream_step(X, y.to(device, dtype), mix.to(device), out.to(device), None, None, 1e-5, dtype) is None
    assert torch.allclose(X.cpu(), new.permute(1, 0, 2), atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("device,dtype", CASES)
def test_embed_streams(device, dtype):
    g = gen(1)
    emb, pos = rnd(g, 30, 24), rnd(g, 50, 24)
    ids, p = torch.tensor([3, 29, 0, 3]), torch.tensor([0, 49, 7, 8], dtype=torch.int32)
    X = seq_ops.embed_streams(ids.to(device), p.to(device), emb.to(device, dtype), pos.to(device, dtype), 3)
    ref = emb[ids] + pos[p.long()]
    assert X.dtype == torch.float32 and X.shape == (4, 3, 24)
    for s in range(3):
        assert torch.equal(X[:, s].cpu(), ref)
    X = seq_ops.embed_streams(ids.to(device), p.to(device), emb.to(device, dtype), None, 1)
    assert torch.equal(X[:, 0].cpu(), emb[ids])


# ------------------------------------------------------------------------------------------ short convolution
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_canon_conv_portions_and_state(device, dtype, taps):
    """Two sequences advance through portions of unequal sizes (1 and 2 tokens too, shorter than the taps) in shared
    steps; the slots start full of another sequence's values, which must never be read."""
    g = gen(taps)
    W, runs = 70, 3
    lens = [23, 9]
    hs = [rnd(g, n, W) for n in lens]
    w = rnd(g, W, taps, s=0.5)
    ref = [h + O.causal_taps(h, w) for h in hs]
    state = (torch.randn(4, runs, max(taps - 1, 1), W, generator=g) * 100).to(device, dtype)
    cuts = [[(0, 1), (1, 3), (3, 4), (4, 12), (12, 14), (14, 23)], [(0, 2), (2, 3), (3, 9)]]
    step = 0
    while any(step < len(c) for c in cuts):
        act = [b for b in range(2) if step < len(cuts[b])]
        portions = [(cuts[b][step][0], cuts[b][step][1] - cuts[b][step][0]) for b in act]
        ctx = step_context(portions, 64, [[0]] * len(act), [[2, 0][b] for b in act], device)
        h = torch.cat([hs[b][cuts[b][step][0]:cuts[b][step][1]] for b in act]).to(device, dtype)
        out = seq_ops.canon_conv(h, w.to(device, dtype), state, 1, ctx)
        want = torch.cat([ref[b][cuts[b][step][0]:cuts[b][step][1]] for b in act])
        assert torch.allclose(out.float().cpu(), want, **tol(dtype, 4)), (taps, step)
        step += 1


# ------------------------------------------------------------------------------------------ latent attention
def paged(c_list, block_size, R, device, dtype, seed):
    """Scatter every sequence's latents into a shuffled block pool (unused rows hold large junk): cache, tables."""
    need = [(len(c) + block_size - 1) // block_size for c in c_list]
    total = sum(need) + 3
    perm = torch.randperm(total, generator=gen(seed)).tolist()
    cache = torch.full((total, block_size, R), 7.0)
    tables = []
    for c, n in zip(c_list, need):
        blocks, perm = perm[:n], perm[n:]
        tables.append(blocks)
        for j in range(len(c)):
            cache[blocks[j // block_size], j % block_size] = c[j]
    return cache.to(device, dtype), tables


def spiked(g, n, R, spikes, u, amp=6.0):
    """Random latents whose rows ``spikes`` point along u: for a query along u those keys' scores stand out."""
    c = rnd(g, n, R, s=0.3)
    for j in spikes:
        if 0 <= j < n:
            c[j] = (u * amp + rnd(g, R, s=0.2)).to(torch.bfloat16).float()
    return c


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,R,bs", [(8, 72, 64), (3, 40, 128), (5, 36, 64), (16, 128, 64), (40, 256, 64), (2, 8, 64)])
def test_latent_attention_prompts_and_decode(device, dtype, H, R, bs):
    """Portions with and without earlier context, single tokens, and a batch of both, against the oracle; every form
    the dispatcher has (portable rows; tiles and split-key decode on the matrix cores for bf16 with R % 8 == 0)."""
    g = gen(H * R)
    u = torch.nn.functional.normalize(rnd(g, R), dim=0)
    # (context before the step, tokens in the step); spikes at the first keys, tile / block borders, far back, the edges
    seqs = [(0, 70), (130, 5), (257, 1), (63, 2), (700, 1), (0, 1), (64, 64), (190, 67)]
    spikes = [0, 1, 5, 62, 63, 64, 65, 127, 128, 129, 191, 192, 255, 256, 257, 699, 700]
    c_list = [spiked(g, p0 + n, R, spikes + [p0 - 1, p0, p0 + 1, p0 + n - 2, p0 + n - 1], u) for p0, n in seqs]
    scale = 0.7
    cache, tables = paged(c_list, bs, R, device, dtype, seed=H)

    def run(sel, **kw):
        ctx = step_context([seqs[i] for i in sel], bs, [tables[i] for i in sel], list(range(len(sel))), device)
        qs, refs = [], []
        for i in sel:
            p0, n = seqs[i]
            # queries along u (so the spiked keys dominate where visible) with a random part per head
            qa = (u[None, None, :] * 3 + rnd(gen(i), n, H, R, s=0.5)).to(torch.bfloat16).float()
            qs.append(qa)
            refs.append(O.absorbed_attention(qa, c_list[i], torch.arange(p0, p0 + n), scale))
        o = seq_ops.latent_attention(torch.cat(qs).to(device, dtype).contiguous(), cache, ctx, scale, **kw)
        assert torch.allclose(o.float().cpu(), torch.cat(refs), **tol(dtype, 4)), sel
        return o
    for sel in ([0], [1], [2], [3], [4], [5], [6], [7], [0, 1, 2, 3, 4, 5, 6, 7], [2, 4, 5], [4, 2]):
        o = run(sel)
        if device == "cuda":
            o_rows = run(sel, force_rows=True)
            assert torch.allclose(o.float(), o_rows.float(), **tol(dtype, 4))


@pytest.mark.parametrize("device,dtype", CASES)
def test_latent_attention_causal_edge_inside_a_portion(device, dtype):
    """One huge key in the middle of a portion: queries before it must not feel it, queries from it on are taken over."""
    g = gen(5)
    H, R, bs, p0, n = 4, 64, 64, 100, 90
    u = torch.nn.functional.normalize(rnd(g, R), dim=0)
    for edge in (100, 101, 127, 128, 129, 150, 189):
        c = spiked(g, p0 + n, R, [edge], u, amp=10.0)
        cache, tables = paged([c], bs, R, device, dtype, seed=edge)
        ctx = step_context([(p0, n)], bs, tables, [0], device)
        qa = (u[None, None, :] * 4).expand(n, H, R).contiguous()
        o = seq_ops.latent_attention(qa.to(device, dtype), cache, ctx, 1.0).float().cpu()
        along = (o @ u)                                            # [n, H]: about 10 where the key is seen, small before
        seen = torch.arange(p0, p0 + n) >= edge
        assert (along[seen] > 8).all() and (along[~seen].abs() < 2).all(), edge
        assert torch.allclose(o, O.absorbed_attention(qa, c, torch.arange(p0, p0 + n), 1.0), **tol(dtype, 10))


@pytest.mark.parametrize("device,dtype", CASES)
def test_latent_norm_store(device, dtype):
    g = gen(9)
    R, bs = 40, 64
    x, w = rnd(g, 6, 100), 1 + rnd(g, R, s=0.1)
    cache = torch.zeros(3, bs, R).to(device, dtype)
    slots = torch.tensor([70, 5, -1, 191, 0, 64], dtype=torch.int32)
    seq_ops.latent_norm_store(x.to(device, dtype)[:, 60:], w.to(device, dtype), 1e-5, cache, slots.to(device))
    ref = O.rms_norm(x[:, 60:], w, 1e-5)
    flat = cache.view(-1, R).float().cpu()
    for t, s in enumerate(slots.tolist()):
        if s >= 0:
            assert torch.allclose(flat[s], ref[t], **tol(dtype, 4))
    assert flat[1].abs().sum() == 0                                # rows nobody named stay untouched


# ------------------------------------------------------------------------------------------ feed-forward pieces
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("F", [8, 392, 1000])
def test_poly_norm(device, dtype, F):
    g = gen(F)
    z, coef = rnd(g, 7, F, s=2.0), torch.tensor([0.6, -0.3, 0.2, 0.05])
    out = seq_ops.poly_norm(z.to(device, dtype), coef.to(device), 1e-5)
    assert torch.allclose(out.float().cpu(), O.poly_norm(z, coef, 1e-5), **tol(dtype, 4))


@pytest.mark.parametrize("device,dtype", CASES)
def test_clamped_glu(device, dtype):
    g = gen(3)
    F, limit = 24, 1.5
    gu = rnd(g, 9, 2 * F, s=2.0)                                       # many values beyond the limit on both sides
    gate, up = gu[:, :F].clamp(max=limit), gu[:, F:].clamp(-limit, limit)
    ref = gate * torch.sigmoid(1.702 * gate) * (up + 1)
    out = seq_ops.clamped_glu(gu.to(device, dtype), limit)
    assert torch.allclose(out.float().cpu(), ref, **tol(dtype, 4))


ROUTES = [(16, 5, 4, 2), (6, 2, 3, 2), (6, 3, 3, 2), (8, 1, 1, 1), (8, 3, 4, 4), (12, 12, 1, 1), (5, 2, 1, 1), (64, 8, 8, 3)]


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("E,top,groups,keep", ROUTES)
def test_moe_route_and_experts(device, dtype, E, top, groups, keep):
    """Grouped top-k routing (the best expert of a dropped group outscores chosen ones: group limits bite) and the
    weighted expert sum with a shared expert."""
    g = gen(E * top)
    T, W, F = 33, 48, 24
    h = rnd(g, T, W)
    rw = rnd(g, E, W, s=3 * W ** -0.5)
    r = dict(experts=E, top=top)
    if groups > 1:
        r["groups"] = dict(count=groups, keep=keep)
    idx_ref, w_ref = O.route(h, rw, r)
    idx, wts = seq_ops.moe_route(h.to(device, dtype), rw.to(device), top, groups, keep)
    order = idx.cpu().long().sort(-1)
    ref_order = idx_ref.sort(-1)
    assert torch.equal(order.values, ref_order.values)
    assert torch.allclose(wts.cpu().gather(1, order.indices), w_ref.gather(1, ref_order.indices), atol=1e-5, rtol=1e-4)
    if groups > 1 and top > keep:          # (with top <= keep the best experts always lie in the best groups)
        free_idx, _ = O.route(h, rw, dict(experts=E, top=top))
        assert not torch.equal(free_idx.sort(-1).values, ref_order.values)       # the test's scores do cross groups
    Wt = {}
    for e in range(E):
        Wt[f"m.e{e}.gate"], Wt[f"m.e{e}.up"], Wt[f"m.e{e}.down"] = rnd(g, F, W, s=0.3), rnd(g, F, W, s=0.3), rnd(g, W, F, s=0.2)
    w_gu = torch.stack([torch.cat([Wt[f"m.e{e}.gate"], Wt[f"m.e{e}.up"]]) for e in range(E)])
    w_down = torch.stack([Wt[f"m.e{e}.down"] for e in range(E)])
    shared = rnd(g, T, W)
    ref = torch.zeros(T, W)
    for t in range(T):
        for e, we in zip(idx_ref[t].tolist(), w_ref[t]):
            ref[t] += we * O.clamped_glu_expert(h[t:t + 1], Wt, f"m.e{e}.", 0.7)[0]
    y = seq_ops.moe_experts(h.to(device, dtype), idx_ref.int().to(device), w_ref.to(device), w_gu.to(device, dtype),
                            w_down.to(device, dtype), 0.7, shared=shared.to(device, dtype))
    assert torch.allclose(y.float().cpu(), ref + shared, **tol(dtype, 6))
    y = seq_ops.moe_experts(h.to(device, dtype), idx_ref.int().to(device), w_ref.to(device), w_gu.to(device, dtype),
                            w_down.to(device, dtype), 0.7)
    assert torch.allclose(y.float().cpu(), ref, **tol(dtype, 6))
    if device == "cuda":                        # both forms of the expert products, whatever the dispatcher picks by size
        forms = ["pairs"] + (["grouped", "tiles128"] if dtype == torch.bfloat16 else [])
        for form in forms:
            for sh in (None, shared):
                y = seq_ops.moe_experts(h.to(device, dtype), idx_ref.int().to(device), w_ref.to(device), w_gu.to(device, dtype),
                                        w_down.to(device, dtype), 0.7, shared=None if sh is None else sh.to(device, dtype), form=form)
                assert torch.allclose(y.float().cpu(), ref + (0 if sh is None else sh), **tol(dtype, 6)), form


@pytest.mark.gpu
@pytest.mark.parametrize("T,W,F,E,top", [(300, 200, 72, 7, 3), (1, 64, 8, 3, 2), (1000, 256, 384, 16, 4), (65, 72, 40, 40, 1)])
def test_moe_grouped_equals_pairs(T, W, F, E, top):
    """Grouped expert products on the matrix cores against the pair-by-pair form: widths and expert sizes that are no
    multiples of the 64-k step or the 128-column tile, experts without any token, one token, more experts than pairs."""
    g = gen(T + W)
    h = rnd(g, T, W).cuda().bfloat16()
    idx = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).int()
    if E > 4:
        idx[idx == 2] = 3 if top == 1 else idx[idx == 2]            # (top 1: expert 2 gets no token at all)
    wts = torch.rand(T, top, generator=g)
    w_gu, w_down, shared = rnd(g, E, 2 * F, W, s=W ** -0.5).cuda().bfloat16(), rnd(g, E, W, F, s=F ** -0.5).cuda().bfloat16(), rnd(g, T, W).cuda().bfloat16()
    a = seq_ops.moe_experts(h, idx.cuda(), wts.cuda(), w_gu, w_down, 1.2, shared=shared, form="pairs").float()
    b = seq_ops.moe_experts(h, idx.cuda(), wts.cuda(), w_gu, w_down, 1.2, shared=shared, form="grouped").float()
    assert torch.allclose(a, b, atol=3e-2, rtol=2e-2)
    assert (a - b).abs().mean() < 2e-3
    c = seq_ops.moe_experts(h, idx.cuda(), wts.cuda(), w_gu, w_down, 1.2, shared=shared, form="tiles128").float()
    assert torch.equal(b, c)          # a row's sums do not depend on the tile it sits in: both grouped forms agree exactly


def test_oracle_absorbed_form_is_the_explicit_one():
    """The oracle's two statements of the attention agree: explicit keys / values, and queries that carry W_uk."""
    g = gen(11)
    T, Wd, H, D, V, R = 9, 20, 3, 4, 6, 10
    m = dict(heads=H, dim=D, vdim=V, kv_rank=R, scale=0.4)
    Wt = {"q": rnd(g, H * D, Wd), "dkv": rnd(g, R, Wd), "dkv.norm": 1 + rnd(g, R, s=0.1), "uk": rnd(g, H * D, R),
          "uv": rnd(g, H * V, R), "o": rnd(g, Wd, H * V)}
    h = rnd(g, T, Wd)
    c = O.rms_norm(h @ Wt["dkv"].T, Wt["dkv.norm"], 1e-5)
    qa = torch.einsum("thd,hdr->thr", (h @ Wt["q"].T).view(T, H, D), Wt["uk"].view(H, D, R))
    ol = O.absorbed_attention(qa, c, torch.arange(T), 0.4)
    y = torch.einsum("thr,hvr->thv", ol, Wt["uv"].view(H, V, R)).reshape(T, H * V) @ Wt["o"].T
    assert torch.allclose(y, O.latent_attention(h, Wt, "", m, 1e-5), atol=1e-4, rtol=1e-4)
