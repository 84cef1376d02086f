"""Every mechanism of nanovllm/hy_ops.py alone against the plain restatement in tests/oracle_lipelix.py: on the CPU the
engine's plumbing operators, on the GPU (marked gpu) the HIP kernels of libhymix in float32 and bfloat16.  Batches are
built by hand: several sequences, portions that start in the middle of a sequence, scattered cache blocks, state slots
that hold stale data."""
import math
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "nano-vllm-hw3_amd"))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import oracle_lipelix as O  # noqa: E402

from nanovllm import hy_ops  # noqa: E402
from nanovllm.seq_ops import StepContext  # noqa: E402

CASES = [("cpu", torch.float32), pytest.param("cuda", torch.float32, marks=pytest.mark.gpu),
         pytest.param("cuda", torch.bfloat16, marks=pytest.mark.gpu)]
F64 = torch.float64


def gen(seed):
    return torch.Generator().manual_seed(seed)


def rnd(g, *shape, s=1.0, dtype=torch.float32):
    """Values the storage type holds exactly, so that oracle and operator start from the same numbers."""
    return (torch.randn(*shape, generator=g) * s).to(dtype)


def tol(dtype, f32=2e-5, bf16=2e-2):
    return f32 if dtype == torch.float32 else bf16


def near(got, ref, dtype, f32=2e-5, bf16=2e-2):
    got, ref = got.detach().to("cpu", F64), ref.to(F64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert torch.isfinite(got).all()
    err = (got - ref).abs().max().item() / max(ref.abs().max().item(), 1e-9)
    assert err < tol(dtype, f32, bf16), f"relative error {err:.3g}"


def batch(portions, block_size=64, device="cpu", seed=0, slots=None):
    """portions = [(pos0, n)] per sequence -> StepContext with shuffled cache blocks and the given (or shuffled) slots."""
    g = gen(seed)
    B = len(portions)
    need = [(p + n + block_size - 1) // block_size for p, n in portions]
    perm = torch.randperm(sum(need) + 3, generator=g).tolist()
    mb = max(need)
    tables = torch.zeros(B, mb, dtype=torch.int32)
    tok_seq, tok_pos, slot_map, qstart = [], [], [], [0]
    for b, (p, n) in enumerate(portions):
        blocks = [perm.pop() for _ in range(need[b])]
        tables[b, :need[b]] = torch.tensor(blocks, dtype=torch.int32)
        for pos in range(p, p + n):
            tok_seq.append(b)
            tok_pos.append(pos)
            slot_map.append(blocks[pos // block_size] * block_size + pos % block_size)
        qstart.append(qstart[-1] + n)
    if slots is None:
        slots = torch.randperm(B + 2, generator=g)[:B].tolist()
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)  # noqa: E731
    return StepContext(tok_seq=i32(tok_seq), tok_pos=i32(tok_pos), qstart=i32(qstart), seq_pos0=i32([p for p, _ in portions]),
                       ctx_lens=i32([p + n for p, n in portions]), seq_slot=i32(slots), slot_mapping=i32(slot_map),
                       block_tables=tables.to(device), num_seqs=B, num_tokens=len(tok_seq), max_q=max(n for _, n in portions),
                       block_size=block_size, qstart_host=qstart), sum(need) + 3


# ------------------------------------------------------------------------------------------ residual side
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("W", [40, 7, 264])
def test_embed_close_and_carry(device, dtype, W):
    g = gen(W)
    T, eps, mult = 11, 1e-4, 0.4
    ctx, _ = batch([(0, 4), (5, 1), (2, 6)], device=device)
    embed = rnd(g, 19, W, dtype=dtype)
    ids = torch.randint(0, 19, (T,), generator=g)
    x = hy_ops.embed_scaled(ids.to(device), embed.to(device), 3.5)
    ref_x = embed[ids].to(F64) * 3.5
    near(x, ref_x, torch.float32)
    y, gate_wide, bias = rnd(g, T, W, dtype=dtype), rnd(g, T, W + 9, dtype=dtype), rnd(g, W, dtype=dtype)
    post_w, next_w, src = 1 + rnd(g, W, s=0.2, dtype=dtype), 1 + rnd(g, W, s=0.2, dtype=dtype), rnd(g, T, W, dtype=dtype)
    state = rnd(g, 6, 3, W, dtype=dtype).to(device)
    before = state.clone()
    gate = gate_wide.to(device)[:, 5:5 + W]                     # a column slice of a wider product
    h = hy_ops.sublayer_close(x, y.to(device), gate, bias.to(device), post_w.to(device), mult, next_w.to(device), eps, dtype,
                              carry=(src.to(device), state, 1, ctx))
    z = y.to(F64) * torch.sigmoid(gate_wide[:, 5:5 + W].to(F64) + bias.to(F64))
    ref_x = ref_x + mult * O.rms(z, eps) * post_w.to(F64)
    near(x, ref_x, torch.float32, f32=3e-6 if dtype == torch.float32 else 1e-2)
    near(h, O.rms(ref_x, eps) * next_w.to(F64), dtype)
    # the carried rows: the last token of every portion, at the sequence's slot and this layer; nothing else moves
    want = before.clone()
    for b, last in enumerate([3, 4, 10]):
        want[int(ctx.seq_slot[b]), 1] = src[last].to(device)
    assert torch.equal(state, want)
    # norm only (no sublayer result), and write only (no next norm)
    x0 = x.clone()
    near(hy_ops.sublayer_close(x, None, None, None, None, mult, next_w.to(device), eps, dtype), O.rms(ref_x, eps) * next_w.to(F64), dtype)
    assert torch.equal(x, x0)
    assert hy_ops.sublayer_close(x, y.to(device), gate, bias.to(device), post_w.to(device), mult, None, eps, dtype) is None
    near(x, ref_x + mult * O.rms(z, eps) * post_w.to(F64), torch.float32, f32=3e-6 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("device,dtype", CASES)
def test_token_shift_portions_and_stale_slots(device, dtype):
    """A sequence cut into portions of 1-5 tokens through its slot equals the whole sequence shifted at once; a sequence
    that starts in a slot full of another's data reads zero before its first token."""
    g = gen(3)
    W, L = 24, 3
    mu = torch.rand(W, generator=g).to(dtype)
    hs = {k: rnd(g, n, W, dtype=dtype) for k, n in (("a", 13), ("b", 6))}
    ref = {k: O.token_shift(v.to(F64), mu.to(F64)) for k, v in hs.items()}
    state = rnd(g, 4, L, W, s=50.0, dtype=dtype).to(device)     # stale: large values that would show
    plan = [[("a", 0, 5), ("b", 0, 1)], [("a", 5, 6), ("b", 1, 3)], [("b", 3, 6), ("a", 6, 8)], [("a", 8, 13)]]
    slot = {"a": 2, "b": 0}
    for step in plan:
        ctx, _ = batch([(a, b - a) for _, a, b in step], device=device, slots=[slot[k] for k, _, _ in step])
        h = torch.cat([hs[k][a:b] for k, a, b in step]).to(device)
        out = hy_ops.token_shift(h, mu.to(device), state, 1, ctx)
        near(out, torch.cat([ref[k][a:b] for k, a, b in step]), dtype, bf16=1e-2)
        # what the closing launch of the sublayer does: the portion's last input is carried
        x = torch.zeros(h.shape[0], W, device=device)
        hy_ops.sublayer_close(x, None, None, None, None, 1.0, None, 1e-5, dtype, carry=(h, state, 1, ctx))


@pytest.mark.parametrize("device,dtype", CASES)
def test_relu_squared(device, dtype):
    g = gen(4)
    z = rnd(g, 9, 50, dtype=dtype)
    near(hy_ops.relu_squared(z.to(device)[:, 7:44]), torch.relu(z[:, 7:44].to(F64)) ** 2, dtype)


# ------------------------------------------------------------------------------------------ attention
def step_context(tables, parts, block_size, device):
    """The step of parts [(sequence, first position, end position)] over fixed per-sequence block tables."""
    tok_seq, tok_pos, slot_map, qstart = [], [], [], [0]
    mb = max(len(t) for t in tables)
    bt = torch.zeros(len(parts), mb, dtype=torch.int32)
    for i, (b, a, e) in enumerate(parts):
        bt[i, :len(tables[b])] = torch.tensor(tables[b], dtype=torch.int32)
        for pos in range(a, e):
            tok_seq.append(i)
            tok_pos.append(pos)
            slot_map.append(tables[b][pos // block_size] * block_size + pos % block_size)
        qstart.append(qstart[-1] + e - a)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)  # noqa: E731
    return StepContext(tok_seq=i32(tok_seq), tok_pos=i32(tok_pos), qstart=i32(qstart), seq_pos0=i32([a for _, a, _ in parts]),
                       ctx_lens=i32([e for _, _, e in parts]), seq_slot=i32(list(range(len(parts)))), slot_mapping=i32(slot_map),
                       block_tables=bt.to(device), num_seqs=len(parts), num_tokens=len(tok_seq),
                       max_q=max(e - a for _, a, e in parts), block_size=block_size, qstart_host=qstart)


def attention_case(device, dtype, H, G, D, V, rot, lens, steps, window=0, keep_first=0, sink=None, proj_norm=False,
                   unit_norm=False, vmix=None, block_size=64, seed=0, plant=None, scale=None, base=50.0):
    """Whole sequences of the given lengths through the oracle's pieces; the same tokens through qkv_prepare +
    paged_attention in ``steps`` = [[(sequence, first position, end position)]], over scattered cache blocks."""
    g = gen(seed)
    eps = 1e-5
    scale = scale if scale is not None else D ** -0.5
    qkv = [rnd(g, n, (H + G) * D + G * V, dtype=dtype) for n in lens]
    if plant:                                    # plant(b, qkv_b): make chosen scores stand out
        for b in range(len(lens)):
            plant(b, qkv[b])
    vf = [rnd(g, n, G * V, dtype=dtype) for n in lens] if vmix is not None else None
    qw, kw = (1 + rnd(g, H * D, s=0.3, dtype=dtype), 1 + rnd(g, G * D, s=0.3, dtype=dtype)) if proj_norm else (None, None)
    sink_t = rnd(g, H, s=2.0) if sink == "learned" else (torch.zeros(H) if sink == "zero" else None)
    inv_freq = hy_ops.rotary_inv_freq(rot, base, device)
    ref = []
    for b, n in enumerate(lens):
        q, k, v = qkv[b].to(F64).split([H * D, G * D, G * V], -1)
        if proj_norm:
            q, k = O.rms(q, eps) * qw.to(F64), O.rms(k, eps) * kw.to(F64)
        q, k, v = q.reshape(n, H, D), k.reshape(n, G, D), v.reshape(n, G, V)
        pos = torch.arange(n)
        q, k = O.rotate(q, pos, rot, base), O.rotate(k, pos, rot, base)
        if unit_norm:
            q, k = O.rms(q, eps), O.rms(k, eps)
        if vmix is not None:
            v = (1 - vmix) * v + vmix * vf[b].to(F64).view(n, G, V)
        if dtype == torch.bfloat16:              # what the operator hands on and the cache holds
            q, k, v = (t.to(dtype).to(F64) for t in (q, k, v))
        s = torch.einsum("ihd,jhd->hij", q, k.repeat_interleave(H // G, 1)) * scale
        ok = O.visible(n, window if window else None, keep_first)
        p = O.softmax_with_sink(s, ok, sink_t.to(F64) if sink_t is not None else torch.full((H,), -math.inf, dtype=F64))
        ref.append(torch.einsum("hij,jhv->ihv", p, v.repeat_interleave(H // G, 1)).reshape(n, H * V))
    need = [(n + block_size - 1) // block_size for n in lens]
    perm = torch.randperm(sum(need) + 2, generator=g).tolist()
    tables = [[perm.pop() for _ in range(k)] for k in need]
    kc = torch.randn(sum(need) + 2, block_size, G, D).to(dtype).to(device) * 40     # stale rows that would show
    vc = torch.randn(sum(need) + 2, block_size, G, V).to(dtype).to(device) * 40
    lam = torch.tensor([vmix if vmix is not None else 0.0], dtype=torch.float32, device=device)
    dev = lambda t: None if t is None else t.to(device)  # noqa: E731
    for parts in steps:
        ctx = step_context(tables, parts, block_size, device)
        x = torch.cat([qkv[b][a:e] for b, a, e in parts]).to(device)
        f = torch.cat([vf[b][a:e] for b, a, e in parts]).to(device) if vmix is not None else None
        q = hy_ops.qkv_prepare(x, H, G, D, V, dev(qw), dev(kw), eps, inv_freq, unit_norm, ctx, kc, vc, f, lam)
        o = hy_ops.paged_attention(q, kc, vc, ctx, scale, dev(sink_t), window, keep_first)
        near(o, torch.cat([ref[b][a:e] for b, a, e in parts]), dtype, f32=3e-5, bf16=3e-2)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,G,D,V,rot", [(4, 2, 16, 8, 8), (3, 3, 24, 40, 24), (6, 1, 8, 72, 4), (2, 2, 80, 16, 80)])
def test_attention_full_causal_with_learned_sink(device, dtype, H, G, D, V, rot):
    """Whole-projection norms, partial rotation, a learned sink; a whole prompt, a portion behind a context that ends in the
    middle of a block, and single tokens, in one batch."""
    steps = [[(0, 0, 70), (1, 0, 3), (2, 0, 1)], [(1, 3, 4), (0, 70, 75), (2, 1, 2)], [(0, 75, 150), (1, 4, 5)]]
    attention_case(device, dtype, H, G, D, V, rot, [150, 5, 2], steps, sink="learned", proj_norm=True, seed=1)
    attention_case(device, dtype, H, G, D, V, rot, [150, 5, 2], steps, sink="learned", proj_norm=True, vmix=0.35, seed=2)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("window,keep", [(9, 3), (64, 5), (70, 0), (5, 7), (1, 1), (300, 2)])
def test_attention_window_edges_stand_out(device, dtype, window, keep):
    """Unit-norm heads, zero sink, window with kept first tokens.  For every query the keys just inside and just outside
    the window and the last kept / first dropped token are made to score far above the rest in turn, each with a value of
    its own, so that a window one token off, or a dropped first token, changes the result by much."""
    H, G, D, V, rot = 2, 1, 16, 8, 8
    n = 200

    def plant(b, x):
        # keys at chosen distances behind some queries point along that query
        q = x[:, :H * D].view(-1, H, D)
        k = x[:, H * D:(H + G) * D].view(-1, G, D)
        for i in range(20, n, 7):
            for j in (i - window + 1, i - window, keep - 1, keep):
                if 0 <= j < i:
                    k[j, 0] = (q[i, b % H].float() * 3).to(x.dtype)
    # sequence 0 as a whole prompt; sequence 1 as a prompt of 100 and then token by token
    steps = [[(0, 0, n), (1, 0, 100)]] + [[(1, t, t + 1)] for t in range(100, n)]
    attention_case(device, dtype, H, G, D, V, rot, [n, n], steps, window=window, keep_first=keep, sink="zero", unit_norm=True,
                   seed=window, plant=plant, scale=1.0, base=1e6)


@pytest.mark.parametrize("device,dtype", CASES)
def test_attention_portions_and_decoding_through_the_cache(device, dtype):
    """The same sequences computed as whole prompts, as portions behind a cached context that ends inside a block, and
    token by token, give the same rows (the cache and the positions are all that links the steps); keys far back stand
    out for the last queries."""
    H, G, D, V, rot, n = 4, 2, 16, 24, 16, 330

    def plant(b, x):
        q = x[:, :H * D].view(-1, H, D)
        k = x[:, H * D:(H + G) * D].view(-1, G, D)
        k[3 + b, 0] = (q[n - 1, 0].float() * 2).to(x.dtype)       # a far key for the last query
        k[64, 1] = (q[n - 2, 3].float() * 2).to(x.dtype)          # the first row of the second block
    steps = [[(0, 0, n), (1, 0, 37)], [(1, 37, 39)], [(1, 39, 200)], [(1, 200, 320)]] + [[(1, t, t + 1)] for t in range(320, n)]
    for window, keep, sink in ((0, 0, "learned"), (75, 6, "zero")):
        attention_case(device, dtype, H, G, D, V, rot, [n, n], steps, window=window, keep_first=keep, sink=sink,
                       unit_norm=window > 0, proj_norm=window == 0, seed=5, plant=plant, base=1e4)


# ------------------------------------------------------------------------------------------ delta rule
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,D,rank", [(3, 8, 5), (1, 40, 16), (2, 64, 3), (2, 72, 8)])
def test_delta_rule_pieces_and_portions(device, dtype, H, D, rank):
    """prepare + recurrence + gate/norm against the oracle's mixer without its output product; then the same sequences
    cut into portions (single tokens included) through state slots that held another sequence's state."""
    g = gen(D)
    W, eps = 32, 1e-5
    hd = H * D
    names = ["r", "k", "v", "g", "a", "w1"]
    w = {"m." + n: rnd(g, hd if n != "w1" else rank, W, s=W ** -0.5) for n in names}
    w.update({"m.w2": rnd(g, hd, rank, s=1.0, dtype=dtype), "m.w0": rnd(g, hd, dtype=dtype), "m.a.b": rnd(g, hd, dtype=dtype),
              "m.norm": 1 + rnd(g, hd, s=0.3, dtype=dtype), "m.o": torch.eye(hd)})
    lens = {"a": 37, "b": 9}
    hs = {k: rnd(g, n, W) for k, n in lens.items()}
    proj = {k: (h @ torch.cat([w["m." + n] for n in names]).T).to(dtype) for k, h in hs.items()}

    def oracle(p):
        """The oracle's mixer fed with the rounded products: identity 'projections' of the product's columns."""
        cols, off = {}, 0
        for n in names:
            size = hd if n != "w1" else rank
            cols[n] = (off, size)
            off += size
        ww = {"m." + n: torch.eye(off, dtype=F64)[a:a + s] for n, (a, s) in cols.items()}
        ww.update({k: v.to(F64) for k, v in w.items() if k[2:] in ("w2", "w0", "a.b", "norm", "o")})
        return O.general_delta(p.to(F64), ww, "m.", dict(heads=H, dim=D), eps)
    ref = {k: oracle(p) for k, p in proj.items()}
    cols = ((0, hd), (hd, hd), (4 * hd, hd), (5 * hd, rank))
    state = rnd(g, 4, H, D, D, s=30.0).to(device)               # stale
    slot = {"a": 1, "b": 3}

    def step(parts):
        ctx, _ = batch([(a, e - a) for _, a, e in parts], device=device, slots=[slot[k] for k, _, _ in parts])
        p = torch.cat([proj[k][a:e] for k, a, e in parts]).to(device)
        prep = hy_ops.delta_prepare(p, cols, w["m.w2"].to(device), w["m.w0"].to(device), w["m.a.b"].to(device), H, D, math.exp(-0.5))
        o = hy_ops.delta_recurrence(prep, p[:, 2 * hd:3 * hd], state, ctx)
        return hy_ops.delta_gate_norm(o, p[:, 3 * hd:4 * hd], w["m.norm"].to(device), eps, dtype)
    near(step([("a", 0, 37), ("b", 0, 9)]), torch.cat([ref["a"], ref["b"]]), dtype, f32=5e-5)
    state.normal_(0, 30.0)
    plan = [[("a", 0, 2), ("b", 0, 1)], [("b", 1, 2), ("a", 2, 19)], [("a", 19, 20)], [("a", 20, 21), ("b", 2, 9)], [("a", 21, 37)]]
    for parts in plan:
        near(step(parts), torch.cat([ref[k][a:e] for k, a, e in parts]), dtype, f32=5e-5)


@pytest.mark.parametrize("device,dtype", CASES)
def test_delta_state_is_float32_over_long_runs(device, dtype):
    """600 tokens in portions of 1 and 7: the state that travels through the slot keeps the whole sequence's result."""
    g = gen(11)
    H, D, n = 2, 16, 600
    prep_in = torch.rand(n, H, 5, D, generator=g)
    prep_in[:, :, 0] = 0.9 + 0.1 * prep_in[:, :, 0]                  # decays close to one: a long memory
    u = torch.nn.functional.normalize(rnd(g, n, H, D), dim=-1)
    prep_in[:, :, 2], prep_in[:, :, 1] = u, u * prep_in[:, :, 1]
    v = rnd(g, n, H * D, dtype=dtype)
    S = torch.zeros(H, D, D, dtype=F64)
    ref = []
    for t in range(n):
        decay, au, uu, k, r = prep_in[t].to(F64).unbind(1)
        uS = torch.einsum("hi,hij->hj", uu, S)
        S = decay[:, :, None] * S - au[:, :, None] * uS[:, None, :] + k[:, :, None] * v[t].to(F64).view(H, D)[:, None, :]
        ref.append(torch.einsum("hij,hi->hj", S, r))
    ref = torch.stack(ref)
    state = rnd(g, 2, H, D, D, s=9.0).to(device)
    a, out, i = 0, [], 0
    while a < n:
        e = min(n, a + (1, 7)[i % 2])
        ctx, _ = batch([(a, e - a)], device=device, slots=[1])
        out.append(hy_ops.delta_recurrence(prep_in[a:e].contiguous().to(device), v[a:e].to(device), state, ctx))
        a, i = e, i + 1
    near(torch.cat(out), ref, torch.float32, f32=2e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,V", [(4, 4, 40, 56), (8, 2, 64, 128), (6, 1, 128, 8), (3, 3, 8, 40), (64, 2, 16, 16)])
@pytest.mark.parametrize("window,keep", [(0, 0), (88, 12), (130, 0), (5, 200)])
def test_matrix_core_attention_equals_portable_form(H, G, D, V, window, keep):
    """bf16: the tile kernel (portions) and the split-key kernel (single tokens) against the portable kernel on the same
    cache, for head sizes on and off the padded tile sizes, grouped heads, windows around tile borders; sequences whose
    portions start inside a block, a batch of single tokens at unequal lengths."""
    g = gen(H * D + window)
    dev, bf, bs = "cuda", torch.bfloat16, 64
    lens = [333, 64, 1, 129, 700]
    need = [(n + bs - 1) // bs for n in lens]
    perm = torch.randperm(sum(need) + 1, generator=g).tolist()
    tables = [[perm.pop() for _ in range(k)] for k in need]
    kc = rnd(g, sum(need) + 1, bs, G, D, dtype=bf).to(dev)
    vc = rnd(g, sum(need) + 1, bs, G, V, dtype=bf).to(dev)
    sink = rnd(g, H, s=2.0).to(dev)
    for parts in ([(b, 0, n) for b, n in enumerate(lens)], [(0, 300, 333), (3, 127, 129), (4, 1, 700)],
                  [(b, n - 1, n) for b, n in enumerate(lens)], [(4, 699, 700)]):
        ctx = step_context(tables, parts, bs, dev)
        q = rnd(g, ctx.num_tokens, H, D, dtype=bf).to(dev)
        for sk in (sink, None):
            ref = hy_ops.paged_attention(q, kc, vc, ctx, 0.3, sk, window, keep, force_rows=True)
            got = hy_ops.paged_attention(q, kc, vc, ctx, 0.3, sk, window, keep)
            near(got, ref.double().cpu(), bf, bf16=1.5e-2)
