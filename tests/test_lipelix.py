"""The Lipelix model family in the engine against the plain restatement in tests/oracle_lipelix.py.

Every test makes its own small configuration and random checkpoint.  ``device`` = "cpu" drives the engine's plumbing
operators (scheduler, block and slot pools, portion batching are the same code as on the GPU); "cuda" (marked gpu) drives
the HIP kernels of libhymix, in float32 against tight bounds and in bfloat16 against the rounding of that format."""
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "nano-vllm-hw3_amd"))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import oracle_lipelix as O  # noqa: E402
from test_pasizen import DEVICES, cut, dtypes_for, replay, tokens, write_model  # noqa: E402  (engine test helpers)


def attn(kind="attention", heads=4, kv_heads=2, dim=16, vdim=8, rot=8, base=100.0, scale=0.4, v_mix=True, window=9, keep=3):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, rot=dict(dims=rot, base=base), scale=scale, v_mix=v_mix)
    if kind == "attention_2":
        m["mask"] = dict(size=window, keep_first=keep)
    return kind, m


def delta(heads=3, dim=8, rank=5):
    return "general_delta", dict(heads=heads, dim=dim, decay_rank=rank)


def config(layers, width=40, vocab=53, eps=1e-5, mult=0.45, emb=5.0):
    return dict(architecture="Lipelix", vocab=vocab, width=width, norm=dict(eps=eps), residual_mult=mult,
                embedding=dict(scale=emb),
                layers=[dict(type=kind, mixer={k: v for k, v in m.items() if k != "decay_rank"}, mlp=dict(kind="dense", ff=ff) if ff else None)
                        for (kind, m), ff in layers]), [m.get("decay_rank") for (kind, m), ff in layers]


DEFAULT = [(attn("attention_2", window=9, keep=3), 24), (delta(), None), (attn("attention", heads=2, kv_heads=2, dim=24, vdim=8, rot=24), 56),
           (attn("attention_2", heads=4, kv_heads=1, dim=8, vdim=16, rot=4, window=70, keep=0, v_mix=False), None), (delta(heads=1, dim=24, rank=2), 16)]


def weights(cfg_ranks, seed=0, sink=1.0):
    """A random checkpoint under the design's tensor names, bf16-representable values."""
    cfg, ranks = cfg_ranks
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def rnd(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16)
    t = {"embed": rnd(cfg["vocab"], W, s=0.3), "final.norm": 1 + rnd(W, s=0.1), "head": rnd(cfg["vocab"], W, s=W ** -0.5)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        t.update({p + "norm1": 1 + rnd(W, s=0.1), p + "norm1b": 1 + rnd(W, s=0.1), p + "shift": torch.rand(W, generator=g).to(torch.bfloat16),
                  p + "rg1": rnd(W, W, s=W ** -0.5), p + "rg1.b": rnd(W, s=0.5)})
        if L["type"] == "general_delta":
            hd, R = m["heads"] * m["dim"], ranks[i]
            for n in ("r", "k", "v", "g", "a"):
                t[p + "mix." + n] = rnd(hd, W, s=2 * W ** -0.5)
            t.update({p + "mix.w1": rnd(R, W, s=W ** -0.5), p + "mix.w2": rnd(hd, R, s=2.0), p + "mix.w0": rnd(hd), p + "mix.a.b": rnd(hd),
                      p + "mix.norm": 1 + rnd(hd, s=0.2), p + "mix.o": rnd(W, hd, s=hd ** -0.5)})
        else:
            H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            t.update({p + "mix.q": rnd(H * D, W, s=2 * W ** -0.5), p + "mix.k": rnd(G * D, W, s=2 * W ** -0.5),
                      p + "mix.v": rnd(G * V, W, s=W ** -0.5), p + "mix.o": rnd(W, H * V, s=(H * V) ** -0.5)})
            if L["type"] == "attention":
                t.update({p + "mix.q.norm": 1 + rnd(H * D, s=0.3), p + "mix.k.norm": 1 + rnd(G * D, s=0.3), p + "mix.sink": rnd(H, s=sink)})
            if m.get("v_mix"):
                t[p + "mix.vmix"] = (torch.rand((), generator=g) * 0.6 + 0.2).to(torch.bfloat16)
        if L["mlp"] is not None:
            ff = L["mlp"]["ff"]
            t.update({p + "norm2": 1 + rnd(W, s=0.1), p + "norm2b": 1 + rnd(W, s=0.1), p + "rg2": rnd(W, W, s=W ** -0.5),
                      p + "rg2.b": rnd(W, s=0.5), p + "mlp.up": rnd(ff, W, s=W ** -0.5), p + "mlp.down": rnd(W, ff, s=ff ** -0.5)})
    return {k: v.to(torch.bfloat16).contiguous() for k, v in t.items()}


def close(got, ref, dtype):
    """Logit rows against the oracle's (difference with its mean removed, relative to the spread of the logits): float32
    to accumulation order, bfloat16 to that format's rounding through the layers."""
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape and np.isfinite(got).all()
    d = got - ref
    d = d - d.mean(-1, keepdims=True)
    err = np.sqrt((d ** 2).mean(-1)) / ref.std()
    bound = 1e-4 if dtype == torch.float32 else 4e-2
    assert err.max() < bound, f"relative error {err.max():.3g} at row {int(err.argmax())}"


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cr = config(DEFAULT)
    w = weights(cr, seed=1)
    return write_model(tmp_path_factory.mktemp("lipelix_default"), cr[0], w), cr[0], w


def forward(cfg, w, toks, **kw):
    return O.forward(cfg, w, toks, **kw).numpy()


# ------------------------------------------------------------------------------------------ whole model, schedules
@pytest.mark.parametrize("device", DEVICES)
def test_whole_prompt_and_layer_trace(model, tmp_path, device):
    """One step per prompt: every position's logits; and the residual after every layer, through the runner itself."""
    path, cfg, w = model
    toks = tokens(90, cfg["vocab"], 3)
    layers = []
    ref = forward(cfg, w, toks, layers_out=layers)
    for dtype in dtypes_for(device):
        got = replay(path, [([("a", toks, list(range(90)))], ["a"])], tmp_path, device, dtype)
        close(got[0], ref, dtype)
    from nanovllm.engine.llm_engine import LLMEngine
    from nanovllm.engine.sequence import ACTIVE, Sequence
    eng = LLMEngine(path, device=device, dtype=torch.float32, max_num_seqs=2, num_kvcache_blocks=4, max_num_batched_tokens=4096)
    seq = Sequence(toks)
    seq.state = ACTIVE
    assert eng.scheduler.reserve_portion(seq, 90)
    trace = []
    eng.model_runner.run_portions([(seq, 90)], trace=trace)
    assert len(trace) == len(layers) == 5
    for got_l, ref_l in zip(trace, layers):
        assert torch.allclose(got_l.cpu().double(), ref_l, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_prefill_equals_token_by_token(model, tmp_path, device):
    """A prompt fed one token per step (cache, shift rows and recurrent state from the very first token) gives the logits
    of the whole prompt in one step; 140 tokens cross two cache-block borders and both windows."""
    path, cfg, w = model
    toks = tokens(140, cfg["vocab"], 4)
    ref = forward(cfg, w, toks)
    steps = [([("a", [t], [0])], ["a"] if i == 139 else []) for i, t in enumerate(toks)]
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=192)
        close(np.concatenate([got[i] for i in range(140)]), ref, dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2], [3, 2, 7, 2, 64, 1, 5], [63, 2, 1, 64], [65, 1, 1, 1, 2], [9, 1, 8, 10]])
def test_portions(model, tmp_path, device, sizes):
    """Prompts cut into portions of several sizes (down to two tokens, across block borders and window edges, single
    tokens between)."""
    path, cfg, w = model
    toks = tokens(133, cfg["vocab"], 5)
    ref = forward(cfg, w, toks)
    parts = cut(133, sizes)
    steps = [([("r", toks[a:b], list(range(b - a)))], ["r"] if b == 133 else []) for a, b in parts]
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=192)
        close(np.concatenate([got[i] for i in range(len(parts))]), ref, dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_and_reused_pages_and_slots(model, tmp_path, device):
    """Unequal requests share steps (prompt portions beside single tokens), more requests than state slots and more
    tokens than cache blocks over the run: blocks and slots are freed and taken again, also by a request whose first
    tokens land in a slot that still holds another request's shift rows and recurrent state.  Each equals itself alone."""
    path, cfg, w = model
    V = cfg["vocab"]
    reqs = {f"q{i}": tokens(n, V, 10 + i) for i, n in enumerate([97, 5, 130, 66, 1, 71, 64])}
    ref = {k: forward(cfg, w, v) for k, v in reqs.items()}
    plan = {"q0": cut(97, [40, 1, 1, 30, 1]), "q1": cut(5, [2, 1]), "q2": cut(130, [64, 3, 1]), "q3": cut(66, [66]),
            "q4": cut(1, [1]), "q5": cut(71, [7, 1]), "q6": cut(64, [62, 2])}
    live, waiting, steps, rows = [], list(reqs), [], []
    cursor = {k: 0 for k in reqs}
    while live or waiting:
        while waiting and len(live) < 3:
            live.append(waiting.pop(0))
        entries, end = [], []
        for k in list(live):
            a, b = plan[k][cursor[k]]
            cursor[k] += 1
            entries.append((k, reqs[k][a:b], list(range(b - a))))
            rows.append((len(steps), k, a, b))
            if b == len(reqs[k]):
                end.append(k)
                live.remove(k)
        steps.append((entries, end))
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=7 * 64, max_live=3)
        at = {}
        for s, k, a, b in rows:
            o = at.get(s, 0)
            close(got[s][o:o + b - a], ref[k][a:b], dtype)
            at[s] = o + b - a


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding(model, tmp_path, device):
    """A short prompt and 200 single-token steps: three block borders and the 70-token window pass over decoded tokens."""
    path, cfg, w = model
    toks = tokens(215, cfg["vocab"], 6)
    ref = forward(cfg, w, toks)
    steps = [([("a", toks[:15], [14])], [])] + [([("a", [t], [0])], []) for t in toks[15:]]
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=256)
        close(np.concatenate([got[i] for i in range(len(steps))]), ref[14:], dtype)


VARIANTS = {
    # one layer of each kind alone; sizes that the default makes equal are unequal here and the other way round
    "delta_only": config([(delta(heads=2, dim=40, rank=1), 8)], width=24, mult=1.0, emb=1.0),
    "window_only_one_head": config([(attn("attention_2", heads=1, kv_heads=1, dim=8, vdim=8, rot=8, window=1, keep=1, v_mix=False), None)]),
    "full_only_no_mix": config([(attn("attention", heads=6, kv_heads=3, dim=4, vdim=20, rot=2, v_mix=False), 12)], width=16),
    "mix_source_is_a_window_layer": config([(delta(), 8), (attn("attention_2", window=64, keep=64), None), (attn("attention"), 8),
                                            (attn("attention_2", window=65, keep=1), 8)], mult=0.1),
    "single_mixing_layer": config([(attn("attention", dim=72, rot=36, heads=2, kv_heads=1, vdim=72), 8), (delta(heads=1, dim=72, rank=9), None)]),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(VARIANTS))
def test_other_shapes(tmp_path, device, name):
    """Other sizes, orders and constants: every mixer alone, one head, a window of one token, windows equal to and one more
    than a cache block, all first tokens kept, no value mixing / one mixing layer / a window layer as the source of the
    mixed values, multiplier and embedding scale of 1, head sizes beyond one wave.  Portions and a batch."""
    cr = VARIANTS[name]
    cfg = cr[0]
    w = weights(cr, seed=7, sink=3.0)
    path = write_model(tmp_path / "m", cfg, w)
    a, b = tokens(150, cfg["vocab"], 8), tokens(9, cfg["vocab"], 9)
    ra, rb = forward(cfg, w, a), forward(cfg, w, b)
    steps = [([("a", a[:31], list(range(31)))], []),
             ([("a", a[31:131], list(range(100))), ("b", b[:2], [0, 1])], []),
             ([("b", b[2:], list(range(7))), ("a", a[131:132], [0])], ["b"])] + \
            [([("a", [t], [0])], []) for t in a[132:]]
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=256)
        close(got[0], ra[:31], dtype)
        close(got[1], np.concatenate([ra[31:131], rb[:2]]), dtype)
        close(got[2], np.concatenate([rb[2:], ra[131:132]]), dtype)
        close(np.concatenate([got[i] for i in range(3, len(steps))]), ra[132:], dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_a_sink_and_a_far_key_show(tmp_path, device):
    """Weights made so that faults show: large sinks (leaving one out moves every row) and keys that point along later
    queries far back (embedding rows repeated at chosen places make a far token's key match the query)."""
    cr = config([(attn("attention", heads=2, kv_heads=1, dim=16, vdim=16, rot=4, scale=1.5, v_mix=False), None)], width=32, mult=1.0)
    cfg = cr[0]
    w = weights(cr, seed=3, sink=4.0)
    w["l0.mix.k"] = w["l0.mix.q"][:16].clone()                 # a token's key is its first head's query: equal tokens attract
    path = write_model(tmp_path / "m", cfg, w)
    toks = tokens(300, cfg["vocab"], 12)
    for far, at in ((2, 290), (63, 291), (64, 292), (129, 299)):
        toks[at] = toks[far]
    ref = forward(cfg, w, toks)
    no_sink = forward(cfg, {**w, "l0.mix.sink": torch.full((2,), -60.0)}, toks)
    assert np.abs(ref - no_sink).max() > 0.05 * ref.std()      # the sink matters in this model
    steps = [([("a", toks[:280], [279])], [])] + [([("a", [t], [0])], []) for t in toks[280:]]
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=320)
        close(np.concatenate([got[i] for i in range(len(steps))]), ref[279:], dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(model, device):
    """LLM.generate (the scheduler's own portions: a 16-token step budget cuts prompts, decoded tokens share steps with
    prompt pieces, five requests over three slots) continues every prompt as the oracle's greedy loop does."""
    from nanovllm import LLM, SamplingParams
    path, cfg, w = model
    prompts = [tokens(n, cfg["vocab"], 20 + n) for n in (37, 3, 18, 1, 70)]

    def greedy(p, n):
        p = list(p)
        for _ in range(n):
            p.append(int(forward(cfg, w, p)[-1].argmax()))
        return p[-n:]
    llm = LLM(path, device=device, dtype=torch.float32, max_num_seqs=3, max_num_batched_tokens=16, num_kvcache_blocks=5)
    out = llm.generate(prompts, SamplingParams(max_tokens=6, ignore_eos=True))
    assert [o["token_ids"] for o in out] == [greedy(p, 6) for p in prompts]
    assert len(llm.scheduler.block_manager.free) == 5 and len(llm.scheduler.slots.free) == 3


def test_scheduler_preempts_when_blocks_run_out(model):
    """Two requests that cannot both grow in a three-block pool: the later one is put back, runs again afterwards from
    its first token (its slot's state is stale by then), and both produce what they produce alone."""
    from nanovllm import LLM, SamplingParams
    path, cfg, w = model
    prompts = [tokens(60, cfg["vocab"], 31), tokens(62, cfg["vocab"], 32)]
    sp = SamplingParams(max_tokens=10, ignore_eos=True)
    alone = [LLM(path, device="cpu", dtype=torch.float32, max_num_seqs=2, num_kvcache_blocks=4).generate([p], sp)[0]["token_ids"]
             for p in prompts]
    llm = LLM(path, device="cpu", dtype=torch.float32, max_num_seqs=2, num_kvcache_blocks=3)
    out = llm.generate(prompts, sp)
    assert [o["token_ids"] for o in out] == alone


def test_registry_config_and_dummy_weights(tmp_path):
    from nanovllm.config import Config
    from nanovllm.models import registry
    assert registry.architecture_of({"architecture": "Lipelix"}) == "Lipelix"
    cfg = config([(attn("attention", kv_heads=2, vdim=8), 8), (attn("attention_2", kv_heads=1, vdim=8), 8)])[0]
    path = write_model(tmp_path / "bad", cfg, {})
    with pytest.raises(ValueError):                            # layers that mix values must agree on their value rows
        Config(path, device="cpu")
    # a model without a checkpoint: random tensors under the checkpoint's names go through the same placement
    from nanovllm import LLM, SamplingParams
    cr = config(DEFAULT)
    path = write_model(tmp_path / "dummy", cr[0], {})
    llm = LLM(path, device="cpu", dtype=torch.float32, load_format="dummy", max_num_seqs=2, num_kvcache_blocks=4)
    out = llm.generate([tokens(20, 53, 1)], SamplingParams(max_tokens=3, ignore_eos=True))
    assert len(out[0]["token_ids"]) == 3


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_captured_decode_steps_equal_eager_steps(model, dtype):
    """Decode-only steps replay a hipGraph per batch-size bucket.  Three requests decode for 70 steps (a block border is
    crossed, the batch shrinks from 3 to 2 to 1: three buckets, padding rows in the bucket of 4) with an eager prefill of
    a fourth request between replays; every step's logits equal those of an engine that runs everything eagerly."""
    from nanovllm.engine.llm_engine import LLMEngine
    from nanovllm.engine.sequence import ACTIVE, Sequence
    path, cfg, w = model
    engines = [LLMEngine(path, dtype=dtype, enforce_eager=eager, max_num_seqs=4, num_kvcache_blocks=12, max_model_len=256,
                         max_num_batched_tokens=4096) for eager in (True, False)]
    assert not engines[0].model_runner.portion_graphs and sorted(engines[1].model_runner.portion_graphs) == [1, 2, 4]
    prompts = [tokens(n, cfg["vocab"], 40 + n) for n in (50, 3, 61)]
    cont = [tokens(70, cfg["vocab"], 50 + i) for i in range(3)]
    outs = []
    for eng in engines:
        seqs, got = [], []
        for p in prompts:
            s = Sequence(p)
            s.state = ACTIVE
            assert eng.scheduler.reserve_portion(s, len(p))
            seqs.append(s)
        got.append(eng.forward_portions([(s, len(s)) for s in seqs]))
        for s in seqs:
            s.num_computed = s.num_tokens
        for step in range(70):
            live = [(i, s) for i, s in enumerate(seqs) if not (i == 1 and step >= 20) and not (i == 2 and step >= 45)]
            for i, s in live:
                s.extend([cont[i][step]])
                assert eng.scheduler.reserve_portion(s, 1)
            got.append(eng.forward_portions([(s, 1) for _, s in live]))
            for _, s in live:
                s.num_computed += 1
            if step == 30:                      # eager work between replays: another request's prompt
                extra = Sequence(tokens(40, cfg["vocab"], 99))
                extra.state = ACTIVE
                assert eng.scheduler.reserve_portion(extra, 40)
                got.append(eng.forward_portions([(extra, 40)]))
                eng.scheduler.release(extra)
        outs.append([g.float().cpu() for g in got])
    assert [a.shape for a in outs[0]] == [b.shape for b in outs[1]]
    close(torch.cat(outs[1]).numpy(), torch.cat(outs[0]).numpy(), dtype)
