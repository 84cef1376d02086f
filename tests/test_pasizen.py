"""The Pasizen model family in the engine against the plain restatement in tests/oracle_pasizen.py.

Every test makes its own small configuration and random checkpoint.  ``device`` = "cpu" drives the engine's plumbing
operators (scheduler, block and slot pools, portion batching are the same code as on the GPU); "cuda" (marked gpu)
drives the HIP kernels of libseqmix, in float32 against tight bounds and in bfloat16 against the rounding of that
format."""
import io
import json
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "nano-vllm-hw3_amd"))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import oracle_pasizen as O  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def mixer(heads=3, dim=8, vdim=16, kv_rank=24, scale=0.3):
    return dict(heads=heads, dim=dim, vdim=vdim, kv_rank=kv_rank, scale=scale)


def dense(ff=40):
    return dict(kind="dense", ff=ff)


def moe(experts=6, top=2, ff=24, limit=1.5, groups=(3, 2), shared=(16, 0.8)):
    r = dict(experts=experts, top=top)
    if groups:
        r["groups"] = dict(count=groups[0], keep=groups[1])
    m = dict(kind="moe", expert=dict(ff=ff, limit=limit), router=r)
    if shared:
        m["shared"] = dict(ff=shared[0], limit=shared[1])
    return m


def config(layers, width=48, vocab=61, streams=3, taps=3, loop=None, max_positions=512, eps=1e-5):
    c = dict(architecture="Pasizen", vocab=vocab, width=width, max_positions=max_positions, norm=dict(eps=eps),
             layers=[dict(type="latent_attention", mixer=m, mlp=f) for m, f in layers])
    if streams:
        c["streams"] = streams
    if taps:
        c["canon"] = dict(taps=taps)
    if loop:
        c["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    return c


DEFAULT_LAYERS = [(mixer(), dense()), (mixer(heads=2, dim=16, vdim=8, kv_rank=40), moe()), (mixer(heads=5, kv_rank=16), None)]


def weights(cfg, seed=0):
    """A random checkpoint under the design's tensor names, bf16-representable values."""
    g = torch.Generator().manual_seed(seed)
    W, S = cfg["width"], cfg.get("streams")

    def rnd(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16)
    t = {"embed": rnd(cfg["vocab"], W), "pos": rnd(cfg["max_positions"], W, s=0.5), "final.norm": 1 + rnd(W, s=0.1),
         "head": rnd(cfg["vocab"], W, s=W ** -0.5)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, D, V, R = m["heads"], m["dim"], m["vdim"], m["kv_rank"]
        t.update({p + "norm1": 1 + rnd(W, s=0.1), p + "mix.q": rnd(H * D, W, s=W ** -0.5), p + "mix.dkv": rnd(R, W, s=W ** -0.5),
                  p + "mix.dkv.norm": 1 + rnd(R, s=0.1), p + "mix.uk": rnd(H * D, R, s=2 * R ** -0.5),
                  p + "mix.uv": rnd(H * V, R, s=R ** -0.5), p + "mix.o": rnd(W, H * V, s=(H * V) ** -0.5)})
        if cfg.get("canon"):
            t[p + "canon1"] = rnd(W, cfg["canon"]["taps"], s=0.4)
        for q in ["hc1"] + (["hc2"] if L["mlp"] is not None else []):
            if S:
                t.update({f"{p}{q}.in": (1.0 / S + rnd(S, s=0.2)), f"{p}{q}.out": 1 + rnd(S, s=0.2),
                          f"{p}{q}.mix": (torch.eye(S) + rnd(S, S, s=0.2)).to(torch.bfloat16)})
        f = L["mlp"]
        if f is None:
            continue
        t[p + "norm2"] = 1 + rnd(W, s=0.1)
        if f["kind"] == "dense":
            t.update({p + "mlp.up": rnd(f["ff"], W, s=W ** -0.5), p + "mlp.down": rnd(W, f["ff"], s=f["ff"] ** -0.5),
                      p + "mlp.act": torch.tensor([0.7, 0.25, 0.1, 0.05]).to(torch.bfloat16)})
            continue
        ff = f["expert"]["ff"]
        t[p + "mlp.router"] = rnd(f["router"]["experts"], W, s=3 * W ** -0.5)
        for e in range(f["router"]["experts"]):
            t.update({f"{p}mlp.e{e}.gate": rnd(ff, W, s=2 * W ** -0.5), f"{p}mlp.e{e}.up": rnd(ff, W, s=2 * W ** -0.5),
                      f"{p}mlp.e{e}.down": rnd(W, ff, s=ff ** -0.5)})
        if f.get("shared"):
            fs = f["shared"]["ff"]
            t.update({p + "mlp.shared.gate": rnd(fs, W, s=2 * W ** -0.5), p + "mlp.shared.up": rnd(fs, W, s=2 * W ** -0.5),
                      p + "mlp.shared.down": rnd(W, fs, s=fs ** -0.5)})
    return {k: v.to(torch.bfloat16).contiguous() for k, v in t.items()}


def write_model(path, cfg, w):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file(w, os.path.join(path, "model.safetensors"))
    return str(path)


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def replay(model_dir, steps, tmp, device, dtype=torch.float32, max_tokens=512, max_live=4):
    """Steps [(entries, end)] with entries [(id, tokens, want)] through nanovllm.trace.replay -> {step: logits}."""
    from nanovllm.trace import replay as run
    lines = [json.dumps(dict(step=i, entries=[dict(id=r, tokens=t, want=w) for r, t, w in entries], end=end))
             for i, (entries, end) in enumerate(steps)]
    out = os.path.join(str(tmp), f"out_{np.random.randint(1 << 30)}")
    log = io.StringIO()
    assert run(model_dir, dtype, out, max_tokens, lines, device=device, max_live=max_live, log=log) == 0
    assert log.getvalue().split() == sum((["done", str(i)] for i in range(len(steps))), [])
    got = {}
    for i, (entries, _) in enumerate(steps):
        n = sum(len(w) for _, _, w in entries)
        if n:
            got[i] = np.fromfile(os.path.join(out, f"{i}.f32"), dtype="<f4").reshape(n, -1)
    return got


def close(got, ref, dtype):
    """Logit rows against the oracle's: float32 to accumulation order, bfloat16 to that format's rounding through the
    layers (difference with its mean removed, relative to the spread of the logits)."""
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape and np.isfinite(got).all()
    d = got - ref
    d = d - d.mean(-1, keepdims=True)
    err = np.sqrt((d ** 2).mean(-1)) / ref.std()
    if dtype == torch.float32:
        assert err.max() < 2e-4, f"relative error {err.max():.3g} at row {int(err.argmax())}"
        return
    # bfloat16: rounding can turn a near-tie of two router scores the other way, which moves that one row by much more
    # than rounding does (these small random routers have such ties in a few percent of the tokens); that is no fault,
    # so the bound is on the bulk of the rows.  float32 above, and the per-mechanism tests in bfloat16, are the sharp ones.
    over = np.nonzero(err > 6e-2)[0]
    assert len(over) <= max(1, 0.15 * len(err)) and (len(err) < 20 or np.median(err) < 3e-2), \
        f"{len(over)} of {len(err)} rows beyond bf16 rounding: {over[:10]}, median {np.median(err):.3g}"


def dtypes_for(device):
    return [torch.float32] if device == "cpu" else [torch.float32, torch.bfloat16]


def cut(n, sizes):
    """[(start, stop)] covering range(n) with portions of the given sizes, cycled."""
    out, a, i = [], 0, 0
    while a < n:
        b = min(n, a + sizes[i % len(sizes)])
        out.append((a, b))
        a, i = b, i + 1
    return out


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cfg = config(DEFAULT_LAYERS, loop=(0, 2, 2))
    w = weights(cfg, seed=1)
    return write_model(tmp_path_factory.mktemp("pasizen_default"), cfg, w), cfg, w


# ------------------------------------------------------------------------------------------ whole model, schedules
@pytest.mark.parametrize("device", DEVICES)
def test_whole_prompt_and_layer_trace(model, tmp_path, device):
    """One step per prompt: every position's logits; and the residual streams after every layer run."""
    path, cfg, w = model
    toks = tokens(70, cfg["vocab"], 3)
    ref, layers = O.forward(cfg, w, toks, return_layers=True)
    for dtype in dtypes_for(device):
        got = replay(path, [([("a", toks, list(range(70)))], ["a"])], tmp_path, device, dtype)
        close(got[0], ref, dtype)
    # the layer trace through the runner itself
    from nanovllm.engine.llm_engine import LLMEngine
    from nanovllm.engine.sequence import ACTIVE, Sequence
    eng = LLMEngine(path, device=device, dtype=torch.float32, max_num_seqs=2, num_kvcache_blocks=4, max_num_batched_tokens=4096)
    seq = Sequence(toks)
    seq.state = ACTIVE
    assert eng.scheduler.reserve_portion(seq, 70)
    trace = []
    eng.model_runner.run_portions([(seq, 70)], trace=trace)
    assert len(trace) == len(O.layer_runs(cfg)) == 5
    for got_l, ref_l in zip(trace, layers):
        assert torch.allclose(got_l.cpu(), ref_l, atol=2e-3, rtol=1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_prefill_equals_token_by_token(model, tmp_path, device):
    """A prompt fed one token per step (decode through cache and state from the very first token) gives the logits of
    the whole prompt in one step; 140 tokens cross two cache-block borders."""
    path, cfg, w = model
    toks = tokens(140, cfg["vocab"], 4)
    ref = O.forward(cfg, w, toks)
    steps = [([("a", [t], [0])], ["a"] if i == 139 else []) for i, t in enumerate(toks)]
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=192)
        close(np.concatenate([got[i] for i in range(140)]), ref, dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2], [3, 2, 7, 2, 64, 1, 5], [63, 2, 1, 64], [65, 1, 1, 1, 2]])
def test_portions(model, tmp_path, device, sizes):
    """Prompts cut into portions of several sizes (down to two tokens, across block borders, single tokens between)."""
    path, cfg, w = model
    toks = tokens(133, cfg["vocab"], 5)
    ref = O.forward(cfg, w, toks)
    parts = cut(133, sizes)
    steps = [([("r", toks[a:b], list(range(b - a)))], ["r"] if b == 133 else []) for a, b in parts]
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=192)
        close(np.concatenate([got[i] for i in range(len(parts))]), ref, dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_and_reused_pages_and_slots(model, tmp_path, device):
    """Unequal requests share steps (prompt portions beside single tokens), more requests than state slots and more
    tokens than cache blocks over the run: blocks and slots are freed and taken again, also by a request whose first
    tokens land in a slot that still holds another request's state.  Each request equals itself run alone."""
    path, cfg, w = model
    V = cfg["vocab"]
    reqs = {f"q{i}": tokens(n, V, 10 + i) for i, n in enumerate([97, 5, 130, 66, 1, 71, 64])}
    ref = {k: O.forward(cfg, w, v) for k, v in reqs.items()}
    plan = {"q0": cut(97, [40, 1, 1, 30, 1]), "q1": cut(5, [2, 1]), "q2": cut(130, [64, 3, 1]), "q3": cut(66, [66]),
            "q4": cut(1, [1]), "q5": cut(71, [7, 1]), "q6": cut(64, [62, 2])}
    order = list(reqs)
    live, waiting, steps, rows = [], list(order), [], []
    cursor = {k: 0 for k in order}
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
    # 3 live requests of at most 130 + 97 + 66 tokens: 3 + 2 + 2 blocks of 64; the run as a whole needs 12
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=7 * 64, max_live=3)
        at = {}
        for s, k, a, b in rows:
            o = at.get(s, 0)
            close(got[s][o:o + b - a], ref[k][a:b], dtype)
            at[s] = o + b - a


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding(model, tmp_path, device):
    """A short prompt and 200 single-token steps: three block borders are crossed while decoding."""
    path, cfg, w = model
    toks = tokens(215, cfg["vocab"], 6)
    ref = O.forward(cfg, w, toks)
    steps = [([("a", toks[:15], [14])], [])] + [([("a", [t], [0])], []) for t in toks[15:]]
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=256)
        close(np.concatenate([got[i] for i in range(len(steps))]), ref[14:], dtype)


VARIANTS = {
    "one_stream_no_loop": config([(mixer(heads=1, dim=8, vdim=8, kv_rank=8), dense(16)), (mixer(), moe(groups=None, shared=None))],
                                 streams=1, taps=2),
    "plain_residual_no_conv": config([(mixer(kv_rank=36), moe(experts=4, top=1, groups=(2, 2))), (mixer(), dense())],
                                     streams=None, taps=None),
    "many_streams_long_taps": config([(mixer(heads=7, dim=4, vdim=4, kv_rank=64), None), (mixer(), moe(top=3, groups=(2, 1)))],
                                     streams=5, taps=6, width=40, loop=(1, 2, 3)),
    "single_tap": config([(mixer(kv_rank=96), dense()), (mixer(), moe(experts=8, top=4, groups=(4, 2), shared=(8, 3.0)))],
                         streams=2, taps=1, loop=(0, 1, 2)),
    "wide_latent": config([(mixer(heads=4, dim=16, vdim=24, kv_rank=136), dense())], streams=4, taps=4, width=64),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(VARIANTS))
def test_other_shapes(tmp_path, device, name):
    """Other sizes and options: one head, heads that do not divide a tile, latent ranks off the multiples of 8 and 32,
    one / many / no streams, 1 / 2 / 6 taps and no convolution, top-1 and ungrouped routing, all groups kept, no shared
    expert, a layer without feed-forward, loops of one layer, of the first layer, and none.  Portions and a batch."""
    cfg = VARIANTS[name]
    w = weights(cfg, seed=7)
    path = write_model(tmp_path / "m", cfg, w)
    a, b = tokens(75, cfg["vocab"], 8), tokens(9, cfg["vocab"], 9)
    ra, rb = O.forward(cfg, w, a), O.forward(cfg, w, b)
    steps = [([("a", a[:31], list(range(31)))], []),
             ([("a", a[31:66], list(range(35))), ("b", b[:2], [0, 1])], []),
             ([("b", b[2:], list(range(7))), ("a", a[66:67], [0])], ["b"])] + \
            [([("a", [t], [0])], []) for t in a[67:]]
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=192)
        close(got[0], ra[:31], dtype)
        close(got[1], np.concatenate([ra[31:66], rb[:2]]), dtype)
        close(got[2], np.concatenate([rb[2:], ra[66:67]]), dtype)
        close(np.concatenate([got[i] for i in range(3, len(steps))]), ra[67:], dtype)


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
            p.append(int(O.forward(cfg, w, p)[-1].argmax()))
        return p[-n:]
    llm = LLM(path, device=device, dtype=torch.float32, max_num_seqs=3, max_num_batched_tokens=16, num_kvcache_blocks=5)
    out = llm.generate(prompts, SamplingParams(max_tokens=6, ignore_eos=True))
    assert [o["token_ids"] for o in out] == [greedy(p, 6) for p in prompts]
    assert len(llm.scheduler.block_manager.free) == 5 and len(llm.scheduler.slots.free) == 3


def test_scheduler_preempts_when_blocks_run_out(model):
    """Two requests that cannot both grow in a three-block pool: the later one is put back, runs again afterwards, and
    both produce what they produce alone."""
    from nanovllm import LLM, SamplingParams
    path, cfg, w = model
    prompts = [tokens(60, cfg["vocab"], 31), tokens(62, cfg["vocab"], 32)]
    sp = SamplingParams(max_tokens=10, ignore_eos=True)
    alone = [LLM(path, device="cpu", dtype=torch.float32, max_num_seqs=2, num_kvcache_blocks=4).generate([p], sp)[0]["token_ids"]
             for p in prompts]
    llm = LLM(path, device="cpu", dtype=torch.float32, max_num_seqs=2, num_kvcache_blocks=3)
    out = llm.generate(prompts, sp)
    assert [o["token_ids"] for o in out] == alone


def test_registry_and_config():
    from nanovllm.models import registry
    assert registry.architecture_of({"architecture": "Pasizen"}) == "Pasizen"
    assert registry.architecture_of({"architectures": ["Qwen3ForCausalLM"]}) == "Qwen3ForCausalLM"
    assert registry.architecture_of({}) == "Qwen3ForCausalLM"
    with pytest.raises(ValueError):
        registry.architecture_of({"architecture": "NoSuchModel"})
    from nanovllm.models.pasizen import layer_run_order
    assert layer_run_order(4, None) == [0, 1, 2, 3]
    assert layer_run_order(4, dict(start=1, stop=3, times=3)) == [0, 1, 2, 1, 2, 1, 2, 3] == O.layer_runs(
        dict(layers=[0] * 4, loop=dict(start=1, stop=3, times=3)))


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
    # (bfloat16: a bucket's GEMMs have other row counts than the eager batch, so rounding differs: all rows as one set)
    close(torch.cat(outs[1]).numpy(), torch.cat(outs[0]).numpy(), dtype)
