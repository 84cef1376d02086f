"""Replay of a token trace through the engine: given token ids are fed step by step and the logits of chosen
positions are written out; nothing is sampled.  The replay drives the engine's own pieces - LLMEngine, its scheduler's
block and slot pools (Scheduler.reserve_portion / release), ModelRunner.run_portions and the model's kernels - exactly as
generation does; only the choice of what runs in a step comes from the trace instead of from Scheduler.schedule_portions.

Input: one JSON object per line,
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
``entries``: per request its next tokens and the places among them whose logits are wanted; ``end``: requests that are
over after the step (their blocks and slot return to the pools).  Output: <out>/<step>.f32 = float32 [wanted, vocab]
for a step that wants something, and a line ``done <step>`` on standard output after every step."""
import json
import os
import sys

import torch


def replay(model, dtype, out_dir, max_tokens, lines, device="cuda", max_live=4, log=sys.stdout):
    from nanovllm.config import Config
    from nanovllm.engine.llm_engine import LLMEngine
    from nanovllm.engine.sequence import ACTIVE, Sequence
    cfg0 = Config(model, device=device, dtype=dtype, enforce_eager=True)
    if not cfg0.runs_portions:
        raise SystemExit("trace replay needs a model family that is stepped with portions of sequences")
    bs = cfg0.kvcache_block_size
    # the cache pool holds max_tokens (every live request rounded up to whole blocks), the state pool max_live requests
    blocks = (int(max_tokens) + bs - 1) // bs + (max_live if bs > 64 else 0)
    engine = LLMEngine(model, device=device, dtype=dtype, enforce_eager=True, max_num_seqs=max_live,
                       num_kvcache_blocks=blocks, max_model_len=cfg0.hf_config.max_position_embeddings,
                       max_num_batched_tokens=1 << 30)
    sch = engine.scheduler
    live = {}
    os.makedirs(out_dir, exist_ok=True)
    for line in lines:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        batch, rows, row0 = [], [], 0
        for e in step["entries"]:
            toks = e["tokens"]
            if not toks:
                continue
            seq = live.get(e["id"])
            if seq is None:
                seq = live[e["id"]] = Sequence(toks)
                seq.state = ACTIVE
            else:
                seq.extend(toks)
            if not sch.reserve_portion(seq, len(toks)):
                raise RuntimeError(f"step {step['step']}: the cache or state pool cannot hold request {e['id']}")
            batch.append((seq, len(toks)))
            rows.extend(row0 + int(w) for w in e.get("want", []))
            row0 += len(toks)
        if batch:
            logits = engine.forward_portions(batch, rows)
            for seq, n in batch:
                seq.num_computed += n
            if rows:
                data = logits.float().cpu().contiguous().numpy().astype("<f4", copy=False)
                tmp = os.path.join(out_dir, f".{step['step']}.part")
                with open(tmp, "wb") as f:
                    f.write(data.tobytes())
                os.replace(tmp, os.path.join(out_dir, f"{step['step']}.f32"))
        for rid in step.get("end", []):
            seq = live.pop(rid, None)
            if seq is not None:
                sch.release(seq)
        print(f"done {step['step']}", file=log, flush=True)
    return 0


def main(argv=None):
    import argparse
    ap = argparse.ArgumentParser(description="replay a token trace through the engine and write the wanted logits")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32")
    ap.add_argument("--max-tokens", type=int, required=True, help="tokens the cache pool is made for")
    ap.add_argument("--max-live", type=int, default=4, help="state slots (requests alive at a time)")
    ap.add_argument("--device", default="cuda", choices=["cuda", "cpu"],
                    help="cpu = engine plumbing with plain torch operators, for hosts without a GPU")
    a = ap.parse_args(argv)
    return replay(a.model, getattr(torch, a.dtype), a.out, a.max_tokens, sys.stdin, device=a.device, max_live=a.max_live)


if __name__ == "__main__":
    sys.exit(main())
