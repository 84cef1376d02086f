"""Pasizen: a decoder-only model whose layers combine a latent-attention mixer behind a short causal convolution with a
PolyNorm dense feed-forward or a routed mixture of clamped-GLU experts, on a multi-stream residual, with learned
absolute positions and a block of layers that may be run several times with the same weights.

Everything that can differ between checkpoints is read from config.json:
  vocab, width, max_positions, norm.eps, streams, canon.taps,
  layers[i] = {type, mixer: {heads, dim, vdim, kv_rank, scale}, mlp: null | {kind: dense, ff} |
               {kind: moe, expert: {ff, limit}, router: {experts, top, groups: {count, keep}}, shared: {ff, limit}}},
  loop = {start, stop, times}: layers start..stop-1 run `times` times in a row; every pass ("layer run") has its own
  cache and convolution state.
Checkpoint tensors: embed, pos, final.norm, head, and per layer l<i>.{norm1, norm2, canon1, hc1.*, hc2.*, mix.*, mlp.*}.

The model is stepped with portions of sequences (nanovllm.seq_ops.StepContext): any mix of prompt pieces and single
decoded tokens in one batch.  Residual streams, norms, softmax and router scores are float32 whatever the model dtype."""
import re

import torch
import torch.nn.functional as F
from torch import nn

from nanovllm import seq_ops
from nanovllm.layers.canon import CausalTaps
from nanovllm.layers.feedforward import ClampedGLU, PolyNormMLP, RoutedExperts
from nanovllm.layers.latent_attention import LatentAttention
from nanovllm.layers.streams import StreamPort

MIXERS = {"latent_attention": LatentAttention}


def layer_run_order(num_layers, loop):
    """Indices of the layers in the order they run."""
    if not loop:
        return list(range(num_layers))
    a, b, n = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * n + list(range(b, num_layers))


class PasizenLayer(nn.Module):
    def __init__(self, cfg, spec):
        super().__init__()
        W, eps, S = cfg.hidden_size, cfg.norm_eps, cfg.streams
        learned = cfg.learned_streams
        m = spec["mixer"]
        if spec["type"] not in MIXERS:
            raise ValueError(f"unknown mixer type {spec['type']!r}")
        self.norm1 = nn.Parameter(torch.ones(W), requires_grad=False)
        self.port1 = StreamPort(S, learned)
        self.canon = CausalTaps(W, cfg.canon_taps) if cfg.canon_taps else None
        self.mixer = LatentAttention(W, m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["scale"], eps)
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp is not None:
            self.norm2 = nn.Parameter(torch.ones(W), requires_grad=False)
            self.port2 = StreamPort(S, learned)
            if mlp["kind"] == "dense":
                self.mlp = PolyNormMLP(W, mlp["ff"], eps)
            elif mlp["kind"] == "moe":
                r, g, sh = mlp["router"], mlp["router"].get("groups"), mlp.get("shared")
                shared = ClampedGLU(W, sh["ff"], sh["limit"]) if sh else None
                self.mlp = RoutedExperts(W, r["experts"], r["top"], mlp["expert"]["ff"], mlp["expert"]["limit"],
                                         g["count"] if g else 1, g["keep"] if g else 1, shared)
            else:
                raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")


class PasizenForCausalLM(nn.Module):
    runs_portions = True           # stepped with portions; owns a latent cache and convolution state per layer run
    default_block_size = 64
    native_library = "seqmix"

    @staticmethod
    def normalize_config(d: dict) -> dict:
        d = dict(d)
        d["vocab_size"], d["hidden_size"] = d["vocab"], d["width"]
        d["max_position_embeddings"] = d.get("max_positions", 1 << 20)
        d["learned_positions"] = "max_positions" in d
        d["norm_eps"] = d["norm"]["eps"]
        d["learned_streams"] = bool(d.get("streams"))
        d["streams"] = d.get("streams") or 1
        d["canon_taps"] = (d.get("canon") or {}).get("taps", 0)
        d["run_order"] = layer_run_order(len(d["layers"]), d.get("loop"))
        d.setdefault("torch_dtype", "bfloat16")
        return d

    def __init__(self, cfg):
        super().__init__()
        self.cfg = cfg
        W = cfg.hidden_size
        self.dtype = torch.get_default_dtype()
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, W), requires_grad=False)
        self.pos = nn.Parameter(torch.empty(cfg.max_position_embeddings, W), requires_grad=False) if cfg.learned_positions else None
        self.layers = nn.ModuleList([PasizenLayer(cfg, spec) for spec in cfg.layers])
        self.final_norm = nn.Parameter(torch.ones(W), requires_grad=False)
        self.head = nn.Parameter(torch.empty(cfg.vocab_size, W), requires_grad=False)
        self.run_order = list(cfg.run_order)
        self.sum_streams = torch.ones(cfg.streams, dtype=torch.float32)
        self._f32_out = None       # whether the vendor GEMM writes float32 from 16-bit operands for the head's shape

    # ------------------------------------------------------------------ checkpoint names
    _SIMPLE = {"norm1": "norm1", "norm2": "norm2", "canon1": "canon.weight", "mix.dkv.norm": "mixer.latent_norm",
               "mix.o": "mixer.o_proj", "mlp.up": "mlp.up", "mlp.down": "mlp.down", "mlp.act": "mlp.coef",
               "mlp.router": "mlp.router", "mlp.shared.down": "mlp.shared.down",
               "hc1.in": "port1.w_in", "hc1.out": "port1.out", "hc1.mix": "port1.mix",
               "hc2.in": "port2.w_in", "hc2.out": "port2.out", "hc2.mix": "port2.mix"}

    def load_checkpoint_tensor(self, params, name, tensor):
        """Place one checkpoint tensor; returns False for a name this model does not know."""
        top = {"embed": "embed", "pos": "pos", "final.norm": "final_norm", "head": "head"}
        if name in top:
            params[top[name]].data.copy_(tensor)
            return True
        m = re.fullmatch(r"l(\d+)\.(.+)", name)
        if not m or int(m.group(1)) >= len(self.layers):
            return False
        i, rest = int(m.group(1)), m.group(2)
        layer, pre = self.layers[i], f"layers.{i}."
        if rest in self._SIMPLE:
            p = params.get(pre + self._SIMPLE[rest])
            if p is None:
                return False
            p.data.copy_(tensor.reshape(p.shape))
            return True
        mx = layer.mixer
        if rest == "mix.q":
            mx.qc_proj.data[:mx.heads * mx.dim].copy_(tensor)
        elif rest == "mix.dkv":
            mx.qc_proj.data[mx.heads * mx.dim:].copy_(tensor)
        elif rest == "mix.uk":
            mx.uk.data.copy_(tensor.view(mx.heads, mx.dim, mx.kv_rank))
        elif rest == "mix.uv":
            mx.uv.data.copy_(tensor.view(mx.heads, mx.vdim, mx.kv_rank))
        elif rest in ("mlp.shared.gate", "mlp.shared.up"):
            sh = layer.mlp.shared
            sh.gate_up.data[(sh.ff if rest.endswith("up") else 0):][:sh.ff].copy_(tensor)
        else:
            e = re.fullmatch(r"mlp\.e(\d+)\.(gate|up|down)", rest)
            if not e or not isinstance(layer.mlp, RoutedExperts):
                return False
            k, which = int(e.group(1)), e.group(2)
            ff = layer.mlp.w_down.shape[2]
            if which == "down":
                layer.mlp.w_down.data[k].copy_(tensor)
            else:
                layer.mlp.w_gu.data[k, (ff if which == "up" else 0):][:ff].copy_(tensor)
        return True

    def checkpoint_tensors(self, seed=0, std=0.05):
        """Random tensors with the checkpoint's names and shapes (benchmarks and tests without a checkpoint), drawn in
        a fixed order from one seeded generator on the model's device."""
        cfg, dev = self.cfg, self.embed.device
        g = torch.Generator(device=dev).manual_seed(seed)
        W, S = cfg.hidden_size, cfg.streams

        def rnd(*shape, s=std):
            return torch.randn(*shape, generator=g, device=dev, dtype=torch.float32) * s
        t = {"embed": rnd(cfg.vocab_size, W, s=1.0), "final.norm": 1 + rnd(W), "head": rnd(cfg.vocab_size, W, s=W ** -0.5)}
        if cfg.learned_positions:
            t["pos"] = rnd(cfg.max_position_embeddings, W, s=0.3)
        for i, spec in enumerate(cfg.layers):
            p, m = f"l{i}.", spec["mixer"]
            H, D, V, R = m["heads"], m["dim"], m["vdim"], m["kv_rank"]
            t.update({p + "norm1": 1 + rnd(W), p + "mix.q": rnd(H * D, W, s=W ** -0.5), p + "mix.dkv": rnd(R, W, s=W ** -0.5),
                      p + "mix.dkv.norm": 1 + rnd(R), p + "mix.uk": rnd(H * D, R, s=R ** -0.5),
                      p + "mix.uv": rnd(H * V, R, s=R ** -0.5), p + "mix.o": rnd(W, H * V, s=(H * V) ** -0.5)})
            if cfg.canon_taps:
                t[p + "canon1"] = rnd(W, cfg.canon_taps, s=0.2)
            ports = ["hc1"] + (["hc2"] if spec.get("mlp") is not None else [])
            if cfg.learned_streams:
                for q in ports:
                    t.update({f"{p}{q}.in": 1.0 / S + rnd(S, s=0.1), f"{p}{q}.out": 1 + rnd(S, s=0.1),
                              f"{p}{q}.mix": torch.eye(S, device=dev) + rnd(S, S, s=0.1)})
            mlp = spec.get("mlp")
            if mlp is None:
                continue
            t[p + "norm2"] = 1 + rnd(W)
            if mlp["kind"] == "dense":
                t.update({p + "mlp.up": rnd(mlp["ff"], W, s=W ** -0.5), p + "mlp.down": rnd(W, mlp["ff"], s=mlp["ff"] ** -0.5),
                          p + "mlp.act": torch.tensor([0.6, 0.3, 0.1, 0.05], device=dev) + rnd(4, s=0.05)})
                continue
            ff = mlp["expert"]["ff"]
            t[p + "mlp.router"] = rnd(mlp["router"]["experts"], W, s=2 * W ** -0.5)
            for e in range(mlp["router"]["experts"]):
                t.update({f"{p}mlp.e{e}.gate": rnd(ff, W, s=2 * W ** -0.5), f"{p}mlp.e{e}.up": rnd(ff, W, s=2 * W ** -0.5),
                          f"{p}mlp.e{e}.down": rnd(W, ff, s=ff ** -0.5)})
            if mlp.get("shared"):
                fs = mlp["shared"]["ff"]
                t.update({p + "mlp.shared.gate": rnd(fs, W, s=2 * W ** -0.5), p + "mlp.shared.up": rnd(fs, W, s=2 * W ** -0.5),
                          p + "mlp.shared.down": rnd(W, fs, s=fs ** -0.5)})
        return {k: v.to(torch.bfloat16) for k, v in t.items()}

    # ------------------------------------------------------------------ cache and state
    def cache_bytes_per_block(self, block_size):
        item = self.dtype.itemsize
        return sum(block_size * self.layers[li].mixer.kv_rank * item for li in self.run_order)

    def state_bytes_per_slot(self):
        taps = self.cfg.canon_taps
        return len(self.run_order) * max(taps - 1, 0) * self.cfg.hidden_size * self.dtype.itemsize

    def allocate_cache(self, num_blocks, block_size, num_slots, device):
        """One latent cache per layer run (a looped layer's passes do not share), and one convolution state tensor
        [slots, runs, taps-1, width] for every sequence slot."""
        self.num_slots = num_slots
        for run, li in enumerate(self.run_order):
            mx = self.layers[li].mixer
            mx.cache[run] = torch.zeros(num_blocks, block_size, mx.kv_rank, dtype=self.dtype, device=device)
        taps = self.cfg.canon_taps
        if taps:
            state = torch.zeros(num_slots, len(self.run_order), max(taps - 1, 1), self.cfg.hidden_size, dtype=self.dtype,
                                device=device)
            for layer in self.layers:
                layer.canon.state = state

    def workspaces(self):
        """Scratch buffers that captured decode graphs address."""
        from nanovllm import _seqmix
        return [_seqmix.decode_workspace]

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids, positions, trace=None):
        """input_ids int64 [T], positions int32 [T] (the step's context is seq_ops.get_step()) -> final-normed hidden
        [T, width].  ``trace``: a list that receives the summed streams after every layer run (debugging)."""
        cfg, dt = self.cfg, self.dtype
        eps = cfg.norm_eps
        X = seq_ops.embed_streams(input_ids, positions, self.embed, self.pos, cfg.streams)
        first = self.layers[self.run_order[0]]
        h = seq_ops.stream_step(X, None, None, None, first.port1.w_in, first.norm1, eps, dt)
        n = len(self.run_order)
        for run, li in enumerate(self.run_order):
            layer = self.layers[li]
            if layer.canon is not None:
                h = layer.canon(h, run)
            y = layer.mixer(h, run)
            port = layer.port1
            if layer.mlp is not None:
                h = seq_ops.stream_step(X, y, port.mix, port.out, layer.port2.w_in, layer.norm2, eps, dt)
                y = layer.mlp(h)
                port = layer.port2
            # the write of this layer's last sublayer and the read (+ norm) of the next layer's first, in one launch
            if run + 1 < n:
                nxt = self.layers[self.run_order[run + 1]]
                w_in, norm_w = nxt.port1.w_in, nxt.norm1
            else:
                w_in, norm_w = self.sum_streams, self.final_norm
            h = seq_ops.stream_step(X, y, port.mix, port.out, w_in, norm_w, eps, dt)
            if trace is not None:
                trace.append(X.sum(1))
        return h

    def compute_logits(self, hidden_states):
        """float32 logits of the given rows: products of the stored values, float32 accumulation AND output."""
        if hidden_states.dtype == torch.float32:
            return F.linear(hidden_states, self.head)
        if hidden_states.is_cuda and self._f32_out is not False:
            try:
                out = torch.mm(hidden_states, self.head.t(), out_dtype=torch.float32)
                self._f32_out = True
                return out
            except RuntimeError:
                if self._f32_out:          # it has worked before: this is another fault
                    raise
                self._f32_out = False      # no such GEMM for this shape: the same sums from widened operands
        return F.linear(hidden_states.float(), self.head.float())
