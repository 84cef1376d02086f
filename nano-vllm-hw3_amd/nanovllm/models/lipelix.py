"""Lipelix: a decoder-only model whose layers are listed one by one in config.json, each with one of three mixers - full
causal rotary attention with a learned sink and normalised q/k projections ("attention"), sliding-window rotary attention
that keeps the first tokens, with unit-norm heads and a zero sink ("attention_2"), or a generalized delta-rule recurrence
("general_delta") - and an optional squared-ReLU feed-forward.  Every sublayer sits between two RMS norms on a float32
residual, its result is gated by a sigmoid of a product of its input and scaled by ``residual_mult``; the mixer reads a
token-shifted input; attention layers that say ``v_mix`` blend their values with those of the first such layer.

Read from config.json: vocab, width, embedding.scale, norm.eps, residual_mult, and per layer
  {type, mixer: {heads, kv_heads, dim, vdim, scale, rot: {dims, base}, v_mix, mask: {size, keep_first}} | {heads, dim},
   mlp: null | {kind: dense, ff}}.
Checkpoint tensors: embed, final.norm, head, and per layer l<i>.{norm1, norm1b, norm2, norm2b, shift, rg1, rg1.b, rg2,
rg2.b, mix.*, mlp.up, mlp.down}.

The model is stepped with portions of sequences (nanovllm.seq_ops.StepContext).  It owns a paged key/value cache per
attention layer and, per state slot, the token-shift row of every layer and the float32 delta-rule state of every
recurrent layer."""
import re

import torch
import torch.nn.functional as F
from torch import nn

from nanovllm import hy_ops, seq_ops
from nanovllm.layers.delta_rule import GeneralDelta
from nanovllm.layers.feedforward import ReluSquaredMLP
from nanovllm.layers.gated_sublayer import GatedPort
from nanovllm.layers.rotary_attention import PagedRotaryAttention
from nanovllm.layers.token_shift import TokenShift

ATTENTION_KINDS = {
    # type -> what distinguishes it
    "attention": dict(proj_norm=True, unit_norm=False, sink="learned", windowed=False),
    "attention_2": dict(proj_norm=False, unit_norm=True, sink="zero", windowed=True),
}


class LipelixLayer(nn.Module):
    def __init__(self, cfg, spec):
        super().__init__()
        W, eps, m = cfg.hidden_size, cfg.norm_eps, spec["mixer"]
        self.kind = spec["type"]
        self.port1 = GatedPort(W)
        self.shift = TokenShift(W)
        if self.kind in ATTENTION_KINDS:
            k = ATTENTION_KINDS[self.kind]
            mask = m.get("mask") or {}
            self.mixer = PagedRotaryAttention(
                W, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], eps, m["rot"]["dims"], m["rot"]["base"],
                proj_norm=k["proj_norm"], unit_norm=k["unit_norm"], sink=k["sink"],
                window=mask.get("size", 0) if k["windowed"] else 0, keep_first=mask.get("keep_first", 0) if k["windowed"] else 0,
                v_mix=bool(m.get("v_mix")))
        elif self.kind == "general_delta":
            self.mixer = GeneralDelta(W, m["heads"], m["dim"], spec["decay_rank"], eps)
        else:
            raise ValueError(f"unknown mixer type {self.kind!r}")
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp is not None:
            if mlp["kind"] != "dense":
                raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
            self.port2 = GatedPort(W, own_gate_weight=False)       # its gate rows ride on the up product
            self.mlp = ReluSquaredMLP(W, mlp["ff"], extra_rows=W)


class LipelixForCausalLM(nn.Module):
    runs_portions = True           # stepped with portions; owns its caches and per-sequence state
    default_block_size = 64
    native_library = "hymix"

    @staticmethod
    def normalize_config(d: dict) -> dict:
        d = dict(d)
        d["vocab_size"], d["hidden_size"] = d["vocab"], d["width"]
        d["max_position_embeddings"] = d.get("max_positions", 1 << 20)
        d["norm_eps"] = d["norm"]["eps"]
        d["embedding_scale"] = (d.get("embedding") or {}).get("scale", 1.0)
        d["residual_mult"] = d.get("residual_mult", 1.0)
        layers = []
        for spec in d["layers"]:
            spec = dict(spec)
            # the rank of the decay's inner projection is a tensor's shape, not a config value: a default until the
            # checkpoint is seen (load_checkpoint_tensor resizes), or what a dummy model asks for
            if spec["type"] == "general_delta":
                spec["decay_rank"] = spec["mixer"].get("decay_rank", 32)
            layers.append(spec)
        d["layers"] = layers
        mixed = [(s["mixer"]["kv_heads"], s["mixer"]["vdim"]) for s in layers if s["type"] in ATTENTION_KINDS and s["mixer"].get("v_mix")]
        if len(set(mixed)) > 1:
            raise ValueError(f"layers that mix values must agree on kv_heads and vdim, got {sorted(set(mixed))}")
        d.setdefault("torch_dtype", "bfloat16")
        return d

    def __init__(self, cfg):
        super().__init__()
        self.cfg = cfg
        W = cfg.hidden_size
        self.dtype = torch.get_default_dtype()
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, W), requires_grad=False)
        self.layers = nn.ModuleList([LipelixLayer(cfg, spec) for spec in cfg.layers])
        self.final_norm = nn.Parameter(torch.ones(W), requires_grad=False)
        self.head = nn.Parameter(torch.empty(cfg.vocab_size, W), requires_grad=False)
        self._f32_out = None       # whether the vendor GEMM writes float32 from 16-bit operands for the head's shape
        # the first layer that mixes values gives them; it blends nothing itself
        self.v_source = next((i for i, l in enumerate(self.layers) if getattr(l.mixer, "v_mix", False)), None)

    # ------------------------------------------------------------------ checkpoint names
    _PORT = {"norm1": "port1.norm", "norm1b": "port1.post_norm", "rg1": "port1.gate_weight", "rg1.b": "port1.gate_bias",
             "norm2": "port2.norm", "norm2b": "port2.post_norm", "rg2.b": "port2.gate_bias", "shift": "shift.mu",
             "mlp.down": "mlp.down", "mix.o": "mixer.o_proj", "mix.q.norm": "mixer.q_norm", "mix.k.norm": "mixer.k_norm",
             "mix.sink": "mixer.sink", "mix.w2": "mixer.w2", "mix.w0": "mixer.w0", "mix.a.b": "mixer.a_bias",
             "mix.norm": "mixer.out_norm"}

    def load_checkpoint_tensor(self, params, name, tensor):
        """Place one checkpoint tensor; returns False for a name this model does not know."""
        top = {"embed": "embed", "final.norm": "final_norm", "head": "head"}
        if name in top:
            params[top[name]].data.copy_(tensor)
            return True
        m = re.fullmatch(r"l(\d+)\.(.+)", name)
        if not m or int(m.group(1)) >= len(self.layers):
            return False
        i, rest = int(m.group(1)), m.group(2)
        layer, pre = self.layers[i], f"layers.{i}."
        mx = layer.mixer
        if isinstance(mx, GeneralDelta) and rest in ("mix.w1", "mix.w2") and tensor.shape[rest == "mix.w2"] != mx.rank:
            self._resize_decay_rank(mx, tensor.shape[rest == "mix.w2"])
            params.update(dict(self.named_parameters()))
        if rest in self._PORT:
            p = params.get(pre + self._PORT[rest])
            if p is None:
                return False
            p.data.copy_(tensor.reshape(p.shape))
            return True
        if rest == "mlp.up" and layer.mlp is not None:
            layer.mlp.up.data[:layer.mlp.ff].copy_(tensor)
        elif rest == "rg2" and layer.mlp is not None:
            layer.mlp.up.data[layer.mlp.ff:].copy_(tensor)
        elif isinstance(mx, PagedRotaryAttention) and rest in ("mix.q", "mix.k", "mix.v"):
            a = mx.heads * mx.dim
            b = a + mx.kv_heads * mx.dim
            lo, hi = {"mix.q": (0, a), "mix.k": (a, b), "mix.v": (b, mx.qkv_proj.shape[0])}[rest]
            mx.qkv_proj.data[lo:hi].copy_(tensor)
        elif isinstance(mx, PagedRotaryAttention) and rest == "mix.vmix":
            if mx.lam is None:
                return False
            mx.lam.data.fill_(float(tensor))
        elif isinstance(mx, GeneralDelta) and rest[4:] in GeneralDelta.ROWS:
            hd = mx.heads * mx.dim
            k = GeneralDelta.ROWS.index(rest[4:])
            mx.in_proj.data[k * hd:(k + 1) * hd].copy_(tensor)
        elif isinstance(mx, GeneralDelta) and rest == "mix.w1":
            mx.in_proj.data[5 * mx.heads * mx.dim:].copy_(tensor)
        else:
            return False
        return True

    @staticmethod
    def _resize_decay_rank(mx, rank):
        """The decay's inner rank is known only from the checkpoint's shapes: remake the two tensors that depend on it
        (rows already placed in the merged product are kept)."""
        hd = mx.heads * mx.dim
        old = mx.in_proj.data
        new = torch.empty(5 * hd + rank, old.shape[1], dtype=old.dtype, device=old.device)
        new[:5 * hd] = old[:5 * hd]
        mx.in_proj = nn.Parameter(new, requires_grad=False)
        mx.w2 = nn.Parameter(torch.empty(hd, rank, dtype=old.dtype, device=old.device), requires_grad=False)
        mx.rank = rank

    def checkpoint_tensors(self, seed=0, std=0.05):
        """Random tensors with the checkpoint's names and shapes (benchmarks and tests without a checkpoint), drawn in
        a fixed order from one seeded generator on the model's device."""
        cfg, dev = self.cfg, self.embed.device
        g = torch.Generator(device=dev).manual_seed(seed)
        W = cfg.hidden_size

        def rnd(*shape, s=std):
            return torch.randn(*shape, generator=g, device=dev, dtype=torch.float32) * s
        t = {"embed": rnd(cfg.vocab_size, W, s=1.0 / max(cfg.embedding_scale, 1e-6)), "final.norm": 1 + rnd(W),
             "head": rnd(cfg.vocab_size, W, s=W ** -0.5)}
        for i, spec in enumerate(cfg.layers):
            p, m = f"l{i}.", spec["mixer"]
            t.update({p + "norm1": 1 + rnd(W), p + "norm1b": 1 + rnd(W), p + "shift": 0.5 + rnd(W, s=0.2),
                      p + "rg1": rnd(W, W, s=W ** -0.5), p + "rg1.b": rnd(W, s=0.5)})
            if spec["type"] in ATTENTION_KINDS:
                H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
                t.update({p + "mix.q": rnd(H * D, W, s=W ** -0.5), p + "mix.k": rnd(G * D, W, s=W ** -0.5),
                          p + "mix.v": rnd(G * V, W, s=W ** -0.5), p + "mix.o": rnd(W, H * V, s=(H * V) ** -0.5)})
                if ATTENTION_KINDS[spec["type"]]["proj_norm"]:
                    t.update({p + "mix.q.norm": 1 + rnd(H * D, s=0.2), p + "mix.k.norm": 1 + rnd(G * D, s=0.2)})
                if ATTENTION_KINDS[spec["type"]]["sink"] == "learned":
                    t[p + "mix.sink"] = rnd(H, s=1.0)
                if m.get("v_mix"):
                    t[p + "mix.vmix"] = torch.rand((), generator=g, device=dev) * 0.6 + 0.2
            else:
                H, D, R = m["heads"], m["dim"], spec["decay_rank"]
                for n in GeneralDelta.ROWS:
                    t[p + "mix." + n] = rnd(H * D, W, s=W ** -0.5)
                t.update({p + "mix.w1": rnd(R, W, s=W ** -0.5), p + "mix.w2": rnd(H * D, R, s=R ** -0.5), p + "mix.w0": rnd(H * D, s=1.0),
                          p + "mix.a.b": rnd(H * D, s=1.0), p + "mix.norm": 1 + rnd(H * D, s=0.2),
                          p + "mix.o": rnd(W, H * D, s=(H * D) ** -0.5)})
            mlp = spec.get("mlp")
            if mlp is not None:
                t.update({p + "norm2": 1 + rnd(W), p + "norm2b": 1 + rnd(W), p + "rg2": rnd(W, W, s=W ** -0.5),
                          p + "rg2.b": rnd(W, s=0.5), p + "mlp.up": rnd(mlp["ff"], W, s=W ** -0.5),
                          p + "mlp.down": rnd(W, mlp["ff"], s=mlp["ff"] ** -0.5)})
        return {k: v.to(torch.bfloat16) for k, v in t.items()}

    # ------------------------------------------------------------------ cache and state
    def _attention_layers(self):
        return [l.mixer for l in self.layers if isinstance(l.mixer, PagedRotaryAttention)]

    def cache_bytes_per_block(self, block_size):
        return sum(block_size * mx.cache_bytes_per_token(self.dtype.itemsize) for mx in self._attention_layers())

    def state_bytes_per_slot(self):
        shift = len(self.layers) * self.cfg.hidden_size * self.dtype.itemsize
        return shift + sum(l.mixer.state_bytes_per_slot() for l in self.layers if isinstance(l.mixer, GeneralDelta))

    def allocate_cache(self, num_blocks, block_size, num_slots, device):
        """A key and a value cache per attention layer (all layers share the sequences' block tables); per state slot
        one token-shift row per layer and one float32 delta-rule state per recurrent layer."""
        self.num_slots = num_slots
        shift = torch.zeros(num_slots, len(self.layers), self.cfg.hidden_size, dtype=self.dtype, device=device)
        for layer in self.layers:
            layer.shift.state = shift
            if isinstance(layer.mixer, PagedRotaryAttention):
                layer.mixer.allocate(num_blocks, block_size, self.dtype, device)
            else:
                layer.mixer.allocate(num_slots, device)

    def workspaces(self):
        from nanovllm import _hymix
        return [_hymix.decode_workspace]

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids, positions, trace=None):
        """input_ids int64 [T], positions int32 [T] (the step's context is seq_ops.get_step()) -> final-normed hidden
        [T, width].  ``trace``: a list that receives the residual after every layer (debugging)."""
        cfg, dt = self.cfg, self.dtype
        eps, mult = cfg.norm_eps, cfg.residual_mult
        ctx = seq_ops.get_step()
        x = hy_ops.embed_scaled(input_ids, self.embed, cfg.embedding_scale)
        h = hy_ops.sublayer_close(x, None, None, None, None, mult, self.layers[0].port1.norm, eps, dt)
        v_first = None
        n = len(self.layers)
        for i, layer in enumerate(self.layers):
            port = layer.port1
            gate = F.linear(h, port.gate_weight)
            hs = layer.shift(h, i)
            if isinstance(layer.mixer, PagedRotaryAttention):
                y, v_own = layer.mixer(hs, v_first if i != self.v_source else None)
                if i == self.v_source:
                    v_first = v_own
            else:
                y = layer.mixer(hs)
            carry = (h, layer.shift.state, i, ctx)         # this layer's shift reads h's last row at the next step
            if layer.mlp is not None:
                h = hy_ops.sublayer_close(x, y, gate, port.gate_bias, port.post_norm, mult, layer.port2.norm, eps, dt, carry)
                y, gate = layer.mlp(h)
                port, carry = layer.port2, None
            # the write of this layer's last sublayer and the norm in front of the next layer's first, in one launch
            next_w = self.layers[i + 1].port1.norm if i + 1 < n else self.final_norm
            h = hy_ops.sublayer_close(x, y, gate, port.gate_bias, port.post_norm, mult, next_w, eps, dt, carry)
            if trace is not None:
                trace.append(x.clone())
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
