import json
import os
from dataclasses import dataclass
from types import SimpleNamespace
from typing import Callable, Optional

import torch


def load_hf_config(model_dir: str) -> SimpleNamespace:
    """config.json -> attribute namespace (no dependency on a particular transformers version)."""
    with open(os.path.join(model_dir, "config.json")) as f:
        d = json.load(f)
    from nanovllm.models import registry
    arch = registry.architecture_of(d)
    normalize = getattr(registry.model_class(arch), "normalize_config", None)
    if normalize is not None:
        # a model family with its own config.json layout brings it to the fields the engine reads
        d = normalize(d)
        d["architecture_name"] = arch
        dt = d.get("torch_dtype", "bfloat16")
        d["torch_dtype"] = getattr(torch, dt) if isinstance(dt, str) else dt
        return SimpleNamespace(**d)
    d["architecture_name"] = arch
    rope_theta = d.get("rope_theta")
    if rope_theta is None:
        rope_theta = (d.get("rope_parameters") or {}).get("rope_theta", 1000000.0)
    d["rope_theta"] = rope_theta
    d.setdefault("head_dim", d["hidden_size"] // d["num_attention_heads"])
    d.setdefault("attention_bias", False)
    d.setdefault("tie_word_embeddings", False)
    d.setdefault("rms_norm_eps", 1e-6)
    d.setdefault("hidden_act", "silu")
    d.setdefault("max_position_embeddings", 40960)
    dt = d.get("torch_dtype", d.get("dtype", "bfloat16"))
    d["torch_dtype"] = getattr(torch, dt) if isinstance(dt, str) else dt
    return SimpleNamespace(**d)


@dataclass
class Config:
    """The reference's Config (nanovllm/config.py:9-35) plus ``load_format``: "auto" reads *.safetensors
    and quantizes as configured; "dummy" random-initialises the weights on the GPU (the benchmark has no
    checkpoint to read); "quantized" reads a pre-quantized checkpoint written by
    nanovllm.utils.checkpoint.save_quantized (its quant_config.json overrides quant_type / linear_dtype)."""
    model: str
    max_num_batched_tokens: int = 16384
    max_num_seqs: int = 512
    max_model_len: int = 4096
    gpu_memory_utilization: float = 0.9
    tensor_parallel_size: int = 1
    enforce_eager: bool = False
    hf_config: Optional[SimpleNamespace] = None
    eos: int = -1
    kvcache_block_size: int = 0        # 0 = the model family's own (256 for the paged K/V cache, 64 for latent caches)
    num_kvcache_blocks: int = -1
    linear_dtype: torch.dtype = torch.bfloat16
    weight_quant_fn: Optional[Callable[[torch.Tensor], torch.Tensor]] = None
    quant_type: Optional[str] = None   # "per_tensor", "per_row", "per_group", "per_row_weight_only"
    group_size: int = 128
    load_format: str = "auto"
    # opt-in, off by default because it changes the logits the reference computes in bf16: the vocabulary
    # projection (311 MB of bf16 per decode step for Qwen3-0.6B) as a per-row weight-only quantized linear
    quantize_lm_head: bool = False
    # "cuda" = the product path (HIP kernels).  "cpu" = plumbing only: the UNQUANTIZED model with plain torch
    # operators, eager, for checking engine wiring on a host without a GPU; every quantized option is refused there.
    device: str = "cuda"
    # compute and storage type of the model; None = what config.json says (bfloat16 if it says nothing)
    dtype: Optional[torch.dtype] = None
    # models that are stepped with portions of sequences (prompt pieces beside decoded tokens in one batch):
    # the most tokens of one sequence in one step (0 = only the step's token budget limits a portion)
    prefill_chunk: int = 0

    def __post_init__(self):
        assert os.path.isdir(self.model), f"{self.model} is not a directory"
        assert 1 <= self.tensor_parallel_size <= 8
        self.hf_config = load_hf_config(self.model)
        if self.dtype is not None:
            self.hf_config.torch_dtype = self.dtype
        from nanovllm.models import registry
        cls = registry.model_class(self.hf_config.architecture_name)
        self.runs_portions = bool(getattr(cls, "runs_portions", False))
        if self.kvcache_block_size == 0:
            self.kvcache_block_size = getattr(cls, "default_block_size", 256)
        assert self.kvcache_block_size % (64 if self.runs_portions else 256) == 0
        self.max_model_len = min(self.max_model_len, self.hf_config.max_position_embeddings)
        # (a model stepped with portions cuts a long prompt over several steps)
        assert self.runs_portions or self.max_num_batched_tokens >= self.max_model_len
        if self.runs_portions:
            assert self.tensor_parallel_size == 1, "this model family runs on one GPU"
            assert self.quant_type is None and self.weight_quant_fn is None and self.load_format != "quantized", \
                "the quantized linears are wired into the Qwen3 decoder only"
        assert self.device in ("cuda", "cpu")
        if self.device == "cpu":
            quantized = (self.quant_type is not None or self.weight_quant_fn is not None or self.quantize_lm_head or
                         self.linear_dtype != torch.bfloat16 or self.load_format == "quantized")
            assert not quantized, "the quantized-linear path is HIP only: device='cpu' runs the unquantized model"
            assert self.tensor_parallel_size == 1
            self.enforce_eager = True
        if self.hf_config.__dict__.get("eos_token_id") is not None and self.eos == -1:
            e = self.hf_config.eos_token_id
            self.eos = e[0] if isinstance(e, (list, tuple)) else e
