"""Model architecture configs.

The reference delegates all model execution to vLLM pods; the
model families its configs pin are Llama-class dense transformers
(`examples/poc/manifests/vllm/vllm-lora-deployment.yaml`: Llama-2-7b) and —
per BASELINE.json — Llama-3-8B, Llama-3-70B (TP=4) and Mixtral 8x7B.  These
presets are random-init shapes (no network ⇒ no checkpoints); weights are
initialised randomly and the benchmark is synthetic-data.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass
class LayerSpec:
    """One layer of a heterogeneous (hybrid) stack: which sequence mixer it
    has ('attention' and 'attention_2' keep paged K/V, 'mingru' keeps a recurrent state
    vector), the mixer's sizes and constants, and its feed-forward (None for
    a layer without one).  'latent_attention' keeps one paged row per token
    (the normalised key/value latent followed by the shared rotated key
    part).  'wkv' keeps a matrix state per head and the previous token's
    input row; 'parallel' keeps paged K/V for its attention branch and a
    matrix state per head for its recurrent branch.  `shift` says the mixer's input is blended with the previous
    token's, which costs one fp32 row of model width per sequence."""

    type: str
    mixer: Dict[str, Any] = field(default_factory=dict)
    mlp: Optional[Dict[str, Any]] = None
    shift: bool = False


@dataclass
class ModelConfig:
    name: str
    # Model family; selects the model class and config reader
    # (models/registry.py).
    architecture: str = "llama"
    vocab_size: int = 128256
    hidden_size: int = 4096
    num_layers: int = 32
    num_heads: int = 32
    num_kv_heads: int = 8
    intermediate_size: int = 14336
    head_dim: int = 128
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    max_position_embeddings: int = 8192
    tie_word_embeddings: bool = False
    # MoE (Mixtral-style); num_experts == 0 means dense.
    num_experts: int = 0
    num_experts_per_tok: int = 2
    # Multi-GPU MoE mode: False = TP-shard every expert's intermediate dim;
    # True = expert parallelism (each rank owns num_experts/world full
    # experts; models/mixtral.py MoEBlock docstring).
    expert_parallel: bool = False
    dtype: str = "bfloat16"
    # Heterogeneous stacks: per-layer specs (None = num_layers identical
    # Llama-style layers), and the number of equal parts the RMS norms split
    # a row into (1 = ordinary RMS norm).
    layer_specs: Optional[List[LayerSpec]] = None
    norm_groups: int = 1
    # Weight-shared loop over a span of layers: (start, stop, times) runs
    # layers start..stop-1 `times` times in a row; every run of a layer has
    # its own cache and state.  None = every layer runs once.
    layer_loop: Optional[Tuple[int, int, int]] = None
    # Folder with config.json + model.safetensors ("" = random init).
    weights_path: str = ""
    # Post-norm stacks: x <- norm(residual_alpha * x + sublayer(x)).
    residual_alpha: float = 1.0
    # logits <- cap * tanh(logits / cap); 0 = no cap.
    logit_softcap: float = 0.0
    # Pre-norm stacks with a scaled branch: x <- x + residual_mult * sublayer(norm(x)).
    residual_mult: float = 1.0
    # The residual as several parallel streams that sub-layers read through a
    # weighted sum and write through a mixing matrix (hyper_connections);
    # one stream without them is the ordinary residual.
    residual_streams: int = 1
    hyper_connections: bool = False

    @property
    def is_moe(self) -> bool:
        if self.layer_specs is not None:
            return any(s.mlp is not None and s.mlp.get("kind") == "moe" for s in self.layer_specs)
        return self.num_experts > 0

    def layer_run_order(self) -> List[int]:
        """Layer indices in the order they execute (a looped span repeats)."""
        n = len(self.layer_specs) if self.layer_specs is not None else self.num_layers
        if self.layer_loop is None:
            return list(range(n))
        a, b, times = self.layer_loop
        return list(range(a)) + list(range(a, b)) * times + list(range(b, n))

    @property
    def kv_bytes_per_token_per_layer(self) -> int:
        # K + V, bf16.
        return 2 * self.num_kv_heads * self.head_dim * 2

    def kv_elems_per_token(self, tp_size: int = 1) -> int:
        """K+V elements one token occupies across all layers that keep a
        paged cache (recurrent layers keep none)."""
        if self.layer_specs is None:
            return self.num_layers * 2 * (self.num_kv_heads // tp_size) * self.head_dim
        total = 0
        for i in self.layer_run_order():
            s = self.layer_specs[i]
            if s.type in ("attention", "attention_2"):
                total += (s.mixer["kv_heads"] // tp_size) * (s.mixer["dim"] + s.mixer["vdim"])
            elif s.type == "latent_attention":
                total += s.mixer["kv_rank"] + s.mixer["rot_dim"]
            elif s.type == "parallel":
                # the attention branch caches normed keys and, as values, the
                # keys as projected
                left = s.mixer["left"]
                total += (left["kv_heads"] // tp_size) * 2 * left["dim"]
        return total

    def state_elems_per_seq(self) -> int:
        """fp32 recurrent-state elements one live sequence occupies."""
        if self.layer_specs is None:
            return 0
        total = 0
        for i in self.layer_run_order():
            s = self.layer_specs[i]
            if s.type == "mingru":
                total += s.mixer["width"]
            elif s.type == "wkv":
                # previous token's input row + one matrix per head
                total += self.hidden_size + s.mixer["heads"] * s.mixer["dim"] ** 2
            elif s.type == "parallel":
                right = s.mixer["right"]
                total += right["heads"] * right["dim"] * right["vdim"]
            if s.shift:
                total += self.hidden_size
        return total

    @property
    def has_recurrent_state(self) -> bool:
        return self.state_elems_per_seq() > 0

    def num_params(self) -> int:
        """Approximate parameter count (dense path)."""
        h, i, v = self.hidden_size, self.intermediate_size, self.vocab_size
        kv = self.num_kv_heads * self.head_dim
        q = self.num_heads * self.head_dim
        attn = h * q + 2 * h * kv + q * h
        if self.is_moe:
            mlp = 3 * h * i * self.num_experts + h * self.num_experts
        else:
            mlp = 3 * h * i
        per_layer = attn + mlp + 2 * h
        emb = v * h * (1 if self.tie_word_embeddings else 2)
        return self.num_layers * per_layer + emb + h


LLAMA3_8B = ModelConfig(name="llama3-8b")

LLAMA3_70B = ModelConfig(
    name="llama3-70b",
    hidden_size=8192,
    num_layers=80,
    num_heads=64,
    num_kv_heads=8,
    intermediate_size=28672,
)

MIXTRAL_8X7B = ModelConfig(
    name="mixtral-8x7b",
    vocab_size=32000,
    hidden_size=4096,
    num_layers=32,
    num_heads=32,
    num_kv_heads=8,
    intermediate_size=14336,
    rope_theta=1e6,
    num_experts=8,
    num_experts_per_tok=2,
)

# 70B-shaped tiny: keeps every ratio TP=4 sharding depends on (64 q heads /
# 8 kv heads GQA grouping, 3.5x intermediate, separate lm_head) at CPU-test
# dims — the 4-rank gloo token-identity test for BASELINE config #4 runs on
# this shape.
TINY_70B = ModelConfig(
    name="tiny-70b",
    vocab_size=512,
    hidden_size=128,
    num_layers=2,
    num_heads=64,
    num_kv_heads=8,
    intermediate_size=448,
    head_dim=16,
    max_position_embeddings=512,
)

# Tiny shapes for CPU tests and smoke runs.
TINY = ModelConfig(
    name="tiny",
    vocab_size=512,
    hidden_size=64,
    num_layers=2,
    num_heads=4,
    num_kv_heads=2,
    intermediate_size=128,
    head_dim=16,
    max_position_embeddings=512,
)

TINY_MOE = ModelConfig(
    name="tiny-moe",
    vocab_size=512,
    hidden_size=64,
    num_layers=2,
    num_heads=4,
    num_kv_heads=2,
    intermediate_size=128,
    head_dim=16,
    max_position_embeddings=512,
    num_experts=4,
    num_experts_per_tok=2,
)

PRESETS = {
    "llama3-8b": LLAMA3_8B,
    "llama3-70b": LLAMA3_70B,
    "tiny-70b": TINY_70B,
    "mixtral-8x7b": MIXTRAL_8X7B,
    "tiny": TINY,
    "tiny-moe": TINY_MOE,
}


def get_model_config(name: str) -> ModelConfig:
    """A preset by name, or a model folder (config.json picks the family)."""
    import os

    if name not in PRESETS and os.path.isfile(os.path.join(name, "config.json")):
        from .registry import config_from_dir

        return config_from_dir(name)
    if name not in PRESETS:
        raise KeyError(f"unknown model preset {name!r}; have {sorted(PRESETS)}")
    return PRESETS[name]
