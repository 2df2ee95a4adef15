"""Potatar: a decoder-only stack with the norm AFTER the residual sum.

config.json lists the layers.  A sub-layer reads the residual itself and the
norm follows the sum,

    x <- norm1(alpha * x + mixer(x));   x <- norm2(alpha * x + ff(x))

with one constant alpha for the whole model; a layer may have no
feed-forward.  The residual stream x is fp32 in every mode; the GEMMs read
its rounding to the activation dtype, which the norm kernel writes alongside.

Mixers:
  * "attention": grouped-query softmax attention; q and k are RMS-normed
    over the whole projection, partially rotated (rotate-half pairs), the
    values are unit-RMS per head; a query sees the keys of its own chunk of
    positions.  Layers with value mixing blend their values with those of
    the first such layer (same tokens) before caching them.
  * "wkv": a matrix-state recurrence with token shift, data-dependent
    per-channel decay and a bonus for the current token.
  * "parallel": two mixers read the same input and their outputs are added
    with fixed scales: softmax attention whose values are its keys, with
    per-head q/k norms, a learned distance bias and scores mixed across
    heads; and linear attention with a constant decay per head.

The feed-forward is down(gelu(up h)); the logits are soft-capped with tanh.

Execution on the engine's flat batch: per sub-layer the fused input GEMM(s),
one prep kernel, the attention or scan kernel, the output GEMM, then one
kernel for sum + norm that also emits the next GEMM's input.
"""

from __future__ import annotations

import os
from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from .config import LayerSpec, ModelConfig
from .hybrid_blocks import GeluMLP, MatrixStateMixer, NormedRotaryAttention, _param

MIXERS = ("attention", "wkv", "parallel")


def config_from_json(raw: dict, path: str = "") -> ModelConfig:
    specs: List[LayerSpec] = []
    # sizes that only the tensors' shapes give: the rank of the decay's
    # low-rank pair and the rows of the distance table
    shapes = {}
    ckpt = os.path.join(path, "model.safetensors") if path else ""
    if ckpt and os.path.isfile(ckpt):
        from .loader import read_safetensors_shapes

        shapes = read_safetensors_shapes(ckpt)
    for i, entry in enumerate(raw["layers"]):
        t = entry["type"]
        if t not in MIXERS:
            raise ValueError(f"layer {i}: unknown mixer type {t!r}")
        mlp = entry.get("mlp")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
        mixer = dict(entry["mixer"])
        if t == "wkv" and f"l{i}.mix.w1" in shapes:
            mixer["decay_rank"] = shapes[f"l{i}.mix.w1"][0]
        if t == "parallel":
            mixer["left"] = dict(mixer["left"])
            if f"l{i}.mix.left.rel" in shapes:
                mixer["left"]["bias_rows"] = shapes[f"l{i}.mix.left.rel"][0]
        specs.append(LayerSpec(type=t, mixer=mixer, mlp=None if mlp is None else dict(mlp)))
    cap = raw.get("logit_softcap")
    return ModelConfig(
        name=os.path.basename(os.path.normpath(path)) or "potatar",
        architecture="potatar",
        vocab_size=int(raw["vocab"]),
        hidden_size=int(raw["width"]),
        num_layers=len(specs),
        rms_norm_eps=float(raw["norm"]["eps"]),
        layer_specs=specs,
        weights_path=path,
        residual_alpha=float(raw.get("postln_alpha", 1.0)),
        logit_softcap=float(cap) if cap else 0.0,
        # angles are computed from the position itself: no table bounds the
        # context
        max_position_embeddings=1 << 30,
    )


def make_config(
    name: str, vocab: int, width: int, layers: List[dict], eps: float = 1e-5,
    alpha: float = 1.0, softcap: float = 0.0,
) -> ModelConfig:
    """A random-init config from the same fields config.json carries."""
    cfg = config_from_json(
        {"vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps},
         "postln_alpha": alpha, "logit_softcap": softcap}
    )
    cfg.name = name
    return cfg


def _attention(hidden: int, m: dict, eps: float, device, dtype) -> NormedRotaryAttention:
    rot = m.get("rot") or {}
    return NormedRotaryAttention(
        hidden, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], eps,
        qk_norm="row", rot_base=rot.get("base", 10000.0), rot_dims=int(rot.get("dims", 0)),
        chunk=int((m.get("mask") or {}).get("size", 0)), values="proj", v_unit_norm=True,
        bias=True, device=device, dtype=dtype,
    )


class PotatarLayer(nn.Module):
    def __init__(self, spec: LayerSpec, hidden: int, eps: float, device, dtype) -> None:
        super().__init__()
        m = spec.mixer
        self.type = spec.type
        self.v_mix = False
        if spec.type == "attention":
            self.mixer = _attention(hidden, m, eps, device, dtype)
            self.v_mix = bool(m.get("v_mix"))
        elif spec.type == "wkv":
            self.mixer = MatrixStateMixer(
                hidden, "wkv", m["heads"], m["dim"], m["dim"], eps,
                decay_rank=int(m.get("decay_rank", 32)), device=device, dtype=dtype,
            )
        else:
            lm, rm = m["left"], m["right"]
            self.left = NormedRotaryAttention(
                hidden, lm["heads"], lm["kv_heads"], lm["dim"], lm.get("vdim", lm["dim"]),
                lm["scale"], eps, qk_norm="head", rot_dims=0,
                chunk=int((lm.get("mask") or {}).get("size", 0)), values="key", bias=True,
                dist_rows=int(lm.get("bias_rows", 32)), dist_far=float(lm["bias_max"]),
                talk=True, device=device, dtype=dtype,
            )
            self.right = MatrixStateMixer(
                hidden, "decay", rm["heads"], rm["dim"], rm["vdim"], eps, decay=rm["decay"],
                device=device, dtype=dtype,
            )
            self.left_scale, self.right_scale = float(m["left_scale"]), float(m["right_scale"])
            self.w_in: Optional[torch.Tensor] = None
            self.b_in: Optional[torch.Tensor] = None
            self.fuse_inputs()
        self.norm1 = _param((hidden,), device, dtype, None)
        self.mlp: Optional[GeluMLP] = None
        if spec.mlp is not None:
            self.mlp = GeluMLP(hidden, spec.mlp["ff"], device=device, dtype=dtype)
            self.norm2 = _param((hidden,), device, dtype, None)
        with torch.no_grad():
            self.norm1.fill_(1.0)
            if self.mlp is not None:
                self.norm2.fill_(1.0)

    def fuse_inputs(self) -> None:
        """One GEMM for both branches of a parallel mixer: rows [left q | left
        k | right q | right k | right v | right gate]; the right branch has
        no biases."""
        l, r = self.left, self.right
        self.w_in = torch.cat([l.w_in.data, r.w_in.data], dim=0).contiguous()
        self.b_in = torch.cat([l.b_in.data, torch.zeros_like(r.w_in.data[:, 0])], dim=0).contiguous()

    def cache_spec(self):
        if self.type == "parallel":
            return [self.left.cache_spec(), self.right.cache_spec()]
        return self.mixer.cache_spec()


class PotatarForCausalLM(nn.Module):
    # the runner builds per-token sequence tables and per-sequence segments
    needs_seq_tables = True
    # no adapter hooks in the mixers: base model only
    supports_lora = False
    # single-token steps have static shapes and no host round trip
    supports_decode_graphs = True

    def __init__(self, cfg: ModelConfig, device="cpu", dtype=torch.bfloat16, tp=None) -> None:
        super().__init__()
        if tp is not None and tp.world_size > 1:
            raise NotImplementedError("Potatar runs on one GPU per engine (no tensor parallelism)")
        assert cfg.layer_specs, "Potatar needs per-layer specs"
        self.cfg = cfg
        self.device_ = torch.device(device)
        self.dtype_ = dtype
        H, V = cfg.hidden_size, cfg.vocab_size
        self.embed = _param((V, H), device, dtype, 1.0)
        self.final_norm = _param((H,), device, dtype, None)
        with torch.no_grad():
            self.final_norm.fill_(1.0)
        self.head = _param((V, H), device, dtype, 1.0 / (H ** 0.5))
        self.layers = nn.ModuleList(
            [PotatarLayer(s, H, cfg.rms_norm_eps, device, dtype) for s in cfg.layer_specs]
        )
        # the first layer with value mixing provides the values the later
        # ones blend in
        self.v_source = next((i for i, l in enumerate(self.layers) if l.v_mix), -1)
        self.v_users = sum(1 for l in self.layers if l.v_mix)
        # prompt rows of the attention layers (plain and head-mixed) run MFMA
        # tile kernels where the shapes allow: the runner then builds 64-row
        # tiles
        on_gpu = self.device_.type == "cuda"
        self.needs_prefill_tiles = any(
            (
                s.type == "attention"
                and ops.tiled_prefill_supported(dtype, s.mixer["dim"], s.mixer["vdim"], on_gpu)
            )
            or (
                s.type == "parallel"
                and ops.mixed_heads_tiles_supported(
                    dtype, s.mixer["left"]["dim"], s.mixer["left"]["dim"],
                    s.mixer["left"]["heads"], on_gpu,
                )
            )
            for s in cfg.layer_specs
        )
        # test/debug hook: when a list, forward() appends the fp32 residual
        # stream after every layer
        self.capture_residuals: Optional[list] = None

    def decode_attention_shape(self):
        return None  # no layer uses the split paged-decode kernel

    def cache_specs(self) -> List:
        return [layer.cache_spec() for layer in self.layers]

    def load_weights(self, tensors) -> None:
        used = set()

        def get(name: str) -> torch.Tensor:
            if name not in tensors:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            used.add(name)
            return tensors[name].to(device=self.device_, dtype=self.dtype_)

        with torch.no_grad():
            self.embed.copy_(get("embed"))
            self.final_norm.copy_(get("final.norm"))
            self.head.copy_(get("head"))
            for i, layer in enumerate(self.layers):
                p = f"l{i}."
                layer.norm1.copy_(get(p + "norm1"))
                if layer.type == "parallel":
                    layer.left.load(get, p + "mix.left.")
                    layer.right.load(get, p + "mix.right.")
                    layer.fuse_inputs()
                else:
                    layer.mixer.load(get, p + "mix.")
                    if layer.type == "attention":
                        # stored for every attention layer; only the layers
                        # after the first value-mixing one use theirs
                        lam = float(tensors[p + "mix.vmix"].float()) if p + "mix.vmix" in tensors else 0.0
                        used.add(p + "mix.vmix")
                        layer.mixer.lam = lam
                if layer.mlp is not None:
                    layer.norm2.copy_(get(p + "norm2"))
                    layer.mlp.load(get, p + "mlp.")
        extra = sorted(set(tensors) - used)
        if extra:
            raise ValueError(f"checkpoint tensors the model does not know: {extra[:8]}")

    def forward(self, input_ids, positions, kv_caches, meta) -> torch.Tensor:
        cfg = self.cfg
        eps, alpha = cfg.rms_norm_eps, cfg.residual_alpha
        h = self.embed.index_select(0, input_ids)  # activation dtype
        x = h.float()                              # the residual, fp32
        v_first = None
        for i, layer in enumerate(self.layers):
            cache = kv_caches[i]
            if layer.type == "attention":
                if layer.v_mix and i == self.v_source and self.v_users > 1:
                    y, v_first = layer.mixer(h, positions, cache, meta, want_v=True)
                else:
                    y = layer.mixer(
                        h, positions, cache, meta, v_first=v_first if layer.v_mix else None
                    )
                x, h = ops.scaled_add_rms_norm(x, alpha, layer.norm1, eps, y)
            elif layer.type == "wkv":
                y = layer.mixer(x, h, cache, meta)
                x, h = ops.scaled_add_rms_norm(x, alpha, layer.norm1, eps, y)
            else:
                proj = F.linear(h, layer.w_in, layer.b_in)
                yl = layer.left(h, positions, cache[:2], meta, proj=proj)
                yr = layer.right(x, h, cache[2:], meta, proj=proj[:, layer.left.n_in :])
                x, h = ops.scaled_add_rms_norm(
                    x, alpha, layer.norm1, eps, yl, layer.left_scale, yr, layer.right_scale
                )
            if layer.mlp is not None:
                x, h = ops.scaled_add_rms_norm(x, alpha, layer.norm2, eps, layer.mlp(h))
            if self.capture_residuals is not None:
                self.capture_residuals.append(x.clone())
        _, hn = ops.scaled_add_rms_norm(x, 1.0, self.final_norm, eps)
        return hn

    def compute_logits(self, hidden: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
        z = (hidden[indices] @ self.head.t()).float()
        if self.cfg.logit_softcap > 0.0:
            z = ops.tanh_softcap(z.contiguous(), self.cfg.logit_softcap)
        return z
