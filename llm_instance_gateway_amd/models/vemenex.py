"""Vemenex: a pre-norm decoder whose residual is kept as several streams.

config.json lists the layers.  Every norm has ONE weight for all
coordinates.  The residual is S parallel fp32 streams, all equal to the
normed embedding at the start; a sub-layer reads a weighted sum of the
streams and writes through a mixing matrix ("hyper-connections"):

    u = sum_s in[s] x_s;  y = sublayer(norm(u));
    x_t <- sum_s mix[s, t] x_s + m * out[t] * y      (all t at once)

with one constant m for the whole model.  A checkpoint without such tensors
runs the ordinary residual x <- x + m * sublayer(norm(x)) through the same
kernel (one stream, unit coefficients).  The model's output is the sum of
the streams, normed, times the head.

Mixers (both sliding-window grouped-query attention over paged K/V, q and k
divided per head by their root mean square after a partial rotation):
  * "attention": interleaved rotation pairs with linear position scaling;
    every visible key weighs sigmoid(score + per-head bias), unnormalised.
  * "attention_2": rotate-half pairs; softmax with a zero-score sink in the
    denominator; one sigmoid output gate per head.

Feed-forward: down(relu(gate h) * up h), or routed clamped-gate experts with
a softmax router, correction offsets, group-limited choice and identity
experts; a layer may have none.

Execution on the engine's flat batch: per sub-layer one `hyper_step` kernel
(the previous sub-layer's write fused with this one's read and norm), the
fused input GEMM, one prep kernel (rotation, norms, cache write), the
attention kernel, the output GEMM.
"""

from __future__ import annotations

import os
from typing import List, Optional

import torch
import torch.nn as nn

from .. import ops
from .config import LayerSpec, ModelConfig
from .hybrid_blocks import GatedReluMLP, GroupRoutedExpertsMLP, NormedRotaryAttention, _param

MIXERS = ("attention", "attention_2")


def config_from_json(raw: dict, path: str = "") -> ModelConfig:
    specs: List[LayerSpec] = []
    for i, entry in enumerate(raw["layers"]):
        t = entry["type"]
        if t not in MIXERS:
            raise ValueError(f"layer {i}: unknown mixer type {t!r}")
        mlp = entry.get("mlp")
        if mlp is not None and mlp.get("kind", "dense") not in ("dense", "moe"):
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
        specs.append(
            LayerSpec(type=t, mixer=dict(entry["mixer"]), mlp=None if mlp is None else dict(mlp))
        )
    # hyper-connections exist when the checkpoint carries their tensors; a
    # config without a checkpoint (random init) has them when it names streams
    hyper = "streams" in raw
    ckpt = os.path.join(path, "model.safetensors") if path else ""
    if ckpt and os.path.isfile(ckpt):
        from .loader import read_safetensors_shapes

        hyper = any(k.endswith(".hc1.in") for k in read_safetensors_shapes(ckpt))
    return ModelConfig(
        name=os.path.basename(os.path.normpath(path)) or "vemenex",
        architecture="vemenex",
        vocab_size=int(raw["vocab"]),
        hidden_size=int(raw["width"]),
        num_layers=len(specs),
        rms_norm_eps=float(raw["norm"]["eps"]),
        layer_specs=specs,
        weights_path=path,
        residual_mult=float(raw.get("residual_mult", 1.0)),
        residual_streams=int(raw.get("streams", 1)) if hyper else 1,
        hyper_connections=hyper,
        # angles are computed from the position itself: no table bounds the
        # context
        max_position_embeddings=1 << 30,
    )


def make_config(
    name: str, vocab: int, width: int, layers: List[dict], eps: float = 1e-6,
    residual_mult: float = 1.0, streams: Optional[int] = None,
) -> ModelConfig:
    """A random-init config from the same fields config.json carries
    (streams None: ordinary residual)."""
    raw = {"vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps},
           "residual_mult": residual_mult}
    if streams is not None:
        raw["streams"] = streams
    cfg = config_from_json(raw)
    cfg.name = name
    return cfg


def _attention(kind: str, hidden: int, m: dict, eps: float, device, dtype) -> NormedRotaryAttention:
    rot = m.get("rot") or {}
    sigmoid = kind == "attention"
    return NormedRotaryAttention(
        hidden, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], eps,
        qk_norm="head_post", rot_base=float(rot.get("base", 10000.0)),
        rot_dims=int(rot.get("dims", 0)),
        rot_layout="interleaved" if sigmoid else "half",
        rot_scale=float((rot.get("scaling") or {}).get("factor", 1.0)),
        window=int((m.get("mask") or {}).get("size", 0)), bias=False,
        weights="sigmoid" if sigmoid else "softmax", score_bias=sigmoid,
        sink=not sigmoid, head_gate=not sigmoid, device=device, dtype=dtype,
    )


def _feed_forward(hidden: int, mlp: dict, device, dtype):
    if mlp.get("kind", "dense") == "dense":
        return GatedReluMLP(hidden, int(mlp["ff"]), device=device, dtype=dtype)
    r = mlp["router"]
    grp = r.get("groups") or {}
    return GroupRoutedExpertsMLP(
        hidden, int(mlp["expert"]["ff"]), int(r["experts"]), int(r["top"]),
        identity=int(r.get("identity", 0)), groups=int(grp.get("count", 1)),
        keep=int(grp.get("keep", grp.get("count", 1))), limit=float(mlp["expert"]["limit"]),
        device=device, dtype=dtype,
    )


class StreamPort(nn.Module):
    """How one sub-layer reads from and writes to the S residual streams, and
    the single weight of the norm on its input.  fp32 whatever the activation
    dtype: they enter the residual sum."""

    def __init__(self, streams: int, device) -> None:
        super().__init__()
        S = streams
        f = dict(device=device, dtype=torch.float32)
        self.w_in = nn.Parameter(torch.full((S,), 1.0 / S, **f), requires_grad=False)
        self.w_out = nn.Parameter(torch.ones(S, **f), requires_grad=False)
        self.mix = nn.Parameter(torch.eye(S, **f), requires_grad=False)
        self.g = nn.Parameter(torch.ones(1, **f), requires_grad=False)

    def randomize(self) -> None:
        with torch.no_grad():
            self.w_in.uniform_(0.2, 0.8)
            self.w_out.uniform_(0.5, 1.5)
            self.mix.add_(torch.empty_like(self.mix).uniform_(-0.2, 0.2))
            self.g.uniform_(0.7, 1.3)


class VemenexLayer(nn.Module):
    def __init__(self, spec: LayerSpec, hidden: int, eps: float, streams: int, device, dtype) -> None:
        super().__init__()
        self.type = spec.type
        self.mixer = _attention(spec.type, hidden, spec.mixer, eps, device, dtype)
        self.port1 = StreamPort(streams, device)
        self.mlp = None
        self.port2: Optional[StreamPort] = None
        if spec.mlp is not None:
            self.mlp = _feed_forward(hidden, spec.mlp, device, dtype)
            self.port2 = StreamPort(streams, device)


class VemenexForCausalLM(nn.Module):
    # the runner builds per-token sequence tables and per-sequence segments
    needs_seq_tables = True
    # no adapter hooks in the mixers: base model only
    supports_lora = False
    # single-token steps have static shapes and no host round trip
    supports_decode_graphs = True

    def __init__(self, cfg: ModelConfig, device="cpu", dtype=torch.bfloat16, tp=None) -> None:
        super().__init__()
        if tp is not None and tp.world_size > 1:
            raise NotImplementedError("Vemenex runs on one GPU per engine (no tensor parallelism)")
        assert cfg.layer_specs, "Vemenex needs per-layer specs"
        self.cfg = cfg
        self.device_ = torch.device(device)
        self.dtype_ = dtype
        H, V = cfg.hidden_size, cfg.vocab_size
        self.streams = cfg.residual_streams
        self.embed = _param((V, H), device, dtype, 1.0)
        # the embedding norm's single weight, spread over the row for the
        # gather + norm kernel
        self.embed_norm = _param((H,), device, dtype, None)
        with torch.no_grad():
            self.embed_norm.fill_(1.0)
        self.head = _param((V, H), device, dtype, 1.0 / (H ** 0.5))
        self.layers = nn.ModuleList(
            [VemenexLayer(s, H, cfg.rms_norm_eps, self.streams, device, dtype) for s in cfg.layer_specs]
        )
        # the output reads the plain sum of the streams
        self.final_port = StreamPort(self.streams, device)
        with torch.no_grad():
            self.final_port.w_in.fill_(1.0)
        if not cfg.weights_path and cfg.hyper_connections:
            for layer in self.layers:
                layer.port1.randomize()
                if layer.port2 is not None:
                    layer.port2.randomize()
        on_gpu = self.device_.type == "cuda"
        self.needs_prefill_tiles = any(
            ops.tiled_prefill_supported(dtype, s.mixer["dim"], s.mixer["vdim"], on_gpu)
            for s in cfg.layer_specs
        )
        # test/debug hook: when a list, forward() appends the fp32 sum of the
        # streams after every layer
        self.capture_residuals: Optional[list] = None

    def decode_attention_shape(self):
        return None  # no layer uses the split paged-decode kernel

    def cache_specs(self) -> List:
        return [layer.mixer.cache_spec() for layer in self.layers]

    def load_weights(self, tensors) -> None:
        used = set()

        def get(name: str) -> torch.Tensor:
            if name not in tensors:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            used.add(name)
            return tensors[name].to(device=self.device_, dtype=self.dtype_)

        def scalar(name: str) -> torch.Tensor:
            return get(name).float().reshape(1)

        def port(p: StreamPort, prefix: str, norm: str) -> None:
            p.g.copy_(scalar(norm))
            if self.cfg.hyper_connections:
                p.w_in.copy_(get(prefix + "in").float())
                p.w_out.copy_(get(prefix + "out").float())
                p.mix.copy_(get(prefix + "mix").float())
            else:
                p.w_in.fill_(1.0)
                p.w_out.fill_(1.0)
                p.mix.fill_(1.0)

        with torch.no_grad():
            self.embed.copy_(get("embed"))
            self.embed_norm.copy_(get("embed.norm").reshape(1).expand(self.cfg.hidden_size))
            self.final_port.g.copy_(scalar("final.norm"))
            self.head.copy_(get("head"))
            for i, layer in enumerate(self.layers):
                p = f"l{i}."
                layer.mixer.load(get, p + "mix.")
                port(layer.port1, p + "hc1.", p + "norm1")
                if layer.mlp is not None:
                    if isinstance(layer.mlp, GroupRoutedExpertsMLP):
                        layer.mlp.load(get, p + "mlp.", has=lambda n: n in tensors)
                    else:
                        layer.mlp.load(get, p + "mlp.")
                    port(layer.port2, p + "hc2.", p + "norm2")
        extra = sorted(set(tensors) - used)
        if extra:
            raise ValueError(f"checkpoint tensors the model does not know: {extra[:8]}")

    def forward(self, input_ids, positions, kv_caches, meta) -> torch.Tensor:
        cfg = self.cfg
        eps, m, dt = cfg.rms_norm_eps, cfg.residual_mult, self.dtype_
        x0 = ops.embed_group_norm(input_ids, self.embed, self.embed_norm, eps, 1)  # fp32
        xs = x0.unsqueeze(1).repeat(1, self.streams, 1)  # [R, S, W]
        y, done = None, None  # the last sub-layer's output and its port, not yet written

        def step(port: StreamPort):
            # the pending write and this sub-layer's read + norm in one pass
            if done is None:
                return ops.hyper_step(xs, None, None, None, m, port.w_in, port.g, eps, dt)
            return ops.hyper_step(xs, y, done.mix, done.w_out, m, port.w_in, port.g, eps, dt)

        for i, layer in enumerate(self.layers):
            h = step(layer.port1)
            y, done = layer.mixer(h, positions, kv_caches[i], meta), layer.port1
            if layer.mlp is not None:
                h = step(layer.port2)
                y, done = layer.mlp(h, meta), layer.port2
            if self.capture_residuals is not None:
                ops.hyper_step(xs, y, done.mix, done.w_out, m, None, None, eps, dt)
                y, done = None, None
                self.capture_residuals.append(xs.sum(dim=1))
        return step(self.final_port)

    def compute_logits(self, hidden: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
        return (hidden[indices] @ self.head.t()).float()
