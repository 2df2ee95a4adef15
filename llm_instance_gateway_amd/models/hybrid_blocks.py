"""Building blocks for hybrid stacks: layers whose sequence mixer is either
paged attention or a recurrence with a per-sequence state slot.

Every block works on the engine's flat token batch (prompt portions and
single decoded tokens side by side) and takes its constants as constructor
arguments, so another model family can assemble them differently.

  * `GatedAttention` — grouped-query attention with independent key and
    value head sizes, projection biases, a configurable score scale, an
    optional logarithmic query temperature and an optional sigmoid output
    gate; K/V live in the paged cache.
  * `MinGRU` — the minimal gated recurrent unit: gates read only the current
    token, the state is an fp32 vector per sequence in a slot pool.
  * `XieluMLP` — two-matrix feed-forward with the xIELU activation.
  * `LatentAttention`, `ReluSquaredMLP`, `ScoredExpertsMLP` — low-rank
    key/value attention and its feed-forwards.
  * `NormedRotaryAttention` — q/k norms before or after a partial rotation in
    either pair layout, chunked or sliding-window visibility, softmax (with
    an optional sink) or unnormalised sigmoid weights, distance bias, head
    mixing, per-head output gate.
  * `MatrixStateMixer`, `GeluMLP` — matrix-state recurrences.
  * `GatedReluMLP`, `GroupRoutedExpertsMLP` — gated feed-forward and routed
    experts with a softmax router, group-limited choice and identity experts.

Projections are library GEMMs over fused weights (one GEMM in, one out per
block); everything between them is one HIP kernel each (ops layer).
"""

from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops


def _param(shape, device, dtype, scale: Optional[float] = None) -> nn.Parameter:
    t = torch.empty(*shape, device=device, dtype=dtype)
    with torch.no_grad():
        if scale is None:
            t.zero_()
        else:
            t.uniform_(-scale, scale)
    return nn.Parameter(t, requires_grad=False)


def softplus64(x: float) -> float:
    return math.log1p(math.exp(-abs(x))) + max(x, 0.0)


class GatedAttention(nn.Module):
    def __init__(
        self, hidden: int, heads: int, kv_heads: int, dim: int, vdim: int,
        scale: float, temp_coef: float = 0.0, temp_every: float = 1.0,
        out_gate: bool = True, device="cpu", dtype=torch.bfloat16,
    ) -> None:
        super().__init__()
        assert heads % kv_heads == 0
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale = float(scale)
        self.temp_coef, self.temp_every = float(temp_coef), float(temp_every)
        self.out_gate = out_gate
        self.nq, self.nk, self.nv = heads * dim, kv_heads * dim, kv_heads * vdim
        self.ng = heads * vdim if out_gate else 0
        n_in = self.nq + self.nk + self.nv + self.ng
        s = 1.0 / math.sqrt(hidden)
        # rows: q | k | v | gate
        self.w_in = _param((n_in, hidden), device, dtype, s)
        self.b_in = _param((n_in,), device, dtype, 0.1)
        with torch.no_grad():
            self.b_in[self.nq + self.nk + self.nv :].zero_()  # the gate has no bias
        self.w_o = _param((hidden, heads * vdim), device, dtype, 1.0 / math.sqrt(heads * vdim))

    def cache_spec(self) -> dict:
        return {"kind": "kv", "kv_heads": self.kv_heads, "k_dim": self.dim, "v_dim": self.vdim}

    def load(self, get, prefix: str) -> None:
        """Copy q/k/v(/g) and o from a checkpoint (`get(name)` returns the
        tensor in this module's dtype/device)."""
        parts = [get(prefix + "q"), get(prefix + "k"), get(prefix + "v")]
        bias = [get(prefix + "q.b"), get(prefix + "k.b"), get(prefix + "v.b")]
        if self.out_gate:
            parts.append(get(prefix + "g"))
            bias.append(torch.zeros(self.ng, device=self.b_in.device, dtype=self.b_in.dtype))
        with torch.no_grad():
            self.w_in.copy_(torch.cat(parts, dim=0))
            self.b_in.copy_(torch.cat(bias, dim=0))
            self.w_o.copy_(get(prefix + "o"))

    def forward(self, h, positions, cache, meta):
        k_cache, v_cache = cache
        proj = F.linear(h, self.w_in, self.b_in)
        a, b, c = self.nq, self.nq + self.nk, self.nq + self.nk + self.nv
        q, k, v = proj[:, :a], proj[:, a:b], proj[:, b:c]
        gate = proj[:, c:] if self.out_gate else None
        ops.kv_scatter(k, v, k_cache, v_cache, meta.slot_mapping)
        if ops.mfma_attention_supported(
            proj.dtype, self.dim, self.vdim, proj.is_cuda, self.heads // self.kv_heads
        ):
            o = self._attend_mfma(q, gate, positions, k_cache, v_cache, meta)
        elif (
            meta.num_prefill_tokens > 0
            and meta.prefill_tile_seq is not None
            and ops.tiled_prefill_supported(proj.dtype, self.dim, self.vdim, proj.is_cuda)
        ):
            # prompt portions on MFMA tiles (temperature and gate fused), the
            # step's single tokens (and pad rows) through the any-shape kernel
            np_, rows = meta.num_prefill_tokens, proj.shape[0]
            o = torch.empty(rows, self.heads * self.vdim, dtype=proj.dtype, device=proj.device)
            ops.paged_attention_prefill_tiles(
                q[:np_], k_cache, v_cache, meta.prefill_block_tables,
                meta.prefill_query_start_locs, meta.prefill_context_lens,
                meta.prefill_tile_seq, meta.prefill_tile_qstart, self.scale, self.heads,
                gate=None if gate is None else gate[:np_], temp_coef=self.temp_coef,
                temp_every=self.temp_every, out=o[:np_],
            )
            if rows > np_:
                ops.paged_attention_general(
                    q[np_:], k_cache, v_cache, meta.seq_block_tables, meta.tok_seq[np_:],
                    positions[np_:], self.scale, self.heads,
                    gate=None if gate is None else gate[np_:], temp_coef=self.temp_coef,
                    temp_every=self.temp_every, out=o[np_:],
                )
        else:
            o = ops.paged_attention_general(
                q, k_cache, v_cache, meta.seq_block_tables, meta.tok_seq, positions,
                self.scale, self.heads, gate=gate, temp_coef=self.temp_coef,
                temp_every=self.temp_every,
            )
        return F.linear(o, self.w_o)

    def _attend_mfma(self, q, gate, positions, k_cache, v_cache, meta):
        """bf16, key size == value size in {64, 128}: the MFMA flash-prefill
        and paged-decode kernels do the softmax(QK^T)V; the temperature is
        folded into q beforehand and the gate applied afterwards."""
        qh = ops.temperature_scale_rows(q, positions, self.temp_coef, self.temp_every)
        qh = qh.view(-1, self.heads, self.dim)
        np_, nd = meta.num_prefill_tokens, meta.num_decode_tokens
        out = torch.zeros_like(qh) if np_ + nd < qh.shape[0] else torch.empty_like(qh)
        if np_ > 0:
            out[:np_] = ops.paged_attention_prefill(
                qh[:np_], k_cache, v_cache, meta.prefill_block_tables,
                meta.prefill_query_start_locs, meta.prefill_context_lens, self.scale,
                tile_seq=meta.prefill_tile_seq, tile_qstart=meta.prefill_tile_qstart,
            )
        if nd > 0:
            out[np_ : np_ + nd] = ops.paged_attention_decode(
                qh[np_ : np_ + nd], k_cache, v_cache, meta.decode_block_tables,
                meta.decode_context_lens, self.scale, max_ctx=meta.max_decode_ctx,
                nsplits=meta.decode_nsplits,
            )
        o = out.view(-1, self.heads * self.vdim)
        if gate is not None:
            ops.sigmoid_gate_mul(o, gate)
        return o


class MinGRU(nn.Module):
    def __init__(self, hidden: int, width: int, device="cpu", dtype=torch.bfloat16) -> None:
        super().__init__()
        self.width = width
        s = 1.0 / math.sqrt(hidden)
        # rows: update gate z | candidate x | output gate g
        self.w_in = _param((3 * width, hidden), device, dtype, s)
        self.b_in = _param((3 * width,), device, dtype, 0.1)
        with torch.no_grad():
            self.b_in[2 * width :].zero_()
        self.w_o = _param((hidden, width), device, dtype, 1.0 / math.sqrt(width))

    def cache_spec(self) -> dict:
        return {"kind": "state", "width": self.width}

    def load(self, get, prefix: str) -> None:
        zero = torch.zeros(self.width, device=self.b_in.device, dtype=self.b_in.dtype)
        with torch.no_grad():
            self.w_in.copy_(torch.cat([get(prefix + "z"), get(prefix + "x"), get(prefix + "g")], dim=0))
            self.b_in.copy_(torch.cat([get(prefix + "z.b"), get(prefix + "x.b"), zero], dim=0))
            self.w_o.copy_(get(prefix + "o"))

    def forward(self, h, positions, cache, meta):
        (state,) = cache
        zxg = F.linear(h, self.w_in, self.b_in)
        s = ops.mingru_scan(
            zxg, state, meta.seg_start, meta.seg_len, meta.seg_slot,
            meta.seg_fresh, meta.max_seg_len,
        )
        covered = meta.num_prefill_tokens + meta.num_decode_tokens
        if covered < s.shape[0]:
            s[covered:].zero_()  # GEMM-bucketing pad rows belong to no segment
        return F.linear(s, self.w_o)


class XieluMLP(nn.Module):
    def __init__(self, hidden: int, ff: int, device="cpu", dtype=torch.bfloat16) -> None:
        super().__init__()
        self.w_up = _param((ff, hidden), device, dtype, 1.0 / math.sqrt(hidden))
        self.w_down = _param((hidden, ff), device, dtype, 1.0 / math.sqrt(ff))
        self.set_act(0.0, 0.0)

    def set_act(self, p: float, q: float) -> None:
        """The activation's two learnable scalars enter through softplus."""
        self.a_pos = softplus64(float(p))
        self.a_neg = 0.5 + softplus64(float(q))

    def load(self, get, prefix: str) -> None:
        with torch.no_grad():
            self.w_up.copy_(get(prefix + "up"))
            self.w_down.copy_(get(prefix + "down"))
        act = get(prefix + "act").float().cpu().tolist()
        self.set_act(act[0], act[1])

    def forward(self, h):
        return F.linear(ops.xielu(F.linear(h, self.w_up), self.a_pos, self.a_neg), self.w_down)


def _mm(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    return F.linear(a, w)


class LatentAttention(nn.Module):
    """Attention whose keys and values are up-projections of one low-rank
    latent per token; only the normalised latent and one rotated key part
    shared by all heads are cached (one paged row of kv_rank + rot_dim
    entries).

    Per head a query has `dim` unrotated and `rot_dim` rotated entries; the
    score is (q_un . W_uk c + q_rot . k_rot) * scale.  The up-projections are
    absorbed so that attention runs in latent space as multi-query attention
    over the cache rows themselves:

        q_lat = W_uk^T q_un        (batched GEMM, per head)
        score = ([q_lat | q_rot] . [c | k_rot]) * scale
        o_lat = sum_j p_j c_j      (values = the leading kv_rank entries of the key rows)
        o     = W_uv o_lat         (batched GEMM, per head)

    which is exact because a softmax with a sink is still linear in the
    values.  Optional per-head sink in the softmax denominator, optional
    sigmoid output gate on the concatenated heads.  Rotation is interleaved
    pairs over the first `rot_dims` entries of the rotated part.
    """

    def __init__(
        self, hidden: int, heads: int, dim: int, rot_dim: int, vdim: int, q_rank: int,
        kv_rank: int, scale: float, rot_base: float, rot_dims: int, eps: float,
        sink: bool = True, out_gate: bool = True, device="cpu", dtype=torch.bfloat16,
    ) -> None:
        super().__init__()
        assert 0 <= rot_dims <= rot_dim and rot_dims % 2 == 0
        self.heads, self.dim, self.rot_dim, self.vdim = heads, dim, rot_dim, vdim
        self.q_rank, self.kv_rank = q_rank, kv_rank
        self.scale, self.eps = float(scale), float(eps)
        self.out_gate = out_gate
        self.row = kv_rank + rot_dim  # one cache row
        s = 1.0 / math.sqrt(hidden)
        self.n_in = q_rank + kv_rank + rot_dim
        self.ng = heads * vdim if out_gate else 0
        # rows: query latent | key/value latent | shared rotated key part | gate
        self.w_in = _param((self.n_in + self.ng, hidden), device, dtype, s)
        self.q_norm = _param((q_rank,), device, dtype, None)
        self.kv_norm = _param((kv_rank,), device, dtype, None)
        with torch.no_grad():
            self.q_norm.fill_(1.0)
            self.kv_norm.fill_(1.0)
        self.w_uq = _param((heads * (dim + rot_dim), q_rank), device, dtype, 1.0 / math.sqrt(q_rank))
        # per head, laid out for batched GEMMs: [H, dim, kv_rank] and [H, kv_rank, vdim]
        self.w_uk = _param((heads, dim, kv_rank), device, dtype, 1.0 / math.sqrt(kv_rank))
        self.w_uv = _param((heads, kv_rank, vdim), device, dtype, 1.0 / math.sqrt(kv_rank))
        self.sink = (
            nn.Parameter(torch.zeros(heads, device=device, dtype=torch.float32), requires_grad=False)
            if sink else None
        )
        self.w_o = _param((hidden, heads * vdim), device, dtype, 1.0 / math.sqrt(heads * vdim))
        self.register_buffer(
            "inv_freq", ops.rotary_inv_freq(rot_base, rot_dims, device), persistent=False
        )

    def cache_spec(self) -> dict:
        return {"kind": "latent", "row": self.row}

    def load(self, get, prefix: str) -> None:
        H, D, R = self.heads, self.dim, self.kv_rank
        parts = [get(prefix + "dq"), get(prefix + "dkv")]
        if self.out_gate:
            parts.append(get(prefix + "g"))
        with torch.no_grad():
            self.w_in.copy_(torch.cat(parts, dim=0))
            self.q_norm.copy_(get(prefix + "dq.norm"))
            self.kv_norm.copy_(get(prefix + "dkv.norm"))
            self.w_uq.copy_(get(prefix + "uq"))
            self.w_uk.copy_(get(prefix + "uk").view(H, D, R))
            self.w_uv.copy_(get(prefix + "uv").view(H, self.vdim, R).transpose(1, 2))
            if self.sink is not None:
                self.sink.copy_(get(prefix + "sink").float())
            self.w_o.copy_(get(prefix + "o"))

    def mfma_rows(self, dtype, on_gpu: bool) -> bool:
        return ops.latent_rows_supported(dtype, self.row, self.kv_rank, on_gpu)


    def forward(self, h, positions, cache, meta):
        lat_cache = cache[0]
        H, D, Rr, Rk = self.heads, self.dim, self.rot_dim, self.kv_rank
        rows = h.shape[0]
        proj = _mm(h, self.w_in)
        cq = ops.latent_kv_prep(
            proj, self.q_rank, Rk, Rr, self.q_norm, self.kv_norm, self.eps, self.inv_freq,
            positions, meta.slot_mapping, lat_cache,
        )
        q = _mm(cq, self.w_uq)  # [rows, H*(D+Rr)]
        qa = torch.empty(rows, H, self.row, dtype=q.dtype, device=q.device)
        # latent-space query part: per head q_un @ W_uk, written in place
        torch.bmm(
            q.view(rows, H, D + Rr)[:, :, :D].transpose(0, 1), self.w_uk,
            out=qa[:, :, :Rk].transpose(0, 1),
        )
        ops.rotate_pack_queries(q, H, D, Rr, self.inv_freq, positions, qa, Rk)
        qa = qa.view(rows, H * self.row)
        v_view = lat_cache[..., :Rk]
        np_ = meta.num_prefill_tokens
        if self.mfma_rows(q.dtype, q.is_cuda) and meta.seg_ctx is not None:
            # every row of the step in one launch: (token, head) row tiles
            # that share each key tile across the heads
            covered = np_ + meta.num_decode_tokens
            o = (torch.zeros if covered < rows else torch.empty)(
                rows, H * Rk, dtype=q.dtype, device=q.device
            )
            ops.latent_attention_rows(
                qa, lat_cache, Rk, meta.seq_block_tables, meta.seg_start, meta.seg_len,
                meta.seg_ctx, meta.max_seg_len, self.scale, H, sink=self.sink, out=o,
            )
        else:
            o = ops.paged_attention_general(
                qa, lat_cache, v_view, meta.seq_block_tables, meta.tok_seq, positions,
                self.scale, H, sink=self.sink,
            )
        # values: per head o_lat @ W_uv, heads concatenated in place
        ov = torch.empty(rows, H, self.vdim, dtype=q.dtype, device=q.device)
        torch.bmm(o.view(rows, H, Rk).transpose(0, 1), self.w_uv, out=ov.transpose(0, 1))
        ov = ov.view(rows, H * self.vdim)
        if self.out_gate:
            ops.sigmoid_gate_mul(ov, proj[:, self.n_in :])
        return _mm(ov, self.w_o)


class ReluSquaredMLP(nn.Module):
    """down(relu(up h)^2)."""

    def __init__(self, hidden: int, ff: int, device="cpu", dtype=torch.bfloat16) -> None:
        super().__init__()
        self.w_up = _param((ff, hidden), device, dtype, 1.0 / math.sqrt(hidden))
        self.w_down = _param((hidden, ff), device, dtype, 1.0 / math.sqrt(ff))

    def load(self, get, prefix: str) -> None:
        with torch.no_grad():
            self.w_up.copy_(get(prefix + "up"))
            self.w_down.copy_(get(prefix + "down"))

    def forward(self, h, meta=None):
        return _mm(ops.relu_squared(_mm(h, self.w_up)), self.w_down)


class ScoredExpertsMLP(nn.Module):
    """Routed gated-SiLU experts whose router scores are independent
    logistics: z = W_r h in fp32, s = sigmoid(z), the `top` largest scores
    pick the experts.  The chosen scores are used as they are (no
    renormalisation) and scale each expert's INPUT: out = sum_e expert_e(s_e h).

    Dispatch: (token, expert) pairs sorted by expert into a capacity-padded
    [E, cap, hidden] batch, gathered and scaled in one kernel, then one
    batched GEMM pair over all experts.  Steps made of single tokens only use
    a dense dispatch (every expert sees every token, unchosen pairs scaled by
    zero, which a bias-free expert maps to exactly zero): static shapes and
    no host round trip, so the step can be replayed from a hipGraph.
    """

    def __init__(
        self, hidden: int, ff: int, experts: int, top: int, device="cpu", dtype=torch.bfloat16
    ) -> None:
        super().__init__()
        assert 1 <= top <= experts
        self.experts, self.top, self.ff = experts, top, ff
        # the router runs in fp32 whatever the activation dtype
        self.w_router = nn.Parameter(
            torch.empty(experts, hidden, device=device, dtype=torch.float32).uniform_(
                -1.0 / math.sqrt(hidden), 1.0 / math.sqrt(hidden)
            ),
            requires_grad=False,
        )
        # pre-transposed for bmm: [E, hidden, gate | up] and [E, ff, hidden]
        self.w13 = _param((experts, hidden, 2 * ff), device, dtype, 1.0 / math.sqrt(hidden))
        self.w2 = _param((experts, ff, hidden), device, dtype, 1.0 / math.sqrt(ff))

    def load(self, get, prefix: str) -> None:
        with torch.no_grad():
            self.w_router.copy_(get(prefix + "router").float())
            for e in range(self.experts):
                p = f"{prefix}e{e}."
                self.w13[e].copy_(torch.cat([get(p + "gate"), get(p + "up")], dim=0).t())
                self.w2[e].copy_(get(p + "down").t())

    def route(self, h: torch.Tensor):
        z = F.linear(h.float(), self.w_router)
        w, idx = torch.topk(torch.sigmoid(z), self.top, dim=-1)
        return w, idx  # fp32 [T, top], int64 [T, top]

    def forward(self, h, meta=None):
        T, hidden = h.shape
        E = self.experts
        w, idx = self.route(h)
        if meta is not None and meta.num_prefill_tokens == 0:
            wd = torch.zeros(T, E, dtype=torch.float32, device=h.device).scatter_(1, idx, w)
            src = torch.arange(T, device=h.device).repeat(E)
            xe = ops.scale_gather_rows(h, src, wd.t().contiguous().view(-1))  # [E*T, hidden]
            act = ops.silu_mul(torch.bmm(xe.view(E, T, hidden), self.w13).view(E * T, -1))
            ye = torch.bmm(act.view(E, T, self.ff), self.w2)
            return ye.float().sum(dim=0).to(h.dtype)
        # (token, expert) pairs into a capacity-padded batch; the chosen score
        # scales the expert's input row
        gather, rows, cap = expert_dispatch_plan(idx, E)
        wpad = torch.zeros(E * cap, dtype=torch.float32, device=h.device)
        wpad.index_copy_(0, rows.reshape(-1), w.reshape(-1))
        xe = ops.scale_gather_rows(h, gather, wpad)
        act = ops.silu_mul(torch.bmm(xe.view(E, cap, hidden), self.w13).view(E * cap, -1))
        ye = torch.bmm(act.view(E, cap, self.ff), self.w2).view(E * cap, hidden)
        # every token owns exactly `top` rows of ye: gather them back in pair
        # order and sum in fp32 (no atomics, the same order every time)
        return ye.index_select(0, rows.reshape(-1)).view(T, self.top, hidden).float().sum(dim=1).to(h.dtype)


class NormedRotaryAttention(nn.Module):
    """Grouped-query softmax attention whose queries and keys are RMS-normed
    before an optional partial rotate-half rotation, with optional chunked
    visibility (a query sees the keys of its own chunk of `chunk` positions,
    counted from the sequence's start).

      * qk_norm "row": one norm over the whole q (and k) projection with
        weights of that size; "head": per head with one weight of size dim
        shared by the heads; "head_post": per head AFTER the rotation, no
        weights; "none".
      * rot_dims entries of every head are rotated; rot_layout "half" pairs
        entry i with i + rot_dims/2, "interleaved" pairs 2i with 2i + 1;
        rot_scale divides every frequency (linear position scaling);
        0 = no rotation.
      * window: a query sees itself and the window - 1 tokens before it
        (0 = no window; may be combined with chunk).
      * weights "softmax", optionally with a zero-score sink in the
        denominator (sink=True), or "sigmoid": every visible key weighs
        sigmoid(score + score_bias[head]), nothing is normalised.
      * head_gate: head h's output is multiplied by sigmoid(W_g x)_h, one
        number per head; the gate rows ride in the fused input GEMM.
      * values "proj": a projection of their own; "key": the keys as
        projected, before their norm (no value weights).
      * v_unit_norm: every head's value is divided by its root mean square.
      * value mixing: `forward(..., v_first=...)` blends the values with
        those another layer computed for the same tokens, (1 - lam) v + lam
        v_first, before they are cached; `want_v` returns this layer's.
      * dist_bias / talk: a per-head bias by distance, added to the scaled
        score, and a [heads, heads] matrix that mixes the heads' scores
        before the softmax.  With either, all heads of a token are scored
        together by the head-mixing kernel.

    Projections (biases optional) are one fused GEMM in, one out; everything
    between the GEMMs and the attention kernel is one prep kernel.  A model
    may pass `proj` (a wider fused projection that starts with this block's
    q | k | v columns) instead of letting the block run its own GEMM.
    """

    def __init__(
        self, hidden: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
        eps: float, qk_norm: str = "row", rot_base: float = 10000.0, rot_dims: int = 0,
        chunk: int = 0, values: str = "proj", v_unit_norm: bool = False, bias: bool = True,
        dist_rows: int = 0, dist_far: float = 0.0, talk: bool = False,
        rot_layout: str = "half", rot_scale: float = 1.0, window: int = 0,
        weights: str = "softmax", score_bias: bool = False, sink: bool = False,
        head_gate: bool = False, device="cpu", dtype=torch.bfloat16,
    ) -> None:
        super().__init__()
        assert heads % kv_heads == 0 and qk_norm in ("none", "row", "head", "head_post")
        assert rot_layout in ("half", "interleaved") and weights in ("softmax", "sigmoid")
        assert not (score_bias and weights != "sigmoid") and not (sink and weights != "softmax")
        assert not ((dist_rows > 0 or talk) and (window > 0 or weights == "sigmoid" or sink or head_gate))
        assert values in ("proj", "key") and (values == "proj" or vdim == dim)
        assert 0 <= rot_dims <= dim and rot_dims % 2 == 0
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.eps, self.chunk = float(scale), float(eps), int(chunk)
        self.qk_norm, self.values, self.v_unit_norm = qk_norm, values, v_unit_norm
        self.nq, self.nk = heads * dim, kv_heads * dim
        self.nv = kv_heads * vdim if values == "proj" else 0
        self.n_in = self.nq + self.nk + self.nv
        self.window, self.weights, self.rot_layout = int(window), weights, rot_layout
        # gate rows follow q | k | v; the fused weight is padded with zero rows
        # to a multiple of 8 so that rows of the projection stay 16-byte aligned
        self.n_gate = heads if head_gate else 0
        n_rows = (self.n_in + self.n_gate + 7) // 8 * 8 if head_gate else self.n_in
        s = 1.0 / math.sqrt(hidden)
        self.w_in = _param((n_rows, hidden), device, dtype, s)
        self.b_in = _param((n_rows,), device, dtype, 0.1 if bias else None)
        with torch.no_grad():
            self.w_in[self.n_in + self.n_gate :].zero_()
            self.b_in[self.n_in :].zero_()
        self.has_bias = bias
        # fp32 whatever the activation dtype: they enter the scores
        self.score_bias = (
            nn.Parameter(torch.empty(heads, device=device).uniform_(-1.0, 1.0), requires_grad=False)
            if score_bias else None
        )
        self.sink = (
            nn.Parameter(torch.zeros(heads, device=device), requires_grad=False) if sink else None
        )
        nw = {"row": (self.nq, self.nk), "head": (dim, dim), "none": (0, 0), "head_post": (0, 0)}[qk_norm]
        self.q_norm = _param((nw[0],), device, dtype, None)
        self.k_norm = _param((nw[1],), device, dtype, None)
        with torch.no_grad():
            self.q_norm.fill_(1.0)
            self.k_norm.fill_(1.0)
        self.w_o = _param((hidden, heads * vdim), device, dtype, 1.0 / math.sqrt(heads * vdim))
        self.b_o = _param((hidden,), device, dtype, 0.1 if bias else None)
        self.lam = 0.0  # value-mixing weight
        self.dist_far = float(dist_far)
        # fp32 whatever the activation dtype: they enter the scores
        self.rel = (
            nn.Parameter(torch.empty(dist_rows, heads, device=device).uniform_(-0.5, 0.5), requires_grad=False)
            if dist_rows > 0 else None
        )
        self.talk = (
            nn.Parameter(
                torch.eye(heads, device=device) + torch.empty(heads, heads, device=device).uniform_(-0.1, 0.1),
                requires_grad=False,
            )
            if talk else None
        )
        self.dist_bias: Optional[torch.Tensor] = None
        self.refresh_tables()
        self.register_buffer(
            "inv_freq",
            ops.rotary_inv_freq(rot_base, rot_dims, device, rot_scale) if rot_dims > 0 else None,
            persistent=False,
        )

    def refresh_tables(self) -> None:
        """Expand the bucketed distance table to one row per distance."""
        if self.rel is not None:
            self.dist_bias = ops.distance_bias_table(self.rel, self.dist_far)

    @property
    def mixes_heads(self) -> bool:
        return self.rel is not None or self.talk is not None

    def cache_spec(self) -> dict:
        return {"kind": "kv", "kv_heads": self.kv_heads, "k_dim": self.dim, "v_dim": self.vdim}

    def load(self, get, prefix: str) -> None:
        names = ["q", "k"] + (["v"] if self.values == "proj" else [])
        if self.n_gate:
            names.append("g")
        with torch.no_grad():
            rows = torch.cat([get(prefix + n) for n in names], dim=0)
            self.w_in.zero_()
            self.w_in[: rows.shape[0]].copy_(rows)
            if self.has_bias:
                names_b = [n for n in names if n != "g"]
                self.b_in[: self.n_in].copy_(torch.cat([get(prefix + n + ".b") for n in names_b], dim=0))
                self.b_o.copy_(get(prefix + "o.b"))
            if self.score_bias is not None:
                self.score_bias.copy_(get(prefix + "pb").float())
            if self.qk_norm in ("row", "head"):
                self.q_norm.copy_(get(prefix + "q.norm"))
                self.k_norm.copy_(get(prefix + "k.norm"))
            self.w_o.copy_(get(prefix + "o"))
            if self.rel is not None:
                self.rel.copy_(get(prefix + "rel").float())
            if self.talk is not None:
                self.talk.copy_(get(prefix + "talk").float())
        self.refresh_tables()

    def forward(self, h, positions, cache, meta, v_first=None, want_v=False, proj=None):
        k_cache, v_cache = cache
        if proj is None:
            proj = F.linear(h, self.w_in, self.b_in if self.has_bias else None)
        q, v_out = ops.qkv_norm_rope_cache(
            proj, self.heads, self.kv_heads, self.dim, self.vdim, self.qk_norm,
            self.q_norm, self.k_norm, self.eps, self.inv_freq, positions, k_cache, v_cache,
            meta.slot_mapping, v_source=self.values, v_unit_norm=self.v_unit_norm,
            v_first=v_first, lam=self.lam, want_v=want_v, rot_layout=self.rot_layout,
        )
        if self.mixes_heads:
            o = self._attend_mixed(q, positions, k_cache, v_cache, meta)
        else:
            gate = proj[:, self.n_in : self.n_in + self.n_gate] if self.n_gate else None
            o = self._attend(q, positions, k_cache, v_cache, meta, gate)
        y = F.linear(o, self.w_o, self.b_o if self.has_bias else None)
        return (y, v_out) if want_v else y

    def _attend_mixed(self, q, positions, k_cache, v_cache, meta):
        """All heads of a token together: prompt portions on MFMA tiles where
        the shape allows, everything else (single tokens, pad rows, fp32)
        through the any-shape head-mixing kernel."""
        np_, rows = meta.num_prefill_tokens, q.shape[0]
        kw = dict(dist_bias=self.dist_bias, talk=self.talk, chunk=self.chunk)
        done = 0
        o = None
        if (
            np_ > 0
            and meta.prefill_tile_seq is not None
            and ops.mixed_heads_tiles_supported(q.dtype, self.dim, self.vdim, self.heads, q.is_cuda)
        ):
            o = torch.empty(rows, self.heads * self.vdim, dtype=q.dtype, device=q.device)
            res = ops.paged_attention_mixed_heads_tiles(
                q[:np_], k_cache, v_cache, meta.prefill_block_tables,
                meta.prefill_query_start_locs, meta.prefill_context_lens,
                meta.prefill_tile_seq, meta.prefill_tile_qstart, self.scale, self.heads,
                out=o[:np_], **kw,
            )
            done = np_ if res is not None else 0
        if done == rows:
            return o
        if done == 0:
            return ops.paged_attention_mixed_heads(
                q, k_cache, v_cache, meta.seq_block_tables, meta.tok_seq, positions,
                self.scale, self.heads, **kw,
            )
        ops.paged_attention_mixed_heads(
            q[done:], k_cache, v_cache, meta.seq_block_tables, meta.tok_seq[done:],
            positions[done:], self.scale, self.heads, out=o[done:], **kw,
        )
        return o

    def _attend(self, q, positions, k_cache, v_cache, meta, gate=None):
        np_, rows = meta.num_prefill_tokens, q.shape[0]
        kw = dict(
            chunk=self.chunk, window=self.window, weights=self.weights,
            score_bias=self.score_bias, sink=self.sink, gate_per_head=gate is not None,
        )
        if (
            np_ > 0
            and meta.prefill_tile_seq is not None
            and ops.tiled_prefill_supported(q.dtype, self.dim, self.vdim, q.is_cuda)
        ):
            # prompt portions on MFMA tiles, the step's single tokens (and
            # pad rows) through the any-shape kernel
            o = torch.empty(rows, self.heads * self.vdim, dtype=q.dtype, device=q.device)
            ops.paged_attention_prefill_tiles(
                q[:np_], k_cache, v_cache, meta.prefill_block_tables,
                meta.prefill_query_start_locs, meta.prefill_context_lens,
                meta.prefill_tile_seq, meta.prefill_tile_qstart, self.scale, self.heads,
                out=o[:np_], gate=None if gate is None else gate[:np_], **kw,
            )
            if rows > np_:
                ops.paged_attention_general(
                    q[np_:], k_cache, v_cache, meta.seq_block_tables, meta.tok_seq[np_:],
                    positions[np_:], self.scale, self.heads, out=o[np_:],
                    gate=None if gate is None else gate[np_:], **kw,
                )
            return o
        return ops.paged_attention_general(
            q, k_cache, v_cache, meta.seq_block_tables, meta.tok_seq, positions,
            self.scale, self.heads, gate=gate, **kw,
        )


class MatrixStateMixer(nn.Module):
    """Recurrent mixers that carry one [dim, vdim] fp32 matrix per head and
    sequence (slot pool), scanned token by token by `ops.matrix_state_scan`.

    kind "wkv": every projection reads its own blend of the input with the
    previous token's (`ops.token_shift_mix`, five blends, one more state row
    per sequence); per-channel per-token decay w = exp(-exp(W_w2 tanh(W_w1 .)
    + w0)) from a low-rank pair; the current token enters the output through
    a bonus u instead of the state; every head's output is divided by its
    root mean square, then times a weight, times silu(gate).

    kind "decay": q, k, v pass through silu, one constant decay per head, the
    output reads the updated state; the concatenated heads are RMS-normed
    together with a weight and multiplied by sigmoid(gate).

    A model may hand "decay" a wider fused projection (`proj`, columns q | k
    | v | gate first) instead of letting the block run its own GEMM.
    """

    def __init__(
        self, hidden: int, kind: str, heads: int, dim: int, vdim: int, eps: float,
        decay=None, decay_rank: int = 0, device="cpu", dtype=torch.bfloat16,
    ) -> None:
        super().__init__()
        assert kind in ("wkv", "decay")
        self.kind, self.heads, self.dim, self.vdim, self.eps = kind, heads, dim, vdim, float(eps)
        self.hidden = hidden
        nk, nv = heads * dim, heads * vdim
        self.nk, self.nv = nk, nv
        s = 1.0 / math.sqrt(hidden)
        if kind == "wkv":
            assert vdim == dim
            # blends in the order r, k, v, gate, decay
            self.mu = _param((5, hidden), device, dtype, None)
            with torch.no_grad():
                self.mu.uniform_(0.0, 1.0)
            # pre-transposed for one batched GEMM: [4, hidden, heads*dim]
            self.w_rkvg = _param((4, hidden, nk), device, dtype, s)
            self.w_d1 = _param((decay_rank, hidden), device, dtype, s)
            # the decay's second projection, its offset and the bonus enter
            # the recurrence: fp32
            self.w_d2 = nn.Parameter(
                torch.empty(nk, decay_rank, device=device).uniform_(-0.1, 0.1), requires_grad=False
            )
            self.d0 = nn.Parameter(torch.empty(nk, device=device).uniform_(-1.0, 0.5), requires_grad=False)
            self.bonus = nn.Parameter(torch.empty(nk, device=device).uniform_(-0.5, 0.5), requires_grad=False)
            self.head_decay = None
        else:
            # rows: q | k | v | gate
            self.w_in = _param((2 * nk + 2 * nv, hidden), device, dtype, s)
            self.head_decay = nn.Parameter(
                torch.tensor([float(d) for d in decay], dtype=torch.float32, device=device),
                requires_grad=False,
            )
            assert self.head_decay.shape == (heads,)
        self.norm = _param((nv,), device, dtype, None)
        with torch.no_grad():
            self.norm.fill_(1.0)
        self.w_o = _param((hidden, nv), device, dtype, 1.0 / math.sqrt(nv))

    def cache_spec(self):
        mat = {"kind": "state", "width": ops.matrix_state_width(self.heads, self.dim, self.vdim)}
        if self.kind == "wkv":
            return [{"kind": "state", "width": self.hidden}, mat]
        return mat

    def load(self, get, prefix: str) -> None:
        with torch.no_grad():
            if self.kind == "wkv":
                self.mu.copy_(torch.stack([get(prefix + "mu." + n) for n in "rkvgw"], dim=0))
                self.w_rkvg.copy_(torch.stack([get(prefix + n).t() for n in "rkvg"], dim=0))
                self.w_d1.copy_(get(prefix + "w1"))
                self.w_d2.copy_(get(prefix + "w2").float())
                self.d0.copy_(get(prefix + "w0").float())
                self.bonus.copy_(get(prefix + "u").float().reshape(-1))
            else:
                self.w_in.copy_(torch.cat([get(prefix + n) for n in "qkvg"], dim=0))
            self.norm.copy_(get(prefix + "norm"))
            self.w_o.copy_(get(prefix + "o"))

    @staticmethod
    def _zero_pad_rows(o, meta) -> None:
        covered = meta.num_prefill_tokens + meta.num_decode_tokens
        if covered < o.shape[0]:
            o[covered:].zero_()  # GEMM-bucketing pad rows belong to no segment

    def forward(self, x, h, cache, meta, proj=None):
        """x: the fp32 rows (token shift reads them), h: the same in the
        activation dtype."""
        seg = (meta.seg_start, meta.seg_len, meta.seg_slot, meta.seg_fresh)
        if self.kind == "wkv":
            shift_state, mat_state = cache
            mixes = ops.token_shift_mix(x, self.mu, shift_state, meta.tok_seq, *seg)
            rkvg = torch.bmm(mixes[:4], self.w_rkvg)  # [4, R, heads*dim]
            low = ops.tanh_act(F.linear(mixes[4], self.w_d1))
            decay_pre = F.linear(low.float(), self.w_d2, self.d0)  # fp32
            o = ops.matrix_state_scan(
                rkvg[0], rkvg[1], rkvg[2], mat_state, *seg, self.heads, self.dim, self.vdim,
                decay_pre=decay_pre, bonus=self.bonus,
            )
            self._zero_pad_rows(o, meta)
            g = ops.group_rms_norm_gate(o, rkvg[3], self.norm, self.vdim, "silu", self.eps)
        else:
            (mat_state,) = cache
            if proj is None:
                proj = F.linear(h, self.w_in)
            a, b, c = self.nk, 2 * self.nk, 2 * self.nk + self.nv
            o = ops.matrix_state_scan(
                proj[:, :a], proj[:, a:b], proj[:, b:c], mat_state, *seg, self.heads,
                self.dim, self.vdim, head_decay=self.head_decay, act_silu=True,
            )
            self._zero_pad_rows(o, meta)
            g = ops.group_rms_norm_gate(o, proj[:, c : c + self.nv], self.norm, self.nv, "sigmoid", self.eps)
        return F.linear(g, self.w_o)


class GeluMLP(nn.Module):
    """down(gelu(up h)) with the exact (erf) gelu."""

    def __init__(self, hidden: int, ff: int, device="cpu", dtype=torch.bfloat16) -> None:
        super().__init__()
        self.w_up = _param((ff, hidden), device, dtype, 1.0 / math.sqrt(hidden))
        self.w_down = _param((hidden, ff), device, dtype, 1.0 / math.sqrt(ff))

    def load(self, get, prefix: str) -> None:
        with torch.no_grad():
            self.w_up.copy_(get(prefix + "up"))
            self.w_down.copy_(get(prefix + "down"))

    def forward(self, h, meta=None):
        return _mm(ops.gelu_erf(_mm(h, self.w_up)), self.w_down)


class GatedReluMLP(nn.Module):
    """down(relu(gate h) * (up h)); gate and up are one fused GEMM."""

    def __init__(self, hidden: int, ff: int, device="cpu", dtype=torch.bfloat16) -> None:
        super().__init__()
        self.w13 = _param((2 * ff, hidden), device, dtype, 1.0 / math.sqrt(hidden))
        self.w_down = _param((hidden, ff), device, dtype, 1.0 / math.sqrt(ff))

    def load(self, get, prefix: str) -> None:
        with torch.no_grad():
            self.w13.copy_(torch.cat([get(prefix + "gate"), get(prefix + "up")], dim=0))
            self.w_down.copy_(get(prefix + "down"))

    def forward(self, h, meta=None):
        return _mm(ops.glu_act(_mm(h, self.w13), "relu"), self.w_down)


def expert_dispatch_plan(idx: torch.Tensor, experts: int):
    """Capacity-padded dispatch of (token, choice) pairs to `experts` batches.

    idx int64 [T, top]; choices >= experts take part in no batch.  Returns
    (gather [experts * cap] int64: the token of every batch row, -1 for
    padding; rows [T, top] int64: the batch row of every pair, -1 for pairs
    outside the batches; cap).  One host round trip (the capacity)."""
    T, top = idx.shape
    dev = idx.device
    flat_e = idx.reshape(-1)
    flat_t = torch.arange(T, device=dev).unsqueeze(1).expand(T, top).reshape(-1)
    order = torch.argsort(flat_e, stable=True)
    se, stok = flat_e[order], flat_t[order]
    inside = se < experts
    counts = torch.bincount(se.clamp(max=experts), minlength=experts + 1)
    cap = max(int(counts[:experts].max()), 1)
    starts = torch.cumsum(counts, 0) - counts
    pos_in_e = torch.arange(se.numel(), device=dev) - starts.index_select(0, se.clamp(max=experts))
    trash = experts * cap  # one spare row takes the pairs outside the batches
    dest = torch.where(inside, se * cap + pos_in_e, torch.full_like(se, trash))
    gather = torch.full((trash + 1,), -1, dtype=torch.int64, device=dev)
    gather.index_copy_(0, dest, stok)
    rows = torch.empty_like(dest)
    rows[order] = torch.where(inside, dest, torch.full_like(dest, -1))
    return gather[:trash], rows.view(T, top), cap


class GroupRoutedExpertsMLP(nn.Module):
    """Routed gated experts behind a softmax router with group-limited choice.

    z = W_r h in fp32 over experts + identity outputs; scores softmax(z);
    the choice adds a per-output correction and only looks at the `keep` best
    of `groups` groups of neighbouring outputs (`ops.grouped_topk_route`);
    the chosen plain scores, divided by their sum, weigh the experts'
    OUTPUTS.  The last `identity` outputs are experts without weights whose
    output is their input.  An expert is down(act(gate h, up h)) with
    g = min(gate, limit), u = clamp(up, -limit, limit), act = g * sigmoid(alpha
    g) * (u + 1).

    Dispatch as `ScoredExpertsMLP`: pairs sorted by expert into a
    capacity-padded [E, cap, hidden] batch and one batched GEMM pair; steps
    of single tokens only let every expert see every token (static shapes,
    no host round trip), the combine picks the chosen ones.
    """

    def __init__(
        self, hidden: int, ff: int, experts: int, top: int, identity: int = 0,
        groups: int = 1, keep: int = 1, limit: float = 7.0, alpha: float = 1.702,
        device="cpu", dtype=torch.bfloat16,
    ) -> None:
        super().__init__()
        n = experts + identity
        assert experts >= 1 and identity >= 0 and n % groups == 0 and 1 <= keep <= groups
        assert 1 <= top <= keep * (n // groups)
        self.experts, self.identity, self.top, self.ff = experts, identity, top, ff
        self.groups, self.keep = groups, keep
        self.limit, self.alpha = float(limit), float(alpha)
        # router and correction are fp32 whatever the activation dtype
        self.w_router = nn.Parameter(
            torch.empty(n, hidden, device=device, dtype=torch.float32).uniform_(
                -1.0 / math.sqrt(hidden), 1.0 / math.sqrt(hidden)
            ),
            requires_grad=False,
        )
        self.correction = nn.Parameter(
            torch.zeros(n, device=device, dtype=torch.float32), requires_grad=False
        )
        # pre-transposed for bmm: [E, hidden, gate | up] and [E, ff, hidden]
        self.w13 = _param((experts, hidden, 2 * ff), device, dtype, 1.0 / math.sqrt(hidden))
        self.w2 = _param((experts, ff, hidden), device, dtype, 1.0 / math.sqrt(ff))

    def load(self, get, prefix: str, has=None) -> None:
        with torch.no_grad():
            self.w_router.copy_(get(prefix + "router").float())
            if has is None or has(prefix + "correction"):
                self.correction.copy_(get(prefix + "correction").float())
            for e in range(self.experts):
                p = f"{prefix}e{e}."
                self.w13[e].copy_(torch.cat([get(p + "gate"), get(p + "up")], dim=0).t())
                self.w2[e].copy_(get(p + "down").t())

    def route(self, h: torch.Tensor):
        z = F.linear(h.float(), self.w_router)
        idx, w = ops.grouped_topk_route(z, self.correction, self.top, self.groups, self.keep)
        return w, idx  # fp32 [T, top], int32 [T, top]

    def _experts(self, xe: torch.Tensor, rows: int) -> torch.Tensor:
        """xe [E, rows, hidden] -> [E * rows, hidden]."""
        E = self.experts
        act = ops.glu_act(torch.bmm(xe, self.w13).view(E * rows, -1), "clamped", self.limit, self.alpha)
        return torch.bmm(act.view(E, rows, self.ff), self.w2).view(E * rows, -1)

    def forward(self, h, meta=None):
        T, hidden = h.shape
        E = self.experts
        w, idx = self.route(h)
        if meta is not None and meta.num_prefill_tokens == 0:
            ye = self._experts(h.unsqueeze(0).expand(E, T, hidden), T)
            return ops.routed_combine(ye, h, None, w, idx=idx, experts=E)
        gather, rows, cap = expert_dispatch_plan(idx.long(), E)
        xe = ops.scale_gather_rows(h, gather, (gather >= 0).float())
        ye = self._experts(xe.view(E, cap, hidden), cap)
        return ops.routed_combine(ye, h, rows.contiguous(), w)
