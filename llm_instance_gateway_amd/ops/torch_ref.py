"""Pure-PyTorch reference implementations of the engine ops.

These are (a) the CPU execution path for tests/simulation, and (b) the fp32
numerics references the HIP/CDNA4 kernels are validated against (SURVEY.md §4:
"GPU kernel unit tests vs PyTorch-ROCm reference outputs").  All math is done
in fp32 and cast back to the input dtype.

Shapes convention (flat token batch, no padding):
  x:            [T, hidden]
  q:            [T, num_heads * head_dim]
  k, v:         [T, num_kv_heads * head_dim]
  k_cache/v_cache: [num_blocks, num_kv_heads, block_size, head_dim]
  slot_mapping: [T] int64, slot = block_id * block_size + offset
  block_tables: [num_seqs, max_blocks] int32
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import torch


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    y = xf * torch.rsqrt(var + eps) * weight.float()
    return y.to(x.dtype)


def fused_add_rms_norm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float
) -> Tuple[torch.Tensor, torch.Tensor]:
    """y = rmsnorm(x + residual); returns (y, x + residual)."""
    s = (x.float() + residual.float())
    var = s.pow(2).mean(dim=-1, keepdim=True)
    y = s * torch.rsqrt(var + eps) * weight.float()
    return y.to(x.dtype), s.to(x.dtype)


def build_cos_sin_cache(
    head_dim: int, max_positions: int, theta: float, device, dtype=torch.float32
) -> torch.Tensor:
    """[max_positions, head_dim] — first half cos, second half sin, matching
    GPT-NeoX-style (Llama) half-rotation RoPE.  Precomputed on host: on-device
    sinf/cosf per element turns a memory-bound op VALU-bound (guide App. B)."""
    inv_freq = 1.0 / (
        theta ** (torch.arange(0, head_dim, 2, device=device, dtype=torch.float64) / head_dim)
    )
    t = torch.arange(max_positions, device=device, dtype=torch.float64)
    freqs = torch.outer(t, inv_freq)  # [P, head_dim/2]
    cache = torch.cat([freqs.cos(), freqs.sin()], dim=-1).to(dtype)
    return cache  # [P, head_dim]


def rotary_embedding(
    positions: torch.Tensor,  # [T] int64
    q: torch.Tensor,  # [T, num_heads * head_dim]
    k: torch.Tensor,  # [T, num_kv_heads * head_dim]
    cos_sin_cache: torch.Tensor,  # [P, head_dim]
    head_dim: int,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Llama (NeoX-style half-rotation) RoPE applied to q and k."""

    def rot(x: torch.Tensor) -> torch.Tensor:
        T = x.shape[0]
        xh = x.float().view(T, -1, head_dim)
        half = head_dim // 2
        cs = cos_sin_cache[positions].float()  # [T, head_dim]
        cos = cs[:, :half].unsqueeze(1)  # [T, 1, half]
        sin = cs[:, half:].unsqueeze(1)
        x1, x2 = xh[..., :half], xh[..., half:]
        o1 = x1 * cos - x2 * sin
        o2 = x2 * cos + x1 * sin
        return torch.cat([o1, o2], dim=-1).view(T, -1).to(x.dtype)

    return rot(q), rot(k)


def reshape_and_cache(
    k: torch.Tensor,
    v: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> None:
    """Scatter new K/V rows into the paged cache (in-place)."""
    num_blocks, kvh, bs, hd = k_cache.shape
    T = k.shape[0]
    kf = k.view(T, kvh, hd)
    vf = v.view(T, kvh, hd)
    blk = torch.div(slot_mapping, bs, rounding_mode="floor")
    off = slot_mapping % bs
    k_cache[blk, :, off, :] = kf.to(k_cache.dtype)
    v_cache[blk, :, off, :] = vf.to(v_cache.dtype)


def _gather_kv(
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_table: torch.Tensor,  # [max_blocks] int32
    context_len: int,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Rebuild contiguous [L, kv_heads, head_dim] K/V for one sequence."""
    nb, kvh, bs, hd = k_cache.shape
    nblk = (context_len + bs - 1) // bs
    ids = block_table[:nblk].long()
    k = k_cache[ids].permute(0, 2, 1, 3).reshape(nblk * bs, kvh, hd)[:context_len]
    v = v_cache[ids].permute(0, 2, 1, 3).reshape(nblk * bs, kvh, hd)[:context_len]
    return k, v


def _sdpa(
    q: torch.Tensor,  # [Tq, H, D]
    k: torch.Tensor,  # [L, KVH, D]
    v: torch.Tensor,
    scale: float,
    causal_offset: Optional[int] = None,
) -> torch.Tensor:
    """fp32 attention; if causal_offset is given, query row i attends to
    keys [0, causal_offset + i]."""
    Tq, H, D = q.shape
    L, KVH, _ = k.shape
    group = H // KVH
    qf = q.float().permute(1, 0, 2)  # [H, Tq, D]
    kf = k.float().repeat_interleave(group, dim=1).permute(1, 0, 2)  # [H, L, D]
    vf = v.float().repeat_interleave(group, dim=1).permute(1, 0, 2)
    scores = torch.bmm(qf, kf.transpose(1, 2)) * scale  # [H, Tq, L]
    if causal_offset is not None:
        pos = torch.arange(Tq, device=q.device).unsqueeze(1) + causal_offset
        keyp = torch.arange(L, device=q.device).unsqueeze(0)
        mask = keyp > pos  # [Tq, L]
        scores.masked_fill_(mask.unsqueeze(0), float("-inf"))
    p = torch.softmax(scores, dim=-1)
    out = torch.bmm(p, vf)  # [H, Tq, D]
    return out.permute(1, 0, 2).to(q.dtype)


def paged_attention_decode(
    q: torch.Tensor,  # [N, num_heads, head_dim]
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,  # [N, max_blocks]
    context_lens: torch.Tensor,  # [N]
    scale: float,
) -> torch.Tensor:
    N, H, D = q.shape
    out = torch.empty_like(q)
    for i in range(N):
        L = int(context_lens[i])
        k, v = _gather_kv(k_cache, v_cache, block_tables[i], L)
        out[i] = _sdpa(q[i : i + 1], k, v, scale)[0]
    return out


def paged_attention_prefill(
    q: torch.Tensor,  # [T, num_heads, head_dim] — all prefill-chunk tokens, flat
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,  # [S, max_blocks]
    query_start_locs: torch.Tensor,  # [S+1] cu lens of chunks
    context_lens: torch.Tensor,  # [S] ctx len AFTER this chunk's KV was cached
    scale: float,
) -> torch.Tensor:
    """Chunked-prefill attention: the chunk's own K/V are already in the cache
    (reshape_and_cache runs first), so query row j of sequence s (global
    position ctx - n + j) attends to cache positions [0, ctx - n + j]."""
    out = torch.empty_like(q)
    S = block_tables.shape[0]
    for s in range(S):
        lo, hi = int(query_start_locs[s]), int(query_start_locs[s + 1])
        n = hi - lo
        L = int(context_lens[s])
        k, v = _gather_kv(k_cache, v_cache, block_tables[s], L)
        out[lo:hi] = _sdpa(q[lo:hi], k, v, scale, causal_offset=L - n)
    return out


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    d = x.shape[-1] // 2
    a = x[..., :d].float()
    b = x[..., d:].float()
    return (a * torch.sigmoid(a) * b).to(x.dtype)


def sgmv_shrink(
    x: torch.Tensor,  # [T, H]
    a_stack: torch.Tensor,  # [S, R, H]
    slots: torch.Tensor,  # [T] int32, -1 = no adapter
) -> torch.Tensor:
    """u[t] = A[slot_t] @ x[t]; zero rows for slot -1."""
    T = x.shape[0]
    R = a_stack.shape[1]
    u = torch.zeros(T, R, dtype=torch.float32, device=x.device)
    for t in range(T):
        s = int(slots[t])
        if s >= 0:
            u[t] = a_stack[s].float() @ x[t].float()
    return u.to(x.dtype)


def sgmv_expand(
    u: torch.Tensor,  # [T, R]
    b_stack: torch.Tensor,  # [S, O, R]
    slots: torch.Tensor,  # [T]
    y: torch.Tensor,  # [T, O] accumulated in-place
    scaling: float = 1.0,
) -> None:
    for t in range(u.shape[0]):
        s = int(slots[t])
        if s >= 0:
            y[t] += (b_stack[s].float() @ u[t].float() * scaling).to(y.dtype)


# -- hybrid-model mechanisms (grouped norm, xIELU, minGRU, general attention) --
# Same rounding points as the HIP kernels: fp32 math, results cast to the
# activation dtype; the residual stream and the recurrent state stay fp32.

def _group_scale(x: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    R, H = x.shape
    xg = x.float().view(R, groups, H // groups)
    return (xg / torch.sqrt(xg.pow(2).mean(dim=-1, keepdim=True) + eps)).view(R, H)


def embed_group_norm(tokens, table, w, eps: float, groups: int) -> torch.Tensor:
    return _group_scale(table[tokens], groups, eps) * w.float()


def group_norm(residual, w, eps: float, groups: int, out_dtype) -> torch.Tensor:
    return (_group_scale(residual, groups, eps) * w.float()).to(out_dtype)


def post_add_pre_norm(residual, y, w_post, w_pre, eps: float, groups: int):
    residual.add_(_group_scale(y, groups, eps) * w_post.float())
    if w_pre is None:
        return None
    return (_group_scale(residual, groups, eps) * w_pre.float()).to(y.dtype)


def xielu(x: torch.Tensor, a_pos: float, a_neg: float) -> torch.Tensor:
    z = x.float()
    neg = a_neg * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z
    pos = a_pos * z * z + 0.5 * z
    return torch.where(z > 0, pos, neg).to(x.dtype)


def sigmoid_gate_mul(x: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    return x.copy_((x.float() * torch.sigmoid(g.float())).to(x.dtype))


def mingru_scan(zxg, state, seg_start, seg_len, seg_slot, seg_fresh, W: int):
    """zxg [R, 3W] = (gate pre-activation | candidate pre-activation | output
    gate); state [slots, W] fp32, updated in place."""
    R = zxg.shape[0]
    out = torch.zeros(R, W, dtype=zxg.dtype, device=zxg.device)
    z = torch.sigmoid(zxg[:, :W].float())
    u = zxg[:, W : 2 * W].float()
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = zxg[:, 2 * W :].float()
    og = g * torch.sigmoid(g)
    for s0, n, slot, fresh in zip(
        seg_start.tolist(), seg_len.tolist(), seg_slot.tolist(), seg_fresh.tolist()
    ):
        if n <= 0:
            continue
        S = torch.zeros(W, dtype=torch.float32, device=zxg.device) if fresh else state[slot].clone()
        for t in range(s0, s0 + n):
            S = (1.0 - z[t]) * S + z[t] * cand[t]
            out[t] = (S * og[t]).to(out.dtype)
        state[slot] = S
    return out


def kv_scatter(k, v, k_cache, v_cache, slot_mapping) -> None:
    nb, G, bs, D = k_cache.shape
    Dv = v_cache.shape[-1]
    T = k.shape[0]
    ok = slot_mapping >= 0
    blk = torch.div(slot_mapping, bs, rounding_mode="floor")[ok]
    off = (slot_mapping % bs)[ok]
    k_cache[blk, :, off, :] = k.reshape(T, G, D)[ok].to(k_cache.dtype)
    v_cache[blk, :, off, :] = v.reshape(T, G, Dv)[ok].to(v_cache.dtype)


def query_temperature(positions: torch.Tensor, coef: float, every: float) -> torch.Tensor:
    n = torch.floor((positions.double() + 1.0) / every)
    return (1.0 + coef * torch.log(n + 1.0)).float()


def paged_attention_general(
    q, k_cache, v_cache, block_tables, tok_seq, positions, scale: float,
    num_heads: int, gate=None, temp_coef: float = 0.0, temp_every: float = 1.0,
    sink=None, chunk: int = 0, window: int = 0, score_bias=None,
    weights: str = "softmax", gate_per_head: bool = False,
):
    """q [R, H*D] (may be a strided view); token r belongs to sequence row
    tok_seq[r] of block_tables (-1: padding row) and sees keys 0..positions[r].
    `sink` [H] fp32 adds exp(sink_h) to head h's softmax denominator (a key
    with that unscaled score and no value).  v_cache may be a view into
    k_cache's rows.  chunk > 0 hides keys of earlier chunks: key j is seen
    only if floor(j / chunk) == floor(position / chunk); window > 0 hides
    keys with position - j >= window.  weights "sigmoid": unnormalised
    sigmoid(score + score_bias[h]) per visible key.  gate_per_head: gate
    [R, H]."""
    R = q.shape[0]
    nb, G, bs, D = k_cache.shape
    Dv = v_cache.shape[-1]
    H = num_heads
    out = torch.zeros(R, H * Dv, dtype=q.dtype, device=q.device)
    seqs = tok_seq.tolist()
    pos = positions.tolist()
    tau = (
        query_temperature(positions, temp_coef, temp_every)
        if temp_coef != 0.0
        else torch.ones(R, dtype=torch.float32, device=q.device)
    )
    r = 0
    while r < R:
        s = seqs[r]
        e = r + 1
        while e < R and seqs[e] == s:
            e += 1
        if s >= 0:
            L = max(pos[r:e]) + 1
            nblk = (L + bs - 1) // bs
            ids = block_tables[s, :nblk].long()
            k = k_cache[ids].permute(0, 2, 1, 3).reshape(nblk * bs, G, D)[:L].float()
            v = v_cache[ids].permute(0, 2, 1, 3).reshape(nblk * bs, G, Dv)[:L].float()
            kf = k.repeat_interleave(H // G, dim=1).permute(1, 0, 2)  # [H, L, D]
            vf = v.repeat_interleave(H // G, dim=1).permute(1, 0, 2)
            qf = q[r:e].float().reshape(e - r, H, D).permute(1, 0, 2)  # [H, n, D]
            sc = torch.bmm(qf, kf.transpose(1, 2)) * (scale * tau[r:e])[None, :, None]
            keyp = torch.arange(L, device=q.device)[None, :]
            mask = keyp > positions[r:e, None]
            if chunk > 0:
                mask = mask | (keyp < (positions[r:e, None] // chunk) * chunk)
            if window > 0:
                mask = mask | (keyp < positions[r:e, None] - window + 1)
            sc.masked_fill_(mask[None], float("-inf"))
            if weights == "sigmoid":
                if score_bias is not None:
                    sc = sc + score_bias.float().view(H, 1, 1)
                pr = torch.sigmoid(sc)  # sigmoid(-inf) = 0
            elif sink is not None:
                sk = sink.float().view(H, 1, 1).expand(H, e - r, 1)
                pr = torch.softmax(torch.cat([sc, sk], dim=-1), dim=-1)[..., :-1]
            else:
                pr = torch.softmax(sc, dim=-1)
            o = torch.bmm(pr, vf).permute(1, 0, 2).reshape(e - r, H * Dv)
            if gate is not None and gate_per_head:
                o = (o.view(e - r, H, Dv) * torch.sigmoid(gate[r:e].float())[:, :, None]).reshape(e - r, H * Dv)
            elif gate is not None:
                o = o * torch.sigmoid(gate[r:e].float())
            out[r:e] = o.to(out.dtype)
        r = e
    return out


def temperature_scale_rows(q, positions, coef: float, every: float):
    if coef == 0.0:
        return q.contiguous().clone()
    tau = query_temperature(positions, coef, every)
    return (q.float() * tau[:, None]).to(q.dtype)


# -- token shift, latent attention, sink softmax, routed feed-forward ----------

def _rms_scale(x: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    return xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)


def residual_add(x, a, b=None) -> torch.Tensor:
    """x += (a + b), x fp32 in place."""
    x.add_(a.float() if b is None else a.float() + b.float())
    return x


def offset_rms_norm(x, w, eps: float, out_dtype) -> torch.Tensor:
    """RMS norm whose stored weight is an offset from one."""
    return (_rms_scale(x, eps) * (1.0 + w.float())).to(out_dtype)


def offset_norm_shift(
    x, w_mix, w_ff, mu, state, tok_seq, seg_start, seg_len, seg_slot, seg_fresh,
    eps: float, out_dtype,
):
    """Two offset-weight RMS norms of the same fp32 rows.  The first one's
    result h is blended with the previous token's, h + (h_prev - h) * mu:
    inside a segment h_prev is the row before, at a segment's first row it is
    the sequence's state (zeros when the sequence starts here); the state
    then takes the segment's last unblended h.  Rows outside every segment
    come out zero.  Returns (mixer input, feed-forward input or None)."""
    n = _rms_scale(x, eps)
    h = n * (1.0 + w_mix.float())
    prev = torch.zeros_like(h)
    live = torch.zeros(h.shape[0], 1, dtype=torch.float32, device=h.device)
    for s0, cnt, slot, fresh in zip(
        seg_start.tolist(), seg_len.tolist(), seg_slot.tolist(), seg_fresh.tolist()
    ):
        if cnt <= 0:
            continue
        if not fresh:
            prev[s0] = state[slot]
        prev[s0 + 1 : s0 + cnt] = h[s0 : s0 + cnt - 1]
        state[slot] = h[s0 + cnt - 1]
        live[s0 : s0 + cnt] = 1.0
    hm = (h + (prev - h) * mu.float()) * live
    hf = None if w_ff is None else (n * (1.0 + w_ff.float()) * live).to(out_dtype)
    return hm.to(out_dtype), hf


def rotary_inv_freq(base: float, dims: int, device=None, divide: float = 1.0) -> torch.Tensor:
    """f_i = base^(-2i/dims) / divide, i < dims/2, evaluated in float64, stored
    fp32 (divide > 1 is linear position scaling)."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims) / float(divide)
    return f.float().to(device)


def _rotate_pairs(v: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """Interleaved rotation of the first 2*len(inv_freq) entries of the last
    axis: pair (2i, 2i+1) turns by positions * inv_freq[i] (fp32 angles)."""
    n = inv_freq.shape[0]
    out = v.float().clone()
    ang = positions.float()[:, None] * inv_freq[None, :]
    c, s = torch.cos(ang), torch.sin(ang)
    while c.dim() < v.dim():
        c, s = c.unsqueeze(1), s.unsqueeze(1)
    a, b = out[..., 0 : 2 * n : 2].clone(), out[..., 1 : 2 * n : 2].clone()
    out[..., 0 : 2 * n : 2] = a * c - b * s
    out[..., 1 : 2 * n : 2] = b * c + a * s
    return out


def latent_kv_prep(
    proj, q_rank: int, kv_rank: int, rot_dim: int, w_q, w_kv, eps: float,
    inv_freq, positions, slot_mapping, cache,
):
    """proj [R, >= q_rank + kv_rank + rot_dim] holds, per row, the query
    latent, the key/value latent and the shared rotated key part.  Returns
    the RMS-normed query latent [R, q_rank]; writes the normed key/value
    latent followed by the rotated key part into cache row slot_mapping[r]
    (cache [blocks, 1, block_size, kv_rank + rot_dim])."""
    a, b = q_rank, q_rank + kv_rank
    cq = (_rms_scale(proj[:, :a], eps) * w_q.float()).to(proj.dtype)
    c = _rms_scale(proj[:, a:b], eps) * w_kv.float()
    kr = _rotate_pairs(proj[:, b : b + rot_dim], positions, inv_freq)
    row = torch.cat([c, kr], dim=-1).to(cache.dtype)
    ok = slot_mapping >= 0
    flat = cache.view(-1, kv_rank + rot_dim)
    flat[slot_mapping[ok]] = row[ok]
    return cq


def rotate_pack_queries(q, heads: int, dim: int, rot_dim: int, inv_freq, positions, out, lead: int):
    """out[r, h, lead:lead+rot_dim] = rotated q[r, h, dim:dim+rot_dim]; q is
    [R, heads*(dim+rot_dim)], out [R, heads, lead+rot_dim]."""
    R = q.shape[0]
    qr = q.view(R, heads, dim + rot_dim)[:, :, dim:]
    out[:, :, lead:] = _rotate_pairs(qr, positions, inv_freq).to(out.dtype)
    return out


def relu_squared(x: torch.Tensor) -> torch.Tensor:
    z = torch.relu(x.float())
    return (z * z).to(x.dtype)


def scale_gather_rows(x, idx, w) -> torch.Tensor:
    """out[i] = w[i] * x[idx[i]] (fp32 product, rounded to x's dtype); rows
    with idx < 0 come out zero."""
    ok = idx >= 0
    rows = x.float()[idx.clamp(min=0)] * (w.float() * ok)[:, None]
    return rows.to(x.dtype)


# -- post-norm residual, query/key norms with rotation, chunked and head-mixed
# -- attention, matrix-state recurrences ------------------------------------------

def scaled_add_rms_norm(x, alpha: float, w, eps: float, y1=None, s1: float = 1.0,
                        y2=None, s2: float = 1.0, out_dtype=None):
    """Norm after the sum: x <- rms(alpha * x + s1 * y1 + s2 * y2) * w, x fp32
    updated in place; also returned rounded to out_dtype.  Without y1 the
    rows are only normed (x is left as it is)."""
    if y1 is None:
        return x, (_rms_scale(x, eps) * w.float()).to(out_dtype)
    t = alpha * x + s1 * y1.float()
    if y2 is not None:
        t = t + s2 * y2.float()
    x.copy_(_rms_scale(t, eps) * w.float())
    return x, x.to(out_dtype)


def _rotate_halves(v: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """v [R, heads, dim]: entry i pairs with entry i + n (n = len(inv_freq))
    and the pair turns by positions * inv_freq[i]; entries from 2n on pass."""
    n = inv_freq.shape[0]
    out = v.float().clone()
    ang = positions.float()[:, None] * inv_freq[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = out[..., :n].clone(), out[..., n : 2 * n].clone()
    out[..., :n] = a * c - b * s
    out[..., n : 2 * n] = b * c + a * s
    return out


def qkv_norm_rope_cache(
    proj, heads: int, kv_heads: int, dim: int, vdim: int, qk_norm: str, w_q, w_k,
    eps: float, inv_freq, positions, v_source: str, v_unit_norm: bool, v_first,
    lam: float, want_v: bool, k_cache, v_cache, slot_mapping, rot_layout: str = "half",
):
    R = proj.shape[0]
    nq, nk = heads * dim, kv_heads * dim
    q, k = proj[:, :nq].float(), proj[:, nq : nq + nk].float()
    if v_source == "key":
        v = k.clone().view(R, kv_heads, vdim)
    else:
        v = proj[:, nq + nk : nq + nk + kv_heads * vdim].float().reshape(R, kv_heads, vdim)
    if qk_norm == "row":
        q = (_rms_scale(q, eps) * w_q.float()).view(R, heads, dim)
        k = (_rms_scale(k, eps) * w_k.float()).view(R, kv_heads, dim)
    elif qk_norm == "head":
        q = _rms_scale(q.reshape(R, heads, dim), eps) * w_q.float()
        k = _rms_scale(k.reshape(R, kv_heads, dim), eps) * w_k.float()
    else:
        q, k = q.reshape(R, heads, dim), k.reshape(R, kv_heads, dim)
    if inv_freq is not None and inv_freq.numel() > 0:
        rot = _rotate_halves if rot_layout == "half" else _rotate_pairs
        q = rot(q, positions, inv_freq)
        k = rot(k, positions, inv_freq)
    if qk_norm == "head_post":
        q, k = _rms_scale(q, eps), _rms_scale(k, eps)
    if v_unit_norm:
        v = _rms_scale(v, eps)
    if v_first is not None:
        v = (1.0 - lam) * v + lam * v_first.view(R, kv_heads, vdim)
    ok = slot_mapping >= 0
    bs = k_cache.shape[2]
    blk = torch.div(slot_mapping, bs, rounding_mode="floor")[ok]
    off = (slot_mapping % bs)[ok]
    k_cache[blk, :, off, :] = k[ok].to(k_cache.dtype)
    v_cache[blk, :, off, :] = v[ok].to(v_cache.dtype)
    return q.reshape(R, nq).to(proj.dtype), (v.reshape(R, kv_heads * vdim).clone() if want_v else None)


def paged_attention_chunked(
    q, k_cache, v_cache, block_tables, tok_seq, positions, scale: float, num_heads: int,
    chunk: int = 0, talk=None, dist_bias=None,
):
    """Token r sees keys j <= positions[r] of its sequence that lie in the
    same chunk (floor(j / chunk) == floor(p / chunk); chunk 0: all of them).
    Optional distance bias dist_bias[min(p - j, N - 1), head] added to the
    scaled score, optional mixing of the heads' scores with talk [H, H]
    before the softmax."""
    R = q.shape[0]
    nb, G, bs, D = k_cache.shape
    Dv = v_cache.shape[-1]
    H = num_heads
    out = torch.zeros(R, H * Dv, dtype=q.dtype, device=q.device)
    seqs, pos = tok_seq.tolist(), positions.tolist()
    for r in range(R):
        s, p = seqs[r], pos[r]
        if s < 0:
            continue
        lo = (p // chunk) * chunk if chunk > 0 else 0
        js = torch.arange(lo, p + 1, device=q.device)
        blk = block_tables[s].long()[js // bs]
        k = k_cache[blk, :, js % bs, :].float().repeat_interleave(H // G, dim=1)  # [L, H, D]
        v = v_cache[blk, :, js % bs, :].float().repeat_interleave(H // G, dim=1)
        sc = torch.einsum("hd,lhd->hl", q[r].float().view(H, D), k) * scale
        if dist_bias is not None:
            sc = sc + dist_bias.float()[(p - js).clamp(max=dist_bias.shape[0] - 1)].t()
        if talk is not None:
            sc = talk.float() @ sc
        pr = torch.softmax(sc, dim=-1)
        out[r] = torch.einsum("hl,lhd->hd", pr, v).reshape(H * Dv).to(out.dtype)
    return out


def token_shift_mix(x, mu, state, seg_start, seg_len, seg_slot, seg_fresh, out_dtype):
    """out[m] = x + (x_prev - x) * mu[m] for every row of every segment; the
    row before a segment's first is the sequence's state (zeros when the
    sequence starts here), which then takes the segment's last row.  Rows of
    no segment come out zero.  x fp32 [R, W], mu [n, W] -> [n, R, W]."""
    prev = torch.zeros_like(x)
    live = torch.zeros(x.shape[0], 1, dtype=torch.float32, device=x.device)
    for s0, cnt, slot, fresh in zip(
        seg_start.tolist(), seg_len.tolist(), seg_slot.tolist(), seg_fresh.tolist()
    ):
        if cnt <= 0:
            continue
        if not fresh:
            prev[s0] = state[slot]
        prev[s0 + 1 : s0 + cnt] = x[s0 : s0 + cnt - 1]
        state[slot] = x[s0 + cnt - 1]
        live[s0 : s0 + cnt] = 1.0
    return ((x[None] + (prev - x)[None] * mu.float()[:, None, :]) * live[None]).to(out_dtype)


def matrix_state_scan(
    q, k, v, state, seg_start, seg_len, seg_slot, seg_fresh, heads: int, dim: int,
    vdim: int, decay_pre=None, head_decay=None, bonus=None, act_silu: bool = False,
):
    """Per head a [dim, vdim] fp32 state S.  With `bonus` u (per head and key
    channel): o_t = (S + diag(u) k_t v_t^T)^T q_t, then S <- diag(w_t) S +
    k_t v_t^T with w_t = exp(-exp(decay_pre_t)).  Without: S <- d_h S + k_t
    v_t^T with the head's constant d_h, then o_t = S^T q_t.  act_silu applies
    silu to q, k and v first.  State rows [slots, heads*dim*vdim] are read
    unless the segment starts its sequence, and written back."""
    R = q.shape[0]
    f = (lambda t: torch.nn.functional.silu(t.float())) if act_silu else (lambda t: t.float())
    qf, kf, vf = f(q).view(R, heads, dim), f(k).view(R, heads, dim), f(v).view(R, heads, vdim)
    out = torch.zeros(R, heads, vdim, dtype=torch.float32, device=q.device)
    w = None
    if decay_pre is not None:
        w = torch.exp(-torch.exp(decay_pre.float())).view(R, heads, dim)
    for s0, n, slot, fresh in zip(
        seg_start.tolist(), seg_len.tolist(), seg_slot.tolist(), seg_fresh.tolist()
    ):
        if n <= 0:
            continue
        S = (
            torch.zeros(heads, dim, vdim, dtype=torch.float32, device=q.device)
            if fresh else state[slot, : heads * dim * vdim].view(heads, dim, vdim).clone()
        )
        for t in range(s0, s0 + n):
            kv = kf[t][:, :, None] * vf[t][:, None, :]
            if bonus is not None:
                out[t] = torch.einsum("hd,hde->he", qf[t], S + bonus.float().view(heads, dim, 1) * kv)
                S = w[t][:, :, None] * S + kv
            else:
                S = head_decay.float().view(heads, 1, 1) * S + kv
                out[t] = torch.einsum("hd,hde->he", qf[t], S)
        state[slot, : heads * dim * vdim] = S.reshape(-1)
    return out.view(R, heads * vdim)


def group_rms_norm_gate(o, gate, w, group: int, gate_act: str, eps: float, out_dtype):
    """Every `group` consecutive entries of a row are divided by their root
    mean square; then times w, times silu(gate) or sigmoid(gate)."""
    R, C = o.shape
    n = _rms_scale(o.view(R, C // group, group), eps).view(R, C) * w.float()
    g = gate.float()
    g = torch.nn.functional.silu(g) if gate_act == "silu" else torch.sigmoid(g)
    return (n * g).to(out_dtype)


def gelu_erf(x: torch.Tensor) -> torch.Tensor:
    z = x.float()
    return (0.5 * z * (1.0 + torch.erf(z * 0.7071067811865476))).to(x.dtype)


def tanh_act(x: torch.Tensor) -> torch.Tensor:
    return torch.tanh(x.float()).to(x.dtype)


def tanh_softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    return x.copy_(cap * torch.tanh(x.float() / cap))


def hyper_step(xs, y, mix, out_w, m: float, in_w, g, eps: float, out_dtype):
    """xs fp32 [R, S, W] in place: with y, x_t <- sum_s mix[s, t] x_s + m *
    out_w[t] * y; with in_w, returns rms(sum_t in_w[t] x_t) * g."""
    if y is not None:
        new = torch.einsum("st,rsw->rtw", mix.float(), xs) + (m * out_w.float())[None, :, None] * y.float()[:, None, :]
        xs.copy_(new)
    if in_w is None:
        return None
    u = torch.einsum("s,rsw->rw", in_w.float(), xs)
    return (_rms_scale(u, eps) * g.float().reshape(())).to(out_dtype)


def grouped_topk_route(z, correction, top: int, groups: int, keep: int):
    T, N = z.shape
    s = torch.softmax(z.float(), dim=-1)
    c = s if correction is None else s + correction.float()[None, :]
    if groups > 1 and keep < groups:
        per = N // groups
        gs = c.view(T, groups, per).max(dim=-1).values
        # stable order: ties go to the lower index
        order = torch.argsort(-gs, dim=-1, stable=True)[:, :keep]
        allowed = torch.zeros(T, groups, dtype=torch.bool, device=z.device).scatter_(1, order, True)
        c = c.masked_fill(~allowed.repeat_interleave(per, dim=1), float("-inf"))
    idx = torch.argsort(-c, dim=-1, stable=True)[:, :top]
    w = s.gather(1, idx)
    return idx.to(torch.int32), w / (w.sum(dim=-1, keepdim=True) + 1e-20)


def routed_combine(ye, x, rows, w):
    T, W = x.shape
    src = torch.cat([ye, x], dim=0).float()
    at = torch.where(rows >= 0, rows, ye.shape[0] + torch.arange(T, device=x.device)[:, None])
    return (src[at] * w[:, :, None]).sum(dim=1).to(x.dtype)


def glu_act(x, kind: str, limit: float, alpha: float):
    F_ = x.shape[1] // 2
    g, u = x[:, :F_].float(), x[:, F_:].float()
    if kind == "relu":
        return (torch.relu(g) * u).to(x.dtype)
    g = g.clamp(max=limit)
    u = u.clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(x.dtype)
