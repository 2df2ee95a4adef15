"""Engine ops: dispatch between the CDNA4 HIP extension and torch references.

Policy:
  * CUDA (= ROCm/HIP) tensors → the in-tree native extension
    ``llm_instance_gateway_amd._C`` (hand-written gfx950 kernels).  If the
    extension is missing on a GPU machine the op RAISES — no silent eager
    fallback (the driver records which .so files GPU processes load).
  * CPU tensors → the fp32 torch reference (`torch_ref`), which is also the
    ground truth the kernels are tested against.
  * ``LIG_FORCE_TORCH_OPS=1`` forces the torch path on GPU — for A/B numerics
    and perf comparisons only.
"""

from __future__ import annotations

import os
from typing import Optional, Tuple

import torch

from . import torch_ref

_EXT = None
_EXT_ERR: Optional[Exception] = None


def _load_ext():
    global _EXT, _EXT_ERR
    if _EXT is not None or _EXT_ERR is not None:
        return _EXT
    try:
        from llm_instance_gateway_amd import _C  # built in-tree by setup.py

        _EXT = _C
    except ImportError as e:
        _EXT_ERR = e
    return _EXT


def native_available() -> bool:
    return _load_ext() is not None


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _use_native(t: torch.Tensor) -> bool:
    if not t.is_cuda:
        return False
    if os.environ.get("LIG_FORCE_TORCH_OPS") == "1":
        return False
    ext = _load_ext()
    if ext is None:
        raise RuntimeError(
            "llm_instance_gateway_amd._C native extension is not built but a "
            "GPU tensor was passed; build it with `python setup.py "
            f"build_ext --inplace` (import error: {_EXT_ERR})"
        )
    return True


# -- public op surface -------------------------------------------------------

def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    if _use_native(x):
        out = torch.empty_like(x)
        _EXT.rms_norm(out, x, weight, eps, _stream())
        return out
    return torch_ref.rms_norm(x, weight, eps)


def fused_add_rms_norm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float
) -> Tuple[torch.Tensor, torch.Tensor]:
    if _use_native(x):
        # In-place: residual += x; x = rmsnorm(residual) written to out.
        out = torch.empty_like(x)
        _EXT.fused_add_rms_norm(out, x, residual, weight, eps, _stream())
        return out, residual
    return torch_ref.fused_add_rms_norm(x, residual, weight, eps)


def rotary_embedding(
    positions: torch.Tensor,
    q: torch.Tensor,
    k: torch.Tensor,
    cos_sin_cache: torch.Tensor,
    head_dim: int,
) -> Tuple[torch.Tensor, torch.Tensor]:
    if _use_native(q):
        _EXT.rotary_embedding(positions, q, k, cos_sin_cache, head_dim, _stream())
        return q, k
    return torch_ref.rotary_embedding(positions, q, k, cos_sin_cache, head_dim)


def reshape_and_cache(
    k: torch.Tensor,
    v: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> None:
    if _use_native(k):
        _EXT.reshape_and_cache(k, v, k_cache, v_cache, slot_mapping, _stream())
        return
    torch_ref.reshape_and_cache(k, v, k_cache, v_cache, slot_mapping)


# Flash-decoding context split (ROADMAP r01 #1, measured in
# profiles/r01_flash_decode_split.txt: 13.7x at N=4/ctx=16k, neutral at
# chip-filling batch).  The single-pass kernel launches N*Hkv workgroups;
# when that is far below the chip's 256 CUs and the context is long, split
# the context across `ns` workgroups + a combine pass (bit-exact merge).
_NUM_CUS = 256
_SPLIT_MIN_CTX = 1024      # short contexts: single-pass latency already fine
_SPLIT_MIN_PER_SPLIT = 256  # keep each split's K/V walk worth a workgroup
_SPLIT_MAX = 32
_SPLIT_SCRATCH: dict = {}   # device -> fp32 scratch tensor
# Superseded scratches stay referenced: a captured hipGraph bakes the pointer
# it saw, so freeing an old scratch after a grow would let the allocator hand
# that memory to live tensors the graph then scribbles over.
_SPLIT_SCRATCH_RETIRED: list = []


def decode_nsplits(n_seqs: int, n_kv_heads: int, max_ctx: int) -> int:
    """Context-split factor for the paged decode kernel (1 = single-pass)."""
    wg = n_seqs * n_kv_heads
    target = 2 * _NUM_CUS
    if wg == 0 or wg >= target or max_ctx < _SPLIT_MIN_CTX:
        return 1
    ns = min(_SPLIT_MAX, (target + wg - 1) // wg)
    ns = min(ns, max(1, max_ctx // _SPLIT_MIN_PER_SPLIT))
    return max(1, ns)


def split_scratch(device, numel: int) -> torch.Tensor:
    """fp32 partials scratch [N, Hq, ns, D+2] (flat).  Cached per device and
    grown monotonically; graph capture preallocates its max so every captured
    graph keeps one stable pointer."""
    t = _SPLIT_SCRATCH.get(device)
    if t is None or t.numel() < numel:
        if t is not None:
            _SPLIT_SCRATCH_RETIRED.append(t)
        t = torch.empty(numel, dtype=torch.float32, device=device)
        _SPLIT_SCRATCH[device] = t
    return t


def paged_attention_decode(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,
    context_lens: torch.Tensor,
    scale: float,
    max_ctx: int = 0,
    nsplits: int = 0,
) -> torch.Tensor:
    """`max_ctx` is a host-side hint (no device sync) driving the split
    heuristic; `nsplits` > 0 pins the factor (the hipGraph path captures a
    bucket-static value)."""
    if _use_native(q):
        out = torch.empty_like(q)
        N, Hq, D = q.shape
        Hkv = k_cache.shape[1]
        ns = nsplits if nsplits > 0 else decode_nsplits(N, Hkv, max_ctx)
        if ns > 1:
            scratch = split_scratch(q.device, N * Hq * ns * (D + 2))
            _EXT.paged_attention_decode_split(
                out, q, k_cache, v_cache, block_tables, context_lens,
                scratch, scale, ns, _stream()
            )
        else:
            _EXT.paged_attention_decode(
                out, q, k_cache, v_cache, block_tables, context_lens, scale,
                _stream()
            )
        return out
    return torch_ref.paged_attention_decode(
        q, k_cache, v_cache, block_tables, context_lens, scale
    )


def paged_attention_prefill(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,
    query_start_locs: torch.Tensor,
    context_lens: torch.Tensor,
    scale: float,
    tok_block_tables: "Optional[torch.Tensor]" = None,
    tok_context_lens: "Optional[torch.Tensor]" = None,
    tile_seq: "Optional[torch.Tensor]" = None,
    tile_qstart: "Optional[torch.Tensor]" = None,
) -> torch.Tensor:
    if _use_native(q):
        head_dim = q.shape[-1]
        if head_dim in (64, 128):
            # MFMA flash-prefill kernel over 64-row query tiles.
            if tile_seq is None or tile_qstart is None:
                qsl = query_start_locs.cpu().tolist()
                ts, tq = [], []
                for s in range(len(qsl) - 1):
                    for qb in range(0, qsl[s + 1] - qsl[s], 64):
                        ts.append(s)
                        tq.append(qb)
                dev = q.device
                tile_seq = torch.tensor(ts, dtype=torch.int32, device=dev)
                tile_qstart = torch.tensor(tq, dtype=torch.int32, device=dev)
            out = torch.empty_like(q)
            _EXT.paged_attention_prefill(
                out, q, k_cache, v_cache, tile_seq, tile_qstart,
                query_start_locs, context_lens, block_tables, scale, _stream()
            )
            return out
        if tok_block_tables is not None and tok_context_lens is not None:
            # per-token expansion precomputed once per step by the model runner
            return paged_attention_decode(
                q, k_cache, v_cache, tok_block_tables, tok_context_lens, scale
            )
        # v1 native path: run each chunk query row as a "decode" against its
        # causal context prefix (context = L - n + j + 1).  The GROUP waves of
        # a row share K/V lines via L1/L2, and consecutive rows of a chunk
        # walk overlapping context, so the re-read is largely cache-absorbed.
        # A fused MFMA flash-prefill kernel replaces this (see csrc/).
        n_per = (query_start_locs[1:] - query_start_locs[:-1]).long()
        ctx_end = context_lens.long()
        # per-token causal context length
        tok_in_chunk = torch.cat(
            [torch.arange(int(n), device=q.device) for n in n_per]
        )
        ctx_per_tok = (
            torch.repeat_interleave(ctx_end - n_per, n_per) + tok_in_chunk + 1
        ).int()
        bt_per_tok = torch.repeat_interleave(block_tables, n_per, dim=0).contiguous()
        return paged_attention_decode(
            q, k_cache, v_cache, bt_per_tok, ctx_per_tok, scale
        )
    return torch_ref.paged_attention_prefill(
        q, k_cache, v_cache, block_tables, query_start_locs, context_lens, scale
    )


def quant_fp8_rowwise(x: torch.Tensor):
    """Fused dynamic per-row e4m3 quantization: (x [T,K] bf16) ->
    (xq [T,K] float8_e4m3fn, xs [T,1] fp32) with x ≈ xq.float() * xs.
    One kernel launch vs ~4 for the torch elementwise path (models/quant.py)."""
    if _use_native(x):
        xq = torch.empty_like(x, dtype=torch.float8_e4m3fn)
        xs = torch.empty(x.shape[0], dtype=torch.float32, device=x.device)
        _EXT.quant_fp8_rowwise(xq, xs, x, _stream())
        return xq, xs.unsqueeze(1)
    # CPU reference of the KERNEL's exact semantics (amax clamp 1e-6,
    # matching models/quant.Fp8Linear._quant_input's activation path)
    amax = x.abs().amax(dim=-1, keepdim=True).float().clamp_(min=1e-6)
    xs = amax / 448.0
    xq = (x / xs).clamp_(-448.0, 448.0).to(torch.float8_e4m3fn)
    return xq, xs


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    if _use_native(x):
        d = x.shape[-1] // 2
        out = torch.empty(*x.shape[:-1], d, dtype=x.dtype, device=x.device)
        _EXT.silu_and_mul(out, x, _stream())
        return out
    return torch_ref.silu_and_mul(x)


build_cos_sin_cache = torch_ref.build_cos_sin_cache


def sgmv_shrink(x, a_stack, slots):
    if _use_native(x):
        T = x.shape[0]
        R = a_stack.shape[1]
        u = torch.zeros(T, R, dtype=x.dtype, device=x.device)
        _EXT.sgmv_shrink(u, x, a_stack, slots, _stream())
        return u
    return torch_ref.sgmv_shrink(x, a_stack, slots)


def sgmv_expand(u, b_stack, slots, y, scaling=1.0):
    if _use_native(u):
        _EXT.sgmv_expand(y, u, b_stack, slots, float(scaling), _stream())
        return
    torch_ref.sgmv_expand(u, b_stack, slots, y, scaling)


# MEASURED DEAD END (benchmarks/bench_gemm.py on MI355X): the hand-written
# skinny-M MFMA GEMM (ops/csrc/skinny_gemm.hip) reaches only ~0.5 TB/s of W
# streaming vs hipBLASLt's 2.4 TB/s at M=128 — and the CDNA guide's own
# best-effort decode-projection recipe tops out at 1.3-1.6 TB/s ("per-CU
# load-path/latency-bound ... nowhere near the HBM roofline").  hipBLASLt
# wins this regime; dispatch is disabled (LIG_SKINNY_GEMM_MAX_M to
# re-enable for experiments), kernel + microbench kept as evidence.
SKINNY_GEMM_MAX_M = int(os.environ.get("LIG_SKINNY_GEMM_MAX_M", "0"))


def linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """y = x @ weight.T (nn.Linear, no bias).  Dispatch: custom MFMA kernel
    for decode-sized M on GPU; library GEMM otherwise."""
    if (
        x.is_cuda
        and x.dtype == torch.bfloat16
        and 0 < x.shape[0] <= SKINNY_GEMM_MAX_M
        and weight.shape[1] % 32 == 0
        and weight.shape[0] % 64 == 0
        and _use_native(x)
    ):
        out = torch.empty(
            x.shape[0], weight.shape[0], dtype=x.dtype, device=x.device
        )
        _EXT.skinny_gemm(out, x.contiguous(), weight, _stream())
        return out
    return torch.nn.functional.linear(x, weight)


# -- hybrid-model mechanisms ---------------------------------------------------
# Grouped RMS norm over an fp32 residual, xIELU, the minGRU scan and paged
# attention for any head sizes live in the light ctypes library (ops/hybrid.py,
# plain C ABI, built by one hipcc call).  Storage dtype is bf16 or fp32; the
# math is fp32 either way.

def _use_hybrid(t: torch.Tensor) -> bool:
    if not t.is_cuda:
        return False
    return os.environ.get("LIG_FORCE_TORCH_OPS") != "1"


def _hl():
    from . import hybrid

    return hybrid.lib()


def _is_f32(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return 1
    if t.dtype == torch.bfloat16:
        return 0
    raise TypeError(f"hybrid kernels take bf16 or fp32 storage, got {t.dtype}")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def embed_group_norm(tokens, table, w, eps: float, groups: int) -> torch.Tensor:
    """residual[r] = group_norm(table[tokens[r]]) * w, fp32."""
    H = table.shape[1]
    assert H % groups == 0
    if _use_hybrid(table):
        R = tokens.shape[0]
        res = torch.empty(R, H, dtype=torch.float32, device=table.device)
        _hl().lig_embed_group_norm(
            _ptr(res), _ptr(table), _ptr(tokens), _ptr(w), float(eps), R, H,
            groups, _is_f32(table), _stream(),
        )
        return res
    return torch_ref.embed_group_norm(tokens, table, w, eps, groups)


def group_norm(residual, w, eps: float, groups: int) -> torch.Tensor:
    """fp32 residual -> normalised activations in w's dtype."""
    R, H = residual.shape
    assert residual.dtype == torch.float32 and H % groups == 0
    if _use_hybrid(residual):
        out = torch.empty(R, H, dtype=w.dtype, device=residual.device)
        _hl().lig_group_norm(
            _ptr(out), _ptr(residual), _ptr(w), float(eps), R, H, groups,
            _is_f32(w), _stream(),
        )
        return out
    return torch_ref.group_norm(residual, w, eps, groups, w.dtype)


def post_add_pre_norm(residual, y, w_post, w_pre, eps: float, groups: int):
    """residual += group_norm(y) * w_post (in place); returns
    group_norm(residual) * w_pre in y's dtype (None when w_pre is None)."""
    R, H = residual.shape
    assert residual.dtype == torch.float32 and y.shape == residual.shape
    if _use_hybrid(residual):
        assert y.is_contiguous() and residual.is_contiguous()
        out = None if w_pre is None else torch.empty_like(y)
        _hl().lig_post_add_pre_norm(
            _ptr(out), _ptr(residual), _ptr(y), _ptr(w_post), _ptr(w_pre),
            float(eps), R, H, groups, _is_f32(y), _stream(),
        )
        return out
    return torch_ref.post_add_pre_norm(residual, y, w_post, w_pre, eps, groups)


def xielu(x: torch.Tensor, a_pos: float, a_neg: float) -> torch.Tensor:
    if _use_hybrid(x):
        assert x.is_contiguous()
        out = torch.empty_like(x)
        _hl().lig_xielu(
            _ptr(out), _ptr(x), float(a_pos), float(a_neg), x.numel(),
            _is_f32(x), _stream(),
        )
        return out
    return torch_ref.xielu(x, a_pos, a_neg)


def sigmoid_gate_mul(x: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """x *= sigmoid(g) in place; g may be a column-block view (row stride)."""
    if _use_hybrid(x):
        assert x.is_contiguous() and g.stride(-1) == 1 and g.shape == x.shape
        R, C = x.shape
        _hl().lig_sigmoid_gate_mul(
            _ptr(x), _ptr(g), g.stride(0), R, C, _is_f32(x), _stream()
        )
        return x
    return torch_ref.sigmoid_gate_mul(x, g)


MINGRU_CHUNKED_MIN_LEN = 128


def mingru_scan(zxg, state, seg_start, seg_len, seg_slot, seg_fresh, max_len: int):
    """minGRU over the segments of a flat batch.  zxg [R, 3W] holds the gate
    and candidate pre-activations and the output gate; state [slots, W] fp32
    is read (unless the segment starts its sequence) and updated in place.
    Rows outside every segment are left untouched (undefined)."""
    R, W3 = zxg.shape
    W = W3 // 3
    assert state.dtype == torch.float32 and state.shape[1] == W
    if _use_hybrid(zxg):
        assert zxg.is_contiguous()
        out = torch.empty(R, W, dtype=zxg.dtype, device=zxg.device)
        es = zxg.element_size()
        base = zxg.data_ptr()
        # long portions: three-pass scan over 32-step chunks (scratch holds
        # each chunk's (decay product, local state) pair)
        scratch = None
        if max_len >= MINGRU_CHUNKED_MIN_LEN:
            nchunk = (int(max_len) + 31) // 32
            scratch = torch.empty(
                2 * seg_start.shape[0] * nchunk * W, dtype=torch.float32, device=zxg.device
            )
        _hl().lig_mingru_scan(
            _ptr(out), base, base + W * es, base + 2 * W * es, W3, _ptr(state),
            _ptr(scratch), _ptr(seg_start), _ptr(seg_len), _ptr(seg_slot), _ptr(seg_fresh),
            seg_start.shape[0], int(max_len), W, _is_f32(zxg), _stream(),
        )
        return out
    return torch_ref.mingru_scan(zxg, state, seg_start, seg_len, seg_slot, seg_fresh, W)


def kv_scatter(k, v, k_cache, v_cache, slot_mapping) -> None:
    """Write K [R, G*D] / V [R, G*Dv] rows (column-block views sharing one
    row stride) into caches whose K and V head sizes may differ."""
    if _use_hybrid(k):
        nb, G, bs, D = k_cache.shape
        Dv = v_cache.shape[-1]
        assert k.stride(0) == v.stride(0) and k.stride(1) == 1 and v.stride(1) == 1
        assert k.shape[1] == G * D and v.shape[1] == G * Dv
        assert k_cache.dtype == k.dtype and slot_mapping.dtype == torch.int64
        _hl().lig_kv_scatter(
            _ptr(k), _ptr(v), k.stride(0), _ptr(k_cache), _ptr(v_cache),
            _ptr(slot_mapping), k.shape[0], G, D, Dv, bs, _is_f32(k), _stream(),
        )
        return
    torch_ref.kv_scatter(k, v, k_cache, v_cache, slot_mapping)


def _value_row_stride(v_cache: torch.Tensor) -> int:
    """Entries between consecutive value rows of a [blocks, G, BS, Dv] cache
    (or of a view of the leading Dv entries of a wider cache's rows)."""
    nb, G, bs, Dv = v_cache.shape
    v_row = v_cache.stride(2)
    assert v_cache.stride(3) == 1 and v_row >= Dv
    assert v_cache.stride(1) == bs * v_row and v_cache.stride(0) == G * bs * v_row
    return v_row


def paged_attention_general(
    q, k_cache, v_cache, block_tables, tok_seq, positions, scale: float,
    num_heads: int, gate=None, temp_coef: float = 0.0, temp_every: float = 1.0,
    out: Optional[torch.Tensor] = None, sink: Optional[torch.Tensor] = None,
    chunk: int = 0, window: int = 0, score_bias: Optional[torch.Tensor] = None,
    weights: str = "softmax", gate_per_head: bool = False,
) -> torch.Tensor:
    """Causal paged attention for any key/value head sizes; token r of the
    flat batch attends keys 0..positions[r] of sequence tok_seq[r].  Optional
    query temperature 1 + coef*ln(floor((p+1)/every)+1), sigmoid output gate
    and per-head softmax sink (fp32 [heads]: exp(sink) joins the denominator).
    q/gate may be column-block views with a row stride; v_cache may be a view
    of the leading entries of k_cache's rows (a latent cache).  chunk > 0:
    only keys of the query's own chunk, floor(j/chunk) == floor(p/chunk).
    window > 0: only keys j with p - j < window.  weights "sigmoid": every
    visible key weighs sigmoid(score + score_bias[head]) (fp32 [heads],
    optional) and nothing is normalised.  gate_per_head: gate is [R, heads],
    one logistic gate per head."""
    assert weights in ("softmax", "sigmoid") and (weights == "sigmoid" or score_bias is None)
    if _use_hybrid(q):
        nb, G, bs, D = k_cache.shape
        Dv = v_cache.shape[-1]
        v_row = _value_row_stride(v_cache)
        if sink is not None:
            assert sink.dtype == torch.float32 and sink.shape == (num_heads,) and sink.is_contiguous()
        R = q.shape[0]
        assert q.shape[1] == num_heads * D and q.stride(1) == 1
        assert num_heads % G == 0 and Dv <= 512
        assert block_tables.dtype == torch.int32 and tok_seq.dtype == torch.int32
        assert positions.dtype == torch.int64 and block_tables.is_contiguous()
        if gate is not None:
            gcols = num_heads if gate_per_head else num_heads * Dv
            assert gate.shape == (R, gcols) and gate.stride(1) == 1 and gate.dtype == q.dtype
        if score_bias is not None:
            assert score_bias.dtype == torch.float32 and score_bias.shape == (num_heads,)
            assert score_bias.is_contiguous()
        if out is None:
            out = torch.empty(R, num_heads * Dv, dtype=q.dtype, device=q.device)
        assert out.shape == (R, num_heads * Dv) and out.is_contiguous() and out.dtype == q.dtype
        ev = float(temp_every)
        ev_int = int(ev) if ev == int(ev) and ev >= 1 else 0
        _hl().lig_paged_attention_general(
            _ptr(out), _ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache),
            _ptr(block_tables), block_tables.shape[1], _ptr(tok_seq),
            _ptr(positions), _ptr(gate), 0 if gate is None else gate.stride(0),
            _ptr(sink), float(scale), float(temp_coef), ev, ev_int, R, num_heads,
            G, D, Dv, v_row, bs, int(chunk), int(window), _ptr(score_bias),
            int(weights == "sigmoid"), int(bool(gate_per_head and gate is not None)),
            _is_f32(q), _stream(),
        )
        return out
    res = torch_ref.paged_attention_general(
        q, k_cache, v_cache, block_tables, tok_seq, positions, scale, num_heads,
        gate, temp_coef, temp_every, sink, chunk, window, score_bias, weights,
        gate_per_head,
    )
    if out is not None:
        out.copy_(res)
        return out
    return res


def temperature_scale_rows(q, positions, coef: float, every: float) -> torch.Tensor:
    """Contiguous copy of q [R, C] (may be a strided column block) with row r
    multiplied by 1 + coef*ln(floor((positions[r]+1)/every)+1)."""
    if _use_hybrid(q):
        R, C = q.shape
        assert q.stride(1) == 1 and positions.dtype == torch.int64
        out = torch.empty(R, C, dtype=q.dtype, device=q.device)
        ev = float(every)
        ev_int = int(ev) if ev == int(ev) and ev >= 1 else 0
        _hl().lig_temperature_scale_rows(
            _ptr(out), _ptr(q), q.stride(0), _ptr(positions), float(coef), ev,
            ev_int, R, C, _is_f32(q), _stream(),
        )
        return out
    return torch_ref.temperature_scale_rows(q, positions, coef, every)


def mfma_attention_supported(
    q_dtype, k_dim: int, v_dim: int, is_cuda: bool, group: int = 1
) -> bool:
    """The MFMA flash-prefill / paged-decode kernels of the torch extension
    serve bf16 caches with equal key and value head size 64 or 128 and at
    most 16 query heads per key/value head."""
    return (
        is_cuda
        and q_dtype == torch.bfloat16
        and k_dim == v_dim
        and k_dim in (64, 128)
        and 1 <= group <= 16
        and os.environ.get("LIG_FORCE_TORCH_OPS") != "1"
        and os.environ.get("LIG_GENERAL_ATTENTION") != "1"
        and native_available()
    )


def tiled_prefill_supported(q_dtype, k_dim: int, v_dim: int, is_cuda: bool) -> bool:
    """The MFMA prefill kernel of the light library: bf16, key and value head
    sizes independent, each a multiple of 8 and at most 128."""
    return (
        is_cuda
        and q_dtype == torch.bfloat16
        and k_dim % 8 == 0
        and v_dim % 8 == 0
        and 0 < k_dim <= 128
        and 0 < v_dim <= 128
        and os.environ.get("LIG_FORCE_TORCH_OPS") != "1"
        and os.environ.get("LIG_GENERAL_ATTENTION") != "1"
    )


def paged_attention_prefill_tiles(
    q, k_cache, v_cache, block_tables, query_start_locs, context_lens, tile_seq,
    tile_qstart, scale: float, num_heads: int, gate=None, temp_coef: float = 0.0,
    temp_every: float = 1.0, out: Optional[torch.Tensor] = None,
    sink: Optional[torch.Tensor] = None, chunk: int = 0, window: int = 0,
    score_bias: Optional[torch.Tensor] = None, weights: str = "softmax",
    gate_per_head: bool = False,
) -> torch.Tensor:
    """Prompt-partition attention on MFMA tiles for any head sizes the kernel
    takes (`tiled_prefill_supported`): q [Tp, H*D] (strided view allowed) are
    the rows of the step's prompt portions, laid out by query_start_locs;
    context_lens count each sequence's tokens after this step; tile_seq /
    tile_qstart name the 64-row query tiles.  Temperature, sigmoid gate and
    softmax sink are fused; v_cache may view the head of k_cache's rows; chunk
    > 0 restricts every row to the keys of its own chunk, window > 0 to the
    last `window` keys up to its own.  weights "sigmoid", score_bias and
    gate_per_head as in `paged_attention_general`.  GPU only."""
    assert weights in ("softmax", "sigmoid") and (weights == "sigmoid" or score_bias is None)
    nb, G, bs, D = k_cache.shape
    Dv = v_cache.shape[-1]
    v_row = _value_row_stride(v_cache)
    if sink is not None:
        assert sink.dtype == torch.float32 and sink.shape == (num_heads,) and sink.is_contiguous()
    Tp = q.shape[0]
    assert q.is_cuda and q.dtype == torch.bfloat16 and q.stride(1) == 1
    assert q.shape[1] == num_heads * D
    for t in (block_tables, query_start_locs, context_lens, tile_seq, tile_qstart):
        assert t.dtype == torch.int32 and t.is_contiguous()
    if gate is not None:
        gcols = num_heads if gate_per_head else num_heads * Dv
        assert gate.shape == (Tp, gcols) and gate.stride(1) == 1 and gate.dtype == q.dtype
    if score_bias is not None:
        assert score_bias.dtype == torch.float32 and score_bias.shape == (num_heads,)
        assert score_bias.is_contiguous()
    if out is None:
        out = torch.empty(Tp, num_heads * Dv, dtype=q.dtype, device=q.device)
    assert out.shape == (Tp, num_heads * Dv) and out.is_contiguous()
    ev = float(temp_every)
    ev_int = int(ev) if ev == int(ev) and ev >= 1 else 0
    rc = _hl().lig_paged_attention_prefill_tiles(
        _ptr(out), _ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(gate),
        0 if gate is None else gate.stride(0), _ptr(sink), _ptr(tile_seq),
        _ptr(tile_qstart), _ptr(query_start_locs), _ptr(context_lens),
        _ptr(block_tables), float(scale), float(temp_coef), ev, ev_int,
        tile_seq.shape[0], num_heads, G, D, Dv, v_row, bs, block_tables.shape[1],
        int(chunk), int(window), _ptr(score_bias), int(weights == "sigmoid"),
        int(bool(gate_per_head and gate is not None)), _stream(),
    )
    if rc != 0:
        raise RuntimeError("paged_attention_prefill_tiles: shape or alignment not served")
    return out


# -- token shift, latent attention, routed feed-forward -------------------------

def latent_rows_supported(q_dtype, row: int, v_dim: int, is_cuda: bool) -> bool:
    """The MFMA multi-query kernel over a latent cache: bf16, cache rows of
    up to 576 entries whose leading v_dim (up to 512) are the values, both
    multiples of 8."""
    return (
        is_cuda
        and q_dtype == torch.bfloat16
        and row % 8 == 0
        and v_dim % 8 == 0
        and 0 < v_dim <= min(row, 512)
        and row <= 576
        and os.environ.get("LIG_FORCE_TORCH_OPS") != "1"
        and os.environ.get("LIG_GENERAL_ATTENTION") != "1"
    )


def latent_rows_nsplit(rows: int, segs: int, heads: int, max_ctx: int) -> int:
    """Context slices for the latent row kernel: 1 when the step's rows fill
    the chip by themselves, else enough slices for about two workgroups per
    CU, each with at least 128 keys of the longest possible context."""
    blocks = (rows * heads + 63) // 64 + segs
    if blocks >= _NUM_CUS or max_ctx < 512:
        return 1
    return max(1, min(32, (2 * _NUM_CUS + blocks - 1) // blocks, max_ctx // 128))


def latent_attention_rows(
    q, cache, v_dim: int, block_tables, seg_start, seg_len, seg_ctx, max_seg_len: int,
    scale: float, num_heads: int, sink: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None, nsplit: int = 0,
) -> torch.Tensor:
    """Causal multi-query attention of every segment of the step (prompt
    portions and single tokens alike) over the paged latent cache
    [blocks, 1, block_size, row]: keys are whole rows, values their leading
    v_dim entries, all heads of a token share them.  q [R, heads*row]
    contiguous; segment s covers rows seg_start[s] .. +seg_len[s] of the flat
    batch, belongs to row s of block_tables and holds seg_ctx[s] tokens after
    this step.  Rows of no segment are left untouched.  nsplit > 1 cuts every
    tile's visible keys into that many slices run by separate workgroups and
    merged afterwards (0: chosen from the row count and the longest context
    the block tables can hold).  GPU, bf16."""
    nb, G, bs, row = cache.shape
    R = q.shape[0]
    assert G == 1 and q.is_cuda and q.dtype == torch.bfloat16 and cache.dtype == q.dtype
    assert q.is_contiguous() and q.shape[1] == num_heads * row and cache.is_contiguous()
    for t in (block_tables, seg_start, seg_len, seg_ctx):
        assert t.dtype == torch.int32 and t.is_contiguous()
    S = seg_start.shape[0]
    assert block_tables.shape[0] >= S and seg_len.shape[0] == S and seg_ctx.shape[0] == S
    if sink is not None:
        assert sink.dtype == torch.float32 and sink.shape == (num_heads,) and sink.is_contiguous()
    if out is None:
        out = torch.empty(R, num_heads * v_dim, dtype=q.dtype, device=q.device)
    assert out.shape == (R, num_heads * v_dim) and out.is_contiguous() and out.dtype == q.dtype
    if nsplit <= 0:
        nsplit = latent_rows_nsplit(R, S, num_heads, block_tables.shape[1] * bs)
    scratch = None
    if nsplit > 1:
        scratch = split_scratch(q.device, R * num_heads * nsplit * (v_dim + 4))
    rc = _hl().lig_latent_attention_rows(
        _ptr(out), _ptr(q), _ptr(cache), _ptr(sink), _ptr(seg_start), _ptr(seg_len),
        _ptr(seg_ctx), _ptr(block_tables), block_tables.shape[1], float(scale), S,
        int(max_seg_len), num_heads, row, v_dim, bs, int(nsplit), _ptr(scratch), _stream(),
    )
    if rc != 0:
        raise RuntimeError("latent_attention_rows: shape or alignment not served")
    return out


def residual_add(x: torch.Tensor, a: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x += a (+ b) in place; x is the fp32 residual, a and b branch outputs."""
    assert x.dtype == torch.float32 and a.shape == x.shape and (b is None or b.shape == x.shape)
    if _use_hybrid(x):
        assert x.is_contiguous() and a.is_contiguous() and (b is None or b.is_contiguous())
        assert b is None or b.dtype == a.dtype
        _hl().lig_residual_add(_ptr(x), _ptr(a), _ptr(b), x.numel(), _is_f32(a), _stream())
        return x
    return torch_ref.residual_add(x, a, b)


def offset_rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """fp32 rows -> x / rms(x) * (1 + w) in w's dtype."""
    assert x.dtype == torch.float32
    if _use_hybrid(x):
        R, H = x.shape
        assert x.is_contiguous()
        out = torch.empty(R, H, dtype=w.dtype, device=x.device)
        _hl().lig_offset_rms_norm(_ptr(out), _ptr(x), _ptr(w), float(eps), R, H, _is_f32(w), _stream())
        return out
    return torch_ref.offset_rms_norm(x, w, eps, w.dtype)


def offset_norm_shift(
    x, w_mix, w_ff, mu, state, tok_seq, seg_start, seg_len, seg_slot, seg_fresh, eps: float,
    add_a: Optional[torch.Tensor] = None, add_b: Optional[torch.Tensor] = None,
):
    """Both input norms of a parallel layer from one pass over the fp32
    residual x [R, H] (weights stored as offsets from one), with the mixer
    branch blended with the previous token's, h + (h_prev - h) * mu.  `state`
    [slots, H] fp32 carries each sequence's last unblended h between steps
    and is updated in place.  w_ff None: no feed-forward branch.

    add_a (and add_b): the previous layer's branch outputs, added on the way
    in; the norms then read x + (add_a + add_b), which is returned as a new
    residual tensor (x itself is left as it was).

    Returns (mixer input, feed-forward input or None, residual) in w_mix's
    dtype / fp32; rows of no segment are zero."""
    assert x.dtype == torch.float32 and state.dtype == torch.float32
    assert add_b is None or add_a is not None
    if _use_hybrid(x):
        R, H = x.shape
        assert x.is_contiguous() and state.shape[1] == H and state.is_contiguous()
        hm = torch.empty(R, H, dtype=w_mix.dtype, device=x.device)
        hf = None if w_ff is None else torch.empty_like(hm)
        x_out = x
        if add_a is not None:
            assert add_a.shape == x.shape and add_a.is_contiguous() and add_a.dtype == w_mix.dtype
            assert add_b is None or (add_b.shape == x.shape and add_b.is_contiguous() and add_b.dtype == add_a.dtype)
            x_out = torch.empty_like(x)
        _hl().lig_offset_norm_shift(
            _ptr(hm), _ptr(hf), _ptr(x), _ptr(add_a), _ptr(add_b),
            _ptr(x_out) if add_a is not None else None, _ptr(w_mix), _ptr(w_ff), _ptr(mu),
            _ptr(state), _ptr(tok_seq), _ptr(seg_start), _ptr(seg_len), _ptr(seg_slot),
            _ptr(seg_fresh), float(eps), R, H, _is_f32(w_mix), _stream(),
        )
        return hm, hf, x_out
    if add_a is not None:
        x = torch_ref.residual_add(x.clone(), add_a, add_b)
    hm, hf = torch_ref.offset_norm_shift(
        x, w_mix, w_ff, mu, state, tok_seq, seg_start, seg_len, seg_slot, seg_fresh, eps,
        w_mix.dtype,
    )
    return hm, hf, x


rotary_inv_freq = torch_ref.rotary_inv_freq


def latent_kv_prep(
    proj, q_rank: int, kv_rank: int, rot_dim: int, w_q, w_kv, eps: float, inv_freq,
    positions, slot_mapping, cache,
) -> torch.Tensor:
    """Per row of the fused projection [query latent | key/value latent |
    shared rotated key part | ...]: returns the RMS-normed query latent and
    writes [normed key/value latent | rotated key part] into the paged latent
    cache [blocks, 1, block_size, kv_rank + rot_dim] at slot_mapping."""
    if _use_hybrid(proj):
        R = proj.shape[0]
        assert proj.stride(1) == 1 and proj.shape[1] >= q_rank + kv_rank + rot_dim
        assert cache.is_contiguous() and cache.shape[1] == 1 and cache.shape[3] == kv_rank + rot_dim
        assert cache.dtype == proj.dtype and inv_freq.dtype == torch.float32
        assert positions.dtype == torch.int64 and slot_mapping.dtype == torch.int64
        assert 2 * inv_freq.shape[0] <= rot_dim
        cq = torch.empty(R, q_rank, dtype=proj.dtype, device=proj.device)
        _hl().lig_latent_kv_prep(
            _ptr(cq), _ptr(proj), proj.stride(0), _ptr(w_q), _ptr(w_kv), _ptr(inv_freq),
            inv_freq.shape[0], _ptr(positions), _ptr(slot_mapping), _ptr(cache), float(eps),
            R, q_rank, kv_rank, rot_dim, _is_f32(proj), _stream(),
        )
        return cq
    return torch_ref.latent_kv_prep(
        proj, q_rank, kv_rank, rot_dim, w_q, w_kv, eps, inv_freq, positions, slot_mapping, cache
    )


def rotate_pack_queries(q, heads: int, dim: int, rot_dim: int, inv_freq, positions, out, lead: int):
    """out[r, h, lead:] = interleaved rotation of q[r, h, dim:dim+rot_dim];
    q [R, heads*(dim+rot_dim)] contiguous, out [R, heads, lead+rot_dim]."""
    if _use_hybrid(q):
        R = q.shape[0]
        assert q.is_contiguous() and out.is_contiguous() and out.dtype == q.dtype
        assert out.shape == (R, heads, lead + rot_dim) and positions.dtype == torch.int64
        _hl().lig_rotate_pack_queries(
            _ptr(out), _ptr(q), _ptr(inv_freq), inv_freq.shape[0], _ptr(positions), R,
            heads, dim, rot_dim, lead, _is_f32(q), _stream(),
        )
        return out
    return torch_ref.rotate_pack_queries(q, heads, dim, rot_dim, inv_freq, positions, out, lead)


def relu_squared(x: torch.Tensor) -> torch.Tensor:
    if _use_hybrid(x):
        assert x.is_contiguous()
        out = torch.empty_like(x)
        _hl().lig_relu_squared(_ptr(out), _ptr(x), x.numel(), _is_f32(x), _stream())
        return out
    return torch_ref.relu_squared(x)


def silu_mul(x: torch.Tensor) -> torch.Tensor:
    """[rows, 2F] fused (gate | up) -> silu(gate) * up [rows, F]; the light
    library's own kernel (bf16 or fp32 storage)."""
    if _use_hybrid(x):
        assert x.is_contiguous() and x.dim() == 2 and x.shape[1] % 2 == 0
        F_ = x.shape[1] // 2
        out = torch.empty(x.shape[0], F_, dtype=x.dtype, device=x.device)
        _hl().lig_silu_mul(_ptr(out), _ptr(x), x.shape[0], F_, _is_f32(x), _stream())
        return out
    return torch_ref.silu_and_mul(x)


def scale_gather_rows(x: torch.Tensor, idx: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """out[i] = w[i] * x[idx[i]]; idx int64 (negative: zero row), w fp32."""
    if _use_hybrid(x):
        assert x.is_contiguous() and idx.dtype == torch.int64 and w.dtype == torch.float32
        assert idx.is_contiguous() and w.is_contiguous() and idx.shape == w.shape
        out = torch.empty(idx.shape[0], x.shape[1], dtype=x.dtype, device=x.device)
        _hl().lig_scale_gather_rows(
            _ptr(out), _ptr(x), _ptr(idx), _ptr(w), idx.shape[0], x.shape[1], _is_f32(x), _stream()
        )
        return out
    return torch_ref.scale_gather_rows(x, idx, w)


# -- post-norm residual, normed/rotated attention inputs, chunked and
# -- head-mixed attention, matrix-state recurrences ----------------------------------

def scaled_add_rms_norm(
    x: torch.Tensor, alpha: float, w: torch.Tensor, eps: float,
    y1: Optional[torch.Tensor] = None, s1: float = 1.0,
    y2: Optional[torch.Tensor] = None, s2: float = 1.0,
):
    """Norm after the sum on the fp32 residual x [R, H], in place:
    x <- rms(alpha * x + s1 * y1 + s2 * y2) * w.  Returns (x, x rounded to
    w's dtype), the second being the next sub-layer's GEMM input.  Without y1
    the rows are only normed and x stays as it is."""
    assert x.dtype == torch.float32 and (y2 is None or y1 is not None)
    if _use_hybrid(x):
        R, H = x.shape
        assert x.is_contiguous() and w.shape == (H,)
        for y in (y1, y2):
            assert y is None or (y.shape == x.shape and y.is_contiguous() and y.dtype == w.dtype)
        h = torch.empty(R, H, dtype=w.dtype, device=x.device)
        _hl().lig_scaled_add_rms_norm(
            _ptr(x), _ptr(h), _ptr(y1), _ptr(y2), _ptr(w), float(alpha), float(s1),
            float(s2), float(eps), R, H, _is_f32(w), _stream(),
        )
        return x, h
    return torch_ref.scaled_add_rms_norm(x, alpha, w, eps, y1, s1, y2, s2, w.dtype)


_QK_NORM_MODES = {"none": 0, "row": 1, "head": 2, "head_post": 3}


def qkv_norm_rope_cache(
    proj, heads: int, kv_heads: int, dim: int, vdim: int, qk_norm: str, w_q, w_k,
    eps: float, inv_freq, positions, k_cache, v_cache, slot_mapping,
    v_source: str = "proj", v_unit_norm: bool = False, v_first=None, lam: float = 0.0,
    want_v: bool = False, rot_layout: str = "half",
):
    """Everything between the fused input projection and the attention
    kernel, one pass per token row of proj = [q | k | v] (or [q | k] with
    v_source "key": the values are the keys as projected).

    qk_norm "row": RMS norm over all of q (and of k) with weights of that
    size; "head": per head, one weight of size dim shared by the heads;
    "none"; "head_post": per head AFTER the rotation, without weights.  The
    rotation turns the first 2*len(inv_freq) entries of every q and k head
    (inv_freq None: no rotation); rot_layout "half" pairs entry i with entry
    i + len(inv_freq), "interleaved" pairs entry 2i with 2i + 1.  Values: optionally
    divided per head by their root mean square, optionally blended with
    v_first (fp32 [R, kv_heads*vdim]) as (1 - lam) v + lam v_first.  Keys and
    values go to the paged caches at slot_mapping; returns (q [R, heads*dim]
    contiguous, the values as cached in fp32 if want_v else None)."""
    mode = _QK_NORM_MODES[qk_norm]
    assert rot_layout in ("half", "interleaved")
    from_key = v_source == "key"
    assert v_source in ("proj", "key") and (not from_key or vdim == dim)
    if _use_hybrid(proj):
        R = proj.shape[0]
        nq, nk, nv = heads * dim, kv_heads * dim, kv_heads * vdim
        assert proj.stride(1) == 1 and proj.shape[1] >= nq + nk + (0 if from_key else nv)
        nb, G, bs, D = k_cache.shape
        assert G == kv_heads and D == dim and v_cache.shape == (nb, G, bs, vdim)
        assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == proj.dtype
        assert positions.dtype == torch.int64 and slot_mapping.dtype == torch.int64
        if mode == 1:
            assert w_q.shape == (nq,) and w_k.shape == (nk,)
        elif mode == 2:
            assert w_q.shape == (dim,) and w_k.shape == (dim,)
        nf = 0
        if inv_freq is not None and inv_freq.numel() > 0:
            nf = inv_freq.shape[0]
            assert inv_freq.dtype == torch.float32 and 2 * nf <= dim
        if v_first is not None:
            assert v_first.dtype == torch.float32 and v_first.shape == (R, nv) and v_first.is_contiguous()
        q_out = torch.empty(R, nq, dtype=proj.dtype, device=proj.device)
        v_out = torch.empty(R, nv, dtype=torch.float32, device=proj.device) if want_v else None
        _hl().lig_qkv_norm_rope_cache(
            _ptr(q_out), _ptr(v_out), _ptr(proj), proj.stride(0),
            _ptr(w_q) if mode in (1, 2) else None, _ptr(w_k) if mode in (1, 2) else None, _ptr(inv_freq) if nf else None, nf, _ptr(positions),
            _ptr(v_first), float(lam), _ptr(k_cache), _ptr(v_cache), _ptr(slot_mapping),
            float(eps), R, heads, kv_heads, dim, vdim, mode, int(from_key),
            int(bool(v_unit_norm)), bs, int(rot_layout == "interleaved"), _is_f32(proj),
            _stream(),
        )
        return q_out, v_out
    return torch_ref.qkv_norm_rope_cache(
        proj, heads, kv_heads, dim, vdim, qk_norm, w_q, w_k, eps, inv_freq, positions,
        v_source, v_unit_norm, v_first, lam, want_v, k_cache, v_cache, slot_mapping,
        rot_layout,
    )


def distance_bias_table(rel: torch.Tensor, far: float) -> torch.Tensor:
    """Expand a bucketed distance table rel [rows, H] into one row per
    distance, fp32 [N, H]: distance n < rows/2 reads row n, larger distances
    row rows/2 + floor(ln(n / (rows/2)) / ln(far / (rows/2)) * (rows - rows/2)),
    capped at the last row.  The table stops at the first distance that
    reaches the last row; all larger distances read that entry."""
    import math

    rows = rel.shape[0]
    half = rows // 2
    idx = []
    n = 0
    while True:
        if n < half:
            b = n
        else:
            b = min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))
        idx.append(b)
        if b == rows - 1 or n > (1 << 22):
            break
        n += 1
    return rel.float()[torch.tensor(idx, dtype=torch.long, device=rel.device)].contiguous()


def paged_attention_mixed_heads(
    q, k_cache, v_cache, block_tables, tok_seq, positions, scale: float, num_heads: int,
    dist_bias: Optional[torch.Tensor] = None, talk: Optional[torch.Tensor] = None,
    chunk: int = 0, out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Causal paged attention whose heads are not independent: token r sees
    keys j <= p = positions[r] of its sequence inside its chunk
    (floor(j/chunk) == floor(p/chunk); chunk 0: all); the scaled score of
    head g gets dist_bias[min(p - j, N - 1), g] (fp32 [N, H]) added, then the
    heads' scores are mixed, s_h <- sum_g talk[h, g] s_g (fp32 [H, H]),
    before an ordinary softmax per head.  One workgroup per token holds all
    heads' scores of a key tile.  Any head sizes, bf16 or fp32 storage."""
    nb, G, bs, D = k_cache.shape
    Dv = v_cache.shape[-1]
    R = q.shape[0]
    if _use_hybrid(q):
        assert q.shape[1] == num_heads * D and q.stride(1) == 1 and num_heads % G == 0
        assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == q.dtype
        assert block_tables.dtype == torch.int32 and tok_seq.dtype == torch.int32
        assert positions.dtype == torch.int64 and block_tables.is_contiguous()
        for t, shp in ((dist_bias, None), (talk, (num_heads, num_heads))):
            if t is not None:
                assert t.dtype == torch.float32 and t.is_contiguous()
                assert shp is None or t.shape == shp
        if dist_bias is not None:
            assert dist_bias.dim() == 2 and dist_bias.shape[1] == num_heads
        if out is None:
            out = torch.empty(R, num_heads * Dv, dtype=q.dtype, device=q.device)
        assert out.shape == (R, num_heads * Dv) and out.is_contiguous() and out.dtype == q.dtype
        rc = _hl().lig_paged_attention_mixed_heads(
            _ptr(out), _ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(block_tables),
            block_tables.shape[1], _ptr(tok_seq), _ptr(positions), _ptr(dist_bias),
            0 if dist_bias is None else dist_bias.shape[0], _ptr(talk), float(scale),
            int(chunk), R, num_heads, G, D, Dv, bs, _is_f32(q), _stream(),
        )
        if rc != 0:
            raise RuntimeError("paged_attention_mixed_heads: more than 64 heads or values wider than 256")
        return out
    rel = dist_bias
    res = torch_ref.paged_attention_chunked(
        q, k_cache, v_cache, block_tables, tok_seq, positions, scale, num_heads, chunk,
        talk=talk, dist_bias=rel,
    )
    if out is not None:
        out.copy_(res)
        return out
    return res


def mixed_heads_tiles_supported(q_dtype, k_dim: int, v_dim: int, heads: int, is_cuda: bool) -> bool:
    """The MFMA head-mixing kernel for prompt rows: bf16, head sizes multiples
    of 8 up to 128, at most 32 heads (a workgroup holds all heads: one wave
    per head up to 16, two heads per wave beyond)."""
    return (
        is_cuda
        and q_dtype == torch.bfloat16
        and k_dim % 8 == 0
        and v_dim % 8 == 0
        and 0 < k_dim <= 128
        and 0 < v_dim <= 128
        and 1 <= heads <= 32
        and os.environ.get("LIG_FORCE_TORCH_OPS") != "1"
        and os.environ.get("LIG_GENERAL_ATTENTION") != "1"
    )


def paged_attention_mixed_heads_tiles(
    q, k_cache, v_cache, block_tables, query_start_locs, context_lens, tile_seq,
    tile_qstart, scale: float, num_heads: int, dist_bias: Optional[torch.Tensor] = None,
    talk: Optional[torch.Tensor] = None, chunk: int = 0, out: Optional[torch.Tensor] = None,
) -> Optional[torch.Tensor]:
    """`paged_attention_mixed_heads` for the step's prompt portions on MFMA
    tiles: q [Tp, H*D] (strided view allowed) laid out by query_start_locs,
    context_lens count each sequence's tokens after this step, tile_seq /
    tile_qstart name the 64-row query tiles (each is run as four 16-row
    workgroups that hold all heads).  Returns None when the shape does not
    fit the kernel's LDS budget (the caller then uses the any-shape kernel).
    GPU, bf16."""
    nb, G, bs, D = k_cache.shape
    Dv = v_cache.shape[-1]
    Tp = q.shape[0]
    assert q.is_cuda and q.dtype == torch.bfloat16 and q.stride(1) == 1
    assert q.shape[1] == num_heads * D and k_cache.is_contiguous() and v_cache.is_contiguous()
    for t in (block_tables, query_start_locs, context_lens, tile_seq, tile_qstart):
        assert t.dtype == torch.int32 and t.is_contiguous()
    for t in (dist_bias, talk):
        assert t is None or (t.dtype == torch.float32 and t.is_contiguous())
    assert dist_bias is None or (dist_bias.dim() == 2 and dist_bias.shape[1] == num_heads)
    assert talk is None or talk.shape == (num_heads, num_heads)
    if out is None:
        out = torch.empty(Tp, num_heads * Dv, dtype=q.dtype, device=q.device)
    assert out.shape == (Tp, num_heads * Dv) and out.is_contiguous()
    rc = _hl().lig_paged_attention_mixed_heads_tiles(
        _ptr(out), _ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(dist_bias),
        0 if dist_bias is None else dist_bias.shape[0], _ptr(talk), _ptr(tile_seq),
        _ptr(tile_qstart), _ptr(query_start_locs), _ptr(context_lens), _ptr(block_tables),
        float(scale), int(chunk), tile_seq.shape[0], num_heads, G, D, Dv, bs,
        block_tables.shape[1], _stream(),
    )
    return out if rc == 0 else None


def token_shift_mix(x, mu, state, tok_seq, seg_start, seg_len, seg_slot, seg_fresh) -> torch.Tensor:
    """Several blends of every row with the row before it, from one pass:
    out[m] = x + (x_prev - x) * mu[m], x fp32 [R, W], mu [n, W] -> [n, R, W]
    in mu's dtype.  Ahead of a segment's first row stands the sequence's
    state row (zeros when the sequence starts here); the state [slots, W]
    fp32 then takes the segment's last row.  Rows of no segment are zero."""
    assert x.dtype == torch.float32 and state.dtype == torch.float32
    if _use_hybrid(x):
        R, W = x.shape
        n = mu.shape[0]
        assert x.is_contiguous() and mu.is_contiguous() and mu.shape == (n, W)
        assert state.is_contiguous() and state.shape[1] == W
        out = torch.empty(n, R, W, dtype=mu.dtype, device=x.device)
        _hl().lig_token_shift_mix(
            _ptr(out), _ptr(x), _ptr(mu), _ptr(state), _ptr(tok_seq), _ptr(seg_start),
            _ptr(seg_len), _ptr(seg_slot), _ptr(seg_fresh), n, R, W, _is_f32(mu), _stream(),
        )
        return out
    return torch_ref.token_shift_mix(x, mu, state, seg_start, seg_len, seg_slot, seg_fresh, mu.dtype)


# key channels per thread the scan kernel is instantiated for
MATRIX_STATE_KEY_CLASSES = (4, 8, 12, 16, 24, 32, 48, 64)


def matrix_state_width(heads: int, dim: int, vdim: int) -> int:
    """fp32 entries of one sequence's matrix state: the scan kernel splits a
    head's key channels over 8 lanes (heads of 32 or more key channels whose
    8 * vdim threads fit a workgroup) or 4, and keeps the state in the order
    its threads hold it, key channels padded to the split times the kernel's
    size class."""
    split = 8 if dim >= 32 and vdim * 8 <= 1024 else 4
    need = (dim + split - 1) // split
    kpt = next((c for c in MATRIX_STATE_KEY_CLASSES if c >= need), None)
    if kpt is None:
        raise ValueError(f"matrix-state heads hold at most 256 key channels, got {dim}")
    return heads * split * kpt * vdim


def matrix_state_scan(
    q, k, v, state, seg_start, seg_len, seg_slot, seg_fresh, heads: int, dim: int,
    vdim: int, decay_pre=None, head_decay=None, bonus=None, act_silu: bool = False,
) -> torch.Tensor:
    """Linear recurrences with one [dim, vdim] fp32 state matrix S per head,
    over the segments of the flat batch; q, k [R, heads*dim] and v
    [R, heads*vdim] may be column-block views.

    With `bonus` u (fp32 [heads*dim]) and decay_pre (fp32 [R, heads*dim]):
        o_t = (S + diag(u) k_t v_t^T)^T q_t;  S <- diag(w_t) S + k_t v_t^T,
        w_t = exp(-exp(decay_pre_t))
    With head_decay d (fp32 [heads]):
        S <- d_h S + k_t v_t^T;  o_t = S^T q_t
    act_silu applies silu to q, k, v on the way in.  state [slots,
    matrix_state_width] is read unless the segment starts its sequence and
    written back; its layout is private to the implementation.  Returns fp32
    [R, heads*vdim]; rows of no segment are left untouched (undefined)."""
    assert (bonus is None) == (decay_pre is None) and (bonus is None) != (head_decay is None)
    assert state.dtype == torch.float32
    if _use_hybrid(q):
        R = q.shape[0]
        assert q.shape[1] == heads * dim and k.shape[1] == heads * dim and v.shape[1] == heads * vdim
        assert q.stride(1) == 1 and k.stride(1) == 1 and v.stride(1) == 1
        assert q.dtype == k.dtype == v.dtype
        assert state.is_contiguous() and state.shape[1] == matrix_state_width(heads, dim, vdim)
        for t, n in ((decay_pre, R * heads * dim), (bonus, heads * dim), (head_decay, heads)):
            if t is not None:
                assert t.dtype == torch.float32 and t.is_contiguous() and t.numel() == n
        S = seg_start.shape[0]
        out = torch.empty(R, heads * vdim, dtype=torch.float32, device=q.device)
        rc = _hl().lig_matrix_state_scan(
            _ptr(out), _ptr(q), q.stride(0), _ptr(k), k.stride(0), _ptr(v), v.stride(0),
            _ptr(decay_pre), _ptr(head_decay), _ptr(bonus), _ptr(state), state.stride(0),
            _ptr(seg_start), _ptr(seg_len), _ptr(seg_slot), _ptr(seg_fresh), S, heads, dim,
            vdim, int(bool(act_silu)), _is_f32(q), _stream(),
        )
        if rc != 0:
            raise RuntimeError("matrix_state_scan: keys or values wider than 256 per head")
        return out
    return torch_ref.matrix_state_scan(
        q, k, v, state, seg_start, seg_len, seg_slot, seg_fresh, heads, dim, vdim,
        decay_pre, head_decay, bonus, act_silu,
    )


def group_rms_norm_gate(o, gate, w, group: int, gate_act: str, eps: float) -> torch.Tensor:
    """o fp32 [R, C]: every `group` consecutive entries are divided by their
    root mean square (group == C: the whole row), then times w [C], times
    silu(gate) or sigmoid(gate); gate [R, C] may be a column-block view.
    Result in w's dtype."""
    assert o.dtype == torch.float32 and gate_act in ("silu", "sigmoid")
    R, C = o.shape
    assert C % group == 0 and gate.shape == (R, C) and w.shape == (C,)
    if _use_hybrid(o):
        assert o.is_contiguous() and gate.stride(1) == 1 and gate.dtype == w.dtype
        out = torch.empty(R, C, dtype=w.dtype, device=o.device)
        _hl().lig_group_rms_norm_gate(
            _ptr(out), _ptr(o), _ptr(gate), gate.stride(0), _ptr(w), int(group),
            1 if gate_act == "silu" else 0, float(eps), R, C, _is_f32(w), _stream(),
        )
        return out
    return torch_ref.group_rms_norm_gate(o, gate, w, group, gate_act, eps, w.dtype)


def gelu_erf(x: torch.Tensor) -> torch.Tensor:
    """The exact gelu, 0.5 z (1 + erf(z / sqrt 2))."""
    if _use_hybrid(x):
        assert x.is_contiguous()
        out = torch.empty_like(x)
        _hl().lig_gelu_erf(_ptr(out), _ptr(x), x.numel(), _is_f32(x), _stream())
        return out
    return torch_ref.gelu_erf(x)


def tanh_act(x: torch.Tensor) -> torch.Tensor:
    if _use_hybrid(x):
        assert x.is_contiguous()
        out = torch.empty_like(x)
        _hl().lig_tanh_act(_ptr(out), _ptr(x), x.numel(), _is_f32(x), _stream())
        return out
    return torch_ref.tanh_act(x)


def tanh_softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x <- cap * tanh(x / cap) in place on fp32 logits."""
    assert x.dtype == torch.float32
    if _use_hybrid(x):
        assert x.is_contiguous()
        _hl().lig_tanh_softcap(_ptr(x), float(cap), x.numel(), _stream())
        return x
    return torch_ref.tanh_softcap(x, cap)


# -- multi-stream residual, grouped router, routed combine ------------------------------

def hyper_step(
    xs: torch.Tensor, y: Optional[torch.Tensor], mix: Optional[torch.Tensor],
    out_w: Optional[torch.Tensor], m: float, in_w: Optional[torch.Tensor],
    g: Optional[torch.Tensor], eps: float, out_dtype,
) -> Optional[torch.Tensor]:
    """One step of a residual kept as S streams, xs fp32 [R, S, W], in place.

    With y [R, W] (the output of the sub-layer that just ran): every stream
    is rewritten from the old ones, x_t <- sum_s mix[s, t] x_s + m * out_w[t]
    * y.  With in_w [S] (the next sub-layer's read): returns h = rms(u) * g
    in out_dtype, u = sum_t in_w[t] x_t, g ONE fp32 weight (tensor of one
    element).  mix, out_w, in_w, g are fp32 device tensors.  S == 1 with
    unit coefficients is the plain pre-norm residual."""
    assert xs.dtype == torch.float32 and xs.dim() == 3 and xs.is_contiguous()
    R, S, W = xs.shape
    if y is not None:
        assert y.shape == (R, W) and y.is_contiguous() and y.dtype == out_dtype
        assert mix.shape == (S, S) and out_w.shape == (S,)
    if in_w is not None:
        assert in_w.shape == (S,) and g.numel() == 1
    if _use_hybrid(xs):
        for t in (mix, out_w, in_w, g):
            assert t is None or (t.dtype == torch.float32 and t.is_contiguous() and t.is_cuda)
        h = torch.empty(R, W, dtype=out_dtype, device=xs.device) if in_w is not None else None
        rc = _hl().lig_hyper_step(
            _ptr(xs), _ptr(y), _ptr(mix), _ptr(out_w), float(m), _ptr(in_w), _ptr(g),
            float(eps), _ptr(h), R, S, W, int(out_dtype == torch.float32), _stream(),
        )
        if rc != 0:
            raise RuntimeError(f"hyper_step: {S} streams not served")
        return h
    return torch_ref.hyper_step(xs, y, mix, out_w, m, in_w, g, eps, out_dtype)


def grouped_topk_route(
    z: torch.Tensor, correction: Optional[torch.Tensor], top: int, groups: int = 1,
    keep: int = 1,
):
    """Softmax router with group-limited choice over fp32 logits z [T, N]:
    scores s = softmax(z); choice scores s + correction; only outputs of the
    `keep` groups (of N/groups neighbours) with the largest best choice score
    can be chosen; the `top` largest choice scores win (ties: lower index).
    Returns (idx int32 [T, top], weights fp32 [T, top] = chosen s over their
    sum + 1e-20)."""
    assert z.dtype == torch.float32 and z.dim() == 2 and z.is_contiguous()
    T, N = z.shape
    assert N % groups == 0 and 1 <= keep <= groups and 1 <= top <= keep * (N // groups)
    if correction is not None:
        assert correction.dtype == torch.float32 and correction.shape == (N,)
    if _use_hybrid(z):
        idx = torch.empty(T, top, dtype=torch.int32, device=z.device)
        w = torch.empty(T, top, dtype=torch.float32, device=z.device)
        rc = _hl().lig_grouped_topk_route(
            _ptr(z), _ptr(correction), T, N, groups, keep, top, _ptr(idx), _ptr(w), _stream()
        )
        if rc != 0:
            raise RuntimeError("grouped_topk_route: shape not served")
        return idx, w
    return torch_ref.grouped_topk_route(z, correction, top, groups, keep)


def routed_combine(
    ye: torch.Tensor, x: torch.Tensor, rows: Optional[torch.Tensor], w: torch.Tensor,
    idx: Optional[torch.Tensor] = None, experts: int = 0,
):
    """out[t] = sum_k w[t, k] * (ye[rows[t, k]] if rows[t, k] >= 0 else x[t]):
    the weighted sum of a token's chosen expert outputs, a negative row
    standing for an identity expert.  rows int64 [T, top], w fp32 [T, top].
    With rows None every expert saw every token (ye is [experts * T, W],
    expert-major) and the rows follow from the choices idx int32 [T, top]:
    idx * T + t, or an identity expert for idx >= experts."""
    T, W = x.shape
    assert ye.dim() == 2 and ye.shape[1] == W and ye.dtype == x.dtype
    assert w.dtype == torch.float32 and w.dim() == 2
    if rows is None:
        assert idx is not None and idx.dtype == torch.int32 and idx.shape == w.shape
        assert ye.shape[0] == experts * T
    else:
        assert rows.dtype == torch.int64 and rows.shape == w.shape
    if _use_hybrid(x):
        assert ye.is_contiguous() and x.is_contiguous() and w.is_contiguous()
        assert (rows if rows is not None else idx).is_contiguous()
        out = torch.empty_like(x)
        _hl().lig_routed_combine(
            _ptr(out), _ptr(ye), _ptr(x), _ptr(rows), _ptr(idx) if rows is None else None,
            int(experts), _ptr(w), T, w.shape[1], W, _is_f32(x), _stream(),
        )
        return out
    if rows is None:
        tok = torch.arange(T, device=x.device).unsqueeze(1)
        il = idx.long()
        rows = torch.where(il < experts, il * T + tok, torch.full_like(il, -1))
    return torch_ref.routed_combine(ye, x, rows, w)


_GLU_KINDS = {"relu": 0, "clamped": 1}


def glu_act(x: torch.Tensor, kind: str, limit: float = 0.0, alpha: float = 1.0) -> torch.Tensor:
    """[rows, 2F] fused (gate | up) -> [rows, F].  "relu": relu(gate) * up.
    "clamped": g = min(gate, limit), u = clamp(up, -limit, limit),
    g * sigmoid(alpha * g) * (u + 1)."""
    k = _GLU_KINDS[kind]
    if _use_hybrid(x):
        assert x.is_contiguous() and x.dim() == 2 and x.shape[1] % 2 == 0
        F_ = x.shape[1] // 2
        out = torch.empty(x.shape[0], F_, dtype=x.dtype, device=x.device)
        _hl().lig_glu_act(
            _ptr(out), _ptr(x), x.shape[0], F_, k, float(limit), float(alpha), _is_f32(x), _stream()
        )
        return out
    return torch_ref.glu_act(x, kind, limit, alpha)
