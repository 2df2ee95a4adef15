#!/usr/bin/env python3
"""Vemenex beside Potatar's attention layers and Mixtral at equal size:
prefill and decode throughput through the engine, and the new kernels beside
the like kernels of those paths against the HBM roofline.

    python bench.py --streams                   # both parts, JSON lines
    python benchmarks/bench_streams.py --part engine|kernels|profile [--sizes s,m]

The closest existing family is Potatar with attention layers only: the same
attention block (q/k norms, partial rotation, a restricted key range, the
same prep, MFMA prompt and any-shape kernels) in front of a dense
feed-forward.  The routed variant stands beside Mixtral with the same
experts.

Engine part: for each size a dense Vemenex stack (sigmoid-weight and
sink-softmax attention alternating, two residual streams, gated relu
feed-forward) beside a Potatar stack of attention layers with the same
width, depth, heads and feed-forward parameters; and a routed Vemenex stack
(8 experts + 2 identity experts in 2 groups of which 1 is kept, 2 per token,
in every layer) beside Mixtral (8 experts, 2 per token).  A sliding window
and a chunk of the same size see different numbers of keys (a chunk starts
anew every `size` positions), so here both masks are as long as the longest
sequence of the workload and every query sees its whole past, as in Mixtral;
the kernel part times both masks at 512 with equal numbers of visible keys.
The same workload goes through LLMEngine.step(): N prompts of L tokens in
budget-sized steps, then K decode steps (hipGraph replay) at batch N.
Random weights, synthetic tokens.

Kernel part: each new kernel or kernel mode and its counterpart, timed with
events at the layer shapes of the sizes above; bytes that must move / time
against 8 TB/s (attention over prompts in useful TFLOP/s).
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

from llm_instance_gateway_amd import ops
from llm_instance_gateway_amd.models.config import ModelConfig
from llm_instance_gateway_amd.models.potatar import make_config as potatar_make
from llm_instance_gateway_amd.models.vemenex import make_config

from bench_hybrid import HBM_BYTES_PER_S, engine_run, timeit

# name: width, layers, heads, kv_heads, head size, three-matrix ff, expert ff, vocab
SIZES = {
    "s": dict(width=2048, layers=8, heads=16, kv_heads=4, dim=128, ff=5632, expert_ff=2048, vocab=32000),
    "m": dict(width=4096, layers=8, heads=32, kv_heads=8, dim=128, ff=9728, expert_ff=3584, vocab=32000),
}
WINDOW = 512
EXPERTS, IDENTITY, TOP = 8, 2, 2


def vemenex_config(name: str, z: dict, routed: bool, mask: int = WINDOW) -> ModelConfig:
    layers = []
    for i in range(z["layers"]):
        kind = "attention" if i % 2 == 0 else "attention_2"
        rot = {"base": 500000.0, "dims": z["dim"] // 2}
        if kind == "attention":
            rot["scaling"] = {"factor": 4.0}
        if routed:
            mlp = {"kind": "moe", "expert": {"ff": z["expert_ff"], "limit": 7.0},
                   "router": {"experts": EXPERTS, "identity": IDENTITY, "top": TOP,
                              "groups": {"count": 2, "keep": 1}}}
        else:
            mlp = {"kind": "dense", "ff": z["ff"]}
        layers.append({
            "type": kind,
            "mixer": {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["dim"],
                      "mask": {"size": mask}, "rot": rot, "scale": 1.0 / math.sqrt(z["dim"])},
            "mlp": mlp,
        })
    return make_config(f"vemenex-{name}{'-routed' if routed else ''}", z["vocab"], z["width"], layers,
                       eps=1e-6, residual_mult=0.5, streams=2)


def potatar_attention_config(name: str, z: dict, mask: int = WINDOW) -> ModelConfig:
    """Attention layers only; the two-matrix feed-forward is widened to the
    parameter count of the three-matrix one."""
    att = {
        "type": "attention",
        "mixer": {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["dim"],
                  "mask": {"size": mask}, "rot": {"base": 10000.0, "dims": z["dim"] // 2},
                  "scale": 1.0 / math.sqrt(z["dim"]), "v_mix": False},
        "mlp": {"ff": z["ff"] * 3 // 2, "kind": "dense"},
    }
    return potatar_make(f"potatar-att-{name}", z["vocab"], z["width"], [dict(att) for _ in range(z["layers"])],
                        eps=1e-6, alpha=2.0, softcap=0.0)


def mixtral_config(name: str, z: dict) -> ModelConfig:
    return ModelConfig(
        name=f"mixtral-{name}", vocab_size=z["vocab"], hidden_size=z["width"],
        num_layers=z["layers"], num_heads=z["heads"], num_kv_heads=z["kv_heads"],
        intermediate_size=z["expert_ff"], head_dim=z["dim"], max_position_embeddings=8192,
        num_experts=EXPERTS, num_experts_per_tok=TOP,
    )


def part_engine(sizes) -> None:
    for name in sizes:
        z = SIZES[name]
        for n_seqs, plen in ((16, 1024), (64, 512)):
            mask = plen + 64 + 1
            row = {"bench": "engine", "size": name, **z, "seqs": n_seqs, "prompt_len": plen, "decode_steps": 64,
                   "mask": mask}
            row["vemenex_dense"] = engine_run(vemenex_config(name, z, False, mask), n_seqs, plen, 64)
            row["potatar_attention"] = engine_run(potatar_attention_config(name, z, mask), n_seqs, plen, 64)
            if plen == 1024:
                row["vemenex_routed"] = engine_run(vemenex_config(name, z, True, mask), n_seqs, plen, 64)
                row["mixtral"] = engine_run(mixtral_config(name, z), n_seqs, plen, 64)
            for k in ("prefill_tok_per_s", "decode_tok_per_s"):
                row["dense_vs_potatar_" + k] = round(row["vemenex_dense"][k] / row["potatar_attention"][k], 3)
                if "mixtral" in row:
                    row["routed_vs_mixtral_" + k] = round(row["vemenex_routed"][k] / row["mixtral"][k], 3)
            print(json.dumps(row), flush=True)


def part_kernels(sizes) -> None:
    dev, bf = "cuda:0", torch.bfloat16
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    f32 = lambda v: torch.tensor(v, dtype=torch.float32, device=dev)
    for name in sizes:
        z = SIZES[name]
        W, FF, EF = z["width"], z["ff"], z["expert_ff"]
        hq, hkv, D = z["heads"], z["kv_heads"], z["dim"]
        for T in (8192, 256):  # a prefill step's rows / a decode batch
            rows = []

            def add(kernel, like, t, nbytes):
                rows.append({"kernel": kernel, "like": like, "us": round(t * 1e6, 2),
                             "GB_per_s": round(nbytes / t / 1e9, 1),
                             "of_roofline": round(nbytes / t / HBM_BYTES_PER_S, 3)})

            y = torch.randn(T, W, device=dev, dtype=bf)
            w = torch.ones(W, device=dev, dtype=bf)
            # the stream step: S streams read and written (4B each way), branch in, GEMM input out (2B)
            for S in (1, 2, 4):
                xs = torch.randn(T, S, W, device=dev)
                mix, ow, iw, g = torch.eye(S, device=dev), torch.ones(S, device=dev), torch.ones(S, device=dev), f32([1.1])
                add(f"hyper_step({S} streams, write + read)", "",
                    timeit(lambda: ops.hyper_step(xs, y, mix, ow, 0.5, iw, g, 1e-6, bf)), T * W * (8 * S + 4))
            x32 = torch.randn(T, W, device=dev)
            add("scaled_add_rms_norm", "hyper_step(1 stream)",
                timeit(lambda: ops.scaled_add_rms_norm(x32, 2.0, w, 1e-6, y)), T * W * 12)
            # activations over a fused gate | up projection: 2 x 2B in, 2B out
            gu = torch.randn(T, 2 * FF, device=dev, dtype=bf)
            add("glu_act(relu)", "", timeit(lambda: ops.glu_act(gu, "relu")), T * FF * 6)
            add("glu_act(clamped)", "", timeit(lambda: ops.glu_act(gu, "clamped", 7.0, 1.702)), T * FF * 6)
            add("silu_mul", "glu_act", timeit(lambda: ops.silu_mul(gu)), T * FF * 6)
            up = torch.randn(T, FF * 3 // 2, device=dev, dtype=bf)
            add("gelu_erf", "glu_act", timeit(lambda: ops.gelu_erf(up)), T * (FF * 3 // 2) * 4)
            # attention prep: reads q|k|v (2B), writes q (2B) and K/V rows (2B)
            bs, nblk = 16, T // 16 + 1
            kc = torch.zeros(nblk, hkv, bs, D, device=dev, dtype=bf)
            vc = torch.zeros_like(kc)
            proj = torch.randn(T, (hq + 2 * hkv) * D + 8 * ((hq + 7) // 8), device=dev, dtype=bf)
            wq, wk = torch.ones(hq * D, device=dev, dtype=bf), torch.ones(hkv * D, device=dev, dtype=bf)
            pos = torch.arange(T, device=dev, dtype=torch.int64) % 1024
            slots = torch.randperm(T, device=dev).to(torch.int64)
            inv = ops.rotary_inv_freq(10000.0, D // 2, dev)
            prep_bytes = T * (hq + 2 * hkv) * D * 4
            for layout in ("interleaved", "half"):
                add(f"qkv_norm_rope_cache({layout} rotation, head norms after it)", "",
                    timeit(lambda: ops.qkv_norm_rope_cache(proj, hq, hkv, D, D, "head_post", None, None, 1e-6,
                                                           inv, pos, kc, vc, slots, rot_layout=layout)), prep_bytes)
            add("qkv_norm_rope_cache(row norms, half rotation, unit values)", "the same kernel, new modes",
                timeit(lambda: ops.qkv_norm_rope_cache(proj, hq, hkv, D, D, "row", wq, wk, 1e-6, inv, pos, kc, vc,
                                                       slots, v_unit_norm=True)), prep_bytes)
            # router: logits in (4B), choices out; routed combine: top rows in, one out
            N = EXPERTS + IDENTITY
            zl = torch.randn(T, N, device=dev)
            corr = torch.zeros(N, device=dev)
            add("grouped_topk_route", "", timeit(lambda: ops.grouped_topk_route(zl, corr, TOP, 2, 1)),
                T * (N * 4 + TOP * 8))
            add("softmax + topk (library, Mixtral's router)", "grouped_topk_route",
                timeit(lambda: torch.topk(torch.softmax(zl, dim=-1), TOP, dim=-1)), T * (N * 4 + TOP * 8))
            ye = torch.randn(T * TOP, W, device=dev, dtype=bf)
            rws = torch.randperm(T * TOP, device=dev).view(T, TOP)
            cw = torch.rand(T, TOP, device=dev)
            add("routed_combine", "", timeit(lambda: ops.routed_combine(ye, y, rws, cw)), T * W * 2 * (TOP + 1))
            add("index_select + weighted sum (library, Mixtral's combine)", "routed_combine",
                timeit(lambda: (ye.index_select(0, rws.view(-1)).view(T, TOP, W).float() * cw[:, :, None]).sum(1).to(bf)),
                T * W * 2 * (TOP + 1))

            # attention kernels
            L = 1024
            sc = 1.0 / math.sqrt(D)
            pb = torch.full((hq,), -2.0, device=dev)
            sink = torch.zeros(hq, device=dev)
            if T >= 1024:
                Sq = T // L
                nb_seq = L // bs
                kcache = torch.randn(Sq * nb_seq + 1, hkv, bs, D, device=dev, dtype=bf)
                vcache = torch.randn_like(kcache)
                tables = torch.arange(Sq * nb_seq, dtype=torch.int32, device=dev).view(Sq, nb_seq)
                qsl, ctxl = i32([i * L for i in range(Sq + 1)]), i32([L] * Sq)
                tseq = i32([s_ for s_ in range(Sq) for _ in range(L // 64)])
                tqs = i32([q0 for _ in range(Sq) for q0 in range(0, L, 64)])
                qv = torch.randn(T, hq * D, device=dev, dtype=bf)
                gate = torch.randn(T, hq, device=dev, dtype=bf)
                win_pairs = sum(min(p + 1, WINDOW) for p in range(L))
                chunk_pairs = sum(p - (p // WINDOW) * WINDOW + 1 for p in range(L))

                def addf(kernel, like, t, flops):
                    rows.append({"kernel": kernel, "like": like, "us": round(t * 1e6, 1),
                                 "TFLOP_per_s": round(flops / t / 1e12, 1)})

                common = (qv, kcache, vcache, tables, qsl, ctxl, tseq, tqs, sc, hq)
                addf(f"paged_attention_prefill_tiles(window={WINDOW}, sigmoid weights + bias)", "",
                     timeit(lambda: ops.paged_attention_prefill_tiles(
                         *common, window=WINDOW, weights="sigmoid", score_bias=pb), 10),
                     4.0 * Sq * win_pairs * D * hq)
                addf(f"paged_attention_prefill_tiles(window={WINDOW}, sink, head gate)", "",
                     timeit(lambda: ops.paged_attention_prefill_tiles(
                         *common, window=WINDOW, sink=sink, gate=gate, gate_per_head=True), 10),
                     4.0 * Sq * win_pairs * D * hq)
                addf(f"paged_attention_prefill_tiles(chunk={WINDOW})", "the same kernel, new modes",
                     timeit(lambda: ops.paged_attention_prefill_tiles(*common, chunk=WINDOW), 10),
                     4.0 * Sq * chunk_pairs * D * hq)
            else:
                # single tokens: T sequences with 1024 cached tokens each, the
                # last WINDOW of them visible; bytes = visible K and V once
                nb_seq = L // bs
                tables = torch.arange(T * nb_seq, dtype=torch.int32, device=dev).view(T, nb_seq)
                posd = torch.full((T,), L - 1, device=dev, dtype=torch.int64)
                tsq = i32(list(range(T)))
                kc2 = torch.randn(T * nb_seq + 1, hkv, bs, D, device=dev, dtype=bf)
                vc2 = torch.randn_like(kc2)
                q2 = torch.randn(T, hq * D, device=dev, dtype=bf)
                gate = torch.randn(T, hq, device=dev, dtype=bf)
                kvbytes = T * WINDOW * hkv * D * 2 * 2
                common = (q2, kc2, vc2, tables, tsq, posd, sc, hq)
                add("paged_attention_general(window, sigmoid weights, single tokens)", "",
                    timeit(lambda: ops.paged_attention_general(
                        *common, window=WINDOW, weights="sigmoid", score_bias=pb), 10), kvbytes)
                add("paged_attention_general(window, sink, head gate, single tokens)", "",
                    timeit(lambda: ops.paged_attention_general(
                        *common, window=WINDOW, sink=sink, gate=gate, gate_per_head=True), 10), kvbytes)
                add("paged_attention_general(chunked, single tokens)", "the same kernel, new modes",
                    timeit(lambda: ops.paged_attention_general(*common, chunk=WINDOW), 10), kvbytes)
            print(json.dumps({"bench": "kernels", "size": name, "rows": T, "kernels": rows}), flush=True)


def main(argv=None) -> None:
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--part", default="engine,kernels")
    ap.add_argument("--sizes", default="s,m")
    args = ap.parse_args(argv)
    assert torch.cuda.is_available(), "this benchmark needs the GPU"
    sizes = [s for s in args.sizes.split(",") if s]
    if "kernels" in args.part:
        part_kernels(sizes)
    if "engine" in args.part:
        part_engine(sizes)
    if "profile" in args.part:
        # Vemenex only: the run to put under a profiler
        for name in sizes:
            print(json.dumps({"bench": "profile", "size": name,
                              "vemenex_dense": engine_run(vemenex_config(name, SIZES[name], False), 16, 1024, 64),
                              "vemenex_routed": engine_run(vemenex_config(name, SIZES[name], True), 16, 1024, 64)}),
                  flush=True)


if __name__ == "__main__":
    main()
