#!/usr/bin/env python3
"""Potatar beside Tikarax at equal size: prefill and decode throughput
through the engine, and the new kernels beside the like kernels of the
Tikarax path against the HBM roofline.

    python bench.py --postnorm                  # both parts, JSON lines
    python benchmarks/bench_postnorm.py --part engine|kernels|profile [--sizes s,m]

Tikarax is the closest existing family: a hybrid stack whose layers
alternate between paged attention of general head sizes and a recurrence
with a state slot per sequence, served by the same light kernel library.

Engine part: for each size a Potatar stack (attention / wkv / attention /
parallel, repeated) and a Tikarax stack (minGRU / gated attention
alternating) with the same width, depth, head sizes and feed-forward run the
same workload through LLMEngine.step(): N prompts of L tokens prefilled in
budget-sized steps, then K decode steps (hipGraph replay) at batch N.
Random weights, synthetic tokens.

Kernel part: each new kernel and its counterpart, timed with events at the
layer shapes of the sizes above; bytes that must move / time against 8 TB/s
(attention over prompts in useful TFLOP/s).
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
from llm_instance_gateway_amd.models.potatar import make_config

from bench_hybrid import HBM_BYTES_PER_S, engine_run, tikarax_config, timeit

# name: width, layers, heads, kv_heads, head size, recurrent head size, ff, vocab
SIZES = {
    "s": dict(width=2048, layers=8, heads=16, kv_heads=4, dim=128, rdim=64, ff=8192, vocab=32000),
    "m": dict(width=4096, layers=8, heads=32, kv_heads=8, dim=128, rdim=64, ff=14336, vocab=32000),
}
CHUNK = 512


def potatar_config(name: str, z: dict) -> ModelConfig:
    W = z["width"]
    rheads = W // z["rdim"]
    att = {
        "type": "attention",
        "mixer": {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["dim"],
                  "mask": {"size": CHUNK}, "rot": {"base": 10000.0, "dims": z["dim"] // 2},
                  "scale": 1.0 / math.sqrt(z["dim"]), "v_mix": True},
    }
    wkv = {"type": "wkv", "mixer": {"heads": rheads, "dim": z["rdim"], "decay_rank": 64}}
    par = {
        "type": "parallel",
        "mixer": {
            "left": {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["rdim"], "vdim": z["rdim"],
                     "mask": {"size": CHUNK}, "bias_max": 256, "bias_rows": 32,
                     "scale": 1.0 / math.sqrt(z["rdim"])},
            "right": {"heads": rheads // 2, "dim": z["rdim"], "vdim": z["rdim"],
                      "decay": [1.0 - 2.0 ** -(1 + 6 * i / max(rheads // 2 - 1, 1)) for i in range(rheads // 2)]},
            "left_scale": 0.8, "right_scale": 0.9,
        },
    }
    order = [att, wkv, att, par]
    layers = []
    for i in range(z["layers"]):
        layer = dict(order[i % 4])
        layer["mlp"] = {"ff": z["ff"], "kind": "dense"}
        layers.append(layer)
    return make_config(f"potatar-{name}", z["vocab"], W, layers, eps=1e-6, alpha=2.0, softcap=30.0)


def part_engine(sizes) -> None:
    for name in sizes:
        z = SIZES[name]
        for n_seqs, plen in ((16, 1024), (64, 512)):
            row = {"bench": "engine", "size": name, **z, "seqs": n_seqs, "prompt_len": plen, "decode_steps": 64}
            row["potatar"] = engine_run(potatar_config(name, z), n_seqs, plen, 64)
            row["tikarax"] = engine_run(tikarax_config(name, z), n_seqs, plen, 64)
            for k in ("prefill_tok_per_s", "decode_tok_per_s"):
                row["ratio_" + k] = round(row["potatar"][k] / row["tikarax"][k], 3)
            print(json.dumps(row), flush=True)


def part_kernels(sizes) -> None:
    dev, bf = "cuda:0", torch.bfloat16
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    for name in sizes:
        z = SIZES[name]
        W, FF = z["width"], z["ff"]
        hq, hkv, D, RD = z["heads"], z["kv_heads"], z["dim"], z["rdim"]
        rh = W // RD
        for T in (8192, 256):  # a prefill step's rows / a decode batch
            rows = []

            def add(kernel, like, t, nbytes):
                rows.append({"kernel": kernel, "like": like, "us": round(t * 1e6, 2),
                             "GB_per_s": round(nbytes / t / 1e9, 1),
                             "of_roofline": round(nbytes / t / HBM_BYTES_PER_S, 3)})

            seg = 1024 if T >= 1024 else 1
            S = T // seg
            segs = (i32([i * seg for i in range(S)]), i32([seg] * S), i32(list(range(S))), i32([0] * S))
            tok_seq = i32([s_ for s_ in range(S) for _ in range(seg)])
            x32 = torch.randn(T, W, device=dev)
            y = torch.randn(T, W, device=dev, dtype=bf)
            w = torch.ones(W, device=dev, dtype=bf)
            # sum + norm: reads residual (4B) + branch (2B), writes residual (4B) + GEMM input (2B)
            add("scaled_add_rms_norm", "", timeit(lambda: ops.scaled_add_rms_norm(x32, 2.0, w, 1e-6, y)), T * W * 12)
            add("post_add_pre_norm(groups=2)", "scaled_add_rms_norm",
                timeit(lambda: ops.post_add_pre_norm(x32, y, w, w, 1e-5, 2)), T * W * 12)
            up = torch.randn(T, FF, device=dev, dtype=bf)
            add("gelu_erf", "", timeit(lambda: ops.gelu_erf(up)), T * FF * 4)
            add("xielu", "gelu_erf", timeit(lambda: ops.xielu(up, 0.7, 1.2)), T * FF * 4)
            # attention prep: reads q|k|v (2B), writes q (2B) and K/V rows (2B)
            bs, nblk = 16, T // 16 + 1
            kc = torch.zeros(nblk, hkv, bs, D, device=dev, dtype=bf)
            vc = torch.zeros_like(kc)
            proj = torch.randn(T, (hq + 2 * hkv) * D, device=dev, dtype=bf)
            wq, wk = torch.ones(hq * D, device=dev, dtype=bf), torch.ones(hkv * D, device=dev, dtype=bf)
            pos = torch.arange(T, device=dev, dtype=torch.int64) % 1024
            slots = torch.randperm(T, device=dev).to(torch.int64)
            inv = ops.rotary_inv_freq(10000.0, D // 2, dev)
            vf = torch.randn(T, hkv * D, device=dev)
            add("qkv_norm_rope_cache(row norms, rotation, unit values, blend)", "",
                timeit(lambda: ops.qkv_norm_rope_cache(proj, hq, hkv, D, D, "row", wq, wk, 1e-6, inv, pos, kc, vc,
                                                       slots, v_unit_norm=True, v_first=vf, lam=0.3)),
                T * (hq + 2 * hkv) * D * 4 + T * hkv * D * 4)
            kview, vview = proj[:, hq * D:(hq + hkv) * D], proj[:, (hq + hkv) * D:]
            add("kv_scatter + temperature_scale_rows", "qkv_norm_rope_cache",
                timeit(lambda: (ops.kv_scatter(kview, vview, kc, vc, slots),
                                ops.temperature_scale_rows(proj[:, : hq * D], pos, 0.25, 128.0))),
                T * (hq + 2 * hkv) * D * 4)
            # token shift: reads the residual (4B) once, writes five blends (2B each)
            mu = torch.rand(5, W, device=dev).to(bf)
            st = torch.zeros(S + 1, W, device=dev)
            add("token_shift_mix(5 blends)", "",
                timeit(lambda: ops.token_shift_mix(x32, mu, st, tok_seq, *segs)), T * W * 14)
            # recurrences: r, k, v in (2B each) + decay pre-activation (4B) + output (4B); state both ways
            rkv = torch.randn(3, T, W, device=dev, dtype=bf) * 0.3
            pre = torch.randn(T, W, device=dev) - 2.0
            u = torch.randn(W, device=dev) * 0.3
            mst = torch.zeros(S + 1, ops.matrix_state_width(rh, RD, RD), device=dev)
            add(f"matrix_state_scan(bonus form, segments of {seg})", "",
                timeit(lambda: ops.matrix_state_scan(rkv[0], rkv[1], rkv[2], mst, *segs, rh, RD, RD,
                                                     decay_pre=pre, bonus=u), 10),
                T * W * 14 + 2 * S * rh * RD * RD * 4)
            hd = torch.full((rh,), 0.97, device=dev)
            add(f"matrix_state_scan(constant decay, segments of {seg})", "",
                timeit(lambda: ops.matrix_state_scan(rkv[0], rkv[1], rkv[2], mst, *segs, rh, RD, RD,
                                                     head_decay=hd, act_silu=True), 10),
                T * W * 10 + 2 * S * rh * RD * RD * 4)
            zxg = torch.randn(T, 3 * W, device=dev, dtype=bf)
            st1 = torch.zeros(S + 1, W, device=dev)
            add(f"mingru_scan(segments of {seg})", "matrix_state_scan",
                timeit(lambda: ops.mingru_scan(zxg, st1, *segs, seg)), T * W * 8 + 2 * S * W * 4)
            o32 = torch.randn(T, W, device=dev)
            add("group_rms_norm_gate(per head, silu)", "",
                timeit(lambda: ops.group_rms_norm_gate(o32, y, w, RD, "silu", 1e-6)), T * W * 8)
            add("group_rms_norm_gate(whole row, sigmoid)", "",
                timeit(lambda: ops.group_rms_norm_gate(o32, y, w, W, "sigmoid", 1e-6)), T * W * 8)
            o16 = torch.randn(T, W, device=dev, dtype=bf)
            add("sigmoid_gate_mul", "group_rms_norm_gate", timeit(lambda: ops.sigmoid_gate_mul(o16, y)), T * W * 6)

            # attention kernels
            L = 1024
            sc = 1.0 / math.sqrt(D)
            lh, lD = hq, RD  # the parallel layer's attention branch
            rel = torch.randn(32, lh, device=dev)
            tab = ops.distance_bias_table(rel, 256.0)
            talk = torch.eye(lh, device=dev) + 0.1 * torch.randn(lh, lh, device=dev)
            if T >= 1024:
                Sq = T // L
                nb_seq = L // bs
                kcache = torch.randn(Sq * nb_seq + 1, hkv, bs, D, device=dev, dtype=bf)
                vcache = torch.randn_like(kcache)
                tables = torch.arange(Sq * nb_seq, dtype=torch.int32, device=dev).view(Sq, nb_seq)
                qsl, ctxl = i32([i * L for i in range(Sq + 1)]), i32([L] * Sq)
                tseq = i32([s_ for s_ in range(Sq) for _ in range(L // 64)])
                tqs = i32([q0 for _ in range(Sq) for q0 in range(0, L, 64)])
                tsq = i32([s_ for s_ in range(Sq) for _ in range(L)])
                posq = torch.arange(L, device=dev, dtype=torch.int64).repeat(Sq)
                qv = torch.randn(T, hq * D, device=dev, dtype=bf)

                def pairs(chunk):  # visible (query, key) pairs of one sequence
                    return sum(p - (p // chunk) * chunk + 1 for p in range(L)) if chunk else L * (L + 1) // 2

                def addf(kernel, like, t, flops):
                    rows.append({"kernel": kernel, "like": like, "us": round(t * 1e6, 1),
                                 "TFLOP_per_s": round(flops / t / 1e12, 1)})

                for chunk in (0, CHUNK):
                    addf(f"paged_attention_prefill_tiles(chunk={chunk})", "same kernel, chunk=0",
                         timeit(lambda: ops.paged_attention_prefill_tiles(
                             qv, kcache, vcache, tables, qsl, ctxl, tseq, tqs, sc, hq, chunk=chunk), 10),
                         4.0 * Sq * pairs(chunk) * D * hq)
                kc2 = torch.randn(Sq * nb_seq + 1, hkv, bs, lD, device=dev, dtype=bf)
                vc2 = torch.randn_like(kc2)
                q2 = torch.randn(T, lh * lD, device=dev, dtype=bf)
                fl2 = 4.0 * Sq * pairs(CHUNK) * lD * lh
                if ops.mixed_heads_tiles_supported(bf, lD, lD, lh, True):
                    addf("paged_attention_mixed_heads_tiles(MFMA, bias + head mixing, chunked)", "paged_attention_prefill_tiles",
                         timeit(lambda: ops.paged_attention_mixed_heads_tiles(
                             q2, kc2, vc2, tables, qsl, ctxl, tseq, tqs, sc, lh, dist_bias=tab, talk=talk,
                             chunk=CHUNK), 10), fl2)
                addf("paged_attention_mixed_heads(bias + head mixing, chunked, prompt rows)", "",
                     timeit(lambda: ops.paged_attention_mixed_heads(
                         q2, kc2, vc2, tables, tsq, posq, sc, lh, dist_bias=tab, talk=talk, chunk=CHUNK), 3), fl2)
                addf("paged_attention_general(chunked, prompt rows)", "paged_attention_mixed_heads",
                     timeit(lambda: ops.paged_attention_general(
                         q2, kc2, vc2, tables, tsq, posq, sc, lh, chunk=CHUNK), 3), fl2)
            else:
                # single tokens: T sequences with 1024 cached tokens each, the
                # last CHUNK of them visible; bytes = visible K and V once
                nb_seq = L // bs
                tables = torch.arange(T * nb_seq, dtype=torch.int32, device=dev).view(T, nb_seq)
                posd = torch.full((T,), L - 1, device=dev, dtype=torch.int64)
                tsq = i32(list(range(T)))
                kc2 = torch.randn(T * nb_seq + 1, hkv, bs, lD, device=dev, dtype=bf)
                vc2 = torch.randn_like(kc2)
                q2 = torch.randn(T, lh * lD, device=dev, dtype=bf)
                kvbytes = T * CHUNK * hkv * lD * 2 * 2
                add("paged_attention_mixed_heads(single tokens)", "",
                    timeit(lambda: ops.paged_attention_mixed_heads(
                        q2, kc2, vc2, tables, tsq, posd, sc, lh, dist_bias=tab, talk=talk, chunk=CHUNK), 10), kvbytes)
                add("paged_attention_general(chunked, single tokens)", "paged_attention_mixed_heads",
                    timeit(lambda: ops.paged_attention_general(
                        q2, kc2, vc2, tables, tsq, posd, sc, lh, chunk=CHUNK), 10), kvbytes)
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
        # Potatar only: the run to put under a profiler
        for name in sizes:
            print(json.dumps({"bench": "profile", "size": name,
                              "potatar": engine_run(potatar_config(name, SIZES[name]), 16, 1024, 64)}),
                  flush=True)


if __name__ == "__main__":
    main()
