"""Potatar through the engine (scheduler, block/state pools, model runner,
kernels) against the slow float64 oracle in potatar_oracle.py.

Every test builds its own small configuration and random bf16 checkpoint in
a temp folder, so the config reader and the safetensors loader are on the
path too.  The CPU parametrisation runs the engine's torch execution path;
the `gpu` one runs the HIP kernels (fp32 storage for sharp comparisons, bf16
for the serving precision).
"""

import json
import math
import struct

import numpy as np
import pytest
import torch

from llm_instance_gateway_amd.engine import EngineConfig, LLMEngine, SamplingParams
from llm_instance_gateway_amd.models.config import get_model_config

import potatar_oracle as O

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]


def att(heads, kv, dim, vdim, chunk, rot_dims, v_mix, mlp=None, base=300.0):
    return {
        "type": "attention",
        "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "mask": {"size": chunk},
                  "rot": {"base": base, "dims": rot_dims}, "scale": 1.3 / math.sqrt(dim), "v_mix": v_mix},
        "mlp": mlp,
    }


def wkv(heads, dim, mlp=None):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim}, "mlp": mlp}


def par(heads, kv, dim, chunk, far, rheads, rdim, rvdim, decay, ls=0.7, rs=1.1, mlp=None):
    return {
        "type": "parallel",
        "mixer": {
            "left": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "mask": {"size": chunk},
                     "bias_max": far, "scale": 1.1 / math.sqrt(dim)},
            "right": {"heads": rheads, "dim": rdim, "vdim": rvdim, "decay": decay},
            "left_scale": ls, "right_scale": rs,
        },
        "mlp": mlp,
    }


def dense(ff):
    return {"kind": "dense", "ff": ff}


# sizes unlike one another; chunks of 24 and 40 positions so that prompts of
# 90 tokens cross several chunk edges; the first attention layer has no value
# mixing, so the values come from the second
CFG_A = {
    "architecture": "Potatar", "vocab": 67, "width": 40, "norm": {"eps": 1e-5}, "postln_alpha": 1.7,
    "logit_softcap": 9.0,
    "layers": [
        att(4, 2, 12, 6, 24, 8, False, dense(56)),
        att(4, 2, 12, 6, 24, 12, True, None),
        wkv(3, 8, dense(24)),
        par(4, 2, 10, 40, 30, 3, 6, 10, [0.5, 0.9, 0.99], mlp=dense(32)),
        att(2, 2, 12, 6, 40, 4, True, dense(16), base=50.0),
        wkv(2, 12, None),
        att(4, 2, 12, 6, 24, 8, True, None),
    ],
    "tables": {"rel_rows": 10, "decay_rank": 5},
}
# degenerate values: one head, one key/value head per query head, sizes that
# are multiples of nothing, rotation over the whole head, a chunk of 1 and a
# chunk longer than any prompt, no cap on the logits, alpha 1
CFG_B = {
    "architecture": "Potatar", "vocab": 29, "width": 18, "norm": {"eps": 1e-3}, "postln_alpha": 1.0,
    "layers": [
        par(1, 1, 5, 1, 9, 1, 3, 5, [0.8], ls=1.0, rs=1.0),
        att(1, 1, 6, 3, 1000, 6, True, dense(7)),
        wkv(1, 5, None),
        att(3, 3, 4, 5, 7, 2, False, None),
    ],
    "tables": {"rel_rows": 4, "decay_rank": 1},
}
# head sizes the MFMA prompt kernel takes (multiples of 8), long enough
# chunks for several 64-row tiles
CFG_C = {
    "architecture": "Potatar", "vocab": 50, "width": 64, "norm": {"eps": 1e-6}, "postln_alpha": 2.0,
    "logit_softcap": 20.0,
    "layers": [
        att(4, 2, 32, 16, 100, 16, True, dense(64)),
        wkv(2, 16, None),
        att(2, 1, 64, 64, 70, 32, False, dense(48)),
        par(2, 1, 16, 100, 120, 2, 16, 8, [0.7, 0.97], mlp=None),
        att(4, 2, 24, 16, 33, 24, True, None),
    ],
    "tables": {"rel_rows": 12, "decay_rank": 4},
}


def make_checkpoint(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    H, V = cfg["width"], cfg["vocab"]
    tab = cfg["tables"]

    def r(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16)

    def near_one(n):
        return (1 + 0.2 * torch.randn(n, generator=g)).to(torch.bfloat16)

    W = {"embed": r(V, H), "final.norm": near_one(H), "head": r(V, H, s=H ** -0.5)}
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % i
        m = layer["mixer"]
        W[p + "norm1"] = near_one(H)
        if layer["type"] == "attention":
            nq, nk, nv = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            for n, rows in (("q", nq), ("k", nk), ("v", nv)):
                W[p + "mix." + n], W[p + "mix." + n + ".b"] = r(rows, H, s=H ** -0.5), r(rows, s=0.3)
            W[p + "mix.q.norm"], W[p + "mix.k.norm"] = near_one(nq), near_one(nk)
            W[p + "mix.vmix"] = torch.tensor(0.2 + 0.1 * i).to(torch.bfloat16)
            W[p + "mix.o"], W[p + "mix.o.b"] = r(H, m["heads"] * m["vdim"], s=(m["heads"] * m["vdim"]) ** -0.5), r(H, s=0.3)
        elif layer["type"] == "wkv":
            n, rank = m["heads"] * m["dim"], tab["decay_rank"]
            for c in "rkvgw":
                W[p + "mix.mu." + c] = torch.rand(H, generator=g).to(torch.bfloat16)
            for c in "rkvg":
                W[p + "mix." + c] = r(n, H, s=H ** -0.5)
            W[p + "mix.w1"], W[p + "mix.w2"] = r(rank, H, s=H ** -0.5), r(n, rank, s=0.5)
            W[p + "mix.w0"] = (torch.rand(n, generator=g) * 3 - 3.5).to(torch.bfloat16)
            W[p + "mix.u"] = r(m["heads"], m["dim"], s=0.5)
            W[p + "mix.norm"], W[p + "mix.o"] = near_one(n), r(H, n, s=n ** -0.5)
        else:
            lm, rm = m["left"], m["right"]
            q = "mix.left."
            nq, nk = lm["heads"] * lm["dim"], lm["kv_heads"] * lm["dim"]
            W[p + q + "q"], W[p + q + "q.b"] = r(nq, H, s=H ** -0.5), r(nq, s=0.3)
            W[p + q + "k"], W[p + q + "k.b"] = r(nk, H, s=H ** -0.5), r(nk, s=0.3)
            W[p + q + "q.norm"], W[p + q + "k.norm"] = near_one(lm["dim"]), near_one(lm["dim"])
            W[p + q + "rel"] = r(tab["rel_rows"], lm["heads"], s=0.7)
            W[p + q + "talk"] = (torch.eye(lm["heads"]) + 0.3 * torch.randn(lm["heads"], lm["heads"], generator=g)).to(torch.bfloat16)
            W[p + q + "o"], W[p + q + "o.b"] = r(H, nq, s=nq ** -0.5), r(H, s=0.3)
            q = "mix.right."
            nk, nv = rm["heads"] * rm["dim"], rm["heads"] * rm["vdim"]
            W[p + q + "q"], W[p + q + "k"] = r(nk, H, s=H ** -0.5), r(nk, H, s=H ** -0.5)
            W[p + q + "v"], W[p + q + "g"] = r(nv, H, s=H ** -0.5), r(nv, H, s=H ** -0.5)
            W[p + q + "norm"], W[p + q + "o"] = near_one(nv), r(H, nv, s=nv ** -0.5)
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            W[p + "norm2"] = near_one(H)
            W[p + "mlp.up"], W[p + "mlp.down"] = r(ff, H, s=H ** -0.5), r(H, ff, s=ff ** -0.5)
    return W


def write_model(folder, cfg, W):
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps({k: v for k, v in cfg.items() if k != "tables"}))
    header, blobs, at = {}, [], 0
    for name, t in W.items():
        raw = t.contiguous().view(-1).view(torch.uint8).numpy().tobytes()
        header[name] = {"dtype": "BF16", "shape": list(t.shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    hj = json.dumps(header).encode()
    with open(folder / "model.safetensors", "wb") as f:
        f.write(struct.pack("<Q", len(hj)) + hj + b"".join(blobs))
    return str(folder)


def oracle(cfg, W, toks):
    z, streams = O.forward(cfg, {k: v.double().numpy() for k, v in W.items()}, toks)
    return torch.from_numpy(z), torch.from_numpy(streams)


def make_engine(path, device, dtype=torch.float32, blocks=64, block_size=16, seqs=4, budget=4096, **kw):
    mc = get_model_config(path)
    kw.setdefault("enforce_eager", True)
    cfg = EngineConfig(
        model=mc, block_size=block_size, num_kv_blocks=blocks, max_num_seqs=seqs,
        num_state_slots=seqs, max_num_batched_tokens=budget,
        max_model_len=blocks * block_size, watermark_blocks=0, **kw,
    )
    return LLMEngine(cfg, device=device, dtype=dtype)


def row_errs(got, want):
    """Per-row RMS of the mean-free difference over the RMS of the oracle's logits."""
    d = got.double().cpu() - want
    d = d - d.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()


def tol(dtype):
    return 2e-4 if dtype == torch.float32 else 6e-2


def assert_logits(got, want, dtype=torch.float32):
    e = row_errs(got, want)
    assert e.max().item() < tol(dtype), (e.max().item(), int(e.argmax()))


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def replay_all(eng, rid, toks, cuts):
    """Feed toks in portions `cuts`, wanting every position; returns [T, V]."""
    rows, at = [], 0
    for i, n in enumerate(cuts):
        last = i == len(cuts) - 1
        res = eng.replay_step([(rid, toks[at : at + n], list(range(n)))], end=[rid] if last else [])
        rows.append(res[rid].float().cpu())
        at += n
    assert at == len(toks)
    return torch.cat(rows)


def _model(tmp_path_factory, cfg, seed, name):
    W = make_checkpoint(cfg, seed)
    return write_model(tmp_path_factory.mktemp("ptr") / name, cfg, W), W


@pytest.fixture(scope="module")
def model_a(tmp_path_factory):
    return _model(tmp_path_factory, CFG_A, 21, "a")


@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    return _model(tmp_path_factory, CFG_B, 22, "b")


@pytest.fixture(scope="module")
def model_c(tmp_path_factory):
    return _model(tmp_path_factory, CFG_C, 23, "c")


@pytest.fixture(scope="module")
def oracle_a(model_a):
    toks = tokens_for(CFG_A, 90, 5)
    return (toks,) + oracle(CFG_A, model_a[1], toks)


def test_config_reader_sizes_from_shapes(model_a):
    mc = get_model_config(model_a[0])
    assert mc.architecture == "potatar" and mc.residual_alpha == 1.7 and mc.logit_softcap == 9.0
    specs = mc.layer_specs
    assert [s.type for s in specs] == ["attention", "attention", "wkv", "parallel", "attention", "wkv", "attention"]
    # sizes that only the tensors' shapes give
    assert specs[2].mixer["decay_rank"] == 5 and specs[3].mixer["left"]["bias_rows"] == 10
    assert mc.kv_elems_per_token() == 3 * 2 * (12 + 6) + 2 * (12 + 6) + 2 * 2 * 10
    assert mc.state_elems_per_seq() == (40 + 3 * 64) + 3 * 6 * 10 + (40 + 2 * 144)
    assert mc.has_recurrent_state and not mc.is_moe


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_whole_prompt_and_every_layer(model_a, oracle_a, device, dtype):
    if device == "cpu" and dtype == torch.bfloat16:
        pytest.skip("bf16 is the GPU serving precision")
    toks, want, want_res = oracle_a
    eng = make_engine(model_a[0], device, dtype)
    captured = eng.runner.model.capture_residuals = []
    got = replay_all(eng, "w", toks, [len(toks)])
    assert_logits(got, want, dtype)
    assert len(captured) == len(CFG_A["layers"])
    for i, (x, xo) in enumerate(zip(captured, want_res)):
        assert x.dtype == torch.float32, "the residual stream stays fp32"
        e = (x[: len(toks)].double().cpu() - xo).abs().max().item() / xo.abs().max().item()
        assert e < (1e-4 if dtype == torch.float32 else 6e-2), f"layer {i}: {e}"


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("which", ["b", "c"])
def test_other_sizes(model_b, model_c, device, which):
    cfg, (path, W) = (CFG_B, model_b) if which == "b" else (CFG_C, model_c)
    toks = tokens_for(cfg, 75, 6)
    want, _ = oracle(cfg, W, toks)
    eng = make_engine(path, device, block_size=8)
    assert_logits(replay_all(eng, "d", toks, [17, 1, 1, 2, 19, 35]), want)


@pytest.mark.parametrize("device", DEVICES)
def test_first_token_alone(model_a, oracle_a, device):
    toks, want, _ = oracle_a
    eng = make_engine(model_a[0], device)
    assert_logits(replay_all(eng, "f", toks[:1], [1]), want[:1])


@pytest.mark.parametrize("device", DEVICES)
def test_prefill_then_token_by_token(model_a, oracle_a, device):
    toks, want, _ = oracle_a
    eng = make_engine(model_a[0], device)
    # the decoded tokens cross pages and the chunk edges at 40, 48, 72 and 80
    assert_logits(replay_all(eng, "p", toks, [30] + [1] * 60), want)
    eng2 = make_engine(model_a[0], device)
    assert_logits(replay_all(eng2, "q", toks[:50], [1] * 50), want[:50])  # from the very first token


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize(
    "cuts", [[2] * 45, [3, 13, 16, 17, 2, 31, 8], [23, 1, 1, 23, 2, 38, 2], [24, 24, 24, 18], [64, 2, 24]]
)
def test_portions(model_a, oracle_a, device, cuts):
    """Portions that end just before, at and just after chunk edges (24, 40,
    48, 72, 80) and page edges; chunks count from the sequence's start."""
    toks, want, _ = oracle_a
    assert sum(cuts) == len(toks)
    eng = make_engine(model_a[0], device)
    assert_logits(replay_all(eng, "c", toks, cuts), want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_mixed_batch_equals_each_alone_and_pools_are_reused(model_a, device, dtype):
    """Unequal requests share steps (portions beside single tokens), with a
    pool so small that pages and state slots of finished requests are handed
    to later ones; every logit row matches the request run alone."""
    if device == "cpu" and dtype == torch.bfloat16:
        pytest.skip("bf16 is the GPU serving precision")
    lens = {"a": 37, "b": 5, "c": 50, "d": 1, "e": 23, "f": 33}
    toks = {k: tokens_for(CFG_A, n, 100 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: oracle(CFG_A, model_a[1], t)[0] for k, t in toks.items()}
    plan = [
        [("a", 20), ("b", 3)],
        [("a", 1), ("b", 2), ("c", 30), ("d", 1)],           # b, d end: slots free
        [("a", 16), ("e", 7)],                                # c sits this step out; e reuses a freed slot + pages
        [("c", 20), ("e", 1), ("f", 2)],                      # a ended; c comes back and ends
        [("e", 15), ("f", 30)],
        [("f", 1)],
    ]
    eng = make_engine(model_a[0], device, dtype, blocks=9, block_size=16, seqs=4)
    at = {k: 0 for k in toks}
    got = {k: [] for k in toks}
    for step in plan:
        entries, end = [], []
        for rid, n in step:
            entries.append((rid, toks[rid][at[rid] : at[rid] + n], list(range(n))))
            at[rid] += n
            if at[rid] == lens[rid]:
                end.append(rid)
        res = eng.replay_step(entries, end)
        for rid, _ in step:
            got[rid].append(res[rid].float().cpu())
    assert all(at[k] == lens[k] for k in lens)
    bm = eng.scheduler.block_manager
    assert bm.num_free_blocks == 9 and bm.num_free_state_slots == 4
    for k in toks:
        assert_logits(torch.cat(got[k]), want[k], dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_long_prompt_over_dirty_pages_and_slots(model_c, device):
    """A 300-token prompt (several chunks and MFMA tiles) run after another
    request has dirtied every page and state slot of the pool, then decoded
    across a chunk edge."""
    toks = tokens_for(CFG_C, 300, 31)
    want, _ = oracle(CFG_C, model_c[1], toks)
    eng = make_engine(model_c[0], device, blocks=19, block_size=16, seqs=1)
    junk = tokens_for(CFG_C, 304, 32)
    eng.replay_step([("junk", junk, [])], end=["junk"])
    got = replay_all(eng, "x", toks, [250, 1, 1, 28, 2] + [1] * 18)
    assert_logits(got, want)


@pytest.mark.gpu
def test_bf16_prompt_tiles_beside_single_tokens(model_c):
    """bf16 on the GPU: prompt rows of the plain attention layers run the
    MFMA tile kernel with the chunk mask, single tokens the any-shape one."""
    ta, tb = tokens_for(CFG_C, 230, 41), tokens_for(CFG_C, 70, 42)
    wa, wb = oracle(CFG_C, model_c[1], ta)[0], oracle(CFG_C, model_c[1], tb)[0]
    eng = make_engine(model_c[0], "cuda:0", torch.bfloat16)
    assert eng.runner.model.needs_prefill_tiles
    plan = [[("a", 150)], [("a", 1), ("b", 65)], [("a", 60), ("b", 1)], [("a", 1), ("b", 4)], [("a", 18)]]
    at, toks, got = {"a": 0, "b": 0}, {"a": ta, "b": tb}, {"a": [], "b": []}
    for step in plan:
        entries = []
        for rid, n in step:
            entries.append((rid, toks[rid][at[rid] : at[rid] + n], list(range(n))))
            at[rid] += n
        res = eng.replay_step(entries, [r for r, _ in step if at[r] == len(toks[r])])
        for rid, _ in step:
            got[rid].append(res[rid].float().cpu())
    assert_logits(torch.cat(got["a"]), wa, torch.bfloat16)
    assert_logits(torch.cat(got["b"]), wb, torch.bfloat16)


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_scheduler(model_a, device):
    """add_request + generate_all: chunked prefill under a tiny token budget,
    continuous batching of three requests, greedy sampling."""
    W = model_a[1]
    prompts = [tokens_for(CFG_A, n, 200 + n) for n in (19, 7, 26)]
    eng = make_engine(model_a[0], device, budget=8, blocks=32)
    seqs = [eng.add_request(p, SamplingParams(max_new_tokens=6)) for p in prompts]
    done = eng.generate_all(max_steps=200)
    assert len(done) == 3
    for seq, prompt in zip(seqs, prompts):
        toks = list(prompt)
        for step in range(6):
            logits = oracle(CFG_A, W, toks)[0][-1]
            top2 = torch.topk(logits, 2).values
            if float(top2[0] - top2[1]) > 1e-3:  # an unambiguous argmax must match
                assert seq.output_token_ids[step] == int(torch.argmax(logits)), (step, seq.output_token_ids)
            toks.append(seq.output_token_ids[step])
    bm = eng.scheduler.block_manager
    assert bm.num_free_blocks == 32 and bm.num_free_state_slots == 4


@pytest.mark.parametrize("device", DEVICES)
def test_preempted_sequence_recomputes_its_state(model_a, device):
    prompt = tokens_for(CFG_A, 21, 77)
    ref = make_engine(model_a[0], device)
    s0 = ref.add_request(prompt, SamplingParams(max_new_tokens=8))
    ref.generate_all(max_steps=50)
    eng = make_engine(model_a[0], device)
    s1 = eng.add_request(prompt, SamplingParams(max_new_tokens=8))
    for _ in range(4):
        eng.step()
    sch = eng.scheduler
    sch.running.remove(s1)
    sch.block_manager.free(s1)
    s1.preempt()
    sch.waiting.appendleft(s1)
    assert s1.state_slot == -1
    eng.generate_all(max_steps=50)
    assert s1.output_token_ids == s0.output_token_ids


@pytest.mark.gpu
def test_graph_decode_matches_eager(model_a):
    """Decode-only steps replayed from hipGraphs give the tokens of the eager
    engine, replay after replay, with eager prompt steps in between."""
    prompts = [tokens_for(CFG_A, n, 300 + n) for n in (9, 30, 17)]
    outs = []
    for eager in (True, False):
        eng = make_engine(model_a[0], "cuda:0", torch.float32, enforce_eager=eager)
        seqs = [eng.add_request(p, SamplingParams(max_new_tokens=12)) for p in prompts[:2]]
        for _ in range(5):
            eng.step()
        seqs.append(eng.add_request(prompts[2], SamplingParams(max_new_tokens=12)))
        eng.generate_all(max_steps=100)
        outs.append([s.output_token_ids for s in seqs])
    assert outs[0] == outs[1]


def test_served_through_the_pool_and_front_door(tmp_path):
    """A model folder as the pool's base model: worker process, router, HTTP
    front door, greedy completion from prompt token ids."""
    from starlette.testclient import TestClient

    from llm_instance_gateway_amd.api.types import InferenceModel
    from llm_instance_gateway_amd.serving import EnginePool, build_app

    cfg = dict(CFG_A, vocab=300)
    W = make_checkpoint(cfg, 24)
    path = write_model(tmp_path / "served", cfg, W)
    pool = EnginePool(
        path, devices=["cpu"],
        engine_kwargs=dict(num_kv_blocks=64, max_num_seqs=4, max_num_batched_tokens=64, max_model_len=256),
    )
    pool.start()
    try:
        pool.datastore.store_model(InferenceModel(model_name="postnorm"))
        client = TestClient(build_app(pool))
        prompt = tokens_for(cfg, 23, 8)
        r = client.post("/v1/completions", json={"model": "postnorm", "prompt": prompt, "max_tokens": 5})
        assert r.status_code == 200, r.text
        out = r.json()["choices"][0]["token_ids"]
        assert len(out) == 5
        toks = list(prompt)
        for step in range(5):  # workers run bf16: only a clear argmax must match
            logits = oracle(cfg, W, toks)[0][-1]
            top2 = torch.topk(logits, 2).values
            if float(top2[0] - top2[1]) > 0.2:
                assert out[step] == int(torch.argmax(logits)), (step, out)
            toks.append(out[step])
    finally:
        pool.stop()
