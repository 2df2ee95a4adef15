"""The ops behind the Vemenex blocks, each alone, against the float64 oracle
in vemenex_oracle.py.  CPU parametrisation: the torch execution path; `gpu`:
the HIP kernels in fp32 and bf16 storage.

Random inputs hide some faults (one key among many weighs little), so the
attention tests scale one query and one key until a single score stands out,
and place that key where a window, a page or a tile ends.
"""

import numpy as np
import pytest
import torch

from llm_instance_gateway_amd import ops
from llm_instance_gateway_amd.models.hybrid_blocks import (
    GatedReluMLP, GroupRoutedExpertsMLP, expert_dispatch_plan,
)

import vemenex_oracle as O

CASES = [("cpu", torch.float32), pytest.param("cuda:0", torch.float32, marks=pytest.mark.gpu),
         pytest.param("cuda:0", torch.bfloat16, marks=pytest.mark.gpu)]
DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]


def rnd(g, *shape, s=1.0):
    return torch.randn(*shape, generator=g) * s


def close(got, want, dtype, scale=None):
    want = torch.as_tensor(want)
    ref = want.abs().max().item() if scale is None else scale
    err = (got.double().cpu() - want).abs().max().item() / max(ref, 1e-30)
    assert err < (2e-5 if dtype == torch.float32 else 2e-2), err


def i32(v, dev):
    return torch.tensor(v, dtype=torch.int32, device=dev)


# -- the residual as streams ----------------------------------------------------------

@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("S,W", [(1, 7), (2, 64), (3, 50), (4, 36), (5, 12)])
def test_hyper_step(device, dtype, S, W):
    g = torch.Generator().manual_seed(1)
    R, eps, m = 6, 1e-5, 0.6
    xs = rnd(g, R, S, W, s=3.0)
    y = rnd(g, R, W).to(dtype)
    mix, outw = torch.eye(S) + 0.3 * rnd(g, S, S), 0.5 + torch.rand(S, generator=g)
    inw, gw = torch.rand(S, generator=g) + 0.1, torch.tensor([1.3])
    dev = lambda t: t.to(device)
    # read only
    x1 = dev(xs.clone())
    h = ops.hyper_step(x1, None, None, None, m, dev(inw), dev(gw), eps, dtype)
    assert torch.equal(x1.cpu(), xs) and h.dtype == dtype
    xo = xs.double().numpy().transpose(1, 0, 2)  # the oracle keeps [S, R, W]
    close(h, O.scalar_norm(O.hyper_read(xo, inw.double().numpy()), 1.3, eps), dtype)
    # write + read in one pass; the write must use the OLD streams for every target
    h = ops.hyper_step(x1, dev(y), dev(mix), dev(outw), m, dev(inw), dev(gw), eps, dtype)
    xn = O.hyper_write(xo, y.double().numpy(), mix.double().numpy(), outw.double().numpy(), m)
    close(x1, xn.transpose(1, 0, 2), torch.float32)
    close(h, O.scalar_norm(O.hyper_read(xn, inw.double().numpy()), 1.3, eps), dtype)
    # write only
    x2 = dev(xs.clone())
    assert ops.hyper_step(x2, dev(y), dev(mix), dev(outw), m, None, None, eps, dtype) is None
    close(x2, xn.transpose(1, 0, 2), torch.float32)


# -- rotation, norm after rotation, cache write ------------------------------------------

@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("layout,rot,D,Dv,factor", [("interleaved", 6, 10, 6, 4.0), ("half", 4, 10, 6, 1.0),
                                                    ("interleaved", 16, 16, 8, 1.0), ("half", 16, 16, 24, 2.0),
                                                    ("half", 0, 5, 3, 1.0)])
def test_rotate_then_unit_norm_into_cache(device, dtype, layout, rot, D, Dv, factor):
    g = torch.Generator().manual_seed(2)
    R, H, G, eps, bs = 9, 4, 2, 1e-5, 4
    nq, nk, nv = H * D, G * D, G * Dv
    proj = rnd(g, R, nq + nk + nv + 8).to(dtype)  # gate columns ride behind q | k | v
    pos = torch.tensor([0, 1, 2, 40, 41, 1000, 7, 8, 9])
    slots = torch.tensor([5, 0, 11, 6, 3, 10, 9, 8, 2])
    inv_freq = ops.rotary_inv_freq(100.0, rot, device, factor) if rot else None
    kc = torch.full((3, G, bs, D), 7.0, dtype=dtype, device=device)
    vc = torch.full((3, G, bs, Dv), -7.0, dtype=dtype, device=device)
    q, _ = ops.qkv_norm_rope_cache(
        proj.to(device), H, G, D, Dv, "head_post", None, None, eps, inv_freq, pos.to(device),
        kc, vc, slots.to(device), rot_layout=layout,
    )
    P = proj.double().numpy()
    qo, ko = P[:, :nq].reshape(R, H, D), P[:, nq : nq + nk].reshape(R, G, D)
    vo = P[:, nq + nk : nq + nk + nv].reshape(R, G, Dv)
    fr = O.rotary_freqs(100.0, rot, factor) if rot else []
    qo = O.rms(O.rotate(qo, pos.numpy(), fr, layout), eps)
    ko = O.rms(O.rotate(ko, pos.numpy(), fr, layout), eps)
    # angles at position 1000 carry the fp32 rounding of the frequency
    close(q, qo.reshape(R, nq), dtype, scale=30.0 if rot and dtype == torch.float32 else None)
    kflat = kc.permute(0, 2, 1, 3).reshape(-1, G, D)
    vflat = vc.permute(0, 2, 1, 3).reshape(-1, G, Dv)
    close(kflat[slots.to(device)], ko, dtype, scale=30.0 if rot and dtype == torch.float32 else None)
    close(vflat[slots.to(device)], vo, dtype)
    untouched = sorted(set(range(12)) - set(slots.tolist()))
    assert torch.all(kflat[untouched].float() == 7.0) and torch.all(vflat[untouched].float() == -7.0)


# -- windowed attention -------------------------------------------------------------------

def paged_sequence(k, v, bs, table, kc, vc):
    for t in range(k.shape[0]):
        kc[table[t // bs], :, t % bs] = k[t].to(kc.dtype)
        vc[table[t // bs], :, t % bs] = v[t].to(vc.dtype)


def planted(g, T, H, G, D, Dv, dtype, plant, boost=5.0):
    """Random q, k, v with, for every (query, key) in `plant`, that query and
    key pushed along one axis so that their score stands out."""
    q, k, v = rnd(g, T, H, D, s=0.3), rnd(g, T, G, D, s=0.3), rnd(g, T, G, Dv)
    for qi, kj in plant:
        if not 0 <= kj < T:
            continue
        d = torch.zeros(D)
        d[(qi + kj) % D] = 1.0
        q[qi] += boost * d
        k[kj] += boost * d
    return q.to(dtype), k.to(dtype), v.to(dtype)


def window_plant(rows, w):
    """For every row: the oldest key its window keeps, the one just outside,
    its own position and the one after it."""
    out = []
    for r in rows:
        out += [(r, r - w + 1), (r, r - w), (r, r), (r, r + 1)]
    return out


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("kind", ["sigmoid", "sink"])
@pytest.mark.parametrize("window", [1, 7, 16, 50, 64, 65, 1000])
def test_windowed_attention_rows(device, dtype, kind, window):
    """Dominating keys just inside and just outside the window, at page
    borders, at the query itself and one past it; the first tokens of the
    sequence, whose windows reach past its start."""
    g = torch.Generator().manual_seed(3)
    T, H, G, D, Dv, bs, scale = 150, 4, 2, 12, 6, 16, 0.5
    rows = [149, 148, 130, 128, 127, 112, 100, 80, 65, 64, 63, 49, 48, 16, 15, 7, 6, 1, 0]
    # and keys far back (the sequence's first tokens), which only the longest window may see
    far = [(149, 2), (130, 0), (100, 17)]
    q, k, v = planted(g, T, H, G, D, Dv, dtype, window_plant(rows, window) + far)
    kc = torch.full((12, G, bs, D), 7.0, dtype=dtype, device=device)
    vc = torch.full((12, G, bs, Dv), -7.0, dtype=dtype, device=device)
    table = [9, 2, 7, 0, 5, 11, 3, 8, 1, 10]
    paged_sequence(k, v, bs, table, kc, vc)
    pb = rnd(g, H) - 3.0
    gate = rnd(g, T, H, s=2.0).to(dtype)
    qd, kd, vd = q.double().numpy(), k.double().numpy(), v.double().numpy()
    if kind == "sigmoid":
        want = O.windowed_attention(qd, kd, vd, scale, window, "sigmoid", pb.double().numpy())
        kw = dict(weights="sigmoid", score_bias=pb.to(device))
    else:
        want = O.windowed_attention(qd, kd, vd, scale, window, "sink")
        want = want * O.sigmoid(gate.double().numpy())[:, :, None]
        kw = dict(sink=torch.zeros(H, device=device), gate=gate[rows].to(device), gate_per_head=True)
    bt = i32([[0] * 10, table], device)
    got = ops.paged_attention_general(
        q[rows].reshape(len(rows), H * D).to(device), kc, vc, bt, i32([1] * (len(rows) - 1) + [-1], device),
        torch.tensor(rows, device=device), scale, H, window=window, **kw,
    )
    close(got[:-1], want[rows[:-1]].reshape(len(rows) - 1, H * Dv), dtype, scale=np.abs(want).max())
    assert torch.all(got[-1] == 0)  # a row of no sequence


def test_sink_takes_weight_and_sigmoid_weights_do_not_sum_to_one():
    """With scores far below zero the sink holds almost all of the softmax
    (the output vanishes); with one key the sigmoid weight is its logistic,
    not one."""
    T, H, D = 3, 1, 4
    q = np.zeros((T, H, D)); k = np.zeros((T, H, D)); v = np.ones((T, H, 2))
    q[:, 0, 0], k[:, 0, 0] = 10.0, -10.0
    out = O.windowed_attention(q, k, v, 1.0, 5, "sink")
    assert np.all(np.abs(out) < 1e-30)
    kc = torch.zeros(1, 1, 4, D); vc = torch.ones(1, 1, 4, 2)
    kc[0, 0, :3, 0] = -10.0
    got = ops.paged_attention_general(
        torch.tensor(q).float().reshape(T, D), kc, vc, i32([[0]], "cpu"), i32([0] * 3, "cpu"),
        torch.arange(3), 1.0, 1, sink=torch.zeros(1),
    )
    assert got.abs().max().item() < 1e-30
    got = ops.paged_attention_general(
        torch.zeros(1, D), kc, vc, i32([[0]], "cpu"), i32([0], "cpu"), torch.tensor([0]), 1.0, 1,
        weights="sigmoid", score_bias=torch.tensor([-1.0]),
    )
    assert abs(got[0, 0].item() - 1.0 / (1.0 + np.e)) < 1e-6


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["sigmoid", "sink"])
@pytest.mark.parametrize("window,D,Dv", [(1, 32, 16), (50, 32, 16), (64, 96, 32), (33, 24, 40), (200, 64, 64),
                                          (128, 128, 128), (1000, 16, 8)])
def test_windowed_attention_prompt_tiles(kind, window, D, Dv):
    """The MFMA prompt kernel with the window mask: three portions in one
    launch (a whole prompt, a portion that starts inside a sequence, a short
    one), window edges inside and at the borders of 64-row tiles."""
    dev, dtype = "cuda:0", torch.bfloat16
    g = torch.Generator().manual_seed(4)
    H, G, bs, scale = 4, 2, 16, 0.4
    seqs = [(230, 0), (200, 90), (40, 37)]  # (tokens after the step, tokens before it)
    kc = torch.full((40, G, bs, D), 7.0, dtype=dtype, device=dev)
    vc = torch.full((40, G, bs, Dv), -7.0, dtype=dtype, device=dev)
    pb = rnd(g, H) - 3.0
    qs, gs, wants, tables, at = [], [], [], [], 0
    for ctx, done in seqs:
        rows = [ctx - 1, done, done + 1, min(done + 63, ctx - 1), min(done + 64, ctx - 1), (done + ctx) // 2]
        far = [(ctx - 1, 1), (ctx - 1, done)]  # far back, and the portion's first key
        q, k, v = planted(g, ctx, H, G, D, Dv, dtype, window_plant(rows, window) + far, boost=4.0)
        gate = rnd(g, ctx, H, s=2.0).to(dtype)
        nb = (ctx + bs - 1) // bs
        table = list(range(at, at + nb))[::-1]
        at += nb
        paged_sequence(k, v, bs, table, kc, vc)
        qd, kd, vd = q.double().numpy(), k.double().numpy(), v.double().numpy()
        if kind == "sigmoid":
            want = O.windowed_attention(qd, kd, vd, scale, window, "sigmoid", pb.double().numpy())
        else:
            want = O.windowed_attention(qd, kd, vd, scale, window, "sink")
            want = want * O.sigmoid(gate.double().numpy())[:, :, None]
        qs.append(q[done:].reshape(ctx - done, H * D))
        gs.append(gate[done:])
        wants.append(torch.from_numpy(want[done:].reshape(ctx - done, H * Dv)))
        tables.append(table + [0] * (16 - nb))
    lens = [c_ - d_ for c_, d_ in seqs]
    qsl = [0, lens[0], lens[0] + lens[1], sum(lens)]
    ts, tq = [], []
    for si, n in enumerate(lens):
        for qb in range(0, n, 64):
            ts.append(si)
            tq.append(qb)
    if kind == "sigmoid":
        kw = dict(weights="sigmoid", score_bias=pb.to(dev))
    else:
        kw = dict(sink=torch.zeros(H, device=dev), gate=torch.cat(gs).to(dev), gate_per_head=True)
    got = ops.paged_attention_prefill_tiles(
        torch.cat(qs).to(dev), kc, vc, i32(tables, dev), i32(qsl, dev), i32([s[0] for s in seqs], dev),
        i32(ts, dev), i32(tq, dev), scale, H, window=window, **kw,
    )
    close(got, torch.cat(wants), dtype)


# -- feed-forwards ----------------------------------------------------------------------------

@pytest.mark.parametrize("device,dtype", CASES)
def test_glu_activations(device, dtype):
    g = torch.Generator().manual_seed(5)
    for F_ in (12, 7):
        x = rnd(g, 9, 2 * F_, s=2.0).to(dtype)
        gt, up = x[:, :F_].double().numpy(), x[:, F_:].double().numpy()
        close(ops.glu_act(x.to(device), "relu"), np.maximum(gt, 0) * up, dtype)
        for limit in (0.7, 5.0):
            gg, uu = np.minimum(gt, limit), np.clip(up, -limit, limit)
            close(ops.glu_act(x.to(device), "clamped", limit, 1.702),
                  gg * O.sigmoid(1.702 * gg) * (uu + 1), dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("N,groups,keep,top", [(18, 2, 1, 4), (8, 4, 2, 3), (5, 1, 1, 2), (1, 1, 1, 1),
                                                (12, 3, 3, 12), (130, 10, 3, 6), (64, 64, 5, 5)])
def test_grouped_router(device, N, groups, keep, top):
    g = torch.Generator().manual_seed(6)
    T = 40
    z = rnd(g, T, N, s=2.0)
    corr = rnd(g, N, s=0.2)
    # negative choice scores: a barred output must count as minus infinity, not 0
    corr[: N // 2] -= 1.0
    z[3] = z[2]  # equal rows choose equally
    idx, w = ops.grouped_topk_route(z.to(device), corr.to(device), top, groups, keep)
    ci, cw = O.route(z.double().numpy(), corr.double().numpy(), top, groups, keep)
    assert idx.dtype == torch.int32 and w.dtype == torch.float32
    assert np.array_equal(idx.cpu().numpy(), ci)
    close(w, cw, torch.float32)
    assert torch.allclose(w.sum(-1).cpu(), torch.ones(T), atol=1e-5)
    idx2, _ = ops.grouped_topk_route(z.to(device), None, top, groups, keep)
    ci2, _ = O.route(z.double().numpy(), np.zeros(N), top, groups, keep)
    assert np.array_equal(idx2.cpu().numpy(), ci2)


def test_dispatch_plan_leaves_identity_pairs_out():
    idx = torch.tensor([[0, 5], [2, 0], [4, 3], [0, 2]])
    gather, rows, cap = expert_dispatch_plan(idx, 3)  # choices 3, 4, 5 are no batch's
    assert cap == 3 and gather.shape == (9,)
    assert rows.tolist() == [[0, -1], [6, 1], [-1, -1], [2, 7]]
    assert gather.tolist() == [0, 1, 3, -1, -1, -1, 1, 3, -1]


@pytest.mark.parametrize("device,dtype", CASES)
def test_routed_combine(device, dtype):
    g = torch.Generator().manual_seed(7)
    T, W, top = 5, 20, 3
    ye, x = rnd(g, 11, W).to(dtype), rnd(g, T, W).to(dtype)
    rows = torch.tensor([[0, 10, -1], [-1, -1, 3], [4, 4, 4], [7, -1, 2], [1, 9, 5]])
    w = torch.rand(T, top, generator=g)
    got = ops.routed_combine(ye.to(device), x.to(device), rows.to(device), w.to(device))
    want = np.zeros((T, W))
    for t in range(T):
        for k in range(top):
            src = x[t] if rows[t, k] < 0 else ye[rows[t, k]]
            want[t] += w[t, k].item() * src.double().numpy()
    close(got, want, dtype)
    # every expert saw every token: rows follow from the choices
    E = 3
    ye2 = rnd(g, E * T, W).to(dtype)
    idx = torch.tensor([[0, 2, 4], [3, 1, 0], [2, 2, 2], [5, 4, 3], [1, 0, 2]], dtype=torch.int32)
    got = ops.routed_combine(ye2.to(device), x.to(device), None, w.to(device), idx=idx.to(device), experts=E)
    want = np.zeros((T, W))
    for t in range(T):
        for k in range(top):
            e = int(idx[t, k])
            src = x[t] if e >= E else ye2[e * T + t]
            want[t] += w[t, k].item() * src.double().numpy()
    close(got, want, dtype)


@pytest.mark.parametrize("device,dtype", CASES)
def test_gated_relu_mlp(device, dtype):
    g = torch.Generator().manual_seed(8)
    H, ff, T = 24, 17, 6
    W = {"gate": rnd(g, ff, H, s=H ** -0.5).to(dtype), "up": rnd(g, ff, H, s=H ** -0.5).to(dtype),
         "down": rnd(g, H, ff, s=ff ** -0.5).to(dtype)}
    mod = GatedReluMLP(H, ff, device=device, dtype=dtype)
    mod.load(lambda n: W[n].to(device), "")
    h = rnd(g, T, H).to(dtype)
    want = O.dense_ff(h.double().numpy(), {k: v.double().numpy() for k, v in W.items()})
    close(mod(h.to(device)), want, dtype)


class _Meta:
    def __init__(self, prefill):
        self.num_prefill_tokens = prefill


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,ident,groups,keep,top", [(6, 2, 4, 2, 3), (3, 0, 1, 1, 2), (1, 0, 1, 1, 1), (2, 4, 3, 2, 4)])
def test_group_routed_experts_both_dispatch_paths(device, E, ident, groups, keep, top):
    """Sorted capacity-padded dispatch (prompt steps) and dense dispatch
    (single-token steps) against the oracle; identity experts pass the input."""
    g = torch.Generator().manual_seed(9)
    H, ff, T, limit = 20, 9, 23, 0.8
    dtype = torch.float32
    W = {"router": rnd(g, E + ident, H, s=2 * H ** -0.5), "correction": rnd(g, E + ident, s=0.1)}
    for e in range(E):
        W[f"e{e}.gate"], W[f"e{e}.up"] = rnd(g, ff, H, s=2 * H ** -0.5), rnd(g, ff, H, s=2 * H ** -0.5)
        W[f"e{e}.down"] = rnd(g, H, ff, s=ff ** -0.5)
    mod = GroupRoutedExpertsMLP(H, ff, E, top, identity=ident, groups=groups, keep=keep, limit=limit,
                                device=device, dtype=dtype)
    mod.load(lambda n: W[n].to(device), "")
    h = rnd(g, T, H)
    mlp = {"expert": {"ff": ff, "limit": limit},
           "router": {"experts": E, "identity": ident, "top": top, "groups": {"count": groups, "keep": keep}}}
    want = O.moe_ff(h.double().numpy(), {k: v.double().numpy() for k, v in W.items()}, mlp)
    close(mod(h.to(device), _Meta(T)), want, dtype, scale=np.abs(want).max())
    close(mod(h.to(device), _Meta(0)), want, dtype, scale=np.abs(want).max())
