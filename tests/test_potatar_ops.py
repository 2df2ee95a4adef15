"""The ops behind the Potatar blocks, each alone, against the float64 oracle
in potatar_oracle.py.  CPU parametrisation: the torch execution path; `gpu`:
the HIP kernels in fp32 and bf16 storage.

Random inputs hide some faults (one key among hundreds weighs nothing), so
the attention tests scale one query and one key until a single score
dominates, and place that key where a mask, a page or a tile ends.
"""

import math

import numpy as np
import pytest
import torch

from llm_instance_gateway_amd import ops

import potatar_oracle as O

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
CASES = [("cpu", torch.float32), pytest.param("cuda:0", torch.float32, marks=pytest.mark.gpu),
         pytest.param("cuda:0", torch.bfloat16, marks=pytest.mark.gpu)]


def rnd(g, *shape, s=1.0):
    return torch.randn(*shape, generator=g) * s


def q16(t, dtype):
    """Round to the storage type and back: the oracle sees what the op sees."""
    return t.to(dtype).double()


def close(got, want, dtype, scale=None):
    want = torch.as_tensor(want)
    ref = want.abs().max().item() if scale is None else scale
    err = (got.double().cpu() - want).abs().max().item() / max(ref, 1e-30)
    assert err < (2e-5 if dtype == torch.float32 else 2e-2), err


def i32(v, dev):
    return torch.tensor(v, dtype=torch.int32, device=dev)


@pytest.mark.parametrize("device,dtype", CASES)
def test_scaled_add_rms_norm(device, dtype):
    g = torch.Generator().manual_seed(1)
    R, H, eps = 7, 50, 1e-4
    x, y1, y2 = rnd(g, R, H, s=3), rnd(g, R, H).to(dtype), rnd(g, R, H).to(dtype)
    w = (1 + 0.3 * rnd(g, H)).to(dtype)
    for alpha, s1, s2, two in ((2.5, 1.0, 1.0, False), (0.7, 0.8, 0.9, True)):
        xs = x.clone().to(device)
        xo, h = ops.scaled_add_rms_norm(
            xs, alpha, w.to(device), eps, y1.to(device), s1, y2.to(device) if two else None, s2)
        t = alpha * x.double().numpy() + s1 * y1.double().numpy() + (s2 * y2.double().numpy() if two else 0)
        want = O.rms(t, eps) * w.double().numpy()
        assert xo.data_ptr() == xs.data_ptr() and xo.dtype == torch.float32 and h.dtype == dtype
        close(xo, want, torch.float32)
        close(h, want, dtype)
    xs = x.clone().to(device)
    _, h = ops.scaled_add_rms_norm(xs, 1.0, w.to(device), eps)  # norm only
    assert torch.equal(xs.cpu(), x)
    close(h, O.rms(x.double().numpy(), eps) * w.double().numpy(), dtype)


def make_caches(blocks, G, bs, D, Dv, dtype, device, fill=7.0):
    """Caches full of junk: what is not written this test must not be read."""
    k = torch.full((blocks, G, bs, D), fill, dtype=dtype, device=device)
    v = torch.full((blocks, G, bs, Dv), -fill, dtype=dtype, device=device)
    return k, v


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize(
    "mode,rot,from_key,unit,mix",
    [("row", 6, False, True, True), ("head", 0, True, False, False), ("none", 10, False, False, True),
     ("row", 2, False, True, False)],
)
def test_qkv_norm_rope_cache(device, dtype, mode, rot, from_key, unit, mix):
    g = torch.Generator().manual_seed(2)
    R, H, G, D, eps, bs = 9, 4, 2, 10, 1e-5, 4
    Dv = D if from_key else 6
    nq, nk, nv = H * D, G * D, G * Dv
    extra = 5  # further columns of a wider fused projection
    proj = rnd(g, R, nq + nk + (0 if from_key else nv) + extra).to(dtype)
    wq = (1 + 0.3 * rnd(g, nq if mode == "row" else D)).to(dtype)
    wk = (1 + 0.3 * rnd(g, nk if mode == "row" else D)).to(dtype)
    pos = torch.tensor([0, 1, 2, 40, 41, 1000, 7, 8, 9])
    slots = torch.tensor([5, 0, 11, 6, 3, 10, 9, 8, 2])
    v_first = rnd(g, R, nv) if mix else None
    lam = 0.3
    inv_freq = ops.rotary_inv_freq(100.0, rot, device) if rot else None
    kc, vc = make_caches(3, G, bs, D, Dv, dtype, device)
    q, v_out = ops.qkv_norm_rope_cache(
        proj.to(device), H, G, D, Dv, mode, wq.to(device), wk.to(device), eps, inv_freq,
        pos.to(device), kc, vc, slots.to(device), v_source="key" if from_key else "proj",
        v_unit_norm=unit, v_first=None if v_first is None else v_first.to(device), lam=lam,
        want_v=True,
    )
    P = proj.double().numpy()
    qo, ko = P[:, :nq], P[:, nq : nq + nk]
    vo = ko.copy() if from_key else P[:, nq + nk : nq + nk + nv]
    if mode == "row":
        qo, ko = O.rms(qo, eps) * wq.double().numpy(), O.rms(ko, eps) * wk.double().numpy()
    qo, ko = qo.reshape(R, H, D), ko.reshape(R, G, D)
    if mode == "head":
        qo, ko = O.rms(qo, eps) * wq.double().numpy(), O.rms(ko, eps) * wk.double().numpy()
    if rot:
        qo, ko = O.rotate_half(qo, pos.numpy(), 100.0, rot), O.rotate_half(ko, pos.numpy(), 100.0, rot)
    vo = vo.reshape(R, G, Dv)
    if unit:
        vo = O.rms(vo, eps)
    if mix:
        vo = (1 - lam) * vo + lam * v_first.double().numpy().reshape(R, G, Dv)
    # angles at position 1000 carry fp32 rounding of the frequency
    close(q, qo.reshape(R, nq), dtype if dtype == torch.bfloat16 else torch.float32, scale=30.0 if rot else None)
    close(v_out, vo.reshape(R, nv), torch.float32)
    kflat = kc.permute(0, 2, 1, 3).reshape(-1, G, D)
    vflat = vc.permute(0, 2, 1, 3).reshape(-1, G, Dv)
    close(kflat[slots.to(device)], ko, dtype, scale=30.0 if rot else None)
    close(vflat[slots.to(device)], vo, dtype)
    untouched = sorted(set(range(12)) - set(slots.tolist()))
    assert torch.all(kflat[untouched].float() == 7.0) and torch.all(vflat[untouched].float() == -7.0)


def paged_sequence(k, v, bs, table, kc, vc):
    """Write one sequence's keys/values [T, G, *] into the pages `table`."""
    T = k.shape[0]
    for t in range(T):
        kc[table[t // bs], :, t % bs] = k[t].to(kc.dtype)
        vc[table[t // bs], :, t % bs] = v[t].to(vc.dtype)


def planted(g, T, H, G, D, Dv, dtype, plant):
    """Random q, k, v with, for every (query, key) in `plant`, that query and
    key scaled so that their score stands out."""
    q, k, v = rnd(g, T, H, D, s=0.3), rnd(g, T, G, D, s=0.3), rnd(g, T, G, Dv)
    for qi, kj in plant:
        d = torch.zeros(D)
        d[(qi + kj) % D] = 1.0
        q[qi] += 6.0 * d
        k[kj] += 6.0 * d
    return q.to(dtype), k.to(dtype), v.to(dtype)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("chunk", [0, 50, 64, 7])
def test_chunked_attention_rows(device, dtype, chunk):
    """Keys that dominate: far back inside the chunk, the chunk's first key,
    the last key of the chunk before (must not be seen), at a page border, at
    the query's own position, one past it (must not be seen)."""
    g = torch.Generator().manual_seed(3)
    T, H, G, D, Dv, bs, scale = 150, 4, 2, 12, 6, 16, 0.5
    c = chunk or 10 ** 6
    plant = [(149, (149 // c) * c), (149, max((149 // c) * c - 1, 0)), (130, 128), (127, 112),
             (100, 100), (99, 100), (64, 63), (63, 0), (15, 16)]
    q, k, v = planted(g, T, H, G, D, Dv, dtype, plant)
    kc, vc = make_caches(12, G, bs, D, Dv, dtype, device)
    table = [9, 2, 7, 0, 5, 11, 3, 8, 1, 10]
    paged_sequence(k, v, bs, table, kc, vc)
    want = O.chunked_attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), scale, chunk)
    bt = i32([[0] * 10, table], device)
    rows = [149, 148, 130, 127, 100, 99, 64, 63, 16, 15, 0, 50, 49]
    got = ops.paged_attention_general(
        q[rows].reshape(len(rows), H * D).to(device), kc, vc, bt, i32([1] * len(rows), device),
        torch.tensor(rows, device=device), scale, H, chunk=chunk,
    )
    close(got, want[rows].reshape(len(rows), H * Dv), dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("chunk,D,Dv", [(0, 32, 16), (50, 32, 16), (64, 96, 32), (33, 24, 40), (200, 64, 64)])
def test_chunked_attention_prompt_tiles(chunk, D, Dv):
    """The MFMA prompt kernel with the chunk mask: three portions in one
    launch (a whole prompt, a portion that starts inside a chunk, a short
    one), chunk edges inside and at the borders of 64-row tiles."""
    dev, dtype = "cuda:0", torch.bfloat16
    g = torch.Generator().manual_seed(4)
    H, G, bs, scale = 4, 2, 16, 0.4
    c = chunk or 10 ** 6
    seqs = [(230, 0), (200, 90), (40, 37)]  # (tokens after the step, tokens before it)
    kc, vc = make_caches(40, G, bs, D, Dv, dtype, dev)
    qs, wants, tables, at = [], [], [], 0
    for ctx, done in seqs:
        plant = [(ctx - 1, ((ctx - 1) // c) * c), (ctx - 1, max(((ctx - 1) // c) * c - 1, 0)), (done, done),
                 (done + 1, (done // c) * c), (min(done + 64, ctx - 1), done + 63 if done + 63 < ctx else done)]
        q, k, v = planted(g, ctx, H, G, D, Dv, dtype, plant)
        nb = (ctx + bs - 1) // bs
        table = list(range(at, at + nb))[::-1]
        at += nb
        paged_sequence(k, v, bs, table, kc, vc)
        want = O.chunked_attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), scale, chunk)
        qs.append(q[done:].reshape(ctx - done, H * D))
        wants.append(torch.from_numpy(want[done:].reshape(ctx - done, H * Dv)))
        tables.append(table + [0] * (16 - nb))
    lens = [c_ - d_ for c_, d_ in seqs]
    qsl = [0, lens[0], lens[0] + lens[1], sum(lens)]
    ts, tq = [], []
    for si, n in enumerate(lens):
        for qb in range(0, n, 64):
            ts.append(si)
            tq.append(qb)
    got = ops.paged_attention_prefill_tiles(
        torch.cat(qs).to(dev), kc, vc, i32(tables, dev), i32(qsl, dev), i32([s[0] for s in seqs], dev),
        i32(ts, dev), i32(tq, dev), scale, H, chunk=chunk,
    )
    close(got, torch.cat(wants), dtype)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,G,D,chunk,rows_far", [(4, 2, 10, 40, (10, 30.0)), (6, 3, 48, 64, (16, 100.0)),
                                                   (1, 1, 5, 0, (4, 9.0)), (20, 10, 8, 50, (8, 64.0))])
def test_mixed_heads_attention(device, dtype, H, G, D, chunk, rows_far):
    """Distance bias + head mixing; values are rows of their own cache.  The
    bias table has a steep last row, so a wrong bucket for far keys shows;
    the mixing matrix is far from the identity."""
    g = torch.Generator().manual_seed(5)
    T, bs, scale = 140, 16, 0.6
    n_rel, far = rows_far
    c = chunk or 10 ** 6
    plant = [(139, (139 // c) * c), (139, max((139 // c) * c - 1, 0)), (120, 96), (64, 63), (63, 0), (90, 90)]
    q, k, v = planted(g, T, H, G, D, D, dtype, plant)
    rel = rnd(g, n_rel, H, s=0.8)
    rel[-1] += 2.0
    talk = torch.eye(H) + 0.4 * rnd(g, H, H)
    kc, vc = make_caches(10, G, bs, D, D, dtype, device)
    table = [4, 9, 1, 6, 0, 8, 3, 7, 2]
    paged_sequence(k, v, bs, table, kc, vc)
    want = O.chunked_attention(
        q.double().numpy(), k.double().numpy(), v.double().numpy(), scale, chunk,
        bias=O.distance_bias(rel.double().numpy(), T, far), talk=talk.double().numpy(),
    )
    tab = ops.distance_bias_table(rel.to(device), far)
    for n in range(0, 200):
        assert torch.equal(tab[min(n, tab.shape[0] - 1)].cpu(), rel[O.distance_bucket(n, n_rel, far)])
    rows = [139, 138, 120, 90, 64, 63, 41, 40, 39, 1, 0]
    got = ops.paged_attention_mixed_heads(
        q[rows].reshape(len(rows), H * D).to(device), kc, vc, i32([[0] * 9, table], device),
        i32([1] * (len(rows) - 1) + [-1], device), torch.tensor(rows, device=device), scale, H,
        dist_bias=tab, talk=talk.to(device), chunk=chunk,
    )
    close(got[:-1], want[rows[:-1]].reshape(len(rows) - 1, H * D), dtype)
    assert torch.all(got[-1] == 0)  # a row of no sequence
    # without bias and mixing it is ordinary chunked attention
    plain = ops.paged_attention_mixed_heads(
        q[rows].reshape(len(rows), H * D).to(device), kc, vc, i32([[0] * 9, table], device),
        i32([1] * len(rows), device), torch.tensor(rows, device=device), scale, H, chunk=chunk,
    )
    want0 = O.chunked_attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), scale, chunk)
    close(plain, want0[rows].reshape(len(rows), H * D), dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("chunk,H,G,D", [(0, 4, 2, 16), (50, 6, 3, 48), (64, 16, 4, 64), (33, 1, 1, 24), (200, 12, 4, 128), (200, 12, 12, 128),
                                           (64, 32, 8, 64), (50, 20, 5, 32)])
def test_mixed_heads_prompt_tiles(chunk, H, G, D):
    """The MFMA head-mixing kernel: three portions in one launch (a whole
    prompt, a portion that starts inside a chunk, a short one), chunk edges
    inside and at the borders of its 16-row workgroups, a steep last bias row
    and a mixing matrix far from the identity; up to 16 heads a wave serves
    one head, beyond that two."""
    dev, dtype = "cuda:0", torch.bfloat16
    assert ops.mixed_heads_tiles_supported(dtype, D, D, H, True)
    g = torch.Generator().manual_seed(9)
    bs, scale, n_rel, far = 16, 0.4, 12, 90.0
    c = chunk or 10 ** 6
    rel = rnd(g, n_rel, H, s=0.8)
    rel[-1] += 2.0
    talk = torch.eye(H) + 0.4 * rnd(g, H, H)
    tab = ops.distance_bias_table(rel.to(dev), far)
    seqs = [(230, 0), (200, 90), (40, 37)]  # (tokens after the step, tokens before it)
    kc, vc = make_caches(40, G, bs, D, D, dtype, dev)
    qs, wants, tables, at = [], [], [], 0
    for ctx, done in seqs:
        plant = [(ctx - 1, ((ctx - 1) // c) * c), (ctx - 1, max(((ctx - 1) // c) * c - 1, 0)), (done, done),
                 (done + 1, (done // c) * c), (min(done + 16, ctx - 1), done + 15 if done + 15 < ctx else done)]
        q, k, v = planted(g, ctx, H, G, D, D, dtype, plant)
        nb = (ctx + bs - 1) // bs
        table = list(range(at, at + nb))[::-1]
        at += nb
        paged_sequence(k, v, bs, table, kc, vc)
        want = O.chunked_attention(
            q.double().numpy(), k.double().numpy(), v.double().numpy(), scale, chunk,
            bias=O.distance_bias(rel.double().numpy(), ctx, far), talk=talk.double().numpy())
        qs.append(q[done:].reshape(ctx - done, H * D))
        wants.append(torch.from_numpy(want[done:].reshape(ctx - done, H * D)))
        tables.append(table + [0] * (16 - nb))
    lens = [c_ - d_ for c_, d_ in seqs]
    qsl = [0, lens[0], lens[0] + lens[1], sum(lens)]
    ts, tq = [], []
    for si, n in enumerate(lens):
        for qb in range(0, n, 64):
            ts.append(si)
            tq.append(qb)
    got = ops.paged_attention_mixed_heads_tiles(
        torch.cat(qs).to(dev), kc, vc, i32(tables, dev), i32(qsl, dev), i32([s_[0] for s_ in seqs], dev),
        i32(ts, dev), i32(tq, dev), scale, H, dist_bias=tab, talk=talk.to(dev), chunk=chunk,
    )
    if G * D > 1024:  # K and V tiles of every key/value head exceed the LDS budget
        assert got is None
        return
    close(got, torch.cat(wants), dtype)


@pytest.mark.parametrize("device,dtype", CASES)
def test_token_shift_mix_through_reused_slots(device, dtype):
    g = torch.Generator().manual_seed(6)
    W, n = 20, 5
    mu = torch.rand(n, W, generator=g).to(dtype)
    seqs = {0: rnd(g, 9, W), 1: rnd(g, 4, W), 2: rnd(g, 1, W)}
    want = {s: np.stack([O.token_shift(x.double().numpy(), mu[m].double().numpy()) for m in range(n)]) for s, x in seqs.items()}
    state = torch.full((3, W), 99.0, device=device)  # stale content everywhere
    # step 1: seq 0 brings 3 tokens (slot 1), seq 1 brings 1 (slot 0); a pad row at the end
    steps = [
        ([(0, 0, 3, 1), (1, 0, 1, 0)], 1),
        ([(0, 3, 1, 1), (1, 1, 2, 0), (2, 0, 1, 2)], 0),   # seq 2 starts and ends in slot 2
        ([(0, 4, 5, 1), (1, 3, 1, 0)], 2),
    ]
    for plan, pad in steps:
        rows, tok_seq, s_start, s_len, s_slot, s_fresh = [], [], [], [], [], []
        for si, (s, lo, cnt, slot) in enumerate(plan):
            s_start.append(len(tok_seq))
            s_len.append(cnt)
            s_slot.append(slot)
            s_fresh.append(1 if lo == 0 else 0)
            tok_seq += [si] * cnt
            rows.append(seqs[s][lo : lo + cnt])
        x = torch.cat(rows + [rnd(g, pad, W)] if pad else rows)
        tok_seq += [-1] * pad
        out = ops.token_shift_mix(
            x.to(device), mu.to(device), state, i32(tok_seq, device), i32(s_start, device),
            i32(s_len, device), i32(s_slot, device), i32(s_fresh, device),
        )
        assert out.shape == (n, x.shape[0], W) and out.dtype == dtype
        for si, (s, lo, cnt, slot) in enumerate(plan):
            close(out[:, s_start[si] : s_start[si] + cnt], want[s][:, lo : lo + cnt], dtype)
        if pad:
            assert torch.all(out[:, -pad:] == 0)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("bonus", [True, False])
@pytest.mark.parametrize("H,D,Dv", [(3, 8, 8), (2, 5, 3), (1, 48, 48), (2, 33, 20)])
def test_matrix_state_scan(device, dtype, bonus, H, D, Dv):
    """Both recurrences: a prompt in one go, in portions and token by token,
    two sequences per launch through slots with stale content, more tokens
    than one staging tile, head sizes that are no multiple of the key split."""
    if bonus and D != Dv:
        Dv = D
    g = torch.Generator().manual_seed(7)
    lens = {0: 45, 1: 6}
    data, want = {}, {}
    u = rnd(g, H * D, s=0.5)
    decay = torch.tensor([0.6, 0.95, 0.999][:H])
    for s, T in lens.items():
        q, k, v = rnd(g, T, H * D).to(dtype), rnd(g, T, H * D, s=0.5).to(dtype), rnd(g, T, H * Dv).to(dtype)
        pre = rnd(g, T, H * D, s=1.0) - 1.5
        data[s] = (q, k, v, pre)
        qd, kd, vd = (t.double().numpy() for t in (q, k, v))
        if not bonus:
            qd, kd, vd = O.silu(qd), O.silu(kd), O.silu(vd)
        o = np.zeros((T, H, Dv))
        for h in range(H):
            sl, sv = slice(h * D, (h + 1) * D), slice(h * Dv, (h + 1) * Dv)
            if bonus:
                w = np.exp(-np.exp(pre.double().numpy()[:, sl]))
                o[:, h], _ = O.bonus_recurrence(qd[:, sl], kd[:, sl], vd[:, sv], w, u.double().numpy()[sl])
            else:
                o[:, h], _ = O.decay_recurrence(qd[:, sl], kd[:, sl], vd[:, sv], float(decay[h]))
        want[s] = o.reshape(T, H * Dv)
    for cuts0 in ([45], [20, 2, 1, 22], [1] * 45):
        state = torch.full((3, ops.matrix_state_width(H, D, Dv)), 5.0, device=device)
        at = {0: 0, 1: 0}
        for step, n0 in enumerate(cuts0):
            plan = [(0, n0, 2)]
            if step < 3 and at[1] < lens[1]:
                plan.append((1, 2, 0))
            qs, ks, vs, ps, s_start, s_len, s_slot, s_fresh, r = [], [], [], [], [], [], [], [], 0
            for s, n, slot in plan:
                q, k, v, pre = data[s]
                a = at[s]
                qs.append(q[a : a + n]); ks.append(k[a : a + n]); vs.append(v[a : a + n]); ps.append(pre[a : a + n])
                s_start.append(r); s_len.append(n); s_slot.append(slot); s_fresh.append(1 if a == 0 else 0)
                r += n
            # q, k, v as column blocks of one wider projection
            fused = torch.cat([torch.cat(qs), torch.cat(ks), torch.cat(vs)], dim=1).to(device)
            a_, b_ = H * D, 2 * H * D
            out = ops.matrix_state_scan(
                fused[:, :a_], fused[:, a_:b_], fused[:, b_:], state, i32(s_start, device),
                i32(s_len, device), i32(s_slot, device), i32(s_fresh, device), H, D, Dv,
                decay_pre=torch.cat(ps).contiguous().to(device) if bonus else None,
                bonus=u.to(device) if bonus else None,
                head_decay=None if bonus else decay.to(device), act_silu=not bonus,
            )
            assert out.dtype == torch.float32
            for (s, n, slot), r0 in zip(plan, s_start):
                close(out[r0 : r0 + n], want[s][at[s] : at[s] + n], dtype, scale=np.abs(want[s]).max())
                at[s] += n


@pytest.mark.parametrize("device,dtype", CASES)
def test_group_norm_gate_and_activations(device, dtype):
    g = torch.Generator().manual_seed(8)
    R, C, eps = 6, 24, 1e-5
    o, gate = rnd(g, R, C, s=4), rnd(g, R, C + 3).to(dtype)
    w = (1 + 0.3 * rnd(g, C)).to(dtype)
    gd = gate[:, 3:].double().numpy()
    for group, act in ((8, "silu"), (24, "sigmoid"), (1, "silu"), (3, "sigmoid")):
        got = ops.group_rms_norm_gate(o.to(device), gate.to(device)[:, 3:], w.to(device), group, act, eps)
        n = O.rms(o.double().numpy().reshape(R, C // group, group), eps).reshape(R, C) * w.double().numpy()
        close(got, n * (O.silu(gd) if act == "silu" else O.sigmoid(gd)), dtype)
    x = rnd(g, 5, 37, s=2).to(dtype)
    close(ops.gelu_erf(x.to(device)), O.gelu_erf(x.double().numpy()), dtype)
    close(ops.tanh_act(x.to(device)), np.tanh(x.double().numpy()), dtype)
    z = rnd(g, 4, 33, s=20)
    close(ops.tanh_softcap(z.clone().to(device), 15.0), 15.0 * np.tanh(z.double().numpy() / 15.0), torch.float32)
