"""The token-shifted pre-norm stacks of chunked attention and decaying linear attention (Negilorn) against the float64 restatement in
oracle/negilorn.py: every mechanism alone through the C ABI, then whole models through the engine's step function -- whole prompts,
token-by-token decoding, portions, mixed batches, reused pages and slots, a crafted key at every edge of a chunk, greedy generation.
Small random configurations of their own; `be` runs each test on the CPU twin and (gpu) on the MI355X."""
import json
import math
import os
import subprocess

import numpy as np
import pytest
import torch

from oracle import negilorn as ON
from tests.conftest import ROOT

F32, BF16, I32 = torch.float32, torch.bfloat16, torch.int32
TOL = {F32: 3e-5, BF16: 4e-2}


def dev(be, a, dtype=F32):
    return be.t(np.asarray(a, dtype=np.float32)).to(dtype).contiguous()


def ints(be, a):
    return be.t(np.asarray(a, dtype=np.int32))


def rel_err(got, want):
    """rms over the last axis of the difference (mean removed) relative to the rms of the reference"""
    d = np.asarray(got, dtype=np.float64) - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return float((np.sqrt((d * d).mean(-1)) / (np.sqrt((w * w).mean(-1)) + 1e-30)).max())


def close(got, want, tol):
    return np.abs(np.asarray(got, dtype=np.float64) - want).max() <= tol * (1 + np.abs(want).max())


def spans_of(be, lens):
    row0 = np.cumsum([0] + list(lens[:-1]))
    return ints(be, row0), ints(be, lens), len(lens), max(lens)


# ---- row-wise steps and epilogues ------------------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("width", [6, 50, 300, 1030])
def test_scalar_rms_norm_with_additions(be, dtype, width):
    rng = np.random.default_rng(width)
    rows, eps, gain, top = 5, 1e-3, 1.375, 3
    x = rng.standard_normal((rows, width)).astype(np.float32) * 3 + 1
    y = rng.standard_normal((rows, width)).astype(np.float32)
    my = rng.standard_normal((rows * top, width)).astype(np.float32)
    x32, out = be.t(x), torch.zeros((rows, width), dtype=dtype, device=be.device)
    be.ext.add_rms_shift(x32, be.t(y), out, rows, gain, eps, moe_y=be.t(my), top=top, dtype=dtype)
    s = x.astype(np.float64) + y + my.reshape(rows, top, width).sum(1)
    want = np.array([ON.scalar_rms_norm(s[r], gain, eps) for r in range(rows)])
    assert close(be.n(x32), s, 1e-6)
    assert close(be.n(out.float()), want, 3e-6 if dtype is F32 else 1e-2)
    # gathered rows, no addition
    idx = np.array([4, 1, 4], dtype=np.int32)
    out2 = torch.zeros((3, width), dtype=F32, device=be.device)
    be.ext.add_rms_shift(x32, None, out2, 3, gain, eps, row_idx=be.t(idx), dtype=dtype)
    assert close(be.n(out2), np.array([ON.scalar_rms_norm(s[r], gain, eps) for r in idx]), 3e-6)
    # only the additions
    be.ext.add_rms_shift(x32, be.t(y), None, rows, gain, eps, dtype=dtype)
    assert close(be.n(x32), s + y, 1e-6)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_token_shift_over_spans_and_steps(be, dtype):
    """two sequences in two of three slots fed in unequal portions (one token, two, many): every output is the blend with the
    sequence's previous normed row, whichever step brought it; a slot that is used again starts from zeros"""
    rng = np.random.default_rng(3)
    width, eps, gain = 70, 1e-5, 0.75
    shift = ON.bf16_round(rng.uniform(0, 1, size=width))
    prev = torch.full((3, width), 7.0, dtype=F32, device=be.device)          # stale rows of an earlier user
    last = {1: None, 2: None}
    n_tok = {1: 0, 2: 0}
    for step in ([(1, 2), (2, 1)], [(2, 40), (1, 1)], [(1, 1)], [(1, 5), (2, 3)], [(2, 1)], [(1, 1), (2, 1)], [(2, 1), (1, 9)]):
        lens = [n for _s, n in step]
        rows = sum(lens)
        x = rng.standard_normal((rows, width)).astype(np.float32) * 2
        seq = np.concatenate([[s] * n for s, n in step])
        pos = np.concatenate([np.arange(n_tok[s], n_tok[s] + n) for s, n in step])
        out = torch.zeros((rows, width), dtype=dtype, device=be.device)
        hn = torch.zeros((rows, width), dtype=F32, device=be.device)
        be.ext.add_rms_shift(be.t(x), None, out, rows, gain, eps, shift=dev(be, shift, dtype), prev=prev, hn=hn, row_seq=ints(be, seq),
                             row_pos=ints(be, pos), spans=spans_of(be, lens), dtype=dtype)
        got, r = be.n(out.float()), 0
        for s, n in step:
            for _ in range(n):
                a = ON.scalar_rms_norm(x[r].astype(np.float64), gain, eps)
                b = last[s] if last[s] is not None else np.zeros(width)
                assert close(got[r], ON.token_shift(a, b, shift.astype(np.float64)), 3e-6 if dtype is F32 else 1e-2), (step, r)
                last[s] = a
                n_tok[s] += 1
                r += 1
    assert close(be.n(prev)[1], last[1], 3e-6) and close(be.n(prev)[2], last[2], 3e-6) and close(be.n(prev)[0], np.full(width, 7.0), 0)


@pytest.mark.parametrize("dtype,M,N,K", [(F32, 1, 9, 40), (F32, 33, 66, 50), (BF16, 3, 7, 24), (BF16, 17, 40, 64), (BF16, 130, 150, 72)])
@pytest.mark.parametrize("epi", [6, 7, 8])
def test_dense_linear_scale_tanh_and_row_scaled_activation(be, dtype, M, N, K, epi):
    rng = np.random.default_rng(M * 1000 + N * 10 + K + epi)
    x, w = ON.bf16_round(rng.standard_normal((M, K))), ON.bf16_round(rng.standard_normal((N, K)) / math.sqrt(K) * 2)
    rs = rng.uniform(0.1, 1.0, size=M).astype(np.float32)
    acc = x.astype(np.float64) @ w.astype(np.float64).T
    want = {6: acc * 0.3, 7: np.tanh(acc), 8: np.maximum(acc * rs[:, None].astype(np.float64), 0) ** 2}[epi]
    y = torch.full((M, N), float("nan"), dtype=F32, device=be.device)
    be.ext.dense_linear(dev(be, x, dtype), dev(be, w, dtype), y, M, N, K, K, K, N, epi=epi, limit=0.3, aux=be.t(rs), ldaux=1)
    assert close(be.n(y), want, 2e-5)


@pytest.mark.parametrize("shared", [False, True])
@pytest.mark.parametrize("experts,top", [(5, 1), (5, 2), (12, 1), (70, 4), (3, 3)])
def test_sigmoid_router_and_expert_lists(be, experts, top, shared):
    """shared: one more column per row names the expert behind the routed ones, weight 1, and the lists have one more expert"""
    rng = np.random.default_rng(experts * 10 + top)
    rows, per = 37, top + int(shared)
    logits = rng.standard_normal((rows, experts)).astype(np.float32) * 2
    logits[3, :] = 0.25                                          # a tie over all experts: the lowest indices win
    ids = torch.zeros((rows, per), dtype=I32, device=be.device)
    wts = torch.zeros((rows, per), dtype=F32, device=be.device)
    groups = tuple(torch.zeros((n,), dtype=I32, device=be.device) for n in (experts + 1, experts + 1, rows * per))
    be.ext.moe_route_sigmoid(be.t(logits), ids, wts, rows, experts, top, groups=groups, shared_slot=shared)
    gi, gw = be.n(ids), be.n(wts)
    for r in range(rows):
        s = ON.sigmoid(logits[r].astype(np.float64))
        order = sorted(range(experts), key=lambda e: (-s[e], e))[:top]
        assert list(gi[r][:top]) == order, r
        assert close(gw[r][:top], s[order], 1e-6)
        if shared:
            assert gi[r][top] == experts and gw[r][top] == 1.0
    cnt, off, lst = (be.n(t) for t in groups)
    flat = gi.reshape(-1)
    for e in range(experts + int(shared)):
        mine = [p for p in range(rows * per) if flat[p] == e]
        assert cnt[e] == len(mine) and list(lst[off[e]:off[e] + cnt[e]]) == mine


# ---- attention: chunked mask, capped scores, a constant sink, one gate per head, shared rows ------------------------------------------


def attention_case(be, dtype, H, G, dim, vd, chunk, page, lens_by_step, softcap, rot_dims, tiles, seed=0, boost=None):
    """runs kv_rot_append + the attention kernels over steps of spans on two sequences and compares every row with the oracle;
    `tiles`: portions of prompts and single rows through the matrix-core kernels"""
    from exllamav2_amd.window_attn import rotary_tables
    rng = np.random.default_rng(seed)
    width = 24
    m = ON.attn_mixer(heads=H, kv_heads=G, dim=dim, vdim=vd, size=chunk, dims=rot_dims, softcap=softcap,
                      scaling={"factor": 3.0, "original": 40, "low": 2.0, "high": 8.0})["mixer"]
    W = {"l0.mix." + n: ON.bf16_round(rng.standard_normal(s) / math.sqrt(width) * g)
         for n, s, g in (("q", (H * dim, width), 3.0), ("k", (G * dim, width), 3.0), ("v", (G * vd, width), 1.0), ("g", (H, width), 2.0))}
    W["l0.mix.o"] = np.eye(H * vd)
    W64 = {k: v.astype(np.float64) for k, v in W.items()}
    per_seq = max(-(-sum(n for step in lens_by_step for s, n in step if s == q) // page) for q in (0, 1))
    n_pages = 2 * per_seq + 3
    kc = torch.zeros((n_pages, page, G, dim), dtype=dtype, device=be.device)
    vc = torch.zeros((n_pages, page, G, vd), dtype=dtype, device=be.device)
    order = rng.permutation(n_pages)                          # the two sequences' pages lie scattered over the pool
    bt = ints(be, np.array([order[:per_seq], order[per_seq:2 * per_seq]]))
    freq, amp = torch.zeros((1,), dtype=F32, device=be.device), 1.0
    if rot_dims:
        freq, amp = rotary_tables(m["rot"]["base"], rot_dims, m["rot"]["scaling"], be.device)
        assert close(be.n(freq), ON.rotary_frequencies(m["rot"]), 1e-6)
    hist = {0: [], 1: []}
    kvs = {0: [], 1: []}
    off_k, off_v, off_g = H * dim, (H + G) * dim, (H + G) * dim + G * vd
    off_gp = off_g + (-off_g) % 4
    ncat = off_gp + H
    wcat = np.zeros((ncat, width), dtype=np.float32)
    wcat[:off_k], wcat[off_k:off_v], wcat[off_v:off_g], wcat[off_gp:] = W["l0.mix.q"], W["l0.mix.k"], W["l0.mix.v"], W["l0.mix.g"]
    worst = 0.0
    for step in lens_by_step:
        rows = sum(n for _s, n in step)
        hs = ON.bf16_round(rng.standard_normal((rows, width)))
        if boost is not None:
            boost(hs, step, hist)
        seq = np.concatenate([[s] * n for s, n in step])
        pos = np.concatenate([np.arange(len(hist[s]), len(hist[s]) + n) for s, n in step])
        f = be.t((hs.astype(np.float64) @ wcat.astype(np.float64).T).astype(np.float32))
        q = torch.zeros((rows, H * dim), dtype=dtype, device=be.device)
        qs = be.t(np.full(H, m["scale"], dtype=np.float32))
        rs, rp = ints(be, seq), ints(be, pos)
        be.ext.kv_rot_append(f, ncat, 0, off_k, off_v, q, qs, kc, vc, None, None, freq, amp, rot_dims, freq, False, False, rs, rp, bt,
                             page, 0, rows, H, G, dim, vd)
        o = torch.zeros((rows, H * vd), dtype=dtype, device=be.device)
        sink = torch.zeros((H,), dtype=F32, device=be.device)
        common = (q, kc, vc, None, None, sink, f, ncat, off_gp, freq, False, False, rs, rp, bt, page, 0, o)
        var = dict(chunk=chunk, softcap=softcap, gate_head=True)
        if tiles:
            r0 = 0
            t64, t1 = [], []
            for _s, n in step:
                if n == 1:
                    t1.append(r0)
                else:
                    t64 += [(r0 + i, min(64, n - i)) for i in range(0, n, 64)]
                r0 += n
            if t64:
                be.ext.window_attn_tiles(*common, (ints(be, [a for a, _ in t64]), ints(be, [b for _, b in t64]), len(t64)), 64, H, G, dim, vd,
                                         1 << 30, **var)
            if t1:
                nsplit = 3
                po = torch.zeros((rows, H, nsplit, vd), dtype=F32, device=be.device)
                pml = torch.zeros((rows, H, nsplit, 2), dtype=F32, device=be.device)
                be.ext.window_attn_tiles(*common, (ints(be, t1), None, len(t1)), 1, H, G, dim, vd, 1 << 30, nsplit=nsplit, part_o=po, part_ml=pml,
                                         **var)
        else:
            be.ext.window_attn(*common, rows, H, G, dim, vd, 1 << 30, **var)
        got, r = be.n(o.float()), 0
        for s, n in step:
            for _ in range(n):
                p = len(hist[s])
                h = hs[r].astype(np.float64)
                hist[s].append(h)
                kvs[s].append(ON.attention_kv(W64, "l0", m, h, p))
                want = ON.attention_token(W64, "l0", m, h, p, kvs[s])
                worst = max(worst, np.abs(got[r] - want).max() / (1 + np.abs(want).max()))
                r += 1
    return worst


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("H,G,dim,vd,chunk,page,rot", [(4, 2, 16, 8, 6, 4, 8), (3, 3, 12, 20, 1, 3, 12), (2, 1, 10, 6, 50, 32, 0), (6, 2, 48, 48, 17, 8, 48),
                                                     (1, 1, 8, 8, 5, 5, 2)])
def test_chunked_attention_general_kernel(be, dtype, H, G, dim, vd, chunk, page, rot):
    steps = [[(0, 7), (1, 1)], [(0, 1), (1, 12)], [(1, 1)], [(0, 2), (1, 2)], [(0, 30)], [(0, 1), (1, 1)], [(1, 3), (0, 1)]]
    err = attention_case(be, dtype, H, G, dim, vd, chunk, page, steps, softcap=7.0, rot_dims=rot, tiles=False, seed=chunk)
    assert err <= (2e-5 if dtype is F32 else 2e-2)


@pytest.mark.parametrize("H,G,dim,vd,chunk,page", [(4, 2, 32, 32, 20, 16), (2, 2, 64, 64, 96, 64), (34, 2, 32, 32, 7, 8), (2, 1, 128, 64, 33, 256)])
def test_chunked_attention_matrix_core_kernels(be, H, G, dim, vd, chunk, page):
    steps = [[(0, 70), (1, 1)], [(0, 1), (1, 100)], [(1, 1)], [(0, 2), (1, 2)], [(0, 130)], [(0, 1), (1, 1)], [(1, 3), (0, 1)], [(0, 1)], [(0, 1)]]
    err = attention_case(be, BF16, H, G, dim, vd, chunk, page, steps, softcap=5.0, rot_dims=dim // 2, tiles=True, seed=chunk)
    assert err <= 2e-2


def test_soft_cap_saturates_large_scores(be):
    """scores scaled far beyond the cap: without the cap one key would take the whole softmax; with it the weights stay spread"""
    def boost(hs, step, hist):
        hs *= 40.0
    err = attention_case(be, F32, 2, 1, 8, 8, 9, 4, [[(0, 11), (1, 3)], [(0, 1), (1, 1)]], softcap=1.5, rot_dims=4, tiles=False, seed=5, boost=boost)
    assert err <= 2e-5


def test_queries_only_rows_leave_the_cache_alone(be):
    """kv_rot_append without cache tensors (a layer that reads another layer's rows): queries come out as with them"""
    from exllamav2_amd.window_attn import rotary_tables
    rng = np.random.default_rng(0)
    H, G, dim, vd, rows, page = 3, 1, 8, 4, 6, 4
    ncat = (H + G) * dim + G * vd
    f = be.t(rng.standard_normal((rows, ncat)).astype(np.float32))
    freq, amp = rotary_tables(100.0, 8, None, be.device)
    qs = be.t(np.full(H, 0.5, dtype=np.float32))
    rs, rp, bt = ints(be, [0] * rows), ints(be, list(range(5, 5 + rows))), ints(be, [[2, 0, 1]])
    kc = torch.zeros((3, page, G, dim), dtype=F32, device=be.device)
    vc = torch.zeros((3, page, G, vd), dtype=F32, device=be.device)
    qa, qb = (torch.zeros((rows, H * dim), dtype=F32, device=be.device) for _ in range(2))
    be.ext.kv_rot_append(f, ncat, 0, H * dim, (H + G) * dim, qa, qs, kc, vc, None, None, freq, amp, 8, freq, False, False, rs, rp, bt, page, 0, rows, H, G, dim, vd)
    be.ext.kv_rot_append(f, ncat, 0, 0, 0, qb, qs, None, None, None, None, freq, amp, 8, freq, False, False, rs, rp, bt, page, 0, rows, H, G, dim, vd)
    assert np.array_equal(be.n(qa), be.n(qb)) and np.abs(be.n(kc)).sum() > 0


# ---- decaying linear attention ---------------------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_blends_with_the_previous_input(be, dtype):
    rng = np.random.default_rng(1)
    width = 300
    mu = ON.bf16_round(rng.uniform(0, 1, size=(5, width)))
    prev = torch.full((3, width), -3.0, dtype=F32, device=be.device)
    last, n_tok = {0: None, 2: None}, {0: 0, 2: 0}
    for step in ([(0, 3), (2, 1)], [(2, 1), (0, 1)], [(0, 1)], [(2, 33), (0, 2)], [(0, 1), (2, 1)]):
        lens = [n for _s, n in step]
        rows = sum(lens)
        h = rng.standard_normal((rows, width)).astype(np.float32)
        seq = np.concatenate([[s] * n for s, n in step])
        pos = np.concatenate([np.arange(n_tok[s], n_tok[s] + n) for s, n in step])
        out = torch.zeros((5, rows, width), dtype=dtype, device=be.device)
        be.ext.wkv_mix(be.t(h), prev, dev(be, mu, dtype), out, ints(be, seq), ints(be, pos), spans_of(be, lens), rows, width)
        got, r = be.n(out.float()), 0
        for s, n in step:
            for _ in range(n):
                b = last[s] if last[s] is not None else np.zeros(width)
                want = h[r].astype(np.float64) + (b - h[r]) * mu.astype(np.float64)
                assert close(got[:, r], want, 1e-6 if dtype is F32 else 1e-2), (step, r)
                last[s] = h[r].astype(np.float64)
                n_tok[s] += 1
                r += 1
    assert close(be.n(prev)[0], last[0], 0) and close(be.n(prev)[2], last[2], 0)


@pytest.mark.parametrize("chunked", [False, True, "alternating"])
@pytest.mark.parametrize("heads,D", [(3, 8), (2, 64), (1, 5), (4, 32), (2, 100), (1, 128), (1, 192)])
def test_decaying_state_over_spans_and_steps(be, heads, D, chunked):
    """portions of 1 .. 150 tokens of two sequences: the state carried in the slot gives what one pass over the whole sequence gives;
    a slot's stale state is not seen by a sequence that starts at position 0.  Token by token, unrolled in chunks (several chunks, chunks
    that end early, decays fast enough that a factored exponential would overflow), and both forms alternating on the same slots"""
    if chunked and not be.ext.wkv_scan_chunked_supported(D, D):
        pytest.skip("the chunked form does not take this state size")
    rng = np.random.default_rng(heads * 100 + D)
    inner, eps = heads * D, 1e-5
    u = ON.bf16_round(rng.standard_normal((heads, D)) * 0.5)
    nw = ON.bf16_round(1 + rng.standard_normal(inner) * 0.1)
    state = torch.full((3, heads, D, D), 5.0, dtype=F32, device=be.device)
    S = {1: np.zeros((heads, D, D)), 2: np.zeros((heads, D, D))}
    n_tok = {1: 0, 2: 0}
    for n_step, step in enumerate(([(1, 2), (2, 1)], [(2, 37), (1, 1)], [(1, 1)], [(1, 150), (2, 3)], [(2, 1), (1, 1)], [(2, 64), (1, 65)])):
        lens = [n for _s, n in step]
        rows = sum(lens)
        f = rng.standard_normal((4, rows, inner)).astype(np.float32)
        f[1] *= 0.5
        dlog = (rng.standard_normal((rows, inner)) - 1.0).astype(np.float32)
        dlog[:, ::3] += 2.5                                      # channels that forget within a few tokens
        seq = np.concatenate([[s] * n for s, n in step])
        pos = np.concatenate([np.arange(n_tok[s], n_tok[s] + n) for s, n in step])
        out = torch.zeros((rows, inner), dtype=F32, device=be.device)
        if chunked is True or (chunked and n_step % 2 == 1):
            chunk0 = np.cumsum([0] + [-(-n // 64) for n in lens])
            zbuf = torch.zeros((int(chunk0[-1]), heads, D, D), dtype=F32, device=be.device)
            dbuf = torch.zeros((int(chunk0[-1]), heads, D), dtype=F32, device=be.device)
            be.ext.wkv_scan_chunked(be.t(f), rows, be.t(dlog), be.t(u), be.t(nw), out, state, spans_of(be, lens), (ints(be, chunk0[:-1]), 64, int(chunk0[-1])),
                                    ints(be, seq), ints(be, pos), zbuf, dbuf, heads, D, D, eps)
        else:
            be.ext.wkv_scan(be.t(f), rows, be.t(dlog), be.t(u), be.t(nw), out, state, spans_of(be, lens), ints(be, seq), ints(be, pos), heads, D, D, eps)
        got, r = be.n(out), 0
        for s, n in step:
            for _ in range(n):
                rr, kk, vv, gg = (f[i, r].astype(np.float64).reshape(heads, D) for i in range(4))
                w = np.exp(-np.exp(dlog[r].astype(np.float64))).reshape(heads, D)
                o = np.zeros((heads, D))
                for i in range(heads):
                    kv = np.outer(kk[i], vv[i])
                    o[i] = (S[s][i] + u[i].astype(np.float64)[:, None] * kv).T @ rr[i]
                    S[s][i] = w[i][:, None] * S[s][i] + kv
                    o[i] = o[i] / math.sqrt((o[i] ** 2).mean() + eps)
                want = o.reshape(-1) * nw * ON.silu(gg.reshape(-1))
                assert close(got[r], want, 2e-5), (step, r)
                n_tok[s] += 1
                r += 1
    assert close(be.n(state)[1], S[1], 2e-5) and close(be.n(state)[2], S[2], 2e-5) and close(be.n(state)[0], np.full((heads, D, D), 5.0), 0)


# ---- whole models through the engine -----------------------------------------------------------------------------------------------

CONFIGS = {
    # both mixers, both feed-forwards, a layer that reads another layer's keys and values, partial rotation
    "mixed": lambda: ON.small_config([
        ON.layer(ON.attn_mixer(heads=4, kv_heads=2, dim=16, vdim=8, size=6, dims=8), ON.dense_ff(40)),
        ON.layer(ON.wkv_mixer(heads=3, dim=8, rank=5), ON.moe_ff_spec(experts=5, top=2, ff=12, shared=10)),
        ON.layer(ON.attn_mixer(heads=4, kv_heads=2, dim=16, vdim=8, size=6, dims=8, kv_from=0), ON.dense_ff(24)),
        ON.layer(ON.wkv_mixer(heads=2, dim=12, rank=3), ON.moe_ff_spec(experts=4, top=1, ff=9, shared=7))]),
    # linear attention first, chunks of one token, one head, no shared expert, a layer without feed-forward, sharing across two layers,
    # every expert chosen, no frequency rescaling, no soft cap, unscaled logits
    "odd": lambda: ON.small_config([
        ON.layer(ON.wkv_mixer(heads=1, dim=20, rank=1), ON.moe_ff_spec(experts=3, top=3, ff=8, shared=None)),
        ON.layer(ON.attn_mixer(heads=3, kv_heads=1, dim=6, vdim=10, size=1, dims=2, scaling=None, softcap=0.0), None),
        ON.layer(ON.attn_mixer(heads=2, kv_heads=2, dim=12, vdim=6, size=50, dims=12, base=500.0), ON.dense_ff(16)),
        ON.layer(ON.attn_mixer(heads=3, kv_heads=1, dim=6, vdim=10, size=4, dims=2, scaling=None, kv_from=1), ON.moe_ff_spec(experts=7, top=2, ff=5, shared=3)),
        ON.layer(ON.attn_mixer(heads=3, kv_heads=1, dim=6, vdim=10, size=1, dims=2, scaling=None, softcap=3.0, kv_from=1), None)],
        width=28, vocab=50, logit_scale=1.0),
    # head sizes the matrix-core attention takes in bfloat16
    "wide": lambda: ON.small_config([
        ON.layer(ON.attn_mixer(heads=4, kv_heads=2, dim=32, vdim=32, size=9, dims=16), ON.dense_ff(48)),
        ON.layer(ON.wkv_mixer(heads=2, dim=16, rank=6), ON.moe_ff_spec(experts=6, top=2, ff=16, shared=16)),
        ON.layer(ON.attn_mixer(heads=2, kv_heads=1, dim=64, vdim=64, size=70, dims=64, scaling=None), ON.dense_ff(32)),
        ON.layer(ON.attn_mixer(heads=8, kv_heads=2, dim=32, vdim=32, size=5, dims=16, kv_from=0), None)], width=48, vocab=70),
}


def make_engine(be, cfg, W, dtype, max_tokens, page=4, max_seqs=4, graphs=None):
    from exllamav2_amd.config import LayeredConfig
    from exllamav2_amd.engine import Engine
    from exllamav2_amd.layered import LayeredModel
    tensors = {k: be.t(v).to(BF16) for k, v in W.items()}
    model = LayeredModel(LayeredConfig.from_dict_prerms_shift(ON.clean_config(cfg)), device=be.device, dtype=dtype, ext=be.ext).load(tensors)
    return Engine(model, max_tokens=max_tokens, max_seqs=max_seqs, page_size=page, graphs=graphs)


def run_cuts(be, eng, rid, tokens, cuts):
    out, at = [], 0
    for c in cuts:
        out.append(be.n(eng.step([(rid, tokens[at:at + c], list(range(c)))])))
        at += c
    assert at == len(tokens)
    return np.concatenate(out, 0)


def clear_tokens(cfg, W, n, seed, gap=0.008):
    """n random tokens none of whose router decisions is a close call (so that bfloat16 rounding cannot pick another expert: a
    test of rounding must not rest on one); redrawn with the next seed until that holds"""
    for k in range(200):
        toks = [int(t) for t in np.random.default_rng(seed + 1000 * k).integers(0, cfg["vocab"], size=n)]
        gaps = []
        ON.Oracle(cfg, W).feed("g", toks, gaps=gaps)
        if min(gaps) > gap:
            return toks
    raise AssertionError("no token sequence with clear routing found")


@pytest.mark.parametrize("name", sorted(CONFIGS))
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_whole_prompt(be, name, dtype):
    cfg = CONFIGS[name]()
    W = ON.random_model(cfg, seed=1)
    toks = clear_tokens(cfg, W, 23, 2)
    want = ON.Oracle(cfg, W).feed("a", toks)
    eng = make_engine(be, cfg, W, dtype, 32)
    assert rel_err(run_cuts(be, eng, "a", toks, [23]), want) <= TOL[dtype]


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_decoding_and_portions(be, name):
    """the same positions through a whole prompt, token by token from the first token on (chunks, the shift and the recurrent state
    pass over decoded tokens), and in portions down to two tokens that end inside pages and chunks"""
    cfg = CONFIGS[name]()
    W = ON.random_model(cfg, seed=3)
    toks = list(np.random.default_rng(4).integers(0, cfg["vocab"], size=26))
    want = ON.Oracle(cfg, W).feed("a", toks)
    for cuts in ([1] * 26, [2, 3, 2, 5, 2, 1, 1, 4, 2, 2, 2], [9] + [1] * 17, [25, 1], [1, 25]):
        eng = make_engine(be, cfg, W, F32, 28, page=4)
        assert rel_err(run_cuts(be, eng, "a", toks, cuts), want) <= TOL[F32], cuts


def test_mixed_batches_reuse_pages_and_slots(be):
    """five unequal requests over four slots and a pool smaller than their sum: portions beside single tokens, a request left out of
    a step, finished requests' pages and slot (with its shift rows and recurrent state) taken by the next; every position equals the
    request alone"""
    cfg = CONFIGS["mixed"]()
    W = ON.random_model(cfg, seed=5)
    rng = np.random.default_rng(6)
    reqs = {r: list(rng.integers(0, cfg["vocab"], size=n)) for r, n in (("a", 13), ("b", 5), ("c", 9), ("d", 2), ("e", 11))}
    oracle = ON.Oracle(cfg, W)
    want = {r: oracle.feed(r, t) for r, t in reqs.items()}
    eng = make_engine(be, cfg, W, F32, max_tokens=32, page=4, max_seqs=4)
    plan = [[("a", 5), ("b", 2)], [("a", 1), ("b", 3), ("c", 4), ("d", 2)], [("a", 2), ("c", 1)], [("c", 2), ("e", 3), ("a", 1)],
            [("a", 4), ("e", 2), ("c", 2)], [("e", 1)], [("e", 5)]]
    at, got = {r: 0 for r in reqs}, {r: [] for r in reqs}
    for step in plan:
        entries, end = [], []
        for r, n in step:
            entries.append((r, reqs[r][at[r]:at[r] + n], list(range(n))))
            at[r] += n
            if at[r] == len(reqs[r]):
                end.append(r)
        lg = be.n(eng.step(entries, end))
        k = 0
        for r, n in step:
            got[r].append(lg[k:k + n])
            k += n
    assert all(at[r] == len(reqs[r]) for r in reqs)
    assert len(eng.pool.free_pages) == eng.pool.num_pages and len(eng.pool.free_slots) == 4
    assert sum(-(-len(t) // 4) for t in reqs.values()) > eng.pool.num_pages            # pages were used again
    for r in reqs:
        assert rel_err(np.concatenate(got[r], 0), want[r]) <= TOL[F32], r


def test_a_reused_slot_starts_from_zeros(be):
    """one slot, three requests one after the other: the second and third find the first one's shift rows, recurrent state and cached
    keys in their slot and pages and must not see them"""
    cfg = CONFIGS["mixed"]()
    W = ON.random_model(cfg, seed=15)
    rng = np.random.default_rng(16)
    eng = make_engine(be, cfg, W, F32, max_tokens=16, page=4, max_seqs=1)
    for r, n, cuts in (("a", 14, [14]), ("b", 9, [1, 1, 7]), ("c", 12, [2, 10])):
        toks = list(rng.integers(0, cfg["vocab"], size=n))
        want = ON.Oracle(cfg, W).feed(r, toks)
        assert rel_err(run_cuts(be, eng, r, toks, cuts), want) <= TOL[F32], r
        eng.finish(r)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_decode_steps_as_graphs(be, dtype):
    """decoding steps through the engine's persistent-input path (on a GPU: captured once per batch size and replayed; every replay
    is checked): two requests decode side by side, one ends, the other goes on alone, a third joins"""
    cfg = CONFIGS["mixed"]()
    W = ON.random_model(cfg, seed=21)
    reqs = {r: clear_tokens(cfg, W, n, 22 + i) for i, (r, n) in enumerate((("a", 14), ("b", 9), ("c", 8)))}
    oracle = ON.Oracle(cfg, W)
    want = {r: oracle.feed(r, t) for r, t in reqs.items()}
    eng = make_engine(be, cfg, W, dtype, max_tokens=48, page=4, graphs=True)
    got = {r: {} for r in reqs}

    def step(parts, end=()):
        lg = be.n(eng.step([(r, reqs[r][lo:hi], list(range(hi - lo))) for r, lo, hi in parts], end))
        k = 0
        for r, lo, hi in parts:
            for p in range(lo, hi):
                got[r][p] = lg[k]; k += 1

    step([("a", 0, 3), ("b", 0, 2)])
    for i in range(6):
        step([("a", 3 + i, 4 + i), ("b", 2 + i, 3 + i)])
    step([("b", 8, 9)], end=["b"])
    for i in range(3):
        step([("a", 9 + i, 10 + i)])
    step([("c", 0, 4)])
    for i in range(2):
        step([("c", 4 + i, 5 + i), ("a", 12 + i, 13 + i)])
    step([("c", 6, 8)], end=["c", "a"])
    for r in reqs:
        assert sorted(got[r]) == list(range(len(reqs[r])))
        assert rel_err(np.stack([got[r][p] for p in range(len(reqs[r]))]), want[r]) <= TOL[dtype], r
    eng.close()


def test_matrix_core_sizes_in_portions_and_decoding_bf16(be):
    """head sizes of the tile kernels: a prompt of several 64-row tiles that crosses chunk and page borders, then decoding, beside a
    second request"""
    cfg = CONFIGS["wide"]()
    W = ON.random_model(cfg, seed=41)
    reqs = {r: clear_tokens(cfg, W, n, 42 + i, gap=0.004) for i, (r, n) in enumerate((("a", 12), ("b", 160)))}
    oracle = ON.Oracle(cfg, W)
    want = {r: oracle.feed(r, t) for r, t in reqs.items()}
    eng = make_engine(be, cfg, W, BF16, max_tokens=256, page=16, graphs=True)
    got = {r: {} for r in reqs}

    def step(parts, end=()):
        lg = be.n(eng.step([(r, reqs[r][lo:hi], list(range(hi - lo))) for r, lo, hi in parts], end))
        k = 0
        for r, lo, hi in parts:
            for p in range(lo, hi):
                got[r][p] = lg[k]; k += 1

    for i in range(5):
        step([("a", i, i + 1)])                                  # one token per step from the first token on
    step([("b", 0, 139), ("a", 5, 6)])                           # 140 rows: every scratch buffer grows
    for i in range(6, 12):
        step([("a", i, i + 1), ("b", 133 + i, 134 + i)])
    step([("b", 145, 160)])
    for r in reqs:
        assert rel_err(np.stack([got[r][p] for p in range(len(reqs[r]))]), want[r]) <= TOL[BF16], r
    eng.close()


def crafted_model(chunk, seed=31):
    """one attention layer behind a linear-attention layer, made so that token 0's query matches token 1's key and nothing else:
    queries read inputs 0-3, keys inputs 4-7 through the same matrix, values the other inputs; token 0 is marked in inputs 0-3,
    token 1 in 4-7, all other tokens are zero there; no shift, no rotation.  Wherever the mask lets token 0 see a token 1 that key
    takes the softmax -- and a token 1 in the chunk before, one position further back, must not be seen at all."""
    cfg = ON.small_config([ON.layer(ON.wkv_mixer(heads=2, dim=4, rank=2), None),
                           ON.layer(ON.attn_mixer(heads=2, kv_heads=2, dim=8, vdim=8, size=chunk, dims=0, scaling=None, scale=1.0, softcap=30.0),
                                    ON.dense_ff(24))], width=16, vocab=40)
    W = ON.random_model(cfg, seed=seed)
    rng = np.random.default_rng(seed + 1)
    E = W["embed"]
    E[:, :8] = 0.0
    mark = rng.standard_normal(4)
    mark *= 4.0 / np.linalg.norm(mark)
    E[0, :4], E[1, 4:8] = mark, mark
    W["embed"] = ON.bf16_round(E)
    M = rng.standard_normal((16, 4))
    W["l1.mix.q"], W["l1.mix.k"] = np.zeros((16, 16), dtype=np.float32), np.zeros((16, 16), dtype=np.float32)
    W["l1.mix.q"][:, :4], W["l1.mix.k"][:, 4:8] = ON.bf16_round(M), ON.bf16_round(M)
    W["l1.mix.v"][:, :8] = 0.0
    W["l1.mix.v"] = ON.bf16_round(W["l1.mix.v"] * 4)
    W["l1.shift"][:] = 0.0
    W["l0.mix.o"] = ON.bf16_round(W["l0.mix.o"] * 0.05)          # the attention's input is nearly the token's own embedding
    W["l0.mix.o"][:8] = 0.0
    return cfg, W


@pytest.mark.parametrize("chunk,page", [(24, 8), (150, 64), (7, 4)])
def test_a_marked_token_at_every_edge_through_the_engine(be, chunk, page):
    """whole prompt, portions that end right at the edges, and decoding: the marked key sits at the first position of the query's
    chunk, at the last position of the chunk before (not seen), right in front of the query, far back inside a long chunk, and across a
    page border"""
    cfg, W = crafted_model(chunk)
    rng = np.random.default_rng(chunk)
    T = chunk * 3 - 2                                           # the query is the next-to-last position of the third chunk
    query = T - 1
    lo = query // chunk * chunk
    seen_changes, unseen_changes = 0, 0
    for target in sorted({lo, lo - 1, query - 1, lo + 1, 0, chunk - 1, (lo // page + 1) * page - 1, (lo // page + 1) * page} - {query}):
        toks = [int(t) for t in rng.integers(2, cfg["vocab"], size=T)]
        toks[target], toks[query] = 1, 0                      # the marked pair, nowhere else
        base = list(toks)
        base[target] = 2
        want = ON.Oracle(cfg, W).feed("t", toks)
        other = ON.Oracle(cfg, W).feed("t", base)[-1]
        visible = target in ON.chunk_visible(query, chunk)
        assert visible == (lo <= target <= query)
        moved = rel_err(want[-1:], other[None])
        if visible:
            seen_changes += moved > 0.02                        # where it can be seen it matters
        else:
            unseen_changes += moved > 0.02
        plans = [[T], [lo, query - lo, 1], [lo + 1, query - lo - 1, 1], [T - 3, 2, 1], [lo - 2] + [1] * (T - lo + 2),
                 [target + 1] + [2] * ((T - target - 1) // 2) + [1] * ((T - target - 1) % 2)]
        for cuts in (plans if chunk < 100 else plans[1:4]):
            eng = make_engine(be, cfg, W, F32, max_tokens=T + page, page=page)
            got = run_cuts(be, eng, "t", toks, [c for c in cuts if c > 0])
            assert rel_err(got[-4:], want[-4:]) <= TOL[F32], (target, cuts[:3])
    assert seen_changes >= 3


def test_the_state_carries_a_far_token(be):
    """a token 300 positions back reaches the last position only through the recurrent state (chunks of 16 tokens hide it from the
    attention): changing it changes the logits, and portions and decoding carry it like the whole prompt does"""
    cfg = ON.small_config([ON.layer(ON.wkv_mixer(heads=2, dim=8, rank=3), ON.dense_ff(24)),
                           ON.layer(ON.attn_mixer(heads=2, kv_heads=1, dim=8, vdim=8, size=16, dims=4), None)], width=16, vocab=40)
    W = ON.random_model(cfg, seed=51)
    W["l0.mix.w0"] = ON.bf16_round(W["l0.mix.w0"] * 0 - 6.0)      # slow decay: w = exp(-exp(-6)) per token
    W["l0.mix.w2"] = ON.bf16_round(W["l0.mix.w2"] * 0.1)
    rng = np.random.default_rng(52)
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], size=310)]
    other = list(toks)
    other[9] = (toks[9] + 1) % cfg["vocab"]
    want = ON.Oracle(cfg, W).feed("a", toks)
    assert rel_err(ON.Oracle(cfg, W).feed("a", other)[-1:], want[-1:]) > 1e-3
    for cuts in ([310], [100, 2, 65, 143], [290] + [1] * 20):
        eng = make_engine(be, cfg, W, F32, max_tokens=320, page=16)
        assert rel_err(run_cuts(be, eng, "a", toks, cuts)[-8:], want[-8:]) <= TOL[F32], cuts


def test_long_decoding_bf16(be):
    cfg = CONFIGS["mixed"]()
    W = ON.random_model(cfg, seed=7)
    toks = clear_tokens(cfg, W, 60, 8, gap=0.006)
    want = ON.Oracle(cfg, W).feed("a", toks)
    eng = make_engine(be, cfg, W, BF16, 64, page=8)
    assert rel_err(run_cuts(be, eng, "a", toks, [3] + [1] * 57), want) <= TOL[BF16]


def test_greedy_generation_through_the_generator(be):
    from exllamav2_amd.engine import Generator
    cfg = CONFIGS["mixed"]()
    W = ON.random_model(cfg, seed=9)
    rng = np.random.default_rng(10)
    prompts = [list(map(int, rng.integers(0, cfg["vocab"], size=n))) for n in (7, 3, 5, 4, 6)]
    eng = make_engine(be, cfg, W, F32, max_tokens=64, page=4, max_seqs=3)
    out = Generator(eng, chunk=3).generate(prompts, 6)
    oracle = ON.Oracle(cfg, W)
    checked = 0
    for i, p in enumerate(prompts):
        lg = oracle.feed(i, p)[-1]
        for t in out[i]:
            top2 = np.sort(lg)[-2:]
            if top2[1] - top2[0] < 1e-3:
                break                                             # a near tie: later tokens may differ legitimately
            assert t == int(np.argmax(lg))
            checked += 1
            lg = oracle.feed(i, [t])[-1]
        assert len(out[i]) == 6
    assert checked >= 20
    assert len(eng.pool.free_pages) == eng.pool.num_pages


def test_model_directory_registry(be, tmp_path):
    """config.json + model.safetensors -> architectures.load_model picks the class by the architecture name"""
    from safetensors.torch import save_file
    from exllamav2_amd.architectures import load_model, read_config
    from exllamav2_amd.engine import Engine
    cfg = CONFIGS["odd"]()
    W = ON.random_model(cfg, seed=11)
    save_file({k: torch.from_numpy(np.asarray(v)).to(BF16) for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(ON.clean_config(cfg)))
    assert read_config(str(tmp_path))[0] == "Negilorn"
    model = load_model(str(tmp_path), device=be.device, dtype=F32, ext=be.ext)
    toks = [1, 5, 9, 2, 2, 7]
    got = be.n(Engine(model, 16, page_size=4).step([("x", toks, list(range(6)))]))
    assert rel_err(got, ON.Oracle(cfg, W).feed("x", toks)) <= TOL[F32]


def test_sharing_a_later_layer_is_refused(be):
    cfg = ON.small_config([ON.layer(ON.attn_mixer(kv_from=1), None), ON.layer(ON.attn_mixer(), None)])
    W = ON.random_model(ON.small_config([ON.layer(ON.attn_mixer(), None), ON.layer(ON.attn_mixer(), None)]), seed=1)
    with pytest.raises(RuntimeError, match="earlier layer"):
        make_engine(be, cfg, W, F32, 16)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_command_replays_steps(tmp_path, dtype):
    """bin/trace_run in a process of its own: steps on standard input, logits files and `done` lines out"""
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from safetensors.torch import save_file
    cfg = CONFIGS["mixed"]()
    W = ON.random_model(cfg, seed=12)
    mdir = tmp_path / "model"
    mdir.mkdir()
    save_file({k: torch.from_numpy(np.asarray(v)).to(BF16) for k, v in W.items()}, str(mdir / "model.safetensors"))
    (mdir / "config.json").write_text(json.dumps(ON.clean_config(cfg)))
    rng = np.random.default_rng(13)
    a, b = list(map(int, rng.integers(0, cfg["vocab"], size=300))), list(map(int, rng.integers(0, cfg["vocab"], size=9)))
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:290], "want": [0, 289]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[290:295], "want": []}, {"id": "b", "tokens": b[:8], "want": [7]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[8:], "want": [0]}, {"id": "a", "tokens": a[295:], "want": [4]}], "end": ["a", "b"]}]
    out = tmp_path / "out"
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(mdir), "--dtype", dtype, "--out", str(out), "--max-tokens", "512"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600, cwd=str(tmp_path))
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    oracle = ON.Oracle(cfg, W)
    wa, wb = oracle.feed("a", a), oracle.feed("b", b)
    tol = TOL[F32] if dtype == "float32" else TOL[BF16]
    assert rel_err(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1), wa[[0, 289]]) <= tol
    assert rel_err(np.fromfile(out / "1.f32", dtype="<f4").reshape(1, -1), wb[[7]]) <= tol
    assert rel_err(np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1), np.stack([wb[8], wa[299]])) <= tol
