"""The sandwich-normed stacks of attention beside a state-space scan, forget-gate linear attention and gated delta rule (Kilurax)
against the float64 restatement in oracle/kilurax.py: every new mechanism alone through the C ABI, then whole models through the
engine's step function -- whole prompts, token-by-token decoding, portions, mixed batches, reused pages and slots, a crafted key far
back and at page borders, a token only the recurrent state carries, greedy generation.  Small random configurations of their own;
`be` runs each test on the CPU twin and (gpu) on the MI355X."""
import json
import math
import os
import subprocess

import numpy as np
import pytest
import torch

from oracle import kilurax as OK
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


def pos_errs(got, want):
    d = np.asarray(got, dtype=np.float64) - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return np.sqrt((d * d).mean(-1)) / (np.sqrt((w * w).mean(-1)) + 1e-30)


def ok(got, want, dtype, frac=0.9):
    """float32: every position within 3e-5 of the logits' rms.  bfloat16: the typical position within 1.5e-2 and `frac` of them within
    4e-2; single positions may lie further out -- the head norms of the linear-attention mixers divide by the size of a read-out that
    can be next to nothing (a one-term state at a sequence's first tokens, whose sign then hangs on rounding), and in a deep model a
    rounded input can tip a close router decision, which the later positions of the sequence then remember: the design's conditioning
    and not the kernels' -- the float32 runs of the same cases pin the arithmetic."""
    e = pos_errs(got, want)
    if dtype is F32:
        return e.max() <= TOL[F32]
    return np.median(e) <= 1.5e-2 and (e <= TOL[BF16]).mean() >= frac and e.max() <= 2.0


def close(got, want, tol):
    return np.abs(np.asarray(got, dtype=np.float64) - want).max() <= tol * (1 + np.abs(want).max())


def spans_of(be, lens):
    row0 = np.cumsum([0] + list(lens[:-1]))
    return ints(be, row0), ints(be, lens), len(lens), max(lens)


# ---- row-wise steps and epilogues ------------------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("width,groups", [(6, 1), (48, 4), (300, 2), (1030, 5)])
def test_sandwich_norm_with_additions(be, dtype, width, groups):
    rng = np.random.default_rng(width)
    rows, eps, mult, top, ya, yb = 5, 1e-3, 0.375, 3, 1.25, -0.5
    x = rng.standard_normal((rows, width)).astype(np.float32) * 3 + 1
    y, y2 = rng.standard_normal((2, rows, width)).astype(np.float32)
    my = rng.standard_normal((rows * top, width)).astype(np.float32)
    w_out, w_in = OK.bf16_round(1 + 0.3 * rng.standard_normal((2, width)))
    x32, out = be.t(x), torch.zeros((rows, width), dtype=dtype, device=be.device)
    be.ext.sandwich_norm(x32, dev(be, w_out, dtype), mult, dev(be, w_in, dtype), out, rows, groups, eps, y=be.t(y), ya=ya, y2=be.t(y2), yb=yb,
                         moe_y=be.t(my), top=top)
    t = ya * y.astype(np.float64) + yb * y2 + my.reshape(rows, top, width).sum(1)
    s = np.array([x[r] + mult * OK.group_rms_norm(t[r], w_out, groups, eps) for r in range(rows)])
    want = np.array([OK.group_rms_norm(s[r], w_in, groups, eps) for r in range(rows)])
    assert close(be.n(x32), s, 2e-6)
    assert close(be.n(out.float()), want, 3e-6 if dtype is F32 else 1e-2)
    # gathered rows, no addition
    idx = np.array([4, 1, 4], dtype=np.int32)
    out2 = torch.zeros((3, width), dtype=F32, device=be.device)
    be.ext.sandwich_norm(x32, None, 0.0, dev(be, w_in, dtype), out2, 3, groups, eps, row_idx=be.t(idx))
    assert close(be.n(out2), np.array([OK.group_rms_norm(s[r], w_in, groups, eps) for r in idx]), 3e-6)
    # only the addition, one input
    be.ext.sandwich_norm(x32, dev(be, w_out, dtype), mult, None, None, rows, groups, eps, y=be.t(y))
    s2 = np.array([s[r] + mult * OK.group_rms_norm(y[r].astype(np.float64), w_out, groups, eps) for r in range(rows)])
    assert close(be.n(x32), s2, 2e-6)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_input_convolution_over_spans_and_steps(be, dtype, taps):
    """two sequences in two of three slots fed in unequal portions (one token, two, many): every output is the normed row plus the
    convolution over the sequence's last normed rows, whichever step brought them; single-token steps take the fused launch, others
    the two-launch form; a slot that was used before starts from zeros"""
    from exllamav2_amd.rmsnorm import SandwichNorm
    from exllamav2_amd.cache import PagePool, SlotState
    rng = np.random.default_rng(3 + taps)
    width, eps, groups = 70, 1e-5, 2
    w_in = OK.bf16_round(1 + 0.2 * rng.standard_normal(width))
    cw = OK.bf16_round(rng.standard_normal((width, taps)) * 0.5)
    norm = SandwichNorm(be.ext, "n", dev(be, w_in, dtype), None, dev(be, cw, dtype), groups, eps, 1.0)
    pool = PagePool(4, 4, 3, be.device)
    state = norm.make_state(pool, width)
    if state is not None:
        state["tail"].fill_(7.0)                                 # stale rows of an earlier user

    class M:
        def buf(self, tag, shape, dt):
            return torch.zeros(shape, dtype=dt, device=be.device)

    class B:
        pass
    hist = {1: [], 2: []}
    n_tok = {1: 0, 2: 0}
    for step in ([(1, 2), (2, 1)], [(2, 40), (1, 1)], [(1, 1)], [(1, 5), (2, 3)], [(2, 1)], [(1, 1), (2, 1)], [(2, 1), (1, 9)], [(2, 1), (1, 1)]):
        lens = [n for _s, n in step]
        rows = sum(lens)
        x = rng.standard_normal((rows, width)).astype(np.float32) * 2
        b = B()
        b.row_seq = ints(be, np.concatenate([[s] * n for s, n in step]))
        b.row_pos = ints(be, np.concatenate([np.arange(n_tok[s], n_tok[s] + n) for s, n in step]))
        b.spans_dev = spans_of(be, lens)
        out = torch.zeros((rows, width), dtype=dtype, device=be.device)
        norm.forward(be.t(x), None, out, rows, model=M(), batch=b, state=state, dtype=dtype)
        got, r = be.n(out.float()), 0
        for s, n in step:
            for _ in range(n):
                hist[s] = (hist[s] + [OK.group_rms_norm(x[r].astype(np.float64), w_in, groups, eps)])[-taps:]
                assert close(got[r], OK.input_conv(hist[s], cw.astype(np.float64)), 3e-6 if dtype is F32 else 1.5e-2), (step, r)
                n_tok[s] += 1
                r += 1
    if state is not None:
        assert close(be.n(state["tail"])[0], np.full((taps - 1, width), 7.0), 0)         # the unused slot is untouched
        assert close(be.n(state["tail"])[1][-1], hist[1][-1], 3e-6)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("buckets,mul_prev,mul_cur", [(37, 31, 5), (1, 3, 4), (521, 1000003, 7919)])
def test_token_pair_embedding_keeps_the_previous_token(be, dtype, buckets, mul_prev, mul_cur):
    rng = np.random.default_rng(buckets)
    vocab, width, groups, eps, scale = 50, 36, 3, 1e-5, 0.75
    table, pair = OK.bf16_round(rng.standard_normal((vocab, width))), OK.bf16_round(rng.standard_normal((buckets + 1, width)))
    w = OK.bf16_round(1 + 0.2 * rng.standard_normal(width))
    cfg = {"embedding": {"scale": scale, "bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}, "norm": {"groups": groups, "eps": eps}}
    W = {"embed": table.astype(np.float64), "bigram": pair.astype(np.float64), "embed.norm": w.astype(np.float64)}
    prev_tok = torch.full((3,), 11, dtype=I32, device=be.device)              # stale tokens of earlier users
    last, n_tok = {0: None, 2: None}, {0: 0, 2: 0}
    for step in ([(0, 3), (2, 1)], [(2, 1), (0, 1)], [(0, 1)], [(2, 6), (0, 2)], [(2, 1)]):
        lens = [n for _s, n in step]
        rows = sum(lens)
        ids = rng.integers(0, vocab, size=rows)
        seq = np.concatenate([[s] * n for s, n in step])
        pos = np.concatenate([np.arange(n_tok[s], n_tok[s] + n) for s, n in step])
        x32 = torch.zeros((rows, width), dtype=F32, device=be.device)
        be.ext.embed_pair(dev(be, table, dtype), dev(be, pair, dtype), dev(be, w, dtype), ints(be, ids), prev_tok, ints(be, seq), ints(be, pos),
                          spans_of(be, lens), x32, buckets, mul_prev % buckets, mul_cur % buckets, scale, groups, eps)
        got, r = be.n(x32), 0
        for s, n in step:
            for _ in range(n):
                assert close(got[r], OK.embed_token(W, cfg, last[s], ids[r]), 3e-6), (step, r)
                last[s] = int(ids[r])
                n_tok[s] += 1
                r += 1
    assert be.n(prev_tok).tolist() == [last[0], 11, last[2]]


@pytest.mark.parametrize("dtype,M,N,K", [(F32, 1, 9, 40), (F32, 33, 66, 50), (BF16, 3, 7, 24), (BF16, 17, 40, 64), (BF16, 130, 150, 72)])
def test_dense_linear_gated_unit_on_a_weighted_input(be, dtype, M, N, K):
    """the two launches of an expert whose input carries the router's weight s: silu(s g) s from the gate matrix, times the up
    projection = silu(W_gate (s x)) * W_up (s x)"""
    rng = np.random.default_rng(M * 1000 + N * 10 + K)
    x = OK.bf16_round(rng.standard_normal((M, K)))
    wg, wu = OK.bf16_round(rng.standard_normal((2, N, K)) / math.sqrt(K) * 2)
    rs = rng.uniform(0.1, 1.0, size=M).astype(np.float32)
    sx = rs[:, None].astype(np.float64) * x
    want = OK.silu(sx @ wg.astype(np.float64).T) * (sx @ wu.astype(np.float64).T)
    g = torch.full((M, N), float("nan"), dtype=F32, device=be.device)
    y = torch.full((M, N), float("nan"), dtype=F32, device=be.device)
    be.ext.dense_linear(dev(be, x, dtype), dev(be, wg, dtype), g, M, N, K, K, K, N, epi=be.ext.EPI_ROW_SCALED_SILU_SCALED, aux=be.t(rs), ldaux=1)
    be.ext.dense_linear(dev(be, x, dtype), dev(be, wu, dtype), y, M, N, K, K, K, N, epi=be.ext.EPI_AUX_MUL, aux=g, ldaux=N)
    assert close(be.n(y), want, 3e-5)


# ---- the recurrences ------------------------------------------------------------------------------------------------------------------


def scan_steps(rng, slots=(0, 2)):
    """unequal portions of two sequences, single tokens and spans longer than a staging round"""
    return [[(slots[0], 3), (slots[1], 1)], [(slots[1], 1), (slots[0], 1)], [(slots[0], 1)], [(slots[1], 70), (slots[0], 2)], [(slots[1], 1)],
            [(slots[0], 18), (slots[1], 1)], [(slots[0], 32), (slots[1], 33)]]


@pytest.mark.parametrize("cols", [False, True])
@pytest.mark.parametrize("heads,dim,vdim", [(2, 5, 7), (3, 16, 16), (1, 64, 32), (2, 32, 128), (1, 130, 9), (1, 250, 256)])
def test_forget_gate_scan(be, heads, dim, vdim, cols):
    """S <- diag(f) S + (1 - f) v^T, o = S^T silu(q) with f = l + (1 - l) sigmoid(z), head norm, over steps that continue sequences in
    slots with stale state; some channels forget within a few tokens, some hardly at all.  cols: steps with a span of eight rows or more
    take the form that deals value columns to workgroups, the others the fused one, on the same slots"""
    rng = np.random.default_rng(heads * 100 + dim)
    eps = 1e-5
    lower = rng.uniform(0, 0.95, size=heads * dim).astype(np.float32)
    norm_w = (1 + 0.2 * rng.standard_normal(vdim)).astype(np.float32)
    state = torch.full((3, heads, dim, vdim), 5.0, dtype=F32, device=be.device)
    S = {0: np.zeros((heads, dim, vdim)), 2: np.zeros((heads, dim, vdim))}
    n_tok = {0: 0, 2: 0}
    ld = 2 * heads * dim + heads * vdim + 3
    for step in scan_steps(rng)[:4 if dim > 128 else 7]:
        lens = [n for _s, n in step]
        rows = sum(lens)
        f = rng.standard_normal((rows, ld)).astype(np.float32)
        f[:, heads * dim:2 * heads * dim] *= 4.0
        seq = np.concatenate([[s] * n for s, n in step])
        pos = np.concatenate([np.arange(n_tok[s], n_tok[s] + n) for s, n in step])
        out = torch.zeros((rows, heads * vdim), dtype=F32, device=be.device)
        ft = be.t(f)
        o_raw = torch.zeros((rows, heads * vdim), dtype=F32, device=be.device) if cols and max(lens) >= 8 else None
        be.ext.gated_scan(be.ext.SCAN_FORGET_WRITES, ft, ld, 0, heads * dim, ft, ld, 2 * heads * dim, be.t(norm_w), out, state, spans_of(be, lens),
                          ints(be, seq), ints(be, pos), heads, heads, dim, vdim, eps, lower=be.t(lower), o_raw=o_raw)
        got, r = be.n(out), 0
        for s, n in step:
            for _ in range(n):
                row = f[r].astype(np.float64)
                q = OK.silu(row[:heads * dim]).reshape(heads, dim)
                fg = (lower + (1.0 - lower) * OK.sigmoid(row[heads * dim:2 * heads * dim])).reshape(heads, dim)
                v = row[2 * heads * dim:2 * heads * dim + heads * vdim].reshape(heads, vdim)
                want = []
                for i in range(heads):
                    S[s][i] = fg[i][:, None] * S[s][i] + np.outer(1.0 - fg[i], v[i])
                    want.append(OK.group_rms_norm(S[s][i].T @ q[i], norm_w, 1, eps))
                assert close(got[r], np.concatenate(want), 2e-5), (step, r)
                n_tok[s] += 1
                r += 1
    assert close(be.n(state)[0], S[0], 1e-5) and close(be.n(state)[2], S[2], 1e-5) and close(be.n(state)[1], np.full_like(S[0], 5.0), 0)


@pytest.mark.parametrize("cols", [False, True])
@pytest.mark.parametrize("heads,qk_heads,dim,vdim", [(2, 1, 5, 7), (4, 2, 16, 16), (1, 1, 64, 32), (6, 3, 32, 64), (2, 2, 130, 9), (1, 1, 128, 256)])
def test_delta_rule_scan(be, heads, qk_heads, dim, vdim, cols):
    """S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q with unit q / k, the head norm and the output gate, over steps that
    continue sequences in slots with stale state"""
    rng = np.random.default_rng(heads * 100 + dim)
    eps = 1e-5
    a_log, dt_bias = rng.standard_normal((2, heads)).astype(np.float32) - 1.0
    norm_w = (1 + 0.2 * rng.standard_normal(vdim)).astype(np.float32)
    state = torch.full((3, heads, dim, vdim), 5.0, dtype=F32, device=be.device)
    S = {0: np.zeros((heads, dim, vdim)), 2: np.zeros((heads, dim, vdim))}
    n_tok = {0: 0, 2: 0}
    ch = 2 * qk_heads * dim + heads * vdim
    ld = 2 * heads + heads * vdim + 1                            # [beta | dt | gate] + padding
    for step in scan_steps(rng)[:4 if dim > 100 else 7]:
        lens = [n for _s, n in step]
        rows = sum(lens)
        c = rng.standard_normal((rows, ch)).astype(np.float32)
        f = rng.standard_normal((rows, ld)).astype(np.float32) * 2
        seq = np.concatenate([[s] * n for s, n in step])
        pos = np.concatenate([np.arange(n_tok[s], n_tok[s] + n) for s, n in step])
        out = torch.zeros((rows, heads * vdim), dtype=F32, device=be.device)
        ct = be.t(c)
        o_raw = torch.zeros((rows, heads * vdim), dtype=F32, device=be.device) if cols and max(lens) >= 8 else None
        be.ext.gated_scan(be.ext.SCAN_DELTA, be.t(f), ld, 0, qk_heads * dim, ct, ch, 2 * qk_heads * dim, be.t(norm_w), out, state,
                          spans_of(be, lens), ints(be, seq), ints(be, pos), heads, qk_heads, dim, vdim, eps, q_scale=dim ** -0.5,
                          gate_off=2 * heads, beta_off=0, dt_off=heads, dt_bias=be.t(dt_bias), a_log=be.t(a_log), qk=ct, ldqk=ch, o_raw=o_raw)
        got, r = be.n(out), 0
        for s, n in step:
            for _ in range(n):
                cr, fr = c[r].astype(np.float64), f[r].astype(np.float64)
                q, k = cr[:qk_heads * dim].reshape(qk_heads, dim), cr[qk_heads * dim:2 * qk_heads * dim].reshape(qk_heads, dim)
                v = cr[2 * qk_heads * dim:].reshape(heads, vdim)
                beta = OK.sigmoid(fr[:heads])
                decay = np.exp(-np.exp(a_log.astype(np.float64)) * OK.softplus(fr[heads:2 * heads] + dt_bias))
                gate = OK.silu(fr[2 * heads:2 * heads + heads * vdim]).reshape(heads, vdim)
                want = []
                for i in range(heads):
                    g = i // (heads // qk_heads)
                    qi, ki = OK.unit(q[g]) * dim ** -0.5, OK.unit(k[g])
                    Si = decay[i] * S[s][i]
                    Si = Si + np.outer(ki, beta[i] * (v[i] - Si.T @ ki))
                    S[s][i] = Si
                    want.append(OK.group_rms_norm(Si.T @ qi, norm_w, 1, eps) * gate[i])
                assert close(got[r], np.concatenate(want), 3e-5), (step, r)
                n_tok[s] += 1
                r += 1
    assert close(be.n(state)[0], S[0], 1e-5) and close(be.n(state)[2], S[2], 1e-5) and close(be.n(state)[1], np.full_like(S[0], 5.0), 0)


# ---- whole models -----------------------------------------------------------------------------------------------------------------------

CONFIGS = {
    # every mixer, both with and without a feed-forward; sizes differ per layer
    "mixed": lambda: OK.small_config([
        OK.layer(OK.parallel_mixer(), OK.moe_ff_spec(experts=5, top=2, ff=12, shared=10)),
        OK.layer(OK.hgrn2_mixer(heads=3, dim=8, vdim=12), OK.moe_ff_spec(experts=4, top=1, ff=8, shared=8)),
        OK.layer(OK.delta_mixer(heads=4, kv_heads=2, dim=8, vdim=12, conv=4), None),
        OK.layer(OK.parallel_mixer(OK.attn_spec(heads=2, kv_heads=1, dim=12, vdim=20, dims=6), OK.ssm_spec(heads=2, vdim=16, state=4, groups=1, norm_groups=1, conv=2),
                                   left_scale=0.7, right_scale=1.3), OK.moe_ff_spec(experts=7, top=3, ff=6, shared=None))]),
    # the recurrent mixers first, one head, one tap in front of the sublayers, one norm group, every expert chosen, a shared expert as wide
    # as the routed ones, no rotation, one hash bucket, a residual branch at full weight
    "odd": lambda: OK.small_config([
        OK.layer(OK.delta_mixer(heads=1, kv_heads=1, dim=20, vdim=6, conv=1), OK.moe_ff_spec(experts=3, top=3, ff=8, shared=8)),
        OK.layer(OK.hgrn2_mixer(heads=1, dim=6, vdim=30), None),
        OK.layer(OK.parallel_mixer(OK.attn_spec(heads=3, kv_heads=3, dim=6, vdim=10, dims=0), OK.ssm_spec(heads=1, vdim=10, state=3, groups=1, norm_groups=5, conv=5),
                                   left_scale=1.0, right_scale=1.0), OK.moe_ff_spec(experts=9, top=1, ff=5, shared=3)),
        OK.layer(OK.hgrn2_mixer(heads=2, dim=4, vdim=4), OK.moe_ff_spec(experts=2, top=1, ff=16, shared=None))],
        width=30, vocab=50, groups=1, mult=1.0, taps=1, embed_scale=1.0, buckets=1, mul_prev=2, mul_cur=3),
    # head sizes the matrix-core attention takes in bfloat16, more norm groups, longer taps
    "wide": lambda: OK.small_config([
        OK.layer(OK.parallel_mixer(OK.attn_spec(heads=4, kv_heads=2, dim=32, vdim=32, dims=16), OK.ssm_spec(heads=2, vdim=32, state=16, groups=1, norm_groups=2, conv=4)),
                 OK.moe_ff_spec(experts=6, top=2, ff=16, shared=16)),
        OK.layer(OK.delta_mixer(heads=2, kv_heads=1, dim=32, vdim=32, conv=2), None),
        OK.layer(OK.parallel_mixer(OK.attn_spec(heads=2, kv_heads=1, dim=64, vdim=64, dims=64, base=500.0), OK.ssm_spec(heads=4, vdim=16, state=8, groups=2, norm_groups=1, conv=3)),
                 OK.moe_ff_spec(experts=4, top=1, ff=32, shared=8)),
        OK.layer(OK.hgrn2_mixer(heads=2, dim=16, vdim=32), None)], width=64, vocab=70, groups=4, taps=5),
}


def make_engine(be, cfg, W, dtype, max_tokens, page=4, max_seqs=4, graphs=None):
    from exllamav2_amd.config import LayeredConfig
    from exllamav2_amd.engine import Engine
    from exllamav2_amd.layered import LayeredModel
    tensors = {k: be.t(v).to(BF16) for k, v in W.items()}
    model = LayeredModel(LayeredConfig.from_dict_sandwich(cfg), device=be.device, dtype=dtype, ext=be.ext).load(tensors)
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
        OK.Oracle(cfg, W).feed("g", toks, gaps=gaps)
        if min(gaps) > gap:
            return toks
    raise AssertionError("no token sequence with clear routing found")


@pytest.mark.parametrize("name", sorted(CONFIGS))
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_whole_prompt(be, name, dtype):
    cfg = CONFIGS[name]()
    W = OK.random_model(cfg, seed=1)
    toks = clear_tokens(cfg, W, 23, 2, gap=0.03)
    want = OK.Oracle(cfg, W).feed("a", toks)
    eng = make_engine(be, cfg, W, dtype, 32)
    assert ok(run_cuts(be, eng, "a", toks, [23]), want, dtype)


def test_residual_stream_after_every_layer(be):
    """the oracle's stream after each layer against the model's, by running the model cut off after that layer"""
    cfg = CONFIGS["mixed"]()
    W = OK.random_model(cfg, seed=31)
    toks = [int(t) for t in np.random.default_rng(32).integers(0, cfg["vocab"], size=9)]
    trail = []
    OK.Oracle(cfg, W).feed("a", toks, residuals=trail)
    for depth in range(1, len(cfg["layers"]) + 1):
        sub = dict(cfg, layers=cfg["layers"][:depth])
        Ws = dict(W)
        Ws["final.norm"] = np.ones(cfg["width"], dtype=np.float32)
        Ws["head"] = np.eye(cfg["width"], dtype=np.float32)       # logits = the normed stream
        sub["vocab"] = cfg["vocab"]
        Ws["head"] = np.concatenate([Ws["head"], np.zeros((max(cfg["vocab"] - cfg["width"], 0), cfg["width"]), dtype=np.float32)])[:cfg["vocab"]]
        eng = make_engine(be, sub, Ws, F32, 16)
        got = run_cuts(be, eng, "a", toks, [9])[:, :cfg["width"]]
        want = np.array([OK.group_rms_norm(trail[t][depth - 1], np.ones(cfg["width"]), cfg["norm"]["groups"], cfg["norm"]["eps"]) for t in range(9)])
        assert close(got, want[:, :got.shape[1]], 2e-5), depth


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_decoding_and_portions(be, name):
    """the same positions through a whole prompt, token by token from the first token on (the convolutions' tails, the previous token
    and the recurrent state pass over decoded tokens), and in portions down to two tokens that end inside pages"""
    cfg = CONFIGS[name]()
    W = OK.random_model(cfg, seed=3)
    toks = list(np.random.default_rng(4).integers(0, cfg["vocab"], size=26))
    want = OK.Oracle(cfg, W).feed("a", toks)
    for cuts in ([1] * 26, [2, 3, 2, 5, 2, 1, 1, 4, 2, 2, 2], [9] + [1] * 17, [25, 1], [1, 25]):
        eng = make_engine(be, cfg, W, F32, 28, page=4)
        assert rel_err(run_cuts(be, eng, "a", toks, cuts), want) <= TOL[F32], cuts


def test_mixed_batches_reuse_pages_and_slots(be):
    """five unequal requests over four slots and a pool smaller than their sum: portions beside single tokens, a request left out of
    a step, finished requests' pages and slot (with its tails, previous token and recurrent state) taken by the next; every position
    equals the request alone"""
    cfg = CONFIGS["mixed"]()
    W = OK.random_model(cfg, seed=5)
    rng = np.random.default_rng(6)
    reqs = {r: list(rng.integers(0, cfg["vocab"], size=n)) for r, n in (("a", 13), ("b", 5), ("c", 9), ("d", 2), ("e", 11))}
    oracle = OK.Oracle(cfg, W)
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
    """one slot, three requests one after the other: the second and third find the first one's tails, token, recurrent state and
    cached keys in their slot and pages and must not see them"""
    cfg = CONFIGS["mixed"]()
    W = OK.random_model(cfg, seed=15)
    rng = np.random.default_rng(16)
    eng = make_engine(be, cfg, W, F32, max_tokens=16, page=4, max_seqs=1)
    for r, n, cuts in (("a", 14, [14]), ("b", 9, [1, 1, 7]), ("c", 12, [2, 10])):
        toks = list(rng.integers(0, cfg["vocab"], size=n))
        want = OK.Oracle(cfg, W).feed(r, toks)
        assert rel_err(run_cuts(be, eng, r, toks, cuts), want) <= TOL[F32], r
        eng.finish(r)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_decode_steps_as_graphs(be, dtype):
    """decoding steps through the engine's persistent-input path (on a GPU: captured once per batch size and replayed; every replay
    is checked): two requests decode side by side, one ends, the other goes on alone, a third joins"""
    cfg = CONFIGS["mixed"]()
    W = OK.random_model(cfg, seed=21)
    reqs = {r: clear_tokens(cfg, W, n, 22 + i, gap=0.03) for i, (r, n) in enumerate((("a", 14), ("b", 9), ("c", 8)))}
    oracle = OK.Oracle(cfg, W)
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
        assert ok(np.stack([got[r][p] for p in range(len(reqs[r]))]), want[r], dtype), r
    eng.close()


def test_matrix_core_sizes_in_portions_and_decoding_bf16(be):
    """head sizes of the tile kernels: a prompt of several 64-row tiles that crosses page borders, then decoding, beside a second
    request"""
    cfg = CONFIGS["wide"]()
    W = OK.random_model(cfg, seed=41)
    reqs = {r: clear_tokens(cfg, W, n, 42 + i, gap=0.004) for i, (r, n) in enumerate((("a", 12), ("b", 160)))}
    oracle = OK.Oracle(cfg, W)
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
        assert ok(np.stack([got[r][p] for p in range(len(reqs[r]))]), want[r], BF16), r
    eng.close()


def test_head_sizes_of_a_real_model_bf16_and_f32(be):
    """sizes at which every tuned kernel path is taken (attention tiles of 128, the chunked state-space scan, full-state column scans of
    64 and 128 key channels, the vector norm, grouped expert launches): a prompt in portions, then decoding, beside a second request"""
    if be.is_emu:
        pytest.skip("minutes on the CPU twin; the small configurations cover its logic")
    cfg = OK.small_config([
        OK.layer(OK.parallel_mixer(OK.attn_spec(heads=4, kv_heads=2, dim=128, vdim=128, dims=64, base=500000.0),
                                   OK.ssm_spec(heads=8, vdim=32, state=64, groups=2, norm_groups=2, conv=4)), OK.moe_ff_spec(experts=8, top=2, ff=64, shared=96)),
        OK.layer(OK.hgrn2_mixer(heads=2, dim=128, vdim=128), OK.moe_ff_spec(experts=8, top=2, ff=64, shared=64)),
        OK.layer(OK.delta_mixer(heads=4, kv_heads=2, dim=64, vdim=64, conv=4), None),
        OK.layer(OK.delta_mixer(heads=2, kv_heads=2, dim=128, vdim=128, conv=3), OK.moe_ff_spec(experts=4, top=1, ff=128, shared=None)),
        OK.layer(OK.hgrn2_mixer(heads=4, dim=64, vdim=64), None)], width=256, vocab=300, groups=2, taps=4, buckets=251, mul_prev=113, mul_cur=5)
    W = OK.random_model(cfg, seed=61)
    reqs = {"a": clear_tokens(cfg, W, 150, 62, gap=0.002), "b": clear_tokens(cfg, W, 20, 63, gap=0.002)}
    oracle = OK.Oracle(cfg, W)
    want = {r: oracle.feed(r, t) for r, t in reqs.items()}
    for dtype in (F32, BF16):
        eng = make_engine(be, cfg, W, dtype, max_tokens=512, page=64, graphs=True)
        got = {r: {} for r in reqs}

        def step(parts, end=()):
            lg = be.n(eng.step([(r, reqs[r][lo:hi], list(range(hi - lo))) for r, lo, hi in parts], end))
            k = 0
            for r, lo, hi in parts:
                for p in range(lo, hi):
                    got[r][p] = lg[k]; k += 1

        step([("a", 0, 70)])
        step([("a", 70, 135), ("b", 0, 9)])
        step([("a", 135, 137), ("b", 9, 10)])
        for i in range(10):
            step([("a", 137 + i, 138 + i), ("b", 10 + i, 11 + i)])
        step([("a", 147, 150)])
        for r in reqs:
            assert ok(np.stack([got[r][p] for p in range(len(reqs[r]))]), want[r], dtype, frac=0.7), (r, dtype)
        eng.close()


def crafted_model(seed=31):
    """one layer of attention beside a (silenced) state-space scan, made so that token 0's query matches token 1's key and nothing
    else: queries read inputs 0-3, keys inputs 4-7 through the same matrix, values the other inputs; token 0 is marked in inputs 0-3,
    token 1 in 4-7, all other tokens are zero there; no rotation, no input convolution to speak of, no token-pair rows.  Wherever a
    token 1 stands in front of token 0, however far, that key takes the softmax among hundreds."""
    cfg = OK.small_config([OK.layer(OK.parallel_mixer(OK.attn_spec(heads=2, kv_heads=2, dim=8, vdim=8, dims=0, scale=1.0),
                                                      OK.ssm_spec(heads=2, vdim=4, state=4, groups=1, norm_groups=1, conv=2), 1.0, 0.05),
                                    OK.moe_ff_spec(experts=3, top=1, ff=8, shared=8))], width=16, vocab=40, groups=1, taps=2)
    W = OK.random_model(cfg, seed=seed)
    rng = np.random.default_rng(seed + 1)
    E = W["embed"]
    E[:, :8] = 0.0
    mark = rng.standard_normal(4)
    mark *= 6.0 / np.linalg.norm(mark)
    E[0, :4], E[1, 4:8] = mark, mark
    W["embed"] = OK.bf16_round(E)
    W["bigram"][:] = 0.0
    W["embed.norm"][:] = 1.0
    W["l0.norm1"][:] = 1.0
    W["l0.canon1"][:] = 0.0
    M = rng.standard_normal((16, 4))
    W["l0.mix.left.q"], W["l0.mix.left.k"] = np.zeros((16, 16), dtype=np.float32), np.zeros((16, 16), dtype=np.float32)
    W["l0.mix.left.q"][:, :4], W["l0.mix.left.k"][:, 4:8] = OK.bf16_round(M), OK.bf16_round(M)
    W["l0.mix.left.q.b"][:] = 0.0
    W["l0.mix.left.k.b"][:] = 0.0
    W["l0.mix.left.v"][:, :8] = 0.0
    W["l0.mix.left.v"] = OK.bf16_round(W["l0.mix.left.v"] * 4)
    return cfg, W


@pytest.mark.parametrize("page", [4, 64])
def test_a_marked_key_far_back_and_at_page_borders(be, page):
    """whole prompt, portions and decoding: the marked key sits right in front of the query, at the sequence's first token, on both
    sides of a page border and hundreds of tokens back; where it stands it decides the query's logits"""
    cfg, W = crafted_model()
    rng = np.random.default_rng(page)
    T = 330
    query = T - 1
    changes = 0
    for target in (0, 1, page - 1, page, 2 * page, 200, query - page, query - 1):
        toks = [int(t) for t in rng.integers(2, cfg["vocab"], size=T)]
        toks[target], toks[query] = 1, 0                      # the marked pair, nowhere else
        base = list(toks)
        base[target] = 2
        want = OK.Oracle(cfg, W).feed("t", toks)
        other = OK.Oracle(cfg, W).feed("t", base)[-1]
        changes += rel_err(want[-1:], other[None]) > 0.05
        plans = [[T], [target + 1, T - target - 2, 1], [T - 3, 2, 1], [T - 20] + [1] * 20]
        for cuts in plans if target in (0, 200, query - 1) else plans[1:3]:
            eng = make_engine(be, cfg, W, F32, max_tokens=T + page, page=page)
            got = run_cuts(be, eng, "t", toks, [c for c in cuts if c > 0])
            assert rel_err(got[-4:], want[-4:]) <= TOL[F32], (target, cuts[:3])
    assert changes >= 6


@pytest.mark.parametrize("kind", ["hgrn2", "delta"])
def test_the_state_carries_a_far_token(be, kind):
    """a model without attention: a token 300 positions back reaches the last position only through the recurrent state: changing
    it changes the logits, and portions and decoding carry it like the whole prompt does"""
    mixer = OK.hgrn2_mixer(heads=2, dim=8, vdim=8) if kind == "hgrn2" else OK.delta_mixer(heads=2, kv_heads=1, dim=8, vdim=8, conv=2)
    cfg = OK.small_config([OK.layer(mixer, OK.moe_ff_spec(experts=3, top=1, ff=8, shared=8))], width=16, vocab=40)
    W = OK.random_model(cfg, seed=51)
    if kind == "hgrn2":
        W["l0.mix.lower"][:] = OK.bf16_round(np.full(16, 0.996))                    # slow forgetting
    else:
        W["l0.mix.A_log"][:] = -8.0                                                # decay exp(-exp(-8) dt) per token
        W["l0.mix.b"] = OK.bf16_round(W["l0.mix.b"] * 0.1 - 0.0)
    rng = np.random.default_rng(52)
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], size=310)]
    other = list(toks)
    other[9] = (toks[9] + 1) % cfg["vocab"]
    want = OK.Oracle(cfg, W).feed("a", toks)
    assert rel_err(OK.Oracle(cfg, W).feed("a", other)[-1:], want[-1:]) > 1e-3
    for cuts in ([310], [100, 2, 65, 143], [290] + [1] * 20):
        eng = make_engine(be, cfg, W, F32, max_tokens=320, page=16)
        assert rel_err(run_cuts(be, eng, "a", toks, cuts)[-8:], want[-8:]) <= 2 * TOL[F32], cuts


def test_long_decoding_bf16(be):
    cfg = CONFIGS["mixed"]()
    W = OK.random_model(cfg, seed=7)
    toks = clear_tokens(cfg, W, 60, 8, gap=0.006)
    want = OK.Oracle(cfg, W).feed("a", toks)
    eng = make_engine(be, cfg, W, BF16, 64, page=8)
    assert ok(run_cuts(be, eng, "a", toks, [3] + [1] * 57), want, BF16)


def test_greedy_generation_through_the_generator(be):
    from exllamav2_amd.engine import Generator
    cfg = CONFIGS["mixed"]()
    W = OK.random_model(cfg, seed=9)
    rng = np.random.default_rng(10)
    prompts = [list(map(int, rng.integers(0, cfg["vocab"], size=n))) for n in (7, 3, 5, 4, 6)]
    eng = make_engine(be, cfg, W, F32, max_tokens=64, page=4, max_seqs=3)
    out = Generator(eng, chunk=3).generate(prompts, 6)
    oracle = OK.Oracle(cfg, W)
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
    W = OK.random_model(cfg, seed=11)
    save_file({k: torch.from_numpy(np.asarray(v)).to(BF16) for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    assert read_config(str(tmp_path))[0] == "Kilurax"
    model = load_model(str(tmp_path), device=be.device, dtype=F32, ext=be.ext)
    toks = [1, 5, 9, 2, 2, 7]
    got = be.n(Engine(model, 16, page_size=4).step([("x", toks, list(range(6)))]))
    assert rel_err(got, OK.Oracle(cfg, W).feed("x", toks)) <= TOL[F32]


def test_unknown_mixer_and_bad_groups_are_refused(be):
    from exllamav2_amd.config import LayeredConfig
    cfg = CONFIGS["mixed"]()
    with pytest.raises(RuntimeError, match="norm groups"):
        LayeredConfig.from_dict_sandwich(dict(cfg, norm={"eps": 1e-5, "groups": 5}))
    bad = dict(cfg, layers=[dict(cfg["layers"][0], type="nonesuch")])
    with pytest.raises(RuntimeError, match="unknown mixer"):
        make_engine(be, bad, OK.random_model(cfg, seed=1), F32, 16)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_command_replays_steps(tmp_path, dtype):
    """bin/trace_run in a process of its own: steps on standard input, logits files and `done` lines out"""
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from safetensors.torch import save_file
    cfg = CONFIGS["mixed"]()
    W = OK.random_model(cfg, seed=12)
    mdir = tmp_path / "model"
    mdir.mkdir()
    save_file({k: torch.from_numpy(np.asarray(v)).to(BF16) for k, v in W.items()}, str(mdir / "model.safetensors"))
    (mdir / "config.json").write_text(json.dumps(cfg))
    a = clear_tokens(cfg, W, 300, 13, gap=0.002)
    b = clear_tokens(cfg, W, 9, 14)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:290], "want": [0, 289]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[290:295], "want": []}, {"id": "b", "tokens": b[:8], "want": [7]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[8:], "want": [0]}, {"id": "a", "tokens": a[295:], "want": [4]}], "end": ["a", "b"]}]
    out = tmp_path / "out"
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(mdir), "--dtype", dtype, "--out", str(out), "--max-tokens", "512"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600, cwd=str(tmp_path))
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    oracle = OK.Oracle(cfg, W)
    wa, wb = oracle.feed("a", a), oracle.feed("b", b)
    got = np.concatenate([np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(k, -1) for n, k in ((0, 2), (1, 1), (2, 2))])
    want = np.stack([wa[0], wa[289], wb[7], wb[8], wa[299]])
    e = pos_errs(got, want)
    # (five positions of one draw: the typical one pins the arithmetic, the worst may sit where a head norm divides by little)
    assert (np.median(e) <= 3e-6 and e.max() <= 1e-4) if dtype == "float32" else (np.median(e) <= 4e-2 and e.max() <= 0.1), e
