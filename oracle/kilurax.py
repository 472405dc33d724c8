"""Plain float64 restatement of the Kilurax layer stack (sandwich-normed residual steps with a short convolution in front of every
sublayer; softmax attention beside a state-space scan, gated linear attention whose forget gate also writes, gated delta rule;
sparse feed-forwards with sigmoid scores and a shared expert; a hashed token-pair embedding) -- TEST INFRASTRUCTURE ONLY.

One function per mechanism, token by token, written from the equations; nothing is shared with the product path (no pages, no
slots, no batching: a sequence's memory is python lists and per-layer arrays).

Notation: W x with W stored [out, in]; p = a token's position (from 0); n_g(v) = v cut into g equal runs, each divided by
sqrt(mean(run^2) + eps); t = a token, t' = the token before it in the sequence.
    embedding:  x = n_g(embed[t] * scale + bigram[(t' mul_prev + t mul_cur) mod buckets]) w;  row `buckets` of bigram at p = 0
    sublayer:   a = n_g(x) w_in;  h = a + sum_j c[:, j] a_(p - taps + 1 + j)  (rows before p = 0 are zeros);
                x <- x + mult * n_g(f(h)) w_out;   a layer is this with f = mixer, then with f = feed-forward (if it has one)
    parallel:   left_scale * attention(h) + right_scale * ssm(h)
      attention (H query heads over G key / value heads, biases on q, k, v, o): the first `dims` values of every q / k head in
                pairs (i, i + dims / 2) turned by p base^(-2i / dims);  s_j = q . k_j scale for j <= p;  softmax;  W_o heads + b_o
      ssm       [z | u | B | C | d] = W_in h;  (u, B, C) <- silu(conv(u, B, C) + bias);  d <- softplus(d + d_bias);
                head i of group g: S <- exp(-exp(A_i) d_i) S + d_i B_g u_i^T;  y_i = S^T C_g + D_i u_i;
                out = W_o (n_groups(y silu(z)) w)
    hgrn2:      q = silu(W_q h);  f = l + (1 - l) sigmoid(W_f h + b_f);  v = W_v h;  head i: S <- diag(f_i) S + (1 - f_i) v_i^T;
                o_i = S^T q_i;  out = W_o concat_i(n_1(o_i) w)
    delta:      q, k, v = silu(conv(W h)) per channel (no bias);  q, k per head divided by sqrt(sum(.^2) + 1e-6), q also by sqrt(dim);
                beta = sigmoid(W_b h);  g = exp(-exp(A) softplus(W_a h + d_bias));  head i (q / k head i // (heads / kv_heads)):
                S <- g_i S;  u = beta_i (v_i - S^T k);  S <- S + k u^T;  o_i = S^T q;
                out = W_o concat_i(n_1(o_i) w * silu(W_g h)_i)
    moe:        s = sigmoid(W_router h); the `top` largest s choose experts; y = sum_e E_e(s_e h) + E_shared(h),
                E(z) = W_down (silu(W_gate z) * W_up z)
    logits:     head (n_g(x) w_final)
"""
from __future__ import annotations

import math

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def group_rms_norm(v, w, groups, eps):
    parts = v.reshape(groups, -1)
    return (parts / np.sqrt((parts * parts).mean(-1, keepdims=True) + eps)).reshape(-1) * w


def bigram_row(cfg, prev_token, token):
    b = cfg["embedding"]["bigram"]
    if prev_token is None:
        return int(b["buckets"])
    return (int(prev_token) * int(b["mul_prev"]) + int(token) * int(b["mul_cur"])) % int(b["buckets"])


def embed_token(W, cfg, prev_token, token):
    x = W["embed"][int(token)] * cfg["embedding"]["scale"] + W["bigram"][bigram_row(cfg, prev_token, token)]
    return group_rms_norm(x, W["embed.norm"], cfg["norm"]["groups"], cfg["norm"]["eps"])


def causal_conv(history, taps_w, bias=None):
    """history: the inputs up to and including the current token, newest last (a list of vectors); taps_w [channels, taps]: the
    last column weighs the current token"""
    taps = taps_w.shape[1]
    acc = np.zeros(taps_w.shape[0]) if bias is None else bias.copy()
    for j in range(taps):
        back = taps - 1 - j
        if back < len(history):
            acc = acc + taps_w[:, j] * history[len(history) - 1 - back]
    return acc


def input_conv(history, taps_w):
    """what a sublayer reads: its normed row plus the convolution over the last `taps` normed rows"""
    return history[-1] + causal_conv(history, taps_w)


def turn_head(vec, pos, base, dims):
    out = vec.copy()
    half = dims // 2
    for i in range(half):
        a = pos * base ** (-2.0 * i / dims)
        u, v = vec[i], vec[i + half]
        out[i] = u * math.cos(a) - v * math.sin(a)
        out[i + half] = v * math.cos(a) + u * math.sin(a)
    return out


def attention_token(W, key, m, h, pos, kv):
    """appends this token's keys and values to kv, returns the attention's output [width]"""
    H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m["rot"]
    q = (W[key + ".q"] @ h + W[key + ".q.b"]).reshape(H, dim)
    k = (W[key + ".k"] @ h + W[key + ".k.b"]).reshape(G, dim)
    v = (W[key + ".v"] @ h + W[key + ".v.b"]).reshape(G, vd)
    q = np.stack([turn_head(q[i], pos, rot["base"], rot["dims"]) for i in range(H)])
    k = np.stack([turn_head(k[i], pos, rot["base"], rot["dims"]) for i in range(G)])
    kv.append((k, v))
    heads = []
    for i in range(H):
        g = i // (H // G)
        s = np.array([q[i] @ kj[g] for kj, _ in kv]) * m["scale"]
        w = np.exp(s - s.max())
        w = w / w.sum()
        heads.append(sum(wj * vj[g] for wj, (_, vj) in zip(w, kv)))
    return W[key + ".o"] @ np.concatenate(heads) + W[key + ".o.b"]


def ssm_token(W, key, m, h, mem, eps):
    """mem: {"hist": list of the last convolution inputs, "S": [heads, state, vdim]}"""
    H, vd, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * vd
    f = W[key + ".in"] @ h
    z, xbc, d = f[:inner], f[inner:2 * inner + 2 * G * N], f[2 * inner + 2 * G * N:]
    mem["hist"] = (mem["hist"] + [xbc])[-m["conv"]:]
    c = silu(causal_conv(mem["hist"], W[key + ".conv"], W[key + ".conv.b"]))
    u, B, C = c[:inner].reshape(H, vd), c[inner:inner + G * N].reshape(G, N), c[inner + G * N:].reshape(G, N)
    d = softplus(d + W[key + ".dt_bias"])
    y = np.zeros((H, vd))
    for i in range(H):
        g = i // (H // G)
        mem["S"][i] = math.exp(-math.exp(W[key + ".A_log"][i]) * d[i]) * mem["S"][i] + d[i] * np.outer(B[g], u[i])
        y[i] = mem["S"][i].T @ C[g] + W[key + ".D"][i] * u[i]
    gated = y.reshape(-1) * silu(z)
    return W[key + ".o"] @ group_rms_norm(gated, W[key + ".norm"], m["norm_groups"], eps)


def parallel_token(W, key, m, h, pos, mem, eps):
    left = attention_token(W, key + ".left", m["left"], h, pos, mem["kv"])
    right = ssm_token(W, key + ".right", m["right"], h, mem, eps)
    return m["left_scale"] * left + m["right_scale"] * right


def hgrn2_token(W, key, m, h, mem, eps):
    """mem: {"S": [heads, dim, vdim]}"""
    H, dim, vd = m["heads"], m["dim"], m["vdim"]
    q = silu(W[key + ".q"] @ h).reshape(H, dim)
    low = W[key + ".lower"]
    f = (low + (1.0 - low) * sigmoid(W[key + ".f"] @ h + W[key + ".f.b"])).reshape(H, dim)
    v = (W[key + ".v"] @ h).reshape(H, vd)
    out = []
    for i in range(H):
        mem["S"][i] = f[i][:, None] * mem["S"][i] + np.outer(1.0 - f[i], v[i])
        out.append(group_rms_norm(mem["S"][i].T @ q[i], W[key + ".norm"], 1, eps))
    return W[key + ".o"] @ np.concatenate(out)


def unit(v):
    return v / math.sqrt(float(v @ v) + 1e-6)


def delta_token(W, key, m, h, mem, eps):
    """mem: {"hq" / "hk" / "hv": lists of the last convolution inputs, "S": [heads, dim, vdim]}"""
    H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    conv = {}
    for s in "qkv":
        mem["h" + s] = (mem["h" + s] + [W[f"{key}.{s}"] @ h])[-m["conv"]:]
        conv[s] = silu(causal_conv(mem["h" + s], W[f"{key}.{s}.conv"]))
    q, k, v = conv["q"].reshape(G, dim), conv["k"].reshape(G, dim), conv["v"].reshape(H, vd)
    beta = sigmoid(W[key + ".b"] @ h)
    decay = np.exp(-np.exp(W[key + ".A_log"]) * softplus(W[key + ".a"] @ h + W[key + ".dt_bias"]))
    gate = silu(W[key + ".g"] @ h).reshape(H, vd)
    out = []
    for i in range(H):
        g = i // (H // G)
        qi, ki = unit(q[g]) * dim ** -0.5, unit(k[g])
        S = decay[i] * mem["S"][i]
        u = beta[i] * (v[i] - S.T @ ki)
        S = S + np.outer(ki, u)
        mem["S"][i] = S
        out.append(group_rms_norm(S.T @ qi, W[key + ".norm"], 1, eps) * gate[i])
    return W[key + ".o"] @ np.concatenate(out)


def gated_expert(W, key, z):
    return W[key + ".down"] @ (silu(W[key + ".gate"] @ z) * (W[key + ".up"] @ z))


def route(W, key, ms, h):
    """[(expert, weight)] of one token: the `top` largest sigmoid scores, as they are"""
    s = sigmoid(W[key + ".router"] @ h)
    order = np.argsort(-s, kind="stable")[:ms["router"]["top"]]
    return [(int(e), float(s[e])) for e in order]


def route_gap(W, key, ms, h):
    """distance between the last chosen and the first rejected router logit (inf when every expert is chosen)"""
    z = np.sort(W[key + ".router"] @ h)[::-1]
    top = ms["router"]["top"]
    return float(z[top - 1] - z[top]) if top < len(z) else math.inf


def moe_ff(W, key, ms, h):
    y = np.zeros(W[key + ".e0.down"].shape[0])
    for e, w in route(W, key, ms, h):
        y += gated_expert(W, f"{key}.e{e}", w * h)
    if ms.get("shared"):
        y += gated_expert(W, key + ".shared", h)
    return y


class Oracle:
    """feed(seq, tokens) -> logits [len(tokens), vocab] of the sequence's next tokens; state is kept per sequence name"""

    def __init__(self, cfg: dict, weights: dict):
        self.cfg = cfg
        self.W = {k: np.asarray(v, dtype=np.float64) for k, v in weights.items()}
        self.seqs = {}

    def _new(self):
        mem = []
        for spec in self.cfg["layers"]:
            m = spec["mixer"]
            st = {"a1": [], "a2": []}
            if spec["type"] == "parallel":
                r = m["right"]
                st.update(kv=[], hist=[], S=np.zeros((r["heads"], r["state"], r["vdim"])))
            elif spec["type"] == "hgrn2":
                st.update(S=np.zeros((m["heads"], m["dim"], m["vdim"])))
            elif spec["type"] == "delta":
                st.update(hq=[], hk=[], hv=[], S=np.zeros((m["heads"], m["dim"], m["vdim"])))
            else:
                raise ValueError(spec["type"])
            mem.append(st)
        return {"n": 0, "prev": None, "mem": mem}

    def feed(self, seq, tokens, residuals=None, gaps=None):
        """residuals (a list): takes the stream after every layer per token; gaps (a list): takes every token's smallest router gap"""
        cfg, W = self.cfg, self.W
        eps, groups, mult, taps = cfg["norm"]["eps"], cfg["norm"]["groups"], cfg["residual_mult"], cfg["canon"]["taps"]
        st = self.seqs.setdefault(seq, None) or self._new()
        self.seqs[seq] = st
        out = []
        for t in tokens:
            pos = st["n"]
            x = embed_token(W, cfg, st["prev"], t)
            st["prev"] = int(t)
            trail, gap = [], math.inf
            for i, spec in enumerate(cfg["layers"]):
                key, m, mem = f"l{i}", spec["mixer"], st["mem"][i]
                mem["a1"] = (mem["a1"] + [group_rms_norm(x, W[key + ".norm1"], groups, eps)])[-taps:]
                h = input_conv(mem["a1"], W[key + ".canon1"])
                if spec["type"] == "parallel":
                    y = parallel_token(W, key + ".mix", m, h, pos, mem, eps)
                elif spec["type"] == "hgrn2":
                    y = hgrn2_token(W, key + ".mix", m, h, mem, eps)
                else:
                    y = delta_token(W, key + ".mix", m, h, mem, eps)
                x = x + mult * group_rms_norm(y, W[key + ".norm1b"], groups, eps)
                ms = spec.get("mlp")
                if ms is not None:
                    mem["a2"] = (mem["a2"] + [group_rms_norm(x, W[key + ".norm2"], groups, eps)])[-taps:]
                    h2 = input_conv(mem["a2"], W[key + ".canon2"])
                    gap = min(gap, route_gap(W, key + ".mlp", ms, h2))
                    x = x + mult * group_rms_norm(moe_ff(W, key + ".mlp", ms, h2), W[key + ".norm2b"], groups, eps)
                trail.append(x.copy())
            if residuals is not None:
                residuals.append(np.stack(trail))
            if gaps is not None:
                gaps.append(gap)
            out.append(W["head"] @ group_rms_norm(x, W["final.norm"], groups, eps))
            st["n"] += 1
        return np.stack(out)

    def drop(self, seq):
        self.seqs.pop(seq, None)


# ---- small random models for the tests ---------------------------------------------------------------------------------------


def bf16_round(a):
    u = np.asarray(a, dtype=np.float32).view(np.uint32)
    return (((u + 0x7fff + ((u >> 16) & 1)) & 0xffff0000).astype(np.uint32)).view(np.float32)


def attn_spec(heads=4, kv_heads=2, dim=16, vdim=8, dims=None, base=10000.0, scale=None):
    return {"dim": dim, "heads": heads, "kv_heads": kv_heads, "rot": {"base": base, "dims": dim if dims is None else dims},
            "scale": scale if scale is not None else dim ** -0.5, "vdim": vdim}


def ssm_spec(heads=4, vdim=8, state=8, groups=2, norm_groups=2, conv=3):
    return {"conv": conv, "groups": groups, "heads": heads, "norm_groups": norm_groups, "state": state, "vdim": vdim}


def parallel_mixer(left=None, right=None, left_scale=1.25, right_scale=0.75):
    return {"type": "parallel", "mixer": {"left": left or attn_spec(), "left_scale": left_scale, "right": right or ssm_spec(),
                                          "right_scale": right_scale}}


def hgrn2_mixer(heads=3, dim=8, vdim=12):
    return {"type": "hgrn2", "mixer": {"dim": dim, "heads": heads, "vdim": vdim}}


def delta_mixer(heads=4, kv_heads=2, dim=8, vdim=12, conv=3):
    return {"type": "delta", "mixer": {"conv": conv, "dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim}}


def moe_ff_spec(experts=5, top=2, ff=12, shared=10):
    ms = {"expert": {"ff": ff}, "kind": "moe", "router": {"experts": experts, "top": top}}
    if shared:
        ms["shared"] = {"ff": shared}
    return ms


def layer(mix, ff=None):
    return dict(mix, mlp=ff)


def small_config(layers, width=32, vocab=61, eps=1e-5, groups=2, mult=0.625, taps=3, embed_scale=2.0, buckets=37, mul_prev=31, mul_cur=5):
    return {"architecture": "Kilurax", "canon": {"taps": taps},
            "embedding": {"bigram": {"buckets": buckets, "mul_cur": mul_cur, "mul_prev": mul_prev}, "scale": embed_scale},
            "layers": layers, "norm": {"eps": eps, "groups": groups}, "residual_mult": mult, "vocab": vocab, "width": width}


def random_model(cfg: dict, seed: int = 0) -> dict:
    """name -> float32 array (bfloat16-representable values), shapes from the configuration"""
    rng = np.random.default_rng(seed)
    Wd, taps, out = cfg["width"], cfg["canon"]["taps"], {}

    def mat(name, o, i, gain=1.0):
        out[name] = bf16_round(rng.standard_normal((o, i)) * gain / math.sqrt(i))

    def vec(name, n, centre=0.0, spread=0.1):
        out[name] = bf16_round(centre + rng.standard_normal(n) * spread)

    def attention(k, m):
        H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        mat(k + ".q", H * dim, Wd, 2.0); mat(k + ".k", G * dim, Wd, 2.0); mat(k + ".v", G * vd, Wd); mat(k + ".o", Wd, H * vd)
        vec(k + ".q.b", H * dim, 0.0, 0.3); vec(k + ".k.b", G * dim, 0.0, 0.3); vec(k + ".v.b", G * vd, 0.0, 0.3); vec(k + ".o.b", Wd, 0.0, 0.3)

    def ssm(k, m):
        H, vd, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
        inner, ch = H * vd, H * vd + 2 * G * N
        mat(k + ".in", 2 * inner + 2 * G * N + H, Wd)
        out[k + ".conv"] = bf16_round(rng.standard_normal((ch, m["conv"])) / math.sqrt(m["conv"]))
        vec(k + ".conv.b", ch, 0.0, 0.2); vec(k + ".dt_bias", H, -1.0, 0.5); vec(k + ".A_log", H, 0.0, 0.5); vec(k + ".D", H, 1.0, 0.3)
        vec(k + ".norm", inner, 1.0); mat(k + ".o", Wd, inner)

    out["embed"] = bf16_round(rng.standard_normal((cfg["vocab"], Wd)))
    out["bigram"] = bf16_round(rng.standard_normal((cfg["embedding"]["bigram"]["buckets"] + 1, Wd)))
    vec("embed.norm", Wd, 1.0)
    for i, spec in enumerate(cfg["layers"]):
        k, m = f"l{i}", spec["mixer"]
        vec(k + ".norm1", Wd, 1.0); vec(k + ".norm1b", Wd, 1.0)
        out[k + ".canon1"] = bf16_round(rng.standard_normal((Wd, taps)) * 0.4)
        if spec["type"] == "parallel":
            attention(k + ".mix.left", m["left"]); ssm(k + ".mix.right", m["right"])
        elif spec["type"] == "hgrn2":
            H, dim, vd = m["heads"], m["dim"], m["vdim"]
            mat(k + ".mix.q", H * dim, Wd); mat(k + ".mix.f", H * dim, Wd, 2.0); mat(k + ".mix.v", H * vd, Wd)
            vec(k + ".mix.f.b", H * dim, 1.0, 1.0)
            out[k + ".mix.lower"] = bf16_round(rng.uniform(0.0, 0.9, size=H * dim))
            vec(k + ".mix.norm", vd, 1.0); mat(k + ".mix.o", Wd, H * vd)
        else:
            H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            mat(k + ".mix.q", G * dim, Wd, 2.0); mat(k + ".mix.k", G * dim, Wd, 2.0); mat(k + ".mix.v", H * vd, Wd, 2.0)
            for s, n in (("q", G * dim), ("k", G * dim), ("v", H * vd)):
                out[f"{k}.mix.{s}.conv"] = bf16_round(rng.standard_normal((n, m["conv"])) / math.sqrt(m["conv"]))
            mat(k + ".mix.b", H, Wd, 2.0); mat(k + ".mix.a", H, Wd); mat(k + ".mix.g", H * vd, Wd, 2.0)
            vec(k + ".mix.dt_bias", H, -1.0, 0.5); vec(k + ".mix.A_log", H, -1.0, 0.5)
            vec(k + ".mix.norm", vd, 1.0); mat(k + ".mix.o", Wd, H * vd)
        ms = spec.get("mlp")
        if ms is not None:
            vec(k + ".norm2", Wd, 1.0); vec(k + ".norm2b", Wd, 1.0)
            out[k + ".canon2"] = bf16_round(rng.standard_normal((Wd, taps)) * 0.4)
            mat(k + ".mlp.router", ms["router"]["experts"], Wd, 2.0)
            names = [f"e{e}" for e in range(ms["router"]["experts"])] + (["shared"] if ms.get("shared") else [])
            for n in names:
                ff = ms["shared"]["ff"] if n == "shared" else ms["expert"]["ff"]
                mat(f"{k}.mlp.{n}.gate", ff, Wd, 2.0); mat(f"{k}.mlp.{n}.up", ff, Wd, 2.0); mat(f"{k}.mlp.{n}.down", Wd, ff, 2.0)
    vec("final.norm", Wd, 1.0)
    mat("head", cfg["vocab"], Wd)
    return out
