"""Plain float64 restatement of the Negilorn layer stack (chunked attention with shared keys / values and decaying linear attention
behind token-shifted pre-norm residual steps, dense and sparse feed-forwards) -- TEST INFRASTRUCTURE ONLY.

One function per mechanism, token by token, written from the equations; nothing is shared with the product path (no pages, no
slots, no batching: a sequence's memory is python lists and per-layer arrays).

Notation: W x with W stored [out, in]; p = a token's position (from 0); n(v) = v / sqrt(mean(v^2) + eps).
    layer:   a = n(x) g1 (g1 one number);  h = a + (a' - a) * shift, a' = the previous token's a (zeros at p = 0);
             x <- x + mixer(h);   x <- x + ff(n(x) g2)   (absent when the layer has no feed-forward)
    attention (H query heads over G key / value heads, no biases):
             q, k: the first `dims` values of a head in pairs (i, i + dims / 2) turned by p f_i; f_i = base^(-2i / dims), rescaled by
             wavelength l = 2 pi / f: kept where l < original / high, divided by `factor` where l > original / low, blended linearly in
             original / l between the two
             p sees j <= p with floor(j / size) == floor(p / size);  s_j = softcap tanh(q . k_j scale / softcap)
             weights exp(s_j) / (1 + sum exp(s));  head output times sigmoid(W_g h)[head];  out = W_o heads
             kv_from = j: keys and values are those layer j made for the same tokens
    wkv (H heads of D key and D value channels):
             b = the previous token's h (zeros at p = 0);  x_s = h + (b - h) * mu_s for s in r, k, v, g, w
             r, k, v = W_r x_r, W_k x_k, W_v x_v;  gate = silu(W_g x_g);  w = exp(-exp(W_w2 tanh(W_w1 x_w) + w0))
             head i: o = (S + diag(u) k v^T)^T r;  S <- diag(w) S + k v^T;   out = W_o (n_per_head(o) * norm * gate)
    ff:      dense  W_down (silu(W_gate h) * W_up h)
             moe    s = sigmoid(W_router h); the `top` largest s choose experts; y = sum_e E_e(s_e h) + E_shared(h),
                    E(z) = W_down relu(W_up z)^2
    logits:  head (n(x) g_final) * logit_scale
"""
from __future__ import annotations

import math

import numpy as np


def scalar_rms_norm(v, gain, eps):
    return v / math.sqrt(float(np.mean(v * v)) + eps) * float(gain)


def token_shift(a, a_prev, shift):
    return a + (a_prev - a) * shift


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def rotary_frequencies(rot):
    dims = rot["dims"]
    out = []
    for i in range(dims // 2):
        f = rot["base"] ** (-2.0 * i / dims)
        sc = rot.get("scaling")
        if sc:
            wavelength = 2.0 * math.pi / f
            if wavelength > sc["original"] / sc["low"]:
                f = f / sc["factor"]
            elif not wavelength < sc["original"] / sc["high"]:
                s = (sc["original"] / wavelength - sc["low"]) / (sc["high"] - sc["low"])
                f = (1.0 - s) * f / sc["factor"] + s * f
        out.append(f)
    return np.array(out)


def turn_head(vec, pos, freqs, dims):
    """one head's vector: value i and value i + dims / 2 form a pair, the values past `dims` pass unchanged"""
    out = vec.copy()
    half = dims // 2
    for i in range(half):
        a = pos * freqs[i]
        u, v = vec[i], vec[i + half]
        out[i] = u * math.cos(a) - v * math.sin(a)
        out[i + half] = v * math.cos(a) + u * math.sin(a)
    return out


def attention_kv(W, key, m, h, pos):
    """(keys [G, dim] turned, values [G, vdim]) of one token"""
    G, dim, vd = m["kv_heads"], m["dim"], m["vdim"]
    fr = rotary_frequencies(m["rot"])
    k = (W[key + ".mix.k"] @ h).reshape(G, dim)
    v = (W[key + ".mix.v"] @ h).reshape(G, vd)
    return np.stack([turn_head(k[g], pos, fr, m["rot"]["dims"]) for g in range(G)]), v


def chunk_visible(pos, size):
    """positions that position `pos` sees"""
    return [j for j in range(pos + 1) if j // size == pos // size]


def attention_token(W, key, m, h, pos, kv):
    """kv: list over the sequence's tokens of (keys, values) as attention_kv made them (this layer's or the shared layer's)"""
    H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    fr = rotary_frequencies(m["rot"])
    q = (W[key + ".mix.q"] @ h).reshape(H, dim)
    gate = sigmoid(W[key + ".mix.g"] @ h)
    seen = chunk_visible(pos, m["mask"]["size"])
    heads = np.zeros((H, vd))
    for i in range(H):
        g = i // (H // G)
        qi = turn_head(q[i], pos, fr, m["rot"]["dims"])
        s = np.array([float(qi @ kv[j][0][g]) * m["scale"] for j in seen])
        cap = m.get("softcap")
        if cap:
            s = cap * np.tanh(s / cap)
        e = np.exp(s)
        wts = e / (1.0 + e.sum())
        for w, j in zip(wts, seen):
            heads[i] += w * kv[j][1][g]
        heads[i] *= gate[i]
    return W[key + ".mix.o"] @ heads.reshape(-1)


def wkv_token(W, key, m, h, mem, eps):
    """mem: {"b": the previous token's h, "S": [heads, D, D]} -- updated in place"""
    H, D = m["heads"], m["dim"]
    b = mem["b"]
    mem["b"] = h.copy()
    blend = {s: h + (b - h) * W[key + ".mix.mu." + s] for s in "rkvgw"}
    r = (W[key + ".mix.r"] @ blend["r"]).reshape(H, D)
    k = (W[key + ".mix.k"] @ blend["k"]).reshape(H, D)
    v = (W[key + ".mix.v"] @ blend["v"]).reshape(H, D)
    gate = silu(W[key + ".mix.g"] @ blend["g"])
    w = np.exp(-np.exp(W[key + ".mix.w2"] @ np.tanh(W[key + ".mix.w1"] @ blend["w"]) + W[key + ".mix.w0"])).reshape(H, D)
    u = W[key + ".mix.u"]
    out = np.zeros((H, D))
    for i in range(H):
        S = mem["S"][i]
        o = np.zeros(D)
        for c in range(D):                                   # key channel c
            o += r[i][c] * (S[c] + u[i][c] * k[i][c] * v[i])
            S[c] = w[i][c] * S[c] + k[i][c] * v[i]
        out[i] = o / math.sqrt(float(np.mean(o * o)) + eps)
    return W[key + ".mix.o"] @ (out.reshape(-1) * W[key + ".mix.norm"] * gate)


def gated_ff(W, key, h):
    return W[key + ".mlp.down"] @ (silu(W[key + ".mlp.gate"] @ h) * (W[key + ".mlp.up"] @ h))


def relu2_expert(W, key, z):
    return W[key + ".down"] @ np.maximum(W[key + ".up"] @ z, 0.0) ** 2


def route(W, key, ms, h):
    """[(expert, weight)] of one token, best first (the lower index on a tie)"""
    s = sigmoid(W[key + ".mlp.router"] @ h)
    order = sorted(range(len(s)), key=lambda e: (-s[e], e))
    return [(e, float(s[e])) for e in order[:ms["router"]["top"]]]


def route_gap(W, key, ms, h):
    """the distance between the last chosen score and the first one not chosen (inf when every expert is chosen)"""
    s = np.sort(sigmoid(W[key + ".mlp.router"] @ h))[::-1]
    top = ms["router"]["top"]
    return float(s[top - 1] - s[top]) if top < len(s) else math.inf


def moe_ff(W, key, ms, h):
    y = np.zeros(W[key + ".mlp.e0.down"].shape[0])
    for e, w in route(W, key, ms, h):
        y += relu2_expert(W, f"{key}.mlp.e{e}", w * h)
    if ms.get("shared"):
        y += relu2_expert(W, key + ".mlp.shared", h)
    return y


class Oracle:
    """feed(seq, tokens) -> logits [len(tokens), vocab] of the sequence's next tokens; state is kept per sequence name"""

    def __init__(self, cfg: dict, weights: dict):
        self.cfg = cfg
        self.W = {k: np.asarray(v, dtype=np.float64) for k, v in weights.items()}
        self.seqs = {}

    def _new(self):
        Wd = self.cfg["width"]
        mem = []
        for spec in self.cfg["layers"]:
            m = spec["mixer"]
            st = {"a": np.zeros(Wd)}
            if spec["type"] == "wkv":
                st.update(b=np.zeros(Wd), S=np.zeros((m["heads"], m["dim"], m["dim"])))
            else:
                st["kv"] = []
            mem.append(st)
        return {"n": 0, "mem": mem}

    def feed(self, seq, tokens, residuals=None, gaps=None):
        """residuals (a list): takes the stream after every layer per token; gaps (a list): takes every token's smallest router gap"""
        cfg, W, eps = self.cfg, self.W, self.cfg["norm"]["eps"]
        st = self.seqs.setdefault(seq, None) or self._new()
        self.seqs[seq] = st
        out = []
        for t in tokens:
            pos = st["n"]
            x = W["embed"][int(t)].copy()
            trail, gap = [], math.inf
            for i, spec in enumerate(cfg["layers"]):
                key, m, mem = f"l{i}", spec["mixer"], st["mem"][i]
                a = scalar_rms_norm(x, W[key + ".norm1"], eps)
                h = token_shift(a, mem["a"], W[key + ".shift"])
                mem["a"] = a
                if spec["type"] == "wkv":
                    x = x + wkv_token(W, key, m, h, mem, eps)
                elif spec["type"] == "attention":
                    if m.get("kv_from") is None:
                        mem["kv"].append(attention_kv(W, key, m, h, pos))
                        kv = mem["kv"]
                    else:
                        kv = st["mem"][m["kv_from"]]["kv"]
                    x = x + attention_token(W, key, m, h, pos, kv)
                else:
                    raise ValueError(spec["type"])
                ms = spec.get("mlp")
                if ms is not None:
                    h2 = scalar_rms_norm(x, W[key + ".norm2"], eps)
                    if ms["kind"] == "moe":
                        gap = min(gap, route_gap(W, key, ms, h2))
                    x = x + (gated_ff(W, key, h2) if ms["kind"] == "dense" else moe_ff(W, key, ms, h2))
                trail.append(x.copy())
            if residuals is not None:
                residuals.append(np.stack(trail))
            if gaps is not None:
                gaps.append(gap)
            out.append(W["head"] @ scalar_rms_norm(x, W["final.norm"], eps) * cfg.get("logit_scale", 1.0))
            st["n"] += 1
        return np.stack(out)

    def drop(self, seq):
        self.seqs.pop(seq, None)


# ---- small random models for the tests ---------------------------------------------------------------------------------------


def bf16_round(a):
    u = np.asarray(a, dtype=np.float32).view(np.uint32)
    return (((u + 0x7fff + ((u >> 16) & 1)) & 0xffff0000).astype(np.uint32)).view(np.float32)


def attn_mixer(heads=4, kv_heads=2, dim=16, vdim=8, size=6, dims=None, base=10000.0, scaling="default", scale=None, softcap=20.0,
               kv_from=None):
    dims = dim if dims is None else dims
    if scaling == "default":
        scaling = {"factor": 8.0, "original": 64, "low": 1.0, "high": 4.0}
    m = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "mask": {"size": size}, "rot": {"base": base, "dims": dims, "scaling": scaling},
         "scale": scale if scale is not None else dim ** -0.5, "softcap": softcap, "vdim": vdim}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def wkv_mixer(heads=3, dim=8, rank=5):
    return {"type": "wkv", "mixer": {"dim": dim, "heads": heads}, "_rank": rank}


def dense_ff(ff=24):
    return {"ff": ff, "kind": "dense"}


def moe_ff_spec(experts=5, top=2, ff=12, shared=10):
    ms = {"expert": {"ff": ff}, "kind": "moe", "router": {"experts": experts, "top": top}}
    if shared:
        ms["shared"] = {"ff": shared}
    return ms


def layer(mix, ff=None):
    return dict(mix, mlp=ff)


def small_config(layers, width=32, vocab=61, eps=1e-5, logit_scale=0.5):
    return {"architecture": "Negilorn", "layers": layers, "logit_scale": logit_scale, "norm": {"eps": eps}, "vocab": vocab, "width": width}


def random_model(cfg: dict, seed: int = 0) -> dict:
    """name -> float32 array (bfloat16-representable values), shapes from the configuration"""
    rng = np.random.default_rng(seed)
    Wd, out = cfg["width"], {}

    def mat(name, o, i, gain=1.0):
        out[name] = bf16_round(rng.standard_normal((o, i)) * gain / math.sqrt(i))

    def vec(name, n, centre=0.0, spread=0.1):
        out[name] = bf16_round(centre + rng.standard_normal(n) * spread)

    def scalar(name):
        out[name] = bf16_round(np.array(rng.uniform(0.7, 1.4))).reshape(())

    out["embed"] = bf16_round(rng.standard_normal((cfg["vocab"], Wd)))
    for i, spec in enumerate(cfg["layers"]):
        k, m = f"l{i}", spec["mixer"]
        scalar(k + ".norm1")
        out[k + ".shift"] = bf16_round(rng.uniform(0.0, 1.0, size=Wd))
        if spec["type"] == "wkv":
            H, D, rank = m["heads"], m["dim"], spec.get("_rank", 4)
            for s in "rkvgw":
                out[f"{k}.mix.mu.{s}"] = bf16_round(rng.uniform(0.0, 1.0, size=Wd))
            for s in "rkvg":
                mat(f"{k}.mix.{s}", H * D, Wd)
            mat(k + ".mix.w1", rank, Wd); mat(k + ".mix.w2", H * D, rank)
            vec(k + ".mix.w0", H * D, -1.5, 1.0)
            out[k + ".mix.u"] = bf16_round(rng.standard_normal((H, D)) * 0.5)
            vec(k + ".mix.norm", H * D, 1.0)
            mat(k + ".mix.o", Wd, H * D)
        else:
            H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            mat(k + ".mix.q", H * dim, Wd, 2.0)
            if m.get("kv_from") is None:
                mat(k + ".mix.k", G * dim, Wd, 2.0); mat(k + ".mix.v", G * vd, Wd)
            mat(k + ".mix.g", H, Wd); mat(k + ".mix.o", Wd, H * vd)
        ms = spec.get("mlp")
        if ms is not None:
            scalar(k + ".norm2")
            if ms["kind"] == "dense":
                mat(k + ".mlp.gate", ms["ff"], Wd); mat(k + ".mlp.up", ms["ff"], Wd); mat(k + ".mlp.down", Wd, ms["ff"])
            else:
                mat(k + ".mlp.router", ms["router"]["experts"], Wd, 2.0)
                for e in range(ms["router"]["experts"]):
                    mat(f"{k}.mlp.e{e}.up", ms["expert"]["ff"], Wd); mat(f"{k}.mlp.e{e}.down", Wd, ms["expert"]["ff"])
                if ms.get("shared"):
                    mat(k + ".mlp.shared.up", ms["shared"]["ff"], Wd); mat(k + ".mlp.shared.down", Wd, ms["shared"]["ff"])
    scalar("final.norm")
    mat("head", cfg["vocab"], Wd)
    return out


def clean_config(cfg: dict) -> dict:
    """the configuration without the generator's private keys (what goes into a config.json)"""
    layers = [{k: v for k, v in spec.items() if not k.startswith("_")} for spec in cfg["layers"]]
    return dict(cfg, layers=layers)
