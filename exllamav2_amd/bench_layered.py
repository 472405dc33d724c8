"""Prefill and decode throughput of the layer-stack models at layer sizes of real models (random weights), each beside the closest
other model of the package at equal size: the latent-attention / scored-MoE stack beside a Mixtral-style EXL2 stack (same width,
expert width, expert count, depth), the state-space / windowed-attention stack beside a latent-attention stack (same width, depth,
heads, window, feed-forward parameters), the token-shifted chunked-attention / linear-attention stack beside a state-space /
windowed-attention stack (same width, depth, heads, reach, streamed feed-forward parameters).  Used by
`bench.py --design benolix | tibalorn | negilorn`; one JSON object per size and model."""
from __future__ import annotations

import json
import time

import torch

SIZES = {
    # width, heads, dim, rot, vdim, kv_rank, q_rank, window, experts, identity, top, expert ff, dense ff, layers, vocab
    "w2048": dict(width=2048, heads=16, dim=128, rot=64, vdim=128, kv_rank=512, q_rank=768, window=1024, experts=8, identity=2, top=2,
                  ff=5632, dense_ff=5632, layers=4, vocab=32000),
    "w4096": dict(width=4096, heads=32, dim=128, rot=64, vdim=128, kv_rank=512, q_rank=1536, window=2048, experts=8, identity=2, top=2,
                  ff=14336, dense_ff=14336, layers=2, vocab=32000),
}


def layered_config(s: dict) -> dict:
    def mixer(kv_from=None):
        m = {"dim": s["dim"], "heads": s["heads"], "kv_rank": s["kv_rank"], "mask": {"size": s["window"]}, "q_rank": s["q_rank"],
             "rot": {"base": 10000.0, "dims": s["rot"]}, "rot_dim": s["rot"], "scale": (s["dim"] + s["rot"]) ** -0.5, "vdim": s["vdim"]}
        if kv_from is not None:
            m["kv_from"] = kv_from
        return m
    moe = {"expert": {"ff": s["ff"], "limit": 7.0}, "kind": "moe",
           "router": {"experts": s["experts"], "identity": s["identity"], "scale": 1.0, "top": s["top"]}}
    layers = []
    for i in range(s["layers"]):
        layers.append({"type": "latent_attention", "mixer": mixer(None if i % 2 == 0 else i - 1),
                       "mlp": {"ff": s["dense_ff"], "kind": "dense"} if i == 0 else moe})
    return {"architecture": "Benolix", "embedding": {"scale": 1.0}, "layers": layers, "norm": {"eps": 1e-5}, "postln_alpha": 1.0,
            "vocab": s["vocab"], "width": s["width"]}


def random_tensors(cfg: dict, device, seed: int = 0) -> dict:
    g = torch.Generator(device=device).manual_seed(seed)
    T = {}

    def mat(name, out, inp):
        T[name] = (torch.randn((out, inp), device=device, generator=g) / inp ** 0.5).to(torch.bfloat16)

    def vec(name, n, centre):
        T[name] = (centre + 0.1 * torch.randn((n,), device=device, generator=g)).to(torch.bfloat16)

    w = cfg["width"]
    mat("embed", cfg["vocab"], 1); mat("head", cfg["vocab"], w); vec("final.norm", w, 0.0)
    T["embed"] = (torch.randn((cfg["vocab"], w), device=device, generator=g)).to(torch.bfloat16)
    for i, L in enumerate(cfg["layers"]):
        m, k = L["mixer"], f"l{i}"
        H, dim, rd, vd, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        vec(k + ".norm1", w, 0.0); vec(k + ".norm2", w, 0.0)
        mat(k + ".mix.dq", Q, w); vec(k + ".mix.dq.norm", Q, 1.0); mat(k + ".mix.uq", H * (dim + rd), Q)
        if "kv_from" not in m:
            mat(k + ".mix.dkv", R + rd, w); vec(k + ".mix.dkv.norm", R, 1.0)
        mat(k + ".mix.uk", H * dim, R); mat(k + ".mix.uv", H * vd, R); mat(k + ".mix.g", H * vd, w); mat(k + ".mix.o", w, H * vd)
        ms = L["mlp"]
        if ms is None:
            continue
        if ms["kind"] == "dense":
            mat(k + ".mlp.gate", ms["ff"], w); mat(k + ".mlp.up", ms["ff"], w); mat(k + ".mlp.down", w, ms["ff"])
        else:
            r = ms["router"]
            for e in range(r["experts"]):
                mat(f"{k}.mlp.e{e}.gate", ms["expert"]["ff"], w); mat(f"{k}.mlp.e{e}.up", ms["expert"]["ff"], w)
                mat(f"{k}.mlp.e{e}.down", w, ms["expert"]["ff"])
            mat(k + ".mlp.router", r["experts"] + r["identity"], w)
            T[k + ".mlp.correction"] = torch.zeros((r["experts"] + r["identity"],), device=device, dtype=torch.bfloat16)
    return T


def _timed(fn, reps: int):
    """seconds per call; the interpreter's cyclic collector is held off while the clock runs (a full collection of a process that has
    imported torch takes tens of milliseconds and would land in one of a few repetitions)"""
    import gc
    gc.collect()
    gc.disable()
    try:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps
    finally:
        gc.enable()


def bench_layered(size: str, device="cuda:0", prompt: int = 2048, ctx: int = 1024, decode_steps: int = 64, batches=(1, 4)) -> dict:
    from .config import LayeredConfig
    from .engine import Engine
    from .layered import LayeredModel
    s = SIZES[size]
    cfg = layered_config(s)
    model = LayeredModel(LayeredConfig.from_dict(cfg), device=device, dtype=torch.bfloat16).load(random_tensors(cfg, device))
    out = {"design": "benolix", "size": size, "layers": s["layers"], "weight_bytes_per_token": model.weight_bytes()}
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, s["vocab"], (prompt,), generator=g).tolist()
    eng = Engine(model, max_tokens=max(prompt, max(batches) * (ctx + decode_steps + 8)) + 256, max_seqs=max(4, max(batches)))
    eng.step([("warm", toks, [prompt - 1])], ["warm"])
    dt = _timed(lambda: eng.step([("p", toks, [prompt - 1])], ["p"]), 3)
    out["prefill_tokens_per_s"] = prompt / dt
    out["prefill_ms"] = dt * 1e3
    for b in batches:
        ids = [f"d{i}" for i in range(b)]
        eng.step([(r, toks[:ctx], []) for r in ids])
        step = lambda: eng.step([(r, [7], [0]) for r in ids])
        step()
        dt = _timed(step, decode_steps)
        out[f"decode_b{b}_tokens_per_s"] = b / dt
        out[f"decode_b{b}_ms_per_step"] = dt * 1e3
        for r in ids:
            eng.finish(r)
    return out


def bench_quantized_peer(size: str, device="cuda:0", prompt: int = 2048, ctx: int = 1024, decode_steps: int = 64, batches=(1, 4)) -> dict:
    """the package's Mixtral-style EXL2 stack (4.0 bpw) with the same width, expert width / count / top-k, depth and vocabulary"""
    from . import ExLlamaV2, ExLlamaV2Cache, ExLlamaV2Config, GreedyGraphDecoder
    from .synth import synth_checkpoint
    s = SIZES[size]
    out = {"design": "mixtral-exl2-4.0bpw", "size": size, "layers": s["layers"]}
    for b in batches:
        cfg = ExLlamaV2Config(hidden_size=s["width"], intermediate_size=s["ff"], num_hidden_layers=s["layers"],
                              num_attention_heads=s["heads"], num_key_value_heads=max(1, s["heads"] // 4), head_dim=128,
                              vocab_size=s["vocab"], max_seq_len=4096, max_input_len=prompt, max_batch_size=1,
                              num_experts=s["experts"], num_experts_per_token=s["top"], arch="mixtral")
        ck = synth_checkpoint(cfg, device, recipe="4.0bpw", seed=0)
        model = ExLlamaV2(cfg, device=device).load(ck)
        g = torch.Generator().manual_seed(1)
        ids = torch.randint(0, s["vocab"], (1, prompt), generator=g)
        if b == batches[0]:
            cache = ExLlamaV2Cache(model, batch_size=1)
            model.forward(ids, cache)
            def pre():
                cache.current_seq_len = 0
                model.forward(ids, cache)
            dt = _timed(pre, 3)
            out["prefill_tokens_per_s"] = prompt / dt
            out["prefill_ms"] = dt * 1e3
            out["weight_bytes_per_token"] = model.weight_bytes()
            del cache
        cache = ExLlamaV2Cache(model, batch_size=b)
        dec = GreedyGraphDecoder(model, cache, batch_size=b).capture()
        dec.reset(torch.zeros((b,), dtype=torch.int32), ctx)
        dec.run(8)
        dec.reset(torch.zeros((b,), dtype=torch.int32), ctx)
        dt = _timed(lambda: dec.run(1), decode_steps)
        out[f"decode_b{b}_tokens_per_s"] = b / dt
        out[f"decode_b{b}_ms_per_step"] = dt * 1e3
        dec.free(); model.unload()
        del dec, cache, model, ck
        torch.cuda.empty_cache()
    return out


# ---- pre-norm stacks of state-space and windowed-attention mixers (Tibalorn) -----------------------------------------------------

HYBRID_SIZES = {
    # a 3 : 1 pattern of state-space and attention layers; state-space inner width = 2 x width in heads of 64, state 128; attention
    # with grouped heads of 128, a window of 1024 and pooled blocks of 64 behind it; squared-relu feed-forward behind the attention
    "w2048": dict(width=2048, ssm_heads=64, ssm_vdim=64, state=128, groups=1, norm_groups=1, taps=4, heads=16, kv_heads=4, dim=128,
                  vdim=128, window=1024, pool=64, rot_dims=64, ff=8192, pattern="ssa+s", vocab=32000),
    "w4096": dict(width=4096, ssm_heads=128, ssm_vdim=64, state=128, groups=8, norm_groups=8, taps=4, heads=32, kv_heads=8, dim=128,
                  vdim=128, window=2048, pool=64, rot_dims=128, ff=14336, pattern="sa+", vocab=32000),
}


def hybrid_config(s: dict) -> dict:
    """pattern: s = state-space layer, a = attention layer, + = the layer before it has a feed-forward"""
    layers = []
    for ch in s["pattern"]:
        if ch == "+":
            layers[-1]["mlp"] = {"ff": s["ff"], "kind": "dense"}
        elif ch == "s":
            layers.append({"type": "mamba2", "mlp": None,
                           "mixer": {"conv": s["taps"], "groups": s["groups"], "heads": s["ssm_heads"], "norm_groups": s["norm_groups"],
                                     "state": s["state"], "vdim": s["ssm_vdim"]}})
        else:
            layers.append({"type": "attention", "mlp": None,
                           "mixer": {"dim": s["dim"], "heads": s["heads"], "kv_heads": s["kv_heads"], "vdim": s["vdim"],
                                     "mask": {"pool": s["pool"], "size": s["window"]}, "scale": s["dim"] ** -0.5,
                                     "rot": {"base": 500000.0, "dims": s["rot_dims"],
                                             "scaling": {"factor": 8.0, "original": 8192, "fast": 32.0, "slow": 1.0}}}})
    return {"architecture": "Tibalorn", "embedding": {"scale": 1.0}, "layers": layers, "logit_softcap": 30.0, "norm": {"eps": 1e-5},
            "vocab": s["vocab"], "width": s["width"]}


def hybrid_random_tensors(cfg: dict, device, seed: int = 0) -> dict:
    g = torch.Generator(device=device).manual_seed(seed)
    T = {}

    def mat(name, out, inp, gain=1.0):
        T[name] = (torch.randn((out, inp), device=device, generator=g) * gain / inp ** 0.5).to(torch.bfloat16)

    def vec(name, n, centre, spread=0.1):
        T[name] = (centre + spread * torch.randn((n,), device=device, generator=g)).to(torch.bfloat16)

    w = cfg["width"]
    T["embed"] = (torch.randn((cfg["vocab"], w), device=device, generator=g) * 0.5).to(torch.bfloat16)
    vec("final.norm", w, 1.0); vec("final.norm.b", w, 0.0)
    for i, L in enumerate(cfg["layers"]):
        m, k = L["mixer"], f"l{i}"
        vec(k + ".norm1", w, 1.0); vec(k + ".norm1.b", w, 0.0)
        if L["type"] == "mamba2":
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            mat(k + ".mix.in", 2 * inner + 2 * gn + m["heads"], w); mat(k + ".mix.conv", inner + 2 * gn, m["conv"])
            vec(k + ".mix.conv.b", inner + 2 * gn, 0.0); vec(k + ".mix.dt_bias", m["heads"], -1.0, 0.5); vec(k + ".mix.A_log", m["heads"], 0.0, 0.5)
            vec(k + ".mix.D", m["heads"], 1.0); vec(k + ".mix.norm", inner, 1.0); mat(k + ".mix.o", w, inner)
        else:
            H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            mat(k + ".mix.q", H * dim, w); mat(k + ".mix.k", G * dim, w); mat(k + ".mix.v", G * vd, w); mat(k + ".mix.g", H * vd, w)
            vec(k + ".mix.q.b", H * dim, 0.0); vec(k + ".mix.k.b", G * dim, 0.0); vec(k + ".mix.v.b", G * vd, 0.0)
            vec(k + ".mix.temp", H, 1.0); vec(k + ".mix.sink", H, 0.0, 1.0); mat(k + ".mix.o", w, H * vd)
        if L["mlp"] is not None:
            vec(k + ".norm2", w, 1.0); vec(k + ".norm2.b", w, 0.0)
            mat(k + ".mlp.up", L["mlp"]["ff"], w); mat(k + ".mlp.down", w, L["mlp"]["ff"])
    return T


def _bench_engine(model, out, vocab, prompt, ctx, decode_steps, batches):
    from .engine import Engine
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, vocab, (prompt,), generator=g).tolist()
    eng = Engine(model, max_tokens=max(prompt, max(batches) * (ctx + decode_steps + 8)) + 256, max_seqs=max(4, max(batches)))
    eng.step([("warm", toks, [prompt - 1])], ["warm"])
    dt = _timed(lambda: eng.step([("p", toks, [prompt - 1])], ["p"]), 3)
    out["prefill_tokens_per_s"] = prompt / dt
    out["prefill_ms"] = dt * 1e3
    for b in batches:
        ids = [f"d{i}" for i in range(b)]
        eng.step([(r, toks[:ctx], []) for r in ids])
        step = lambda: eng.step([(r, [7], [0]) for r in ids])
        step()
        dt = _timed(step, decode_steps)
        out[f"decode_b{b}_tokens_per_s"] = b / dt
        out[f"decode_b{b}_ms_per_step"] = dt * 1e3
        for r in ids:
            eng.finish(r)
    eng.close()
    return out


def bench_hybrid(size: str, device="cuda:0", prompt: int = 2048, ctx: int = 1024, decode_steps: int = 64, batches=(1, 4)) -> dict:
    from .config import LayeredConfig
    from .layered import LayeredModel
    s = HYBRID_SIZES[size]
    cfg = hybrid_config(s)
    model = LayeredModel(LayeredConfig.from_dict_prenorm(cfg), device=device, dtype=torch.bfloat16).load(hybrid_random_tensors(cfg, device))
    out = {"design": "tibalorn", "size": size, "layers": len(cfg["layers"]), "pattern": s["pattern"], "weight_bytes_per_token": model.weight_bytes()}
    return _bench_engine(model, out, s["vocab"], prompt, ctx, decode_steps, batches)


def bench_hybrid_peer(size: str, device="cuda:0", prompt: int = 2048, ctx: int = 1024, decode_steps: int = 64, batches=(1, 4)) -> dict:
    """the closest model of the package: a latent-attention stack (bfloat16, the same engine) of the same width, depth, head count,
    window and vocabulary, with dense feed-forwards of the same width behind the same layers"""
    from .config import LayeredConfig
    from .layered import LayeredModel
    s = HYBRID_SIZES[size]
    hyb = hybrid_config(s)
    layers = []
    for L in hyb["layers"]:
        mixer = {"dim": s["dim"], "heads": s["heads"], "kv_rank": 512, "mask": {"size": s["window"]}, "q_rank": s["width"] * 3 // 8,
                 "rot": {"base": 10000.0, "dims": 64}, "rot_dim": 64, "scale": (s["dim"] + 64) ** -0.5, "vdim": s["vdim"]}
        layers.append({"type": "latent_attention", "mixer": mixer,
                       "mlp": {"ff": s["ff"] * 2 // 3 // 64 * 64, "kind": "dense"} if L["mlp"] is not None else None})
    cfg = {"architecture": "Benolix", "embedding": {"scale": 1.0}, "layers": layers, "norm": {"eps": 1e-5}, "postln_alpha": 1.0,
           "vocab": s["vocab"], "width": s["width"]}
    model = LayeredModel(LayeredConfig.from_dict(cfg), device=device, dtype=torch.bfloat16).load(random_tensors(cfg, device))
    out = {"design": "benolix-dense-peer", "size": size, "layers": len(layers), "weight_bytes_per_token": model.weight_bytes()}
    return _bench_engine(model, out, s["vocab"], prompt, ctx, decode_steps, batches)


SHIFT_SIZES = {
    # pattern: a = chunked attention, k = the same reading the keys / values of the attention layer before it, w = decaying linear
    # attention; d / m = the layer before has a dense / sparse feed-forward
    "w2048": dict(width=2048, heads=16, kv_heads=4, dim=128, vdim=128, chunk=1024, rot_dims=64, wkv_heads=32, wkv_dim=64, rank=64,
                  ff=5632, experts=8, top=2, expert_ff=2816, shared_ff=2816, pattern="adwmkdwm", vocab=32000),
    "w4096": dict(width=4096, heads=32, kv_heads=8, dim=128, vdim=128, chunk=2048, rot_dims=128, wkv_heads=64, wkv_dim=64, rank=128,
                  ff=14336, experts=8, top=2, expert_ff=7168, shared_ff=7168, pattern="adwm", vocab=32000),
}


def shift_config(s: dict) -> dict:
    layers, last_attn = [], None
    for ch in s["pattern"]:
        if ch == "d":
            layers[-1]["mlp"] = {"ff": s["ff"], "kind": "dense"}
        elif ch == "m":
            layers[-1]["mlp"] = {"expert": {"ff": s["expert_ff"]}, "kind": "moe", "router": {"experts": s["experts"], "top": s["top"]},
                                 "shared": {"ff": s["shared_ff"]}}
        elif ch == "w":
            layers.append({"type": "wkv", "mlp": None, "mixer": {"dim": s["wkv_dim"], "heads": s["wkv_heads"]}})
        else:
            m = {"dim": s["dim"], "heads": s["heads"], "kv_heads": s["kv_heads"], "vdim": s["vdim"], "mask": {"size": s["chunk"]},
                 "scale": s["dim"] ** -0.5, "softcap": 30.0,
                 "rot": {"base": 500000.0, "dims": s["rot_dims"], "scaling": {"factor": 8.0, "original": 8192, "low": 1.0, "high": 4.0}}}
            if ch == "k":
                m["kv_from"] = last_attn
            else:
                last_attn = len(layers)
            layers.append({"type": "attention", "mlp": None, "mixer": m})
    return {"architecture": "Negilorn", "layers": layers, "logit_scale": 0.5, "norm": {"eps": 1e-5}, "vocab": s["vocab"], "width": s["width"]}


def shift_random_tensors(cfg: dict, s: dict, device, seed: int = 0) -> dict:
    g = torch.Generator(device=device).manual_seed(seed)
    T = {}

    def mat(name, out, inp, gain=1.0):
        T[name] = (torch.randn((out, inp), device=device, generator=g) * gain / inp ** 0.5).to(torch.bfloat16)

    def vec(name, n, centre, spread=0.1):
        T[name] = (centre + spread * torch.randn((n,), device=device, generator=g)).to(torch.bfloat16)

    def one(name):
        T[name] = torch.ones((), device=device, dtype=torch.bfloat16)

    w = cfg["width"]
    T["embed"] = (torch.randn((cfg["vocab"], w), device=device, generator=g) * 0.5).to(torch.bfloat16)
    mat("head", cfg["vocab"], w); one("final.norm")
    for i, L in enumerate(cfg["layers"]):
        m, k = L["mixer"], f"l{i}"
        one(k + ".norm1"); vec(k + ".shift", w, 0.3)
        if L["type"] == "wkv":
            inner = m["heads"] * m["dim"]
            for n in "rkvgw":
                vec(f"{k}.mix.mu.{n}", w, 0.5)
            for n in "rkvg":
                mat(f"{k}.mix.{n}", inner, w)
            mat(k + ".mix.w1", s["rank"], w); mat(k + ".mix.w2", inner, s["rank"]); vec(k + ".mix.w0", inner, -1.0, 0.5)
            T[k + ".mix.u"] = (0.3 * torch.randn((m["heads"], m["dim"]), device=device, generator=g)).to(torch.bfloat16)
            vec(k + ".mix.norm", inner, 1.0); mat(k + ".mix.o", w, inner)
        else:
            H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            mat(k + ".mix.q", H * dim, w)
            if "kv_from" not in m:
                mat(k + ".mix.k", G * dim, w); mat(k + ".mix.v", G * vd, w)
            mat(k + ".mix.g", H, w); mat(k + ".mix.o", w, H * vd)
        ms = L["mlp"]
        if ms is not None:
            one(k + ".norm2")
            if ms["kind"] == "dense":
                mat(k + ".mlp.gate", ms["ff"], w); mat(k + ".mlp.up", ms["ff"], w); mat(k + ".mlp.down", w, ms["ff"])
            else:
                mat(k + ".mlp.router", ms["router"]["experts"], w)
                for e in range(ms["router"]["experts"]):
                    mat(f"{k}.mlp.e{e}.up", ms["expert"]["ff"], w); mat(f"{k}.mlp.e{e}.down", w, ms["expert"]["ff"])
                mat(k + ".mlp.shared.up", ms["shared"]["ff"], w); mat(k + ".mlp.shared.down", w, ms["shared"]["ff"])
    return T


def bench_shift(size: str, device="cuda:0", prompt: int = 2048, ctx: int = 1024, decode_steps: int = 64, batches=(1, 4)) -> dict:
    from .config import LayeredConfig
    from .layered import LayeredModel
    s = SHIFT_SIZES[size]
    cfg = shift_config(s)
    model = LayeredModel(LayeredConfig.from_dict_prerms_shift(cfg), device=device, dtype=torch.bfloat16).load(shift_random_tensors(cfg, s, device))
    out = {"design": "negilorn", "size": size, "layers": len(cfg["layers"]), "pattern": s["pattern"], "weight_bytes_per_token": model.weight_bytes()}
    return _bench_engine(model, out, s["vocab"], prompt, ctx, decode_steps, batches)


def bench_shift_peer(size: str, device="cuda:0", prompt: int = 2048, ctx: int = 1024, decode_steps: int = 64, batches=(1, 4)) -> dict:
    """the closest model of the package: a state-space / windowed-attention stack (bfloat16, the same engine) of the same width and
    depth -- a state-space layer for every linear-attention layer (as many heads of the same size, state 128), a windowed
    attention layer of the same heads and reach for every chunked one, a two-matrix feed-forward with the parameters a token
    streams through behind the same layers"""
    from .config import LayeredConfig
    from .layered import LayeredModel
    s = SHIFT_SIZES[size]
    layers = []
    for L in shift_config(s)["layers"]:
        ms = L["mlp"]
        ff = None
        if ms is not None:
            ff = ms["ff"] * 3 // 2 if ms["kind"] == "dense" else s["expert_ff"] * s["top"] + s["shared_ff"]
        if L["type"] == "wkv":
            layers.append({"type": "mamba2", "mixer": {"conv": 4, "groups": 8, "heads": s["wkv_heads"], "norm_groups": 8, "state": 128,
                                                       "vdim": s["wkv_dim"]}, "mlp": {"ff": ff, "kind": "dense"} if ff else None})
        else:
            layers.append({"type": "attention", "mlp": {"ff": ff, "kind": "dense"} if ff else None,
                           "mixer": {"dim": s["dim"], "heads": s["heads"], "kv_heads": s["kv_heads"], "vdim": s["vdim"],
                                     "mask": {"pool": 64, "size": s["chunk"]}, "scale": s["dim"] ** -0.5,
                                     "rot": {"base": 500000.0, "dims": s["rot_dims"],
                                             "scaling": {"factor": 8.0, "original": 8192, "fast": 32.0, "slow": 1.0}}}})
    cfg = {"architecture": "Tibalorn", "embedding": {"scale": 1.0}, "layers": layers, "logit_softcap": 30.0, "norm": {"eps": 1e-5},
           "vocab": s["vocab"], "width": s["width"]}
    model = LayeredModel(LayeredConfig.from_dict_prenorm(cfg), device=device, dtype=torch.bfloat16).load(hybrid_random_tensors(cfg, device))
    out = {"design": "tibalorn-peer", "size": size, "layers": len(layers), "weight_bytes_per_token": model.weight_bytes()}
    return _bench_engine(model, out, s["vocab"], prompt, ctx, decode_steps, batches)


SANDWICH_SIZES = {
    # pattern: p = softmax attention beside a state-space scan, h = linear attention whose forget gate writes, d = gated delta rule;
    # every layer has a sparse feed-forward with a shared expert
    "w2048": dict(width=2048, heads=16, kv_heads=4, dim=128, vdim=128, ssm_heads=32, ssm_vdim=64, state=128, la_heads=16, la_kv_heads=8,
                  la_dim=128, la_vdim=128, experts=8, top=2, expert_ff=2816, shared_ff=2816, pattern="phdp", vocab=32000),
    "w4096": dict(width=4096, heads=32, kv_heads=8, dim=128, vdim=128, ssm_heads=64, ssm_vdim=64, state=128, la_heads=32, la_kv_heads=16,
                  la_dim=128, la_vdim=128, experts=8, top=2, expert_ff=7168, shared_ff=7168, pattern="phd", vocab=32000),
}


def sandwich_config(s: dict) -> dict:
    layers = []
    for ch in s["pattern"]:
        ff = {"expert": {"ff": s["expert_ff"]}, "kind": "moe", "router": {"experts": s["experts"], "top": s["top"]}, "shared": {"ff": s["shared_ff"]}}
        if ch == "p":
            m = {"left": {"dim": s["dim"], "heads": s["heads"], "kv_heads": s["kv_heads"], "vdim": s["vdim"], "scale": s["dim"] ** -0.5,
                          "rot": {"base": 500000.0, "dims": s["dim"]}}, "left_scale": 1.0,
                 "right": {"conv": 4, "groups": 1, "heads": s["ssm_heads"], "norm_groups": 1, "state": s["state"], "vdim": s["ssm_vdim"]},
                 "right_scale": 1.0}
            layers.append({"type": "parallel", "mixer": m, "mlp": ff})
        elif ch == "h":
            layers.append({"type": "hgrn2", "mixer": {"dim": s["la_dim"], "heads": s["la_heads"], "vdim": s["la_vdim"]}, "mlp": ff})
        else:
            layers.append({"type": "delta", "mixer": {"conv": 4, "dim": s["la_dim"], "heads": s["la_heads"], "kv_heads": s["la_kv_heads"],
                                                      "vdim": s["la_vdim"]}, "mlp": ff})
    return {"architecture": "Kilurax", "canon": {"taps": 4}, "embedding": {"bigram": {"buckets": 65521, "mul_cur": 11, "mul_prev": 131}, "scale": 1.0},
            "layers": layers, "norm": {"eps": 1e-5, "groups": 2}, "residual_mult": 0.7, "vocab": s["vocab"], "width": s["width"]}


def sandwich_random_tensors(cfg: dict, device, seed: int = 0) -> dict:
    g = torch.Generator(device=device).manual_seed(seed)
    T = {}

    def mat(name, out, inp, gain=1.0):
        T[name] = (torch.randn((out, inp), device=device, generator=g) * gain / inp ** 0.5).to(torch.bfloat16)

    def vec(name, n, centre, spread=0.1):
        T[name] = (centre + spread * torch.randn((n,), device=device, generator=g)).to(torch.bfloat16)

    w, taps = cfg["width"], cfg["canon"]["taps"]
    T["embed"] = (torch.randn((cfg["vocab"], w), device=device, generator=g) * 0.5).to(torch.bfloat16)
    T["bigram"] = (torch.randn((cfg["embedding"]["bigram"]["buckets"] + 1, w), device=device, generator=g) * 0.5).to(torch.bfloat16)
    vec("embed.norm", w, 1.0); vec("final.norm", w, 1.0); mat("head", cfg["vocab"], w)
    for i, L in enumerate(cfg["layers"]):
        m, k = L["mixer"], f"l{i}"
        for n in ("norm1", "norm1b", "norm2", "norm2b"):
            vec(f"{k}.{n}", w, 1.0)
        for n in ("canon1", "canon2"):
            T[f"{k}.{n}"] = (0.2 * torch.randn((w, taps), device=device, generator=g)).to(torch.bfloat16)
        if L["type"] == "parallel":
            a, r = m["left"], m["right"]
            H, G, dim, vd = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            mat(k + ".mix.left.q", H * dim, w); mat(k + ".mix.left.k", G * dim, w); mat(k + ".mix.left.v", G * vd, w); mat(k + ".mix.left.o", w, H * vd)
            vec(k + ".mix.left.q.b", H * dim, 0.0); vec(k + ".mix.left.k.b", G * dim, 0.0); vec(k + ".mix.left.v.b", G * vd, 0.0); vec(k + ".mix.left.o.b", w, 0.0)
            inner, gn = r["heads"] * r["vdim"], r["groups"] * r["state"]
            mat(k + ".mix.right.in", 2 * inner + 2 * gn + r["heads"], w)
            T[k + ".mix.right.conv"] = (0.5 * torch.randn((inner + 2 * gn, r["conv"]), device=device, generator=g)).to(torch.bfloat16)
            vec(k + ".mix.right.conv.b", inner + 2 * gn, 0.0); vec(k + ".mix.right.dt_bias", r["heads"], -1.0, 0.5)
            vec(k + ".mix.right.A_log", r["heads"], 0.0, 0.5); vec(k + ".mix.right.D", r["heads"], 1.0)
            vec(k + ".mix.right.norm", inner, 1.0); mat(k + ".mix.right.o", w, inner)
        elif L["type"] == "hgrn2":
            H, dim, vd = m["heads"], m["dim"], m["vdim"]
            mat(k + ".mix.q", H * dim, w); mat(k + ".mix.f", H * dim, w); mat(k + ".mix.v", H * vd, w); vec(k + ".mix.f.b", H * dim, 1.0, 1.0)
            T[k + ".mix.lower"] = (0.9 * torch.rand((H * dim,), device=device, generator=g)).to(torch.bfloat16)
            vec(k + ".mix.norm", vd, 1.0); mat(k + ".mix.o", w, H * vd)
        else:
            H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            mat(k + ".mix.q", G * dim, w); mat(k + ".mix.k", G * dim, w); mat(k + ".mix.v", H * vd, w)
            for n, c in (("q", G * dim), ("k", G * dim), ("v", H * vd)):
                T[f"{k}.mix.{n}.conv"] = (0.5 * torch.randn((c, m["conv"]), device=device, generator=g)).to(torch.bfloat16)
            mat(k + ".mix.b", H, w); mat(k + ".mix.a", H, w); mat(k + ".mix.g", H * vd, w)
            vec(k + ".mix.dt_bias", H, -1.0, 0.5); vec(k + ".mix.A_log", H, -1.0, 0.5); vec(k + ".mix.norm", vd, 1.0); mat(k + ".mix.o", w, H * vd)
        ms = L["mlp"]
        mat(k + ".mlp.router", ms["router"]["experts"], w)
        for n, ff in [(f"e{e}", ms["expert"]["ff"]) for e in range(ms["router"]["experts"])] + [("shared", ms["shared"]["ff"])]:
            mat(f"{k}.mlp.{n}.gate", ff, w); mat(f"{k}.mlp.{n}.up", ff, w); mat(f"{k}.mlp.{n}.down", w, ff)
    return T


def bench_sandwich(size: str, device="cuda:0", prompt: int = 2048, ctx: int = 1024, decode_steps: int = 64, batches=(1, 4)) -> dict:
    from .config import LayeredConfig
    from .layered import LayeredModel
    s = SANDWICH_SIZES[size]
    cfg = sandwich_config(s)
    model = LayeredModel(LayeredConfig.from_dict_sandwich(cfg), device=device, dtype=torch.bfloat16).load(sandwich_random_tensors(cfg, device))
    out = {"design": "kilurax", "size": size, "layers": len(cfg["layers"]), "pattern": s["pattern"], "weight_bytes_per_token": model.weight_bytes()}
    return _bench_engine(model, out, s["vocab"], prompt, ctx, decode_steps, batches)


def bench_sandwich_peer(size: str, device="cuda:0", prompt: int = 2048, ctx: int = 1024, decode_steps: int = 64, batches=(1, 4)) -> dict:
    """the closest model of the package: a token-shifted stack of chunked attention and decaying linear attention (bfloat16, the same
    engine) of the same width and depth -- an attention layer of the same heads (one chunk over the whole context) for every layer of
    attention beside a state-space scan, a decaying linear attention of the same state size per head for every other linear-attention
    layer, the same sparse feed-forward (two-matrix experts half as wide again, so that a token streams the same bytes)"""
    from .config import LayeredConfig
    from .layered import LayeredModel
    s = SANDWICH_SIZES[size]
    layers = []
    for ch in s["pattern"]:
        ff = {"expert": {"ff": s["expert_ff"] * 3 // 2}, "kind": "moe", "router": {"experts": s["experts"], "top": s["top"]},
              "shared": {"ff": s["shared_ff"] * 3 // 2}}
        if ch == "p":
            m = {"dim": s["dim"], "heads": s["heads"], "kv_heads": s["kv_heads"], "vdim": s["vdim"], "mask": {"size": 1 << 20},
                 "scale": s["dim"] ** -0.5, "softcap": 30.0, "rot": {"base": 500000.0, "dims": s["dim"]}}
            layers.append({"type": "attention", "mlp": ff, "mixer": m})
        else:
            layers.append({"type": "wkv", "mlp": ff, "mixer": {"dim": s["la_dim"], "heads": s["la_heads"]}})
    cfg = {"architecture": "Negilorn", "layers": layers, "logit_scale": 0.5, "norm": {"eps": 1e-5}, "vocab": s["vocab"], "width": s["width"]}
    model = LayeredModel(LayeredConfig.from_dict_prerms_shift(cfg), device=device, dtype=torch.bfloat16).load(
        shift_random_tensors(cfg, dict(rank=64), device))
    out = {"design": "negilorn-peer", "size": size, "layers": len(layers), "weight_bytes_per_token": model.weight_bytes()}
    return _bench_engine(model, out, s["vocab"], prompt, ctx, decode_steps, batches)


def run(sizes, device="cuda:0", peer: bool = True, design: str = "benolix"):
    for size in sizes:
        if design == "kilurax":
            print(json.dumps(bench_sandwich(size, device)), flush=True)
            if peer:
                print(json.dumps(bench_sandwich_peer(size, device)), flush=True)
            continue
        if design == "negilorn":
            print(json.dumps(bench_shift(size, device)), flush=True)
            if peer:
                print(json.dumps(bench_shift_peer(size, device)), flush=True)
            continue
        if design == "tibalorn":
            print(json.dumps(bench_hybrid(size, device)), flush=True)
            if peer:
                print(json.dumps(bench_hybrid_peer(size, device)), flush=True)
            continue
        print(json.dumps(bench_layered(size, device)), flush=True)
        if peer:
            print(json.dumps(bench_quantized_peer(size, device)), flush=True)
