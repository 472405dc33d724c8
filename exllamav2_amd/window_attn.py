"""Grouped-head attention with a sliding window, pooled blocks behind the window, a sink in the softmax and rotated values
(beside LatentAttention and the quantized ExLlamaV2Attention).

Per token at position p, with h the layer input:
    [q | k | v | g] = W h + bias                      one dense linear (g has no bias)
    q, k: the first rot_dims values of every head turned by p * f_i, amplitudes times `amp` (rotary_tables: plain frequencies, or
          blended between f_i and f_i / factor by a ramp for long contexts); v: all vdim values turned by p * base^(-2m / vdim)
    the cache keeps the turned k and v per token, and per block of `pool` tokens their mean (cache.PagedKV)
    head i (key / value head i // (heads / kv_heads)) sees the tokens 0 <= p - j < window and the blocks wholly in front of the window:
          weights exp(s_j) / (exp(sink_i) + sum exp(s)),  s_j = q_i . k_j * scale * temp_i
    out = W_o (turn_back(sum_j w_j v_j, p) * sigmoid(g))                       (csrc/window_attn.hip)
Everything the design leaves open is a constructor parameter: head counts, sizes, window, block size, rotary base / dims / scaling /
pair layout, score scale, and the variants
    chunk        a chunked mask instead of the window: p sees j <= p with floor(j / chunk) == floor(p / chunk)
    softcap      s_j <- softcap * tanh(s_j / softcap)
    sink_one     the denominator holds a constant 1 (a sink of score 0) instead of a learned exp(sink_i)
    kv_from      the layer has no key / value projections: it attends over the rows layer `kv_from` cached, with its own queries
biases (on q, k, v and on the output projection), per-head temperature, the learned sink and the output gate are used when the
checkpoint has them (none of them: plain causal softmax attention); a gate tensor of one row per head gates whole heads, one of
heads x vdim rows gates every output value.  `out_tag` names the scratch buffer of the result, for a layer that runs two mixers side
by side."""
from __future__ import annotations

import math

import torch

from .cache import PagedKV
from .dense_linear import DenseLinear


def rotary_tables(base: float, dims: int, scaling: dict | None, device):
    """(frequencies fp32 [dims / 2], amplitude): f_i = base^(-2i / dims); with `scaling` = {factor, original, fast, slow} the
    frequency of pair i is f_i / factor * r_i + f_i (1 - r_i), r_i a ramp from 0 to 1 between the pair that makes `fast` turns
    over `original` positions and the one that makes `slow` turns, and cos / sin are multiplied by 0.1 ln(factor) + 1.
    With `scaling` = {factor, original, low, high} the choice goes by wavelength l_i = 2 pi / f_i: f_i where l_i < original / high,
    f_i / factor where l_i > original / low, and between the two (1 - s) f_i / factor + s f_i with
    s = (original / l_i - low) / (high - low); amplitude 1.  Made in double precision, handed to the kernels as fp32."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / dims)
    amp = 1.0
    if scaling and "low" in scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])
        low, high = float(scaling["low"]), float(scaling["high"])
        wavelen = 2.0 * math.pi / f
        s = (orig / wavelen - low) / (high - low) if high != low else torch.ones_like(f)
        blend = (1.0 - s) * f / factor + s * f
        f = torch.where(wavelen < orig / high, f, torch.where(wavelen > orig / low, f / factor, blend))
    elif scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])

        def pair_of(turns):
            return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        amp = 0.1 * math.log(factor) + 1.0
    return f.to(torch.float32).to(device), amp


class WindowAttention:
    MAX_SPLIT = 16                                            # decoded tokens: workgroups that share one row's key list

    def __init__(self, model, key: str, layer_idx: int, *, heads: int, kv_heads: int, dim: int, vdim: int, window: int, pool: int,
                 rot_base: float, rot_dims: int, rot_scaling: dict | None, scale: float, rotate_values: bool = True,
                 interleaved: bool = False, chunk: int = 0, softcap: float = 0.0, sink_one: bool = False, kv_from: int | None = None,
                 out_tag: str = "mix.y"):
        self.model, self.ext, self.key, self.layer_idx = model, model.ext, key, layer_idx
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.window, self.pool, self.scale = window, pool, scale
        self.rot_base, self.rot_dims, self.rot_scaling = rot_base, rot_dims, rot_scaling
        self.rotate_values, self.interleaved = rotate_values, interleaved
        self.chunk, self.softcap, self.sink_one, self.kv_from = int(chunk), float(softcap), bool(sink_one), kv_from
        self.out_tag = out_tag
        if heads % kv_heads or rot_dims > dim or rot_dims % 2 or (rotate_values and vdim % 2) or window <= 0 or pool < 0 \
                or chunk < 0 or (chunk and pool) or softcap < 0:
            raise ValueError(f"{key}: inconsistent attention sizes")
        self.tiles_ok = self.ext.window_attn_tiles_supported(model.dtype, dim, vdim) and (self.heads * vdim) % 4 == 0

    def load(self, get):
        """`get(name)` returns the device tensor `<layer>.mix.<name>` in the model's operand dtype; `get(name, optional=True)`
        returns None for a tensor the checkpoint does not have"""
        H, G, dim, vd, width, f32 = self.heads, self.kv_heads, self.dim, self.vdim, self.model.width, torch.float32
        dev = self.model.device
        own_kv = self.kv_from is None
        q, g = get("q"), get("g", optional=True)
        parts, names = [q], ["q"]
        if own_kv:
            k, v = get("k"), get("v")
            if tuple(k.shape) != (G * dim, width) or tuple(v.shape) != (G * vd, width):
                raise RuntimeError(f"{self.key}: tensor shapes do not match the mixer's sizes")
            parts += [k, v]
            names += ["k", "v"]
        self.gated = g is not None
        self.gate_head = self.gated and tuple(g.shape) == (H, width) and vd != 1
        if tuple(q.shape) != (H * dim, width) or (self.gated and tuple(g.shape) not in ((H * vd, width), (H, width))):
            raise RuntimeError(f"{self.key}: tensor shapes do not match the mixer's sizes")
        # one linear for everything that reads the layer input: [q | k | v | g]; the gate's columns start at a multiple of 4
        pad = (-sum(p.shape[0] for p in parts)) % 4 if self.gated else 0
        if pad:
            parts.append(torch.zeros((pad, width), dtype=q.dtype, device=dev))
        self.off_k = H * dim
        self.off_v = self.off_k + (G * dim if own_kv else 0)
        self.off_g = sum(p.shape[0] for p in parts)
        self.front = DenseLinear(self.ext, self.key + ".front", torch.cat(parts + ([g] if self.gated else []), 0))
        biases = [get(n + ".b", optional=True) for n in names]
        self.front_bias = None
        if any(b is not None for b in biases):
            self.front_bias = torch.zeros((self.front.out_features,), dtype=f32, device=dev)
            at = 0
            for b, part in zip(biases, parts):
                if b is not None:
                    self.front_bias[at:at + part.shape[0]] = b.to(f32)
                at += part.shape[0]
        temp = get("temp", optional=True)
        self.q_scale = ((temp.to(f32) if temp is not None else torch.ones((H,), dtype=f32, device=dev)) * self.scale).contiguous()
        sink = get("sink", optional=True)
        if self.sink_one:
            self.sink = torch.zeros((H,), dtype=f32, device=dev)
        else:
            self.sink = sink.to(f32).contiguous() if sink is not None else None
        self.o = DenseLinear(self.ext, self.key + ".o", get("o"))
        ob = get("o.b", optional=True)
        self.o_bias = ob.to(f32).contiguous() if ob is not None else None
        if self.q_scale.numel() != H or (self.sink is not None and self.sink.numel() != H) or tuple(self.o.weight.shape) != (width, H * vd):
            raise RuntimeError(f"{self.key}: tensor shapes do not match the mixer's sizes")
        self.freq, self.amp = rotary_tables(self.rot_base, self.rot_dims, self.rot_scaling, dev) if self.rot_dims else \
            (torch.zeros((1,), dtype=f32, device=dev), 1.0)
        self.vfreq, _ = rotary_tables(self.rot_base, vd, None, dev)
        return self

    def weight_bytes(self) -> int:
        return self.front.weight_bytes() + self.o.weight_bytes()

    def make_state(self, pool, dtype):
        if self.kv_from is not None:
            return None                                       # it reads the rows of the layer it shares with
        return PagedKV(pool, self.kv_heads, self.dim, self.vdim, self.pool, dtype)

    def check_kv_source(self, src) -> None:
        """the layer whose cached keys and values this one reads must hold rows of the same shape, rotated the same way"""
        mine = (self.kv_heads, self.dim, self.vdim, self.rot_base, self.rot_dims, self.rot_scaling, self.rotate_values, self.interleaved, self.pool)
        if not isinstance(src, WindowAttention) or src.kv_from is not None or mine != (
                src.kv_heads, src.dim, src.vdim, src.rot_base, src.rot_dims, src.rot_scaling, src.rotate_values, src.interleaved, src.pool):
            raise RuntimeError(f"{self.key}: layer {self.kv_from} does not cache keys and values of this layer's shape and rotation")

    def forward(self, xh: torch.Tensor, rows: int, batch, cache) -> torch.Tensor:
        """xh: the normed layer input in the operand dtype [rows, width]; returns the mixer's output, fp32 [rows, width]"""
        ext, m, f32 = self.ext, self.model, torch.float32
        H, G, dim, vd = self.heads, self.kv_heads, self.dim, self.vdim
        st, page = cache.layer(self.layer_idx if self.kv_from is None else self.kv_from), cache.pool.page_size
        own = self.kv_from is None
        ncat = self.front.out_features
        f = self.front.forward(xh, rows, out=m.buf("mix.f", (rows, ncat), f32), bias=self.front_bias)        # [q | k | v | g] fp32
        q = m.buf("attn.q", (rows, H * dim), m.dtype)
        ext.kv_rot_append(f, ncat, 0, self.off_k, self.off_v, q, self.q_scale, st.k if own else None, st.v if own else None,
                          st.k_pool if own else None, st.v_pool if own else None, self.freq, self.amp,
                          self.rot_dims, self.vfreq, self.rotate_values, self.interleaved, batch.row_seq, batch.row_pos, batch.block_table,
                          page, self.pool if own else 0, rows, H, G, dim, vd)
        o = m.buf("attn.o", (rows, H * vd), m.dtype)
        common = (q, st.k, st.v, st.k_pool, st.v_pool, self.sink, f if self.gated else None, ncat, self.off_g, self.vfreq, self.rotate_values, self.interleaved,
                  batch.row_seq, batch.row_pos, batch.block_table, page, self.pool, o)
        var = dict(chunk=self.chunk, softcap=self.softcap, gate_head=self.gate_head)
        reach = self.chunk or self.window                     # the most tokens a position sees
        if self.tiles_ok and (batch.prompt_tiles is not None or batch.tiles1 is not None):
            # matrix-core kernels: portions of prompts as tiles of <= 64 positions x one head per workgroup, decoded tokens as one
            # row x one key / value head per workgroup (its query heads share the pass over the keys)
            if batch.prompt_tiles is not None:
                row0, nrow, n, size = batch.prompt_tiles
                ext.window_attn_tiles(*common, (row0, nrow, n), size, H, G, dim, vd, self.window, **var)
            if batch.tiles1 is not None:
                row0, n, max_pos = batch.tiles1
                # the longest key list among the rows: window tokens + pooled blocks; its steps of 128 entries go to up to 16 workgroups
                entries = min(reach, max_pos + 1) + (max(0, max_pos - self.window + 1) // self.pool if self.pool else 0)
                nsplit = max(1, min(self.MAX_SPLIT, -(-entries // 128)))
                part_o = part_ml = None
                if nsplit > 1:
                    part_o = m.buf("attn.part_o", (rows, H, nsplit, vd), f32)
                    part_ml = m.buf("attn.part_ml", (rows, H, nsplit, 2), f32)
                ext.window_attn_tiles(*common, (row0, None, n), 1, H, G, dim, vd, self.window, nsplit=nsplit, part_o=part_o, part_ml=part_ml,
                                      **var)
        else:
            ext.window_attn(*common, rows, H, G, dim, vd, self.window, **var)
        return self.o.forward(o, rows, out=m.buf(self.out_tag, (rows, m.width), f32), bias=self.o_bias)
