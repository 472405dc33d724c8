"""Linear attention with a per-channel, data-dependent decay (RWKV-style time mixing), beside the attention and state-space mixers.

Per token, with h the mixer's input and h' the previous token's input (zeros at a sequence's start):
    x_s = h + (h' - h) * mu_s                          five blends, s in (r, k, v, g, w)                (csrc/wkv.hip: wkv_mix_kernel)
    r, k, v = W_r x_r, W_k x_k, W_v x_v                heads x dim each;   gate = silu(W_g x_g)
    d = W_w2 tanh(W_w1 x_w) + w0;  w = exp(-exp(d))    decay per head and key channel, in (0, 1)
    head i:  o = (S_i + diag(u_i) k v^T)^T r;  S_i <- diag(w) S_i + k v^T        S fp32 [dim, dim] per slot  (wkv_scan_kernel token by
             token for decoded tokens and short portions; wkv_chunk_* unrolled in chunks of 64 tokens for portions of prompts)
    out = W_o (o / rms_per_head(o) * norm * gate)
Between steps a sequence keeps S and its last input row in its slot (cache.SlotState).  The mixer reads its input in fp32
(`input_f32`): the blends are rounded to the operand dtype once, after blending.  Head count, head size and the rank of the decay's
bottleneck come from the configuration and the tensors' shapes."""
from __future__ import annotations

import torch

from .cache import SlotState
from .dense_linear import DenseLinear


class DecayLinearAttention:
    input_f32 = True                                          # forward() takes the normed layer input as fp32 rows
    MIXES = ("r", "k", "v", "g", "w")
    CHUNKED_FROM = 8                                          # longest span of a step from which the chunked scan is taken

    def __init__(self, model, key: str, layer_idx: int, *, heads: int, dim: int):
        self.model, self.ext, self.key, self.layer_idx = model, model.ext, key, layer_idx
        self.heads, self.dim = heads, dim
        self.inner = heads * dim
        if heads <= 0 or dim <= 0:
            raise ValueError(f"{key}: {heads} heads of {dim}")
        self.kv_from = None
        self.chunked_ok = self.ext.wkv_scan_chunked_supported(dim, dim)

    def load(self, get):
        """`get(name)` returns the device tensor `<layer>.mix.<name>` in the model's operand dtype"""
        width, inner, f32 = self.model.width, self.inner, torch.float32
        self.mu = torch.stack([get("mu." + n).reshape(-1) for n in self.MIXES], 0).contiguous()                 # [5, width]
        proj = [get(n) for n in ("r", "k", "v", "g")]
        w1, w2 = get("w1"), get("w2")
        self.rank = w1.shape[0]
        if any(tuple(t.shape) != (inner, width) for t in proj) or self.mu.shape[1] != width or w1.shape[1] != width \
                or tuple(w2.shape) != (inner, self.rank):
            raise RuntimeError(f"{self.key}: tensor shapes do not match the mixer's sizes")
        self.rkvg = DenseLinear(self.ext, self.key + ".rkvg", torch.stack(proj, 0))                               # [4, inner, width]
        self.w1 = DenseLinear(self.ext, self.key + ".w1", w1)
        self.w2 = DenseLinear(self.ext, self.key + ".w2", w2)
        self.w0 = get("w0").to(f32).reshape(-1).contiguous()
        self.u = get("u").to(f32).contiguous()
        self.norm_w = get("norm").to(f32).reshape(-1).contiguous()
        self.o = DenseLinear(self.ext, self.key + ".o", get("o"))
        if self.w0.numel() != inner or tuple(self.u.shape) != (self.heads, self.dim) or self.norm_w.numel() != inner \
                or tuple(self.o.weight.shape) != (width, inner):
            raise RuntimeError(f"{self.key}: tensor shapes do not match the mixer's sizes")
        return self

    def weight_bytes(self) -> int:
        return self.rkvg.weight_bytes() + self.w1.weight_bytes() + self.w2.weight_bytes() + self.o.weight_bytes()

    def make_state(self, pool, dtype):
        return SlotState(pool, {"prev": (self.model.width,), "S": (self.heads, self.dim, self.dim)})

    def forward(self, h32: torch.Tensor, rows: int, batch, cache) -> torch.Tensor:
        """h32: the normed (and shifted) layer input, fp32 [rows, width]; returns the mixer's output, fp32 [rows, width]"""
        ext, m, f32 = self.ext, self.model, torch.float32
        st = cache.layer(self.layer_idx)
        width, inner = m.width, self.inner
        x = m.buf("wkv.x", (5, rows, width), m.dtype)
        ext.wkv_mix(h32, st["prev"], self.mu, x, batch.row_seq, batch.row_pos, batch.spans_dev, rows, width)
        f = m.buf("wkv.f", (4, rows, inner), f32)
        ext.dense_linear(x, self.rkvg.weight, f, rows, inner, width, width, width, inner, batch=4, sxb=rows * width, swb=inner * width,
                         syb=rows * inner)
        t = self.w1.forward(x, rows, out=m.buf("wkv.t", (rows, self.rank), m.dtype), epi=ext.EPI_TANH, x_off=4 * rows * width, ldx=width)
        d = self.w2.forward(t, rows, out=m.buf("wkv.d", (rows, inner), f32), bias=self.w0)
        g = m.buf("wkv.g", (rows, inner), m.dtype)
        if batch.span_chunks is not None and batch.spans_dev[3] >= self.CHUNKED_FROM and self.chunked_ok:
            # portions of prompts: the recurrence unrolled in chunks, every (chunk, head) independent work
            total = batch.span_chunks[2]
            zbuf = m.buf("wkv.z", (total, self.heads, self.dim, self.dim), f32)
            dbuf = m.buf("wkv.dk", (total, self.heads, self.dim), f32)
            ext.wkv_scan_chunked(f, rows, d, self.u, self.norm_w, g, st["S"], batch.spans_dev, batch.span_chunks, batch.row_seq, batch.row_pos,
                                 zbuf, dbuf, self.heads, self.dim, self.dim, m.norm_eps)
        else:
            # decoded tokens and short portions: one pass per (span, head) with the state in registers
            ext.wkv_scan(f, rows, d, self.u, self.norm_w, g, st["S"], batch.spans_dev, batch.row_seq, batch.row_pos, self.heads, self.dim,
                         self.dim, m.norm_eps)
        return self.o.forward(g, rows, out=m.buf("mix.y", (rows, width), f32))
