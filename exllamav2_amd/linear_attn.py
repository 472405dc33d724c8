"""Linear-attention mixers over a matrix state per head (csrc/gated_scan.hip), beside the state-space and the decaying mixers.

ForgetGateLinearAttention -- the forget gate also decides what is written; no key projection:
    [zq | zf | v] = W h (+ b_f on zf)                 one dense linear;  q = silu(zq): heads x dim;  v: heads x vdim
    f = l + (1 - l) sigmoid(zf)                       per head and key channel, l = a learned lower bound in the checkpoint
    head i: S_i <- diag(f_i) S_i + (1 - f_i) v_i^T;   o_i = S_i^T q_i
    out = W_o concat_i(o_i / rms(o_i) * w)            w [vdim] shared by the heads

GatedDeltaRule -- one decay per head and a delta-rule write:
    [q | k | v | zb | za | zg] = W h                  one dense linear; q, k: kv_heads x dim; v, zg: heads x vdim; zb, za: heads
    (q, k, v) <- silu(conv(q, k, v))                  causal convolution per channel over the last `taps` tokens, no bias
    q, k per head / sqrt(sum(.^2) + 1e-6), q also / sqrt(dim);  beta = sigmoid(zb);  g = exp(-exp(A) softplus(za + a_bias))
    head i (q / k head i // (heads / kv_heads)):  S_i <- g_i S_i;  u = beta_i (v_i - S_i^T k);  S_i <- S_i + k u^T;  o_i = S_i^T q
    out = W_o concat_i(o_i / rms(o_i) * w * silu(zg_i))

Gates, decays, unit norms and the state are fp32 (inside the scan kernel, from the linear's fp32 outputs).  Between steps a sequence
keeps S -- and the delta rule the last taps - 1 convolution inputs -- in its slot (cache.SlotState).  Head counts and sizes are
constructor parameters."""
from __future__ import annotations

import os

import torch

from .cache import SlotState
from .dense_linear import DenseLinear


# longest span of a step from which the column-split scan is taken (EXL2_SCAN_COLS_FROM: kernel-tuning A/B runs)
COLS_FROM = int(os.environ.get("EXL2_SCAN_COLS_FROM", "1"))


class ForgetGateLinearAttention:
    def __init__(self, model, key: str, layer_idx, *, heads: int, dim: int, vdim: int, out_tag: str = "mix.y"):
        self.model, self.ext, self.key, self.layer_idx = model, model.ext, key, layer_idx
        self.heads, self.dim, self.vdim, self.out_tag = heads, dim, vdim, out_tag
        if heads <= 0 or dim <= 0 or vdim <= 0:
            raise ValueError(f"{key}: {heads} heads of {dim} x {vdim}")
        self.kv_from = None
        self.cols_ok = self.ext.gated_scan_cols_supported(dim, vdim)

    def load(self, get):
        H, dim, vd, width, f32 = self.heads, self.dim, self.vdim, self.model.width, torch.float32
        q, f, v = get("q"), get("f"), get("v")
        if tuple(q.shape) != (H * dim, width) or tuple(f.shape) != (H * dim, width) or tuple(v.shape) != (H * vd, width):
            raise RuntimeError(f"{self.key}: tensor shapes do not match the mixer's sizes")
        self.front = DenseLinear(self.ext, self.key + ".front", torch.cat([q, f, v], 0))
        self.front_bias = torch.zeros((self.front.out_features,), dtype=f32, device=self.model.device)
        fb = get("f.b", optional=True)
        if fb is not None:
            self.front_bias[H * dim:2 * H * dim] = fb.to(f32)
        self.lower = get("lower").to(f32).reshape(-1).contiguous()
        self.norm_w = get("norm").to(f32).reshape(-1).contiguous()
        self.o = DenseLinear(self.ext, self.key + ".o", get("o"))
        if self.lower.numel() != H * dim or self.norm_w.numel() != vd or tuple(self.o.weight.shape) != (width, H * vd):
            raise RuntimeError(f"{self.key}: tensor shapes do not match the mixer's sizes")
        return self

    def weight_bytes(self) -> int:
        return self.front.weight_bytes() + self.o.weight_bytes()

    def make_state(self, pool, dtype):
        return SlotState(pool, {"S": (self.heads, self.dim, self.vdim)})

    def forward(self, xh: torch.Tensor, rows: int, batch, cache) -> torch.Tensor:
        """xh: the layer input in the operand dtype [rows, width]; returns the mixer's output, fp32 [rows, width]"""
        ext, m, f32 = self.ext, self.model, torch.float32
        st = cache.layer(self.layer_idx)
        H, dim, vd = self.heads, self.dim, self.vdim
        n = self.front.out_features
        f = self.front.forward(xh, rows, out=m.buf("mix.f", (rows, n), f32), bias=self.front_bias)             # [zq | zf | v]
        g = m.buf("la.g", (rows, H * vd), m.dtype)
        # the walk dealt to (head, value columns) workgroups + a head-norm launch (state shapes outside that kernel, or a raised
        # COLS_FROM for short spans: the fused launch of one workgroup per head)
        o_raw = m.buf("la.o", (rows, H * vd), f32) if self.cols_ok and batch.spans_dev[3] >= COLS_FROM else None
        ext.gated_scan(ext.SCAN_FORGET_WRITES, f, n, 0, H * dim, f, n, 2 * H * dim, self.norm_w, g, st["S"], batch.spans_dev,
                       batch.row_seq, batch.row_pos, H, H, dim, vd, m.norm_eps, lower=self.lower, o_raw=o_raw)
        return self.o.forward(g, rows, out=m.buf(self.out_tag, (rows, m.width), f32))


class GatedDeltaRule:
    def __init__(self, model, key: str, layer_idx, *, heads: int, kv_heads: int, dim: int, vdim: int, taps: int, out_tag: str = "mix.y"):
        self.model, self.ext, self.key, self.layer_idx = model, model.ext, key, layer_idx
        self.heads, self.kv_heads, self.dim, self.vdim, self.taps, self.out_tag = heads, kv_heads, dim, vdim, taps, out_tag
        if heads <= 0 or kv_heads <= 0 or heads % kv_heads or dim <= 0 or vdim <= 0 or taps < 1:
            raise ValueError(f"{key}: {heads} heads over {kv_heads} query / key heads of {dim} x {vdim}, {taps} taps")
        self.channels = 2 * kv_heads * dim + heads * vdim         # what passes the convolution: [q | k | v]
        self.kv_from = None
        self.cols_ok = self.ext.gated_scan_cols_supported(dim, vdim)

    def load(self, get):
        H, G, dim, vd, width, f32 = self.heads, self.kv_heads, self.dim, self.vdim, self.model.width, torch.float32
        q, k, v, b, a, g = (get(n) for n in ("q", "k", "v", "b", "a", "g"))
        if tuple(q.shape) != (G * dim, width) or tuple(k.shape) != (G * dim, width) or tuple(v.shape) != (H * vd, width) \
                or tuple(b.shape) != (H, width) or tuple(a.shape) != (H, width) or tuple(g.shape) != (H * vd, width):
            raise RuntimeError(f"{self.key}: tensor shapes do not match the mixer's sizes")
        self.front = DenseLinear(self.ext, self.key + ".front", torch.cat([q, k, v, b, a, g], 0))
        self.off_b = self.channels
        self.off_a = self.off_b + H
        self.off_g = self.off_a + H
        convs = [get(n + ".conv") for n in ("q", "k", "v")]
        if any(c.dim() != 2 or c.shape[1] != self.taps for c in convs) or [c.shape[0] for c in convs] != [G * dim, G * dim, H * vd]:
            raise RuntimeError(f"{self.key}: convolution weights do not match the mixer's sizes")
        self.conv_w = torch.cat(convs, 0).contiguous()
        self.dt_bias, self.a_log = (get(n).to(f32).reshape(-1).contiguous() for n in ("dt_bias", "A_log"))
        self.norm_w = get("norm").to(f32).reshape(-1).contiguous()
        self.o = DenseLinear(self.ext, self.key + ".o", get("o"))
        if self.dt_bias.numel() != H or self.a_log.numel() != H or self.norm_w.numel() != vd or tuple(self.o.weight.shape) != (width, H * vd):
            raise RuntimeError(f"{self.key}: tensor shapes do not match the mixer's sizes")
        return self

    def weight_bytes(self) -> int:
        return self.front.weight_bytes() + self.o.weight_bytes()

    def make_state(self, pool, dtype):
        return SlotState(pool, {"tail": (max(self.taps - 1, 1), self.channels), "S": (self.heads, self.dim, self.vdim)})

    def forward(self, xh: torch.Tensor, rows: int, batch, cache) -> torch.Tensor:
        """xh: the layer input in the operand dtype [rows, width]; returns the mixer's output, fp32 [rows, width]"""
        ext, m, f32 = self.ext, self.model, torch.float32
        st = cache.layer(self.layer_idx)
        H, G, dim, vd, ch = self.heads, self.kv_heads, self.dim, self.vdim, self.channels
        n = self.front.out_features
        f = self.front.forward(xh, rows, out=m.buf("mix.f", (rows, n), f32))                                   # [q | k | v | zb | za | zg]
        c = m.buf("la.c", (rows, ch), f32)
        ext.conv_silu_rows(f, n, 0, self.conv_w, None, c, st["tail"], batch.spans_dev, batch.row_seq, batch.row_pos, ch, self.taps)
        g = m.buf("la.g", (rows, H * vd), m.dtype)
        o_raw = m.buf("la.o", (rows, H * vd), f32) if self.cols_ok and batch.spans_dev[3] >= COLS_FROM else None
        ext.gated_scan(ext.SCAN_DELTA, f, n, 0, G * dim, c, ch, 2 * G * dim, self.norm_w, g, st["S"], batch.spans_dev, batch.row_seq,
                       batch.row_pos, H, G, dim, vd, m.norm_eps, q_scale=dim ** -0.5, gate_off=self.off_g, beta_off=self.off_b,
                       dt_off=self.off_a, dt_bias=self.dt_bias, a_log=self.a_log, qk=c, ldqk=ch, o_raw=o_raw)
        return self.o.forward(g, rows, out=m.buf(self.out_tag, (rows, m.width), f32))
