"""State-space mixer with a scalar decay per head (selective scan), beside the attention mixers.

Per token, with h the layer input:
    [z | u | B | C | d] = W_in h                      one dense linear; u: heads x vdim, B / C: groups x state, d: heads
    (u, B, C) <- silu(conv(u, B, C) + bias)           causal convolution per channel over the last `taps` tokens
    d <- softplus(d + d_bias);  head i (group i // (heads / groups)):
    S_i <- exp(-exp(A_i) d_i) S_i + d_i B u_i^T;  y_i = S_i^T C + D_i u_i          (csrc/ssm.hip; S fp32 [state, vdim] per slot)
    out = W_o (rms_per_norm_group(y * silu(z)) * w_norm)
Between steps a sequence keeps S and the last taps - 1 convolution inputs in its slot (cache.SlotState).  Everything the design
leaves open is a constructor parameter: head count, vdim, state size, groups, norm groups, taps."""
from __future__ import annotations

import torch

from .cache import SlotState
from .dense_linear import DenseLinear


class StateSpaceMixer:
    CHUNKED_FROM = 8                                          # longest span of a step from which the chunked scan is taken

    def __init__(self, model, key: str, layer_idx: int, *, heads: int, vdim: int, state: int, groups: int, norm_groups: int, taps: int,
                 out_tag: str = "mix.y"):
        self.model, self.ext, self.key, self.layer_idx = model, model.ext, key, layer_idx
        self.heads, self.vdim, self.state, self.groups, self.norm_groups, self.taps = heads, vdim, state, groups, norm_groups, taps
        self.inner = heads * vdim
        self.channels = self.inner + 2 * groups * state
        if heads % groups or self.inner % norm_groups:
            raise ValueError(f"{key}: {heads} heads in {groups} groups, {self.inner} values in {norm_groups} norm groups")
        self.kv_from = None
        self.out_tag = out_tag                                    # scratch buffer of the result (a layer may run two mixers side by side)
        self.chunked_ok = self.ext.ssm_scan_chunked_supported(state, vdim) and self.inner % 4 == 0 and self.channels % 4 == 0

    def load(self, get):
        """`get(name)` returns the device tensor `<layer>.mix.<name>` in the model's operand dtype"""
        width, f32 = self.model.width, torch.float32
        self.front = DenseLinear(self.ext, self.key + ".in", get("in"))
        self.n_front = 2 * self.inner + 2 * self.groups * self.state + self.heads
        self.conv_w, self.conv_b = get("conv").contiguous(), get("conv.b").contiguous()
        self.dt_bias, self.a_log, self.d = (get(n).to(f32).contiguous() for n in ("dt_bias", "A_log", "D"))
        self.norm_w = get("norm").contiguous()
        self.o = DenseLinear(self.ext, self.key + ".o", get("o"))
        if tuple(self.front.weight.shape) != (self.n_front, width) or tuple(self.conv_w.shape) != (self.channels, self.taps) \
                or self.conv_b.numel() != self.channels or self.norm_w.numel() != self.inner \
                or tuple(self.o.weight.shape) != (width, self.inner) or any(t.numel() != self.heads for t in (self.dt_bias, self.a_log, self.d)):
            raise RuntimeError(f"{self.key}: tensor shapes do not match the mixer's sizes")
        return self

    def weight_bytes(self) -> int:
        return self.front.weight_bytes() + self.o.weight_bytes()

    def make_state(self, pool, dtype):
        return SlotState(pool, {"tail": (max(self.taps - 1, 1), self.channels), "S": (self.heads, self.state, self.vdim)})

    def forward(self, xh: torch.Tensor, rows: int, batch, cache) -> torch.Tensor:
        """xh: the normed layer input in the operand dtype [rows, width]; returns the mixer's output, fp32 [rows, width]"""
        ext, m, f32 = self.ext, self.model, torch.float32
        st = cache.layer(self.layer_idx)
        inner, gn = self.inner, self.groups * self.state
        f = self.front.forward(xh, rows, out=m.buf("mix.f", (rows, self.n_front), f32))              # [z | u B C | d]
        c = m.buf("ssm.c", (rows, self.channels), f32)
        ext.conv_silu_rows(f, self.n_front, inner, self.conv_w, self.conv_b, c, st["tail"], batch.spans_dev, batch.row_seq, batch.row_pos,
                           self.channels, self.taps)
        y = m.buf("ssm.y", (rows, inner), f32)
        scan_args = (c, self.channels, 0, inner, inner + gn, f, self.n_front, 2 * inner + 2 * gn, self.dt_bias, self.a_log, self.d, y, st["S"],
                     batch.spans_dev)
        if batch.span_chunks is not None and batch.spans_dev[3] >= self.CHUNKED_FROM and self.chunked_ok:
            # portions of prompts: the recurrence unrolled in chunks, every (chunk, head) independent work
            total = batch.span_chunks[2]
            zbuf = m.buf("ssm.z", (total, self.heads, self.state, self.vdim), f32)
            dbuf = m.buf("ssm.d", (total, self.heads), f32)
            ext.ssm_scan_chunked(*scan_args, batch.span_chunks, batch.row_seq, batch.row_pos, zbuf, dbuf, self.heads, self.groups,
                                 self.state, self.vdim)
        else:
            # decoded tokens and short portions: one pass per (span, head) with the state in registers
            ext.ssm_scan(*scan_args, batch.row_seq, batch.row_pos, self.heads, self.groups, self.state, self.vdim)
        g = m.buf("ssm.g", (rows, inner), m.dtype)
        ext.gated_group_norm(y, f, self.n_front, self.norm_w, g, rows, inner, self.norm_groups, m.norm_eps)
        return self.o.forward(g, rows, out=m.buf(self.out_tag, (rows, m.width), f32))
