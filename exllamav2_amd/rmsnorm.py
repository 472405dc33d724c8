"""ExLlamaV2RMSNorm (reference rmsnorm.py:115-211)."""
from __future__ import annotations

import torch


class ExLlamaV2RMSNorm:
    def __init__(self, ext, key: str, weight: torch.Tensor, eps: float):
        self.ext = ext
        self.key = key
        self.weight = weight
        self.variance_epsilon = eps

    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        """rmsnorm.py:128-150 -> ext_c.rms_norm"""
        out = torch.empty_like(hidden_states)
        d = hidden_states.shape[-1]
        self.ext.rms_norm(hidden_states.view(-1, d), self.weight, out.view(-1, d), self.variance_epsilon)
        return out

    def forward_torch(self, hidden_states: torch.Tensor) -> torch.Tensor:
        """rmsnorm.py:187-211 (fp32 torch reference path)"""
        variance = hidden_states.to(torch.float32).pow(2).mean(-1, keepdim=True)
        hidden_states = hidden_states * torch.rsqrt(variance + self.variance_epsilon)
        hidden_states = hidden_states.to(self.weight.dtype)
        return hidden_states * self.weight


class PostNorm:
    """The residual step of a post-norm layer, x <- rms_norm(alpha x + sublayer(x)) (1 + w), as ONE launch in place on the fp32
    residual stream (csrc/rowops.hip: post_norm_kernel); it also leaves the operand-dtype copy the next linears read.  The weight is
    stored around zero.  `moe` routes the mixture of a token's chosen experts (identity experts included) through the same launch."""

    def __init__(self, ext, key: str, weight: torch.Tensor, eps: float, alpha: float):
        self.ext, self.key, self.weight, self.eps, self.alpha = ext, key, weight.contiguous(), eps, alpha

    def forward(self, x32: torch.Tensor, xh, y, rows: int, moe=None) -> None:
        self.ext.post_norm(x32, xh, y, self.weight, rows, self.alpha, self.eps, moe=moe)


class PreLayerNorm:
    """The norm in front of a sublayer of a pre-norm layer: (x - mean) / sqrt(var + eps) * w + b.  It runs fused with the residual
    addition of the sublayer BEFORE it (csrc/rowops.hip: add_layer_norm_kernel): `forward` adds `y` (that sublayer's fp32 output, or
    None at the start of the stack) into the fp32 stream and leaves the normalised rows in the operand dtype."""

    def __init__(self, ext, key: str, weight: torch.Tensor, bias: torch.Tensor | None, eps: float):
        self.ext, self.key, self.weight, self.eps = ext, key, weight.contiguous(), eps
        self.bias = bias.contiguous() if bias is not None else None
        if self.bias is not None and self.bias.shape != self.weight.shape:
            raise RuntimeError(f"{key}: weight and bias differ in shape")

    def forward(self, x32: torch.Tensor, y, out: torch.Tensor, rows: int, row_idx=None) -> None:
        self.ext.add_layer_norm(x32, y, self.weight, self.bias, out, rows, self.eps, row_idx=row_idx)


class PreShiftRMSNorm:
    """The norm in front of a sublayer of a pre-norm layer whose gain is ONE number: x / sqrt(mean(x^2) + eps) * g, optionally
    followed by a token shift  h + (h' - h) * shift  towards the previous token's normed row h' (zeros at a sequence's start).
    Like PreLayerNorm it runs fused with the residual addition of the sublayer before it -- a linear's fp32 output and / or the
    `top` expert outputs of every row (csrc/rowops.hip: add_rms_shift_kernel).  The previous row is per-sequence state:
    `make_state` asks the pool for one fp32 row per slot; steps of single tokens shift and roll it inside the norm's launch."""

    def __init__(self, ext, key: str, gain: torch.Tensor, eps: float, shift: torch.Tensor | None = None):
        if gain.numel() != 1:
            raise RuntimeError(f"{key}: the gain of this norm is one number, got {tuple(gain.shape)}")
        self.ext, self.key, self.eps = ext, key, eps
        self.gain = float(gain.to(torch.float32).reshape(()).item())
        self.shift = shift.contiguous() if shift is not None else None

    def make_state(self, pool, width: int):
        from .cache import SlotState
        return SlotState(pool, {"prev": (width,)}) if self.shift is not None else None

    def forward(self, x32: torch.Tensor, pending, out: torch.Tensor | None, rows: int, batch=None, state=None, hn=None, row_idx=None,
                dtype=None) -> None:
        """pending: None or (y fp32 [rows, width] | None, expert outputs fp32 [rows * top, width] | None, top)"""
        y, moe_y, top = pending if pending is not None else (None, None, 0)
        kw = {}
        if self.shift is not None and out is not None:
            kw = dict(shift=self.shift, prev=state["prev"], hn=hn, row_seq=batch.row_seq, row_pos=batch.row_pos, spans=batch.spans_dev)
        self.ext.add_rms_shift(x32, y, out, rows, self.gain, self.eps, moe_y=moe_y, top=top, row_idx=row_idx, dtype=dtype, **kw)


class SandwichNorm:
    """The two norms around one sublayer of a sandwich-normed layer, x <- x + mult * n_g(f(conv_in(n_g(x) w_in))) w_out, where n_g is
    an RMS norm taken separately over `groups` equal runs of the row and conv_in(a) = a + a short causal convolution of a over the
    sequence (weights [width, taps], optional).  `forward` runs what lies BETWEEN two sublayers as one launch (csrc/rowops.hip:
    sandwich_norm_kernel): the norm behind the previous sublayer (`pending`: its outputs and its SandwichNorm), the residual
    addition, and this sublayer's norm in front.  The convolution's history is per-sequence state: `make_state` asks the pool for
    the last taps - 1 normed rows per slot; steps of single tokens convolve and roll it inside the norm's launch, steps with longer
    spans write the normed rows in fp32 and convolve in a second launch (csrc/ssm.hip: conv_silu_kernel in its residual form)."""

    def __init__(self, ext, key: str, w_in: torch.Tensor, w_out: torch.Tensor | None, conv_w: torch.Tensor | None, groups: int, eps: float,
                 mult: float):
        self.ext, self.key, self.groups, self.eps, self.mult = ext, key, int(groups), float(eps), float(mult)
        self.w_in = w_in.contiguous()
        self.w_out = w_out.contiguous() if w_out is not None else None
        self.conv_w = conv_w.contiguous() if conv_w is not None else None
        width = self.w_in.numel()
        if width % self.groups or (self.w_out is not None and self.w_out.numel() != width):
            raise RuntimeError(f"{key}: {width} values in {groups} groups")
        self.taps = 0
        if self.conv_w is not None:
            if self.conv_w.dim() != 2 or self.conv_w.shape[0] != width:
                raise RuntimeError(f"{key}: the input convolution's weights are {tuple(self.conv_w.shape)}, the rows {width} wide")
            self.taps = int(self.conv_w.shape[1])

    def make_state(self, pool, width: int):
        from .cache import SlotState
        return SlotState(pool, {"tail": (max(self.taps - 1, 1), width)}) if self.taps > 1 else None

    @staticmethod
    def _pending_args(pending) -> dict:
        """pending: None or (the sublayer's SandwichNorm, y | None, ya, y2 | None, yb, expert rows | None, rows per token)"""
        if pending is None:
            return dict(w_out=None, mult=0.0)
        norm, y, ya, y2, yb, moe_y, top = pending
        return dict(w_out=norm.w_out, mult=norm.mult, y=y, ya=ya, y2=y2, yb=yb, moe_y=moe_y, top=top)

    def forward(self, x32: torch.Tensor, pending, out: torch.Tensor | None, rows: int, model=None, batch=None, state=None, row_idx=None,
                dtype=None) -> None:
        """out (operand dtype or fp32, [rows, width]) takes what this norm's sublayer reads; None: only the pending addition"""
        ext, pa = self.ext, self._pending_args(pending)
        w_out, mult = pa.pop("w_out"), pa.pop("mult")
        if out is None:
            ext.sandwich_norm(x32, w_out, mult, None, None, rows, self.groups, self.eps, dtype=dtype, **pa)
        elif self.conv_w is None or row_idx is not None:
            ext.sandwich_norm(x32, w_out, mult, self.w_in, out, rows, self.groups, self.eps, row_idx=row_idx, dtype=dtype, **pa)
        elif self.taps == 1 or batch.spans_dev[3] == 1:
            # no history needed, or single-token spans: norm, convolution and the roll of the slot's tail in one launch
            ext.sandwich_norm(x32, w_out, mult, self.w_in, out, rows, self.groups, self.eps, conv_w=self.conv_w,
                              tail=state["tail"] if state is not None else None, row_seq=batch.row_seq, row_pos=batch.row_pos,
                              taps=self.taps, dtype=dtype, **pa)
        else:
            width = x32.shape[-1]
            hn = model.buf("hn", (rows, width), torch.float32)
            ext.sandwich_norm(x32, w_out, mult, self.w_in, hn, rows, self.groups, self.eps, dtype=dtype, **pa)
            ext.conv_rows(hn, width, 0, self.conv_w, None, out, state["tail"], batch.spans_dev, batch.row_seq, batch.row_pos, width,
                          self.taps, residual=True)
