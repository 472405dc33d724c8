"""ExLlamaV2MoEMLP (reference moe_mlp.py:25-364): Mixtral-style sparse MLP over per-expert q_matrix handles.

The reference runs its fused extension path only for <= 4 rows and otherwise loops over experts in torch with a host
sync per layer (moe_mlp.py:238, 255-323).  Here the fused path (ext_c.q_moe_mlp_forward_) takes every decode-sized batch:
routing weights stay on the device, each expert's kernels see all rows and skip the ones not routed to them."""
from __future__ import annotations

import torch

from .ext import none_tensor
from .linear import ExLlamaV2Linear


class ExLlamaV2MoEMLP:
    def __init__(self, model, key: str, layer_idx: int, num_experts: int, num_experts_per_token: int):
        cfg = model.config
        self.model, self.ext, self.key, self.layer_idx = model, model.ext, key, layer_idx
        self.num_experts, self.num_experts_per_token = num_experts, num_experts_per_token
        h, inter = cfg.hidden_size, cfg.intermediate_size
        mk = lambda e, name, k, n: ExLlamaV2Linear(self.ext, f"{key}.block_sparse_moe.experts.{e}.{name}", k, n, model)
        self.w1 = [mk(e, "w1", h, inter) for e in range(num_experts)]       # gate projection
        self.w2 = [mk(e, "w2", inter, h) for e in range(num_experts)]       # down projection
        self.w3 = [mk(e, "w3", h, inter) for e in range(num_experts)]       # up projection
        self.gate = None
        self.q_handle = None

    def load(self, ck: dict):
        cfg, m = self.model.config, self.model
        for lin in self.w1 + self.w2 + self.w3:
            lin.load(ck[lin.key])
        self.post_attention_layernorm = ck[self.key + ".post_attention_layernorm"]
        self.gate = ck[self.key + ".block_sparse_moe.gate"]                  # fp16 [E, hidden] (nn.Linear weight)
        self.temp_logits = torch.empty((m.max_rows, self.num_experts), dtype=torch.float16, device=m.device)
        self.q_handle = self.ext.make_q_moe_mlp(                             # moe_mlp.py:114-133
            self.post_attention_layernorm, none_tensor, True, cfg.norm_eps, self.gate, self.num_experts,
            self.num_experts_per_token, [l.q_handle for l in self.w1], [l.q_handle for l in self.w2],
            [l.q_handle for l in self.w3], m.temp_state, none_tensor, m.temp_a, m.temp_b, self.temp_logits, none_tensor,
            m.max_rows, False)
        return self

    def unload(self):
        if self.q_handle is not None:
            self.ext.free_q_moe_mlp(self.q_handle)
            self.q_handle = None
        for lin in self.w1 + self.w2 + self.w3:
            lin.unload()

    def forward(self, hidden_states: torch.Tensor):
        """moe_mlp.py:238-253: ext_c.q_moe_mlp_forward_ in place (x += sum_e w_e * down_e(act(gate_e n) * up_e n))."""
        h = hidden_states.shape[-1]
        self.ext.q_moe_mlp_forward_(self.q_handle, hidden_states.view(-1, h))
        return hidden_states


class ScoredMoEMLP:
    """Sparse MoE over unquantized experts with a score-corrected router and identity experts.

    Router: logits in fp32, scores = softmax over ALL router outputs; the `top` largest (score + correction) are chosen, their
    weights are the uncorrected scores divided by their sum, times `route_scale`.  The last `identity` router outputs are experts
    without tensors whose output is the token itself.  A real expert is the clamped gated unit
    W_down(g sigmoid(1.702 g) (u + 1)), g = min(W_gate h, limit), u = clamp(W_up h, +-limit), evaluated in the up projection's
    epilogue.  Few rows (decoding): every (token, choice) pair is one row that names its expert's slab.  Many rows: the pairs are
    listed per expert on the device and one grouped launch per projection runs all experts (no host round trip either way).
    forward returns (None, mixture): the weighted sum is taken inside the residual step's launch (rmsnorm.PostNorm)."""

    PAIR_ROWS_MAX = 64                                   # (token, choice) pairs up to which rows pick their slab individually

    def __init__(self, model, key: str, layer_idx: int, *, experts: int, identity: int, top: int, route_scale: float, ff: int,
                 limit: float):
        self.model, self.ext, self.key, self.layer_idx = model, model.ext, key, layer_idx
        self.experts, self.identity, self.top, self.route_scale, self.ff, self.limit = experts, identity, top, route_scale, ff, limit

    def load(self, get):
        from .dense_linear import DenseLinear
        E = self.experts
        self.router = DenseLinear(self.ext, self.key + ".router", get("router"))
        if self.router.out_features != E + self.identity:
            raise RuntimeError(f"{self.key}: router has {self.router.out_features} outputs for {E} + {self.identity} experts")
        self.correction = get("correction").to(torch.float32).contiguous()
        if E:
            stack = lambda name: torch.stack([get(f"e{e}.{name}") for e in range(E)], 0)
            self.gate = DenseLinear(self.ext, self.key + ".gate", stack("gate"))
            self.up = DenseLinear(self.ext, self.key + ".up", stack("up"))
            self.down = DenseLinear(self.ext, self.key + ".down", stack("down"))
        return self

    def weight_bytes(self) -> int:
        """bytes one token streams: the router and `top` experts (an upper bound when identity experts are chosen)"""
        n = self.router.weight_bytes()
        if self.experts:
            n += (self.gate.weight_bytes() + self.up.weight_bytes() + self.down.weight_bytes()) // self.experts * min(self.top, self.experts)
        return n

    def forward(self, xh: torch.Tensor, rows: int):
        ext, m = self.ext, self.model
        E, top, ff, width = self.experts, self.top, self.ff, m.width
        dev, dt = m.device, m.dtype
        n_total = E + self.identity
        logits = self.router.forward(xh, rows, out=m.buf("moe.logits", (rows, n_total), torch.float32))
        ids = m.buf("moe.ids", (rows, top), torch.int32)
        wts = m.buf("moe.wts", (rows, top), torch.float32)
        pairs = rows * top
        grouped = pairs > self.PAIR_ROWS_MAX and E > 0
        groups = None
        if grouped:
            groups = (m.buf("moe.count", (E,), torch.int32), m.buf("moe.offset", (E,), torch.int32), m.buf("moe.rows", (pairs,), torch.int32))
        ext.moe_route_scored(logits, self.correction, ids, wts, rows, n_total, top, self.route_scale, E, groups=groups)
        if E == 0:
            return None, (None, ids, wts, 0)
        g = m.buf("ff.g", (pairs, ff), torch.float32)
        a = m.buf("ff.a", (pairs, ff), dt)
        y = m.buf("ff.y", (pairs, width), torch.float32)
        if grouped:
            kw = dict(batch=E, groups=groups)
        else:
            kw = dict(w_sel=ids.view(-1), n_sel=E)
        ext.dense_linear(xh, self.gate.weight, g, pairs, ff, width, width, width, ff, swb=ff * width, x_div=top, **kw)
        ext.dense_linear(xh, self.up.weight, a, pairs, ff, width, width, width, ff, swb=ff * width, x_div=top,
                         aux=g, ldaux=ff, epi=ext.EPI_CLAMPED_GLU, limit=self.limit, **kw)
        ext.dense_linear(a, self.down.weight, y, pairs, width, ff, ff, ff, width, swb=width * ff, **kw)
        return None, (y, ids, wts, E)


class SigmoidMoEMLP:
    """Sparse MoE whose router scores every expert on its own: s = sigmoid(W_router h) in fp32, the `top` largest are chosen and
    weigh their experts as they are (no renormalisation).  The weight multiplies the expert's INPUT: the token's part is
    sum_e expert_e(s_e h), expert(z) = W_down act(W_up z) with act = relu^2 and no gate matrix; since W_up (s h) = s (W_up h) the
    up projection runs on h and the weight enters in its epilogue, in front of the activation (csrc/dense.hip).  A shared expert of
    the same form (its own width) runs for every token: as wide as the routed ones it is stacked behind them and rides their
    launches as one more pair per token, otherwise it runs as a feed-forward of its own.  `act="silu_glu"`: experts are gated units
    W_down (silu(W_gate z) * W_up z); with z = s h the gate launch leaves silu(s g) s and the up launch multiplies by it, so both
    matrices still run on h.  Few rows: every (token, choice) pair names its expert's slab; many rows:
    one grouped launch per projection.  forward returns (y | None, mixture): y is the shared expert's output, the chosen experts'
    rows are added by the residual step's launch (rmsnorm.PreShiftRMSNorm)."""

    PAIR_ROWS_MAX = 64

    def __init__(self, model, key: str, layer_idx: int, *, experts: int, top: int, ff: int, shared_ff: int | None, route_scale: float = 1.0,
                 act: str = "relu2"):
        self.model, self.ext, self.key, self.layer_idx = model, model.ext, key, layer_idx
        self.experts, self.top, self.ff, self.shared_ff, self.route_scale = experts, top, ff, shared_ff, route_scale
        self.glu = act == "silu_glu"
        if not 0 < top <= experts:
            raise ValueError(f"{key}: top {top} of {experts} experts")
        if act not in ("relu2", "silu_glu"):
            raise ValueError(f"{key}: unknown expert form '{act}'")

    def load(self, get):
        from .dense_linear import DenseLinear
        from .mlp import DenseActMLP, DenseGatedMLP
        E, width = self.experts, self.model.width
        self.router = DenseLinear(self.ext, self.key + ".router", get("router"))
        # a shared expert as wide as the routed ones is stacked behind them as expert E: the router's launch names it for every token
        # with weight 1 and the two expert launches run it with the chosen ones
        self.merged = bool(self.shared_ff) and self.shared_ff == self.ff
        names = [f"e{e}" for e in range(E)] + (["shared"] if self.merged else [])
        stack = lambda name: torch.stack([get(f"{n}.{name}") for n in names], 0)
        self.up = DenseLinear(self.ext, self.key + ".up", stack("up"))
        self.down = DenseLinear(self.ext, self.key + ".down", stack("down"))
        self.gate = DenseLinear(self.ext, self.key + ".gate", stack("gate")) if self.glu else None
        self.slabs = len(names)
        if tuple(self.router.weight.shape) != (E, width) or tuple(self.up.weight.shape) != (self.slabs, self.ff, width) \
                or tuple(self.down.weight.shape) != (self.slabs, width, self.ff) \
                or (self.glu and tuple(self.gate.weight.shape) != (self.slabs, self.ff, width)):
            raise RuntimeError(f"{self.key}: tensor shapes do not match the feed-forward's sizes")
        self.shared = None
        if self.shared_ff and not self.merged:
            form = DenseGatedMLP if self.glu else DenseActMLP
            self.shared = form(self.model, self.key + ".shared", self.layer_idx).load(lambda n: get("shared." + n))
            if self.shared.up.out_features != self.shared_ff:
                raise RuntimeError(f"{self.key}: the shared expert is {self.shared.up.out_features} wide, config says {self.shared_ff}")
        return self

    def weight_bytes(self) -> int:
        per_slab = (self.up.weight_bytes() + self.down.weight_bytes() + (self.gate.weight_bytes() if self.glu else 0)) // self.slabs
        n = self.router.weight_bytes() + per_slab * (self.top + int(self.merged))
        return n + (self.shared.weight_bytes() if self.shared is not None else 0)

    def forward(self, xh: torch.Tensor, rows: int):
        ext, m = self.ext, self.model
        E, top, ff, width, dt = self.experts, self.top, self.ff, m.width, m.dtype
        logits = self.router.forward(xh, rows, out=m.buf("moe.logits", (rows, E), torch.float32))
        per_row, S = top + int(self.merged), self.slabs          # (token, expert) pairs per row; weight slabs
        ids = m.buf("moe.ids", (rows, per_row), torch.int32)
        wts = m.buf("moe.wts", (rows, per_row), torch.float32)
        pairs = rows * per_row
        grouped = pairs > self.PAIR_ROWS_MAX
        groups = None
        if grouped:
            groups = (m.buf("moe.count", (S,), torch.int32), m.buf("moe.offset", (S,), torch.int32), m.buf("moe.rows", (pairs,), torch.int32))
        ext.moe_route_sigmoid(logits, ids, wts, rows, E, top, self.route_scale, groups=groups, shared_slot=self.merged)
        a = m.buf("moe.a", (pairs, ff), dt)
        y = m.buf("moe.y", (pairs, width), torch.float32)
        kw = dict(batch=S, groups=groups) if grouped else dict(w_sel=ids.view(-1), n_sel=S)
        if self.glu:
            g = m.buf("moe.g", (pairs, ff), torch.float32)
            ext.dense_linear(xh, self.gate.weight, g, pairs, ff, width, width, width, ff, swb=ff * width, x_div=per_row,
                             aux=wts, ldaux=1, epi=ext.EPI_ROW_SCALED_SILU_SCALED, **kw)
            ext.dense_linear(xh, self.up.weight, a, pairs, ff, width, width, width, ff, swb=ff * width, x_div=per_row,
                             aux=g, ldaux=ff, epi=ext.EPI_AUX_MUL, **kw)
        else:
            ext.dense_linear(xh, self.up.weight, a, pairs, ff, width, width, width, ff, swb=ff * width, x_div=per_row,
                             aux=wts, ldaux=1, epi=ext.EPI_ROW_SCALED_RELU_SQUARED, **kw)
        ext.dense_linear(a, self.down.weight, y, pairs, width, ff, ff, ff, width, swb=width * ff, **kw)
        ys = self.shared.forward(xh, rows)[0] if self.shared is not None else None
        return ys, (y, ids, wts, S)
