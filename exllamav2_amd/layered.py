"""Config-driven decoder stack over unquantized weights: each layer is a mixer and an optional feed-forward taken from two
registries, on an fp32 residual stream.  The residual style is the configuration's: post-norm steps
x <- norm(alpha x + sublayer(x)) (1 + w)  (RMS norm, a `head` matrix), or pre-norm steps  x <- x + sublayer(layer_norm(x))  (weight and
bias, logits from the embedding table, optional soft cap), or pre-norm steps with scalar-gain RMS norms and a token shift in front
of every mixer (a `head` matrix, scaled logits), or sandwich-normed steps  x <- x + mult n_g(sublayer(conv_in(n_g(x) w))) w'  with
grouped RMS norms, a short input convolution and a token-pair table beside the embedding.  Mixers: latent attention, windowed /
chunked / plain causal attention (pooled blocks, sinks, shared keys and values), state-space scan, decaying linear attention, linear
attention whose forget gate writes, gated delta rule, two mixers side by side; a stack may mix them -- each keeps what it needs between steps (pages
of keys and values, per-slot recurrent state) under one page pool.

The model has ONE forward, `step(batch, cache)`: the rows of a step are a flat list of tokens, each with its sequence slot and
position, so whole prompts, portions of prompts and single decoded tokens of several requests run through the same launches
(exllamav2_amd.engine builds the batches).  Operand dtype bfloat16 (weights, linear inputs, cache rows; fp32 accumulation) or
float32 (everything in true 32-bit); norms, softmax, routing, rotation and the residual stream are fp32 in both."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .cache import LatentCache, LayerStates, PagePool
from .config import LayeredConfig
from .dense_linear import DenseLinear
from .ext import ext_c
from .latent_attn import LatentAttention
from .linear_attn import ForgetGateLinearAttention, GatedDeltaRule
from .mlp import DenseActMLP, DenseGatedMLP
from .moe_mlp import ScoredMoEMLP, SigmoidMoEMLP
from .parallel_mixer import ParallelMixer
from .rmsnorm import PostNorm, PreLayerNorm, PreShiftRMSNorm, SandwichNorm
from .ssm import StateSpaceMixer
from .window_attn import WindowAttention
from .wkv import DecayLinearAttention


def _latent_attention(model, key, idx, spec):
    m = spec["mixer"]
    return LatentAttention(model, key, idx, heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
                           kv_rank=int(m["kv_rank"]), q_rank=int(m["q_rank"]), window=int(m["mask"]["size"]),
                           rot_base=float(m["rot"]["base"]), rot_dims=int(m["rot"]["dims"]), scale=float(m["scale"]),
                           kv_from=(int(m["kv_from"]) if m.get("kv_from") is not None else None))


def _window_attention(model, key, idx, spec):
    m = spec["mixer"]
    mask, rot = m.get("mask") or {}, m.get("rot") or {}
    common = dict(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads") or m["heads"]), dim=int(m["dim"]), vdim=int(m.get("vdim") or m["dim"]),
                  rot_base=float(rot.get("base", 10000.0)), rot_dims=int(rot.get("dims", 0)), rot_scaling=rot.get("scaling"),
                  scale=float(m["scale"]))
    if model.config.attention_mask == "chunk":
        # chunks from position 0, capped scores, a constant 1 in the softmax denominator, values as they are, maybe another layer's rows
        return WindowAttention(model, key, idx, window=1 << 30, pool=0, chunk=int(mask.get("size") or 0), softcap=float(m.get("softcap") or 0.0),
                               sink_one=True, rotate_values=False, kv_from=(int(m["kv_from"]) if m.get("kv_from") is not None else None),
                               **common)
    return WindowAttention(model, key, idx, window=int(mask.get("size") or (1 << 30)), pool=int(mask.get("pool") or 0), **common)


def _decay_linear_attention(model, key, idx, spec):
    m = spec["mixer"]
    return DecayLinearAttention(model, key, idx, heads=int(m["heads"]), dim=int(m["dim"]))


def _state_space(model, key, idx, spec):
    m = spec["mixer"]
    return StateSpaceMixer(model, key, idx, heads=int(m["heads"]), vdim=int(m["vdim"]), state=int(m["state"]),
                           groups=int(m.get("groups", 1)), norm_groups=int(m.get("norm_groups", 1)), taps=int(m["conv"]))


def _causal_attention(model, key, idx, m, out_tag="mix.y"):
    """plain causal softmax attention: every earlier token is visible, no sink, no gate, values as they are"""
    rot = m.get("rot") or {}
    return WindowAttention(model, key, idx, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads") or m["heads"]), dim=int(m["dim"]),
                           vdim=int(m.get("vdim") or m["dim"]), window=1 << 30, pool=0, rot_base=float(rot.get("base", 10000.0)),
                           rot_dims=int(rot.get("dims", 0)), rot_scaling=rot.get("scaling"), scale=float(m["scale"]), rotate_values=False,
                           out_tag=out_tag)


def _parallel(model, key, idx, spec):
    """softmax attention (left) beside a state-space scan (right) on the same input"""
    m = spec["mixer"]
    r = m["right"]
    left = _causal_attention(model, key + ".left", (idx, "left"), m["left"], out_tag="mix.y.left")
    right = StateSpaceMixer(model, key + ".right", (idx, "right"), heads=int(r["heads"]), vdim=int(r["vdim"]), state=int(r["state"]),
                            groups=int(r.get("groups", 1)), norm_groups=int(r.get("norm_groups", 1)), taps=int(r["conv"]),
                            out_tag="mix.y.right")
    return ParallelMixer(model, key, idx, left, right, float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0)))


def _forget_gate_attention(model, key, idx, spec):
    m = spec["mixer"]
    return ForgetGateLinearAttention(model, key, idx, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]))


def _delta_rule(model, key, idx, spec):
    m = spec["mixer"]
    return GatedDeltaRule(model, key, idx, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads") or m["heads"]), dim=int(m["dim"]),
                          vdim=int(m["vdim"]), taps=int(m["conv"]))


def _dense_mlp(model, key, idx, spec):
    if model.config.residual == "pre_ln":                      # two matrices, squared relu between them
        return DenseActMLP(model, key, idx)
    return DenseGatedMLP(model, key, idx)


def _moe_mlp(model, key, idx, spec):
    r, e = spec["router"], spec["expert"]
    if model.config.residual in ("pre_rms_shift", "sandwich"):        # sigmoid scores weigh the experts' inputs; a shared expert beside them
        shared = spec.get("shared")
        return SigmoidMoEMLP(model, key, idx, experts=int(r["experts"]), top=int(r["top"]), ff=int(e["ff"]),
                             shared_ff=(int(shared["ff"]) if shared else None), route_scale=float(r.get("scale", 1.0)),
                             act="silu_glu" if model.config.residual == "sandwich" else "relu2")
    return ScoredMoEMLP(model, key, idx, experts=int(r["experts"]), identity=int(r.get("identity", 0)), top=int(r["top"]),
                        route_scale=float(r["scale"]), ff=int(e["ff"]), limit=float(e["limit"]))


# config `type` -> builder(model, key, layer index, layer spec)
MIXERS = {"latent_attention": _latent_attention, "attention": _window_attention, "mamba2": _state_space, "wkv": _decay_linear_attention,
          "parallel": _parallel, "hgrn2": _forget_gate_attention, "delta": _delta_rule}
FEED_FORWARDS = {"dense": _dense_mlp, "moe": _moe_mlp}       # config `mlp.kind` -> builder(model, key, layer index, mlp spec)


SPAN_CHUNK = 64                                           # rows per chunk of the chunked scan (csrc/ssm.hip: SSD_L)


@dataclass
class StepBatch:
    """Device-side description of one step: int32 tensors ids / row_seq / row_pos [rows], block_table [slots, pages],
    logit_rows [n_logits] (rows whose logits are wanted)."""
    ids: torch.Tensor
    row_seq: torch.Tensor
    row_pos: torch.Tensor
    block_table: torch.Tensor
    logit_rows: torch.Tensor
    rows: int
    n_logits: int
    # rows grouped for tiled attention kernels: portions of prompts in tiles of <= 16 consecutive positions of one sequence
    # (row0 int32 [n], rows int32 [n], n) and single decoded tokens (row0 int32 [n], n, largest position among them)
    tiles16: tuple | None = None
    tiles1: tuple | None = None
    # the portions of prompts again in tiles of <= 64 consecutive positions (row0 int32 [n], rows int32 [n], n, tile size)
    prompt_tiles: tuple | None = None
    # the runs of consecutive rows that one sequence brings (recurrent mixers walk them in order): (first row int32 [n],
    # rows int32 [n], n, longest run)
    spans_dev: tuple | None = None
    # the spans cut into chunks of SPAN_CHUNK rows: (number of chunks in front of each span int32 [n], SPAN_CHUNK, chunks in all)
    span_chunks: tuple | None = None
    # host-side view of the same rows, one tuple per request in the step: (first row, rows, sequence slot, first position)
    spans: list | None = None
    # logit_rows is 0 .. rows - 1 in order (every row's logits are wanted, as in decoding): a model may skip the gather
    logits_all_rows: bool = False


class LayeredModel:
    graph_safe_step = True                                # step() is launches on device-resident inputs only: an engine may capture it

    def __init__(self, config: LayeredConfig, device="cuda:0", dtype=torch.bfloat16, ext=None):
        if dtype not in (torch.bfloat16, torch.float32):
            raise RuntimeError("LayeredModel: operand dtype is bfloat16 or float32")
        self.config, self.device, self.dtype, self.ext = config, torch.device(device), dtype, ext or ext_c
        self.width, self.vocab, self.norm_eps = config.width, config.vocab, config.norm_eps
        self.layers = []
        self.loaded = False
        self._scratch = {}
        self.scratch_epoch = 0                            # counts (re)allocations of scratch buffers: a graph captured before one is stale
        self.frozen = False                               # True while a step is being captured into a graph: scratch may not grow

    def buf(self, tag: str, shape, dtype) -> torch.Tensor:
        """A view of the model's scratch arena: one persistent buffer per tag (grown on demand), so the addresses a step uses stay
        the same from step to step -- what a captured graph needs -- and nothing is allocated on the hot path.  Tags are unique
        among the buffers that are alive at the same time; layers run one after the other and share them."""
        n = 1
        for d in shape:
            n *= int(d)
        t = self._scratch.get(tag)
        if t is None or t.dtype is not dtype or t.numel() < n:
            if self.frozen:
                raise RuntimeError(f"scratch buffer '{tag}' would have to grow while a step is being captured")
            t = torch.empty((max(n, 1),), dtype=dtype, device=self.device)
            self._scratch[tag] = t
            self.scratch_epoch += 1
        return t[:n].view(*shape)

    # ---- loading --------------------------------------------------------------------------------------------------------------

    def load(self, tensors: dict):
        """tensors: name -> device tensor as stored (bfloat16 weights); converted once to the operand dtype"""
        cfg = self.config
        conv = lambda t: t.to(self.dtype).contiguous() if t.is_floating_point() else t

        def need(name, optional=False):
            if name not in tensors:
                if optional:
                    return None
                raise RuntimeError(f"checkpoint has no tensor '{name}'")
            return conv(tensors[name])

        self.embed = need("embed")
        if tuple(self.embed.shape) != (cfg.vocab, cfg.width):
            raise RuntimeError(f"embed is {tuple(self.embed.shape)}, config says {(cfg.vocab, cfg.width)}")
        pre = cfg.residual in ("pre_ln", "pre_rms_shift", "sandwich")

        def make_norm(name, shift=None):
            if cfg.residual == "sandwich":
                # `<layer>.norm1` / `.norm2` in front of a sublayer, `.norm1b` / `.norm2b` behind it, `.canon1` / `.canon2` its input convolution
                inner = name != "final.norm"
                conv = need(name.replace("norm", "canon"), optional=cfg.input_conv_taps <= 0) if inner else None
                return SandwichNorm(self.ext, name, need(name), need(name + "b") if inner else None, conv,
                                    cfg.norm_groups, cfg.norm_eps, cfg.residual_mult)
            if cfg.residual == "pre_rms_shift":
                return PreShiftRMSNorm(self.ext, name, need(name), cfg.norm_eps, shift=need(shift) if shift else None)
            if pre:
                return PreLayerNorm(self.ext, name, need(name), need(name + ".b") if name + ".b" in tensors else None, cfg.norm_eps)
            return PostNorm(self.ext, name, need(name), cfg.norm_eps, cfg.postln_alpha)

        self.layers = []
        for i, spec in enumerate(cfg.layers):
            key = f"l{i}"
            if spec["type"] not in MIXERS:
                raise RuntimeError(f"layer {i}: unknown mixer type '{spec['type']}' (known: {sorted(MIXERS)})")
            mixer = MIXERS[spec["type"]](self, key, i, spec).load(lambda n, optional=False, k=key: need(f"{k}.mix.{n}", optional))
            norm1 = make_norm(key + ".norm1", shift=(key + ".shift") if cfg.residual == "pre_rms_shift" else None)
            ff, norm2 = None, None
            ms = spec.get("mlp")
            if ms is not None:
                if ms["kind"] not in FEED_FORWARDS:
                    raise RuntimeError(f"layer {i}: unknown feed-forward kind '{ms['kind']}' (known: {sorted(FEED_FORWARDS)})")
                ff = FEED_FORWARDS[ms["kind"]](self, key + ".mlp", i, ms).load(lambda n, k=key: need(f"{k}.mlp.{n}"))
            if ff is not None or (not pre and key + ".norm2" in tensors):
                norm2 = make_norm(key + ".norm2")
            self.layers.append((mixer, norm1, ff, norm2))
        for i, (mixer, *_rest) in enumerate(self.layers):
            j = getattr(mixer, "kv_from", None)
            if j is not None:
                if not (0 <= j < len(self.layers)) or getattr(self.layers[j][0], "kv_from", 0) is not None:
                    raise RuntimeError(f"layer {i}: kv_from {j} does not name a layer with keys and values of its own")
                src = self.layers[j][0]
                if hasattr(mixer, "check_kv_source"):
                    if j >= i:
                        raise RuntimeError(f"layer {i}: kv_from {j} must name an earlier layer (its rows of the step are cached first)")
                    mixer.check_kv_source(src)
                elif (src.kv_rank, src.rot_dim, src.rot_dims, src.rot_base) != (mixer.kv_rank, mixer.rot_dim, mixer.rot_dims, mixer.rot_base):
                    raise RuntimeError(f"layer {i}: its latent sizes / rotation differ from layer {j}'s, whose cache it reads")
        if pre:
            self.final_norm = make_norm("final.norm")
            # the sublayers in order, each with the norm in front of it: (norm, module, is a mixer)
            self.sublayers = []
            for i, (mixer, norm1, ff, norm2) in enumerate(self.layers):
                self.sublayers.append((norm1, mixer, True, i))
                if ff is not None:
                    self.sublayers.append((norm2, ff, False, i))
        else:
            self.final_norm = need("final.norm")
        self.pair_table = self.embed_norm = None
        if cfg.residual == "sandwich":
            self.embed_norm = need("embed.norm")
            if cfg.pair_embedding is not None:
                self.pair_table = need("bigram")
                if tuple(self.pair_table.shape) != (cfg.pair_embedding["buckets"] + 1, cfg.width):
                    raise RuntimeError(f"bigram is {tuple(self.pair_table.shape)}, config says {(cfg.pair_embedding['buckets'] + 1, cfg.width)}")
        self.head = DenseLinear(self.ext, "head", self.embed if cfg.tied_head else need("head"))
        self.loaded = True
        return self

    def weight_bytes(self) -> int:
        """bytes a decoded token streams (a tied output table counts once: the embedding reads one row of it)"""
        n = self.head.weight_bytes()
        for mixer, _n1, ff, _n2 in self.layers:
            n += mixer.weight_bytes() + (ff.weight_bytes() if ff is not None else 0)
        return n

    # ---- cache ----------------------------------------------------------------------------------------------------------------

    def make_cache(self, pool: PagePool):
        if any(hasattr(mixer, "make_state") or hasattr(mixer, "make_states") for mixer, *_rest in self.layers):
            norm_states = {i: norm1.make_state(pool, self.width) for i, (_m, norm1, *_r) in enumerate(self.layers) if hasattr(norm1, "make_state")}
            norm_states.update({(i, "ff"): norm2.make_state(pool, self.width) for i, (_m, _n1, _ff, norm2) in enumerate(self.layers)
                                if norm2 is not None and hasattr(norm2, "make_state")})
            if getattr(self, "pair_table", None) is not None:
                from .cache import SlotState
                norm_states["embed"] = SlotState(pool, {"prev_token": ()}, dtype=torch.int32)
            per_layer = {}
            for i, (mixer, *_rest) in enumerate(self.layers):
                if hasattr(mixer, "make_states"):                 # several states under keys of the mixer's own ((layer, "left"), ...)
                    per_layer.update(mixer.make_states(pool, self.dtype))
                else:
                    per_layer[i] = mixer.make_state(pool, self.dtype)
            return LayerStates(pool, per_layer, norm_states=norm_states)
        widths, owner = {}, {}
        for i, (mixer, *_rest) in enumerate(self.layers):
            if mixer.kv_from is None:
                widths[i] = mixer.cache_row_width
                owner[i] = i
            else:
                owner[i] = mixer.kv_from
        return LatentCache(pool, widths, owner, self.dtype)

    # ---- forward ----------------------------------------------------------------------------------------------------------------

    def step(self, batch: StepBatch, cache) -> torch.Tensor | None:
        """Runs the batch's rows through all layers, appending to the cache; returns fp32 logits [n_logits, vocab] (None if
        no row wants them)."""
        ext, cfg, rows = self.ext, self.config, batch.rows
        if cfg.residual == "pre_ln":
            return self._step_pre_norm(batch, cache)
        if cfg.residual == "pre_rms_shift":
            return self._step_pre_rms_shift(batch, cache)
        if cfg.residual == "sandwich":
            return self._step_sandwich(batch, cache)
        x32 = self.buf("x32", (rows, self.width), torch.float32)
        xh = x32 if self.dtype is torch.float32 else self.buf("xh", (rows, self.width), self.dtype)
        ext.embed_scale(self.embed, batch.ids, x32, xh, cfg.embedding_scale)
        for mixer, norm1, ff, norm2 in self.layers:
            y = mixer.forward(xh, rows, batch, cache)
            norm1.forward(x32, xh, y, rows)
            if norm2 is not None:
                if ff is None:
                    y, mix = self.buf("zero", (rows, self.width), torch.float32).zero_(), None
                else:
                    y, mix = ff.forward(xh, rows)
                norm2.forward(x32, xh, y, rows, moe=mix)
        if batch.n_logits == 0:
            return None
        xn = self.buf("xn", (batch.n_logits, self.width), self.dtype)
        ext.rms_rows(x32, self.width, self.final_norm, True, xn, self.width, batch.n_logits, self.width, cfg.norm_eps,
                     row_idx=batch.logit_rows)
        return self.head.forward(xn, batch.n_logits, out=self.buf("logits", (batch.n_logits, self.vocab), torch.float32))

    def _step_pre_norm(self, batch: StepBatch, cache) -> torch.Tensor | None:
        """x <- x + sublayer(layer_norm(x)): every residual addition runs in ONE launch with the layer norm of the sublayer that
        follows it; the last addition stands alone and the final norm is taken of the rows whose logits are wanted only."""
        ext, cfg, rows = self.ext, self.config, batch.rows
        x32 = self.buf("x32", (rows, self.width), torch.float32)
        xh = self.buf("xh", (rows, self.width), self.dtype)
        ext.embed_scale(self.embed, batch.ids, x32, None, cfg.embedding_scale)
        y = None
        for norm, module, is_mixer, _layer in self.sublayers:
            norm.forward(x32, y, xh, rows)
            y = module.forward(xh, rows, batch, cache) if is_mixer else module.forward(xh, rows)[0]
        if y is not None:
            ext.add_layer_norm(x32, y, None, None, None, rows, cfg.norm_eps)
        if batch.n_logits == 0:
            return None
        xn = self.buf("xn", (batch.n_logits, self.width), self.dtype)
        self.final_norm.forward(x32, None, xn, batch.n_logits, row_idx=batch.logit_rows)
        cap = cfg.logit_softcap
        return self.head.forward(xn, batch.n_logits, out=self.buf("logits", (batch.n_logits, self.vocab), torch.float32),
                                 epi=ext.EPI_SOFT_CAP if cap > 0 else ext.EPI_NONE, limit=cap)

    def _step_pre_rms_shift(self, batch: StepBatch, cache) -> torch.Tensor | None:
        """x <- x + mixer(shift(norm1(x))), x <- x + ff(norm2(x)) with scalar-gain RMS norms: as in the layer-norm stacks every
        residual addition -- a linear's output, a shared expert's, the chosen experts' rows -- runs in the launch of the norm that
        follows it, which also shifts the normed rows towards the previous token's (kept per slot) in front of a mixer.  A mixer
        that blends its input further (`input_f32`) gets fp32 rows.  Logits: head(norm(x)) * logit_scale, for the wanted rows."""
        ext, cfg, rows, f32 = self.ext, self.config, batch.rows, torch.float32
        x32 = self.buf("x32", (rows, self.width), f32)
        xh = self.buf("xh", (rows, self.width), self.dtype)
        ext.embed_scale(self.embed, batch.ids, x32, None, 1.0)
        multi = batch.spans_dev[3] > 1                        # spans of several rows: the shift reads the normed rows from a buffer
        pending = None
        for norm, module, is_mixer, layer in self.sublayers:
            if is_mixer:
                out = self.buf("xh32", (rows, self.width), f32) if getattr(module, "input_f32", False) else xh
                hn = self.buf("hn", (rows, self.width), f32) if multi else None
                norm.forward(x32, pending, out, rows, batch=batch, state=cache.norm_state(layer), hn=hn, dtype=self.dtype)
                pending = (module.forward(out, rows, batch, cache), None, 0)
            else:
                norm.forward(x32, pending, xh, rows, dtype=self.dtype)
                y, mix = module.forward(xh, rows)
                pending = (y, mix[0], mix[1].shape[-1]) if mix is not None else (y, None, 0)
        xn = self.buf("xn", (max(batch.n_logits, 1), self.width), self.dtype)
        if batch.logits_all_rows and batch.n_logits == rows:
            self.final_norm.forward(x32, pending, xn, rows, dtype=self.dtype)       # the last addition and the final norm in one launch
        else:
            if pending is not None:
                self.final_norm.forward(x32, pending, None, rows, dtype=self.dtype)
            if batch.n_logits == 0:
                return None
            self.final_norm.forward(x32, None, xn, batch.n_logits, row_idx=batch.logit_rows, dtype=self.dtype)
        scaled = cfg.logit_scale != 1.0
        return self.head.forward(xn, batch.n_logits, out=self.buf("logits", (batch.n_logits, self.vocab), f32),
                                 epi=ext.EPI_SCALE if scaled else ext.EPI_NONE, limit=cfg.logit_scale)

    def _step_sandwich(self, batch: StepBatch, cache) -> torch.Tensor | None:
        """x <- x + mult n_g(mixer(conv_in(n_g(x) w1))) w1b, x <- x + mult n_g(ff(conv_in(n_g(x) w2))) w2b: what lies between two
        sublayers -- the norm behind the first (over a linear's output, the weighted results of two mixers side by side, or a shared
        expert's output plus the chosen experts' rows), the residual addition, the norm in front of the second and, in steps of single
        tokens, its input convolution -- is one launch.  The embedding adds a row of the token-pair table chosen by the previous and the
        current token (the previous token is kept per slot) and is normed.  Logits: head(n_g(x) w) for the wanted rows."""
        ext, cfg, rows, f32 = self.ext, self.config, batch.rows, torch.float32
        x32 = self.buf("x32", (rows, self.width), f32)
        xh = self.buf("xh", (rows, self.width), self.dtype)
        pe = cfg.pair_embedding or {"buckets": 0, "mul_prev": 0, "mul_cur": 0}
        est = cache.norm_state("embed")
        nb = max(pe["buckets"], 1)                             # (the multipliers reduced first: the hash stays inside 64 bits)
        ext.embed_pair(self.embed, self.pair_table, self.embed_norm, batch.ids, est["prev_token"] if est is not None else None, batch.row_seq,
                       batch.row_pos, batch.spans_dev, x32, pe["buckets"], pe["mul_prev"] % nb, pe["mul_cur"] % nb, cfg.embedding_scale,
                       cfg.norm_groups, cfg.norm_eps)
        pending = None
        for norm, module, is_mixer, layer in self.sublayers:
            norm.forward(x32, pending, xh, rows, model=self, batch=batch, state=cache.norm_state(layer if is_mixer else (layer, "ff")),
                         dtype=self.dtype)
            if is_mixer:
                y = module.forward(xh, rows, batch, cache)
                pending = (norm,) + (tuple(y) if isinstance(y, tuple) else (y, 1.0, None, 1.0)) + (None, 0)
            else:
                y, mix = module.forward(xh, rows)
                pending = (norm, y, 1.0, None, 1.0) + ((mix[0], mix[1].shape[-1]) if mix is not None else (None, 0))
        xn = self.buf("xn", (max(batch.n_logits, 1), self.width), self.dtype)
        if batch.logits_all_rows and batch.n_logits == rows:
            self.final_norm.forward(x32, pending, xn, rows, dtype=self.dtype)       # the last addition and the final norm in one launch
        else:
            if pending is not None:
                self.final_norm.forward(x32, pending, None, rows, dtype=self.dtype)
            if batch.n_logits == 0:
                return None
            self.final_norm.forward(x32, None, xn, batch.n_logits, row_idx=batch.logit_rows, dtype=self.dtype)
        return self.head.forward(xn, batch.n_logits, out=self.buf("logits", (batch.n_logits, self.vocab), f32))
