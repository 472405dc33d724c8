"""Model hyper-parameters the hot path needs (subset of the reference's ExLlamaV2Config, config.py:58-196)."""
from __future__ import annotations

from dataclasses import dataclass, field


@dataclass
class ExLlamaV2Config:
    hidden_size: int = 4096
    intermediate_size: int = 11008
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    num_key_value_heads: int = 32
    head_dim: int = 128
    vocab_size: int = 32000
    max_seq_len: int = 4096
    norm_eps: float = 1e-5
    rotary_embedding_base: float = 10000.0
    rope_style: int = 2                     # RopeStyle.NEOX (architecture.py:109-112)
    max_batch_size: int = 1
    max_input_len: int = 2048               # chunk size of forward (config.py:196, model.py:833)
    arch: str = "llama"
    num_experts: int = 0                    # > 0: Mixtral-style sparse MLP (moe_mlp.py), experts per token below
    num_experts_per_token: int = 2

    @staticmethod
    def llama2_7b(**kw):
        return ExLlamaV2Config(**kw)

    @staticmethod
    def tinyllama_1b(**kw):
        return ExLlamaV2Config(hidden_size=2048, intermediate_size=5632, num_hidden_layers=22, num_attention_heads=32,
                               num_key_value_heads=4, head_dim=64, vocab_size=32000, max_seq_len=2048, **kw)

    @staticmethod
    def llama2_70b(**kw):
        return ExLlamaV2Config(hidden_size=8192, intermediate_size=28672, num_hidden_layers=80, num_attention_heads=64,
                               num_key_value_heads=8, head_dim=128, **kw)

    @staticmethod
    def mixtral_8x7b(**kw):
        return ExLlamaV2Config(hidden_size=4096, intermediate_size=14336, num_hidden_layers=32, num_attention_heads=32,
                               num_key_value_heads=8, head_dim=128, vocab_size=32000, num_experts=8,
                               num_experts_per_token=2, arch="mixtral", **kw)

    @staticmethod
    def tiny_test(**kw):
        d = dict(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                 num_key_value_heads=2, head_dim=64, vocab_size=320, max_seq_len=512, max_input_len=64)
        d.update(kw)
        return ExLlamaV2Config(**d)


@dataclass
class LayeredConfig:
    """A model described layer by layer in its config.json: `layers` is a list of {"type": <mixer kind>, "mixer": {sizes},
    "mlp": {"kind": "dense" | "moe", ...} | None}; tensors of layer i are named `l<i>.*`.  Every size and constant comes from
    the file (or a tensor's shape); nothing is assumed equal across layers."""
    architecture: str = ""
    vocab: int = 0
    width: int = 0
    norm_eps: float = 1e-5
    postln_alpha: float = 1.0
    embedding_scale: float = 1.0
    layers: list = field(default_factory=list)
    # "post_rms": x <- rms_norm(alpha x + f(x)) (1 + w);  "pre_ln": x <- x + f(layer_norm(x));
    # "pre_rms_shift": x <- x + f(shift(rms_norm(x) * g)), g ONE number per norm, shift = a blend with the previous token's normed row
    residual: str = "post_rms"
    tied_head: bool = False           # logits from the embedding table itself (no `head` tensor)
    logit_softcap: float = 0.0        # > 0: logits <- c tanh(logits / c)
    logit_scale: float = 1.0          # logits <- logits * s
    attention_mask: str = "window"    # what an attention layer's mask.size means: "window" (sliding) or "chunk" (blocks from position 0)
    # "sandwich": x <- x + residual_mult * n_g(f(conv_in(n_g(x) w_in))) w_out with RMS norms over `norm_groups` equal runs of the row and
    # a causal convolution of `input_conv_taps` taps beside the identity in front of every sublayer (0: none)
    norm_groups: int = 1
    residual_mult: float = 1.0
    input_conv_taps: int = 0
    pair_embedding: dict | None = None   # {"buckets", "mul_prev", "mul_cur"}: a hashed (previous token, token) table added to the embedding

    @staticmethod
    def from_dict_prenorm(d: dict) -> "LayeredConfig":
        """pre-norm stacks with layer norms (weight and bias), a tied output table and an optional soft cap on the logits"""
        try:
            cfg = LayeredConfig(architecture=str(d["architecture"]), vocab=int(d["vocab"]), width=int(d["width"]),
                                norm_eps=float(d["norm"]["eps"]), embedding_scale=float(d["embedding"]["scale"]),
                                layers=list(d["layers"]), residual="pre_ln", tied_head=True,
                                logit_softcap=float(d.get("logit_softcap") or 0.0))
        except KeyError as e:
            raise RuntimeError(f"config.json: missing key {e}") from e
        if cfg.vocab <= 0 or cfg.width <= 0 or not cfg.layers:
            raise RuntimeError("config.json: vocab, width and layers must be given")
        return cfg

    @staticmethod
    def from_dict_prerms_shift(d: dict) -> "LayeredConfig":
        """pre-norm stacks with scalar-gain RMS norms and a token shift in front of every mixer, a `head` matrix and scaled logits"""
        try:
            cfg = LayeredConfig(architecture=str(d["architecture"]), vocab=int(d["vocab"]), width=int(d["width"]),
                                norm_eps=float(d["norm"]["eps"]), layers=list(d["layers"]), residual="pre_rms_shift",
                                logit_scale=float(d.get("logit_scale", 1.0)), attention_mask="chunk")
        except KeyError as e:
            raise RuntimeError(f"config.json: missing key {e}") from e
        if cfg.vocab <= 0 or cfg.width <= 0 or not cfg.layers:
            raise RuntimeError("config.json: vocab, width and layers must be given")
        return cfg

    @staticmethod
    def from_dict_sandwich(d: dict) -> "LayeredConfig":
        """stacks whose sublayers stand between two grouped RMS norms behind a short input convolution, with a scaled residual branch,
        a token-pair table beside the embedding and a `head` matrix"""
        try:
            emb = d["embedding"]
            pair = emb.get("bigram")
            cfg = LayeredConfig(architecture=str(d["architecture"]), vocab=int(d["vocab"]), width=int(d["width"]),
                                norm_eps=float(d["norm"]["eps"]), norm_groups=int(d["norm"].get("groups", 1)),
                                embedding_scale=float(emb.get("scale", 1.0)), layers=list(d["layers"]), residual="sandwich",
                                residual_mult=float(d.get("residual_mult", 1.0)), input_conv_taps=int((d.get("canon") or {}).get("taps", 0)),
                                pair_embedding=({"buckets": int(pair["buckets"]), "mul_prev": int(pair["mul_prev"]),
                                                 "mul_cur": int(pair["mul_cur"])} if pair else None))
        except KeyError as e:
            raise RuntimeError(f"config.json: missing key {e}") from e
        if cfg.vocab <= 0 or cfg.width <= 0 or not cfg.layers:
            raise RuntimeError("config.json: vocab, width and layers must be given")
        if cfg.norm_groups <= 0 or cfg.width % cfg.norm_groups:
            raise RuntimeError(f"config.json: {cfg.width} values do not split into {cfg.norm_groups} norm groups")
        if cfg.pair_embedding is not None and cfg.pair_embedding["buckets"] <= 0:
            raise RuntimeError("config.json: the token-pair table needs a positive number of buckets")
        return cfg

    @staticmethod
    def from_dict(d: dict) -> "LayeredConfig":
        try:
            cfg = LayeredConfig(architecture=str(d["architecture"]), vocab=int(d["vocab"]), width=int(d["width"]),
                                norm_eps=float(d["norm"]["eps"]), postln_alpha=float(d["postln_alpha"]),
                                embedding_scale=float(d["embedding"]["scale"]), layers=list(d["layers"]))
        except KeyError as e:
            raise RuntimeError(f"config.json: missing key {e}") from e
        if cfg.vocab <= 0 or cfg.width <= 0 or not cfg.layers:
            raise RuntimeError("config.json: vocab, width and layers must be given")
        return cfg
