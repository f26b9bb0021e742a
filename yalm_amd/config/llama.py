"""Typed configuration of the Llama / Mistral dense decoder, read from the keys of
the architecture's own config.json (the keys convert.py:22-54 reads, plus
`rope_scaling` and `sliding_window`, which the reference lacks)."""
from dataclasses import dataclass, field
from typing import List, Optional

from .spec import LayerSpec, ModelSpec, PartSpec


KV_SINKS = 2          # positions kept as attention sinks under a shortened context (src/model.h:12)


class ConfigError(ValueError):
    pass


@dataclass(frozen=True)
class RopeScaling:
    """The `rope_scaling` object of config.json; only the llama3 kind."""
    rope_type: str
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int

    @staticmethod
    def from_dict(d):
        kind = d.get("rope_type", d.get("type"))
        if kind in (None, "default"):
            return None
        if kind != "llama3":
            raise ConfigError("rope_scaling type %r is not supported (only 'llama3')" % (kind,))
        try:
            rs = RopeScaling("llama3", float(d["factor"]), float(d["low_freq_factor"]), float(d["high_freq_factor"]),
                             int(d["original_max_position_embeddings"]))
        except KeyError as e:
            raise ConfigError("rope_scaling lacks the key %s" % e) from None
        if rs.factor <= 0 or rs.high_freq_factor <= rs.low_freq_factor or rs.original_max_position_embeddings <= 0:
            raise ConfigError("rope_scaling has impossible values: %r" % (rs,))
        return rs

    def to_dict(self):
        return {"rope_type": self.rope_type, "factor": self.factor, "low_freq_factor": self.low_freq_factor,
                "high_freq_factor": self.high_freq_factor,
                "original_max_position_embeddings": self.original_max_position_embeddings}


@dataclass(frozen=True)
class LlamaConfig:
    architecture: str
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float = 10000.0
    partial_rotary_factor: float = 1.0
    rope_scaling: Optional[RopeScaling] = None
    sliding_window: int = 0                   # 0: every key is visible
    attention_sinks: int = 0                  # with a window: the first positions stay visible beside it
    tie_word_embeddings: bool = True
    hidden_act: str = "silu"
    bos_token_id: Optional[int] = None
    eos_token_ids: List[int] = field(default_factory=list)

    ARCHITECTURES = ("LlamaForCausalLM", "MistralForCausalLM")

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d):
        def need(key):
            if key not in d or d[key] is None:
                raise ConfigError("config.json lacks the key %r" % key)
            return d[key]

        archs = d.get("architectures") or []
        arch = archs[0] if archs else None
        if arch not in cls.ARCHITECTURES:
            raise ConfigError("architecture %r is not one of %s" % (arch, list(cls.ARCHITECTURES)))
        if d.get("attention_bias", False) or d.get("mlp_bias", False):
            raise ConfigError("attention_bias / mlp_bias are not supported")            # convert.py:48-49
        hidden = int(need("hidden_size"))
        heads = int(need("num_attention_heads"))
        head_dim = d.get("head_dim")
        head_dim = int(head_dim) if head_dim is not None else hidden // heads           # convert.py:34
        kv = d.get("num_key_value_heads")
        kv = int(kv) if kv is not None else heads                                        # convert.py:37
        eos = d.get("eos_token_id")
        eos_ids = [] if eos is None else ([int(e) for e in eos] if isinstance(eos, (list, tuple)) else [int(eos)])
        rs = d.get("rope_scaling")
        window = d.get("sliding_window")
        cfg = cls(
            architecture=arch, hidden_size=hidden, intermediate_size=int(need("intermediate_size")),
            num_hidden_layers=int(need("num_hidden_layers")), num_attention_heads=heads, num_key_value_heads=kv,
            head_dim=head_dim, vocab_size=int(need("vocab_size")),
            max_position_embeddings=int(need("max_position_embeddings")), rms_norm_eps=float(need("rms_norm_eps")),
            rope_theta=float(d.get("rope_theta", 10000.0)),
            partial_rotary_factor=float(d.get("partial_rotary_factor", 1.0)),
            rope_scaling=RopeScaling.from_dict(rs) if rs else None,
            sliding_window=int(window) if window else 0,
            attention_sinks=int(d.get("attention_sinks") or 0),
            # convert.py:241, 200-204: the head is a tensor of its own only if the key is exactly false
            tie_word_embeddings=d.get("tie_word_embeddings", None) is not False,
            hidden_act=d.get("hidden_act", "silu"),
            bos_token_id=None if d.get("bos_token_id") is None else int(d["bos_token_id"]),
            eos_token_ids=eos_ids)
        cfg.validate()
        return cfg

    def validate(self):
        def positive(name):
            if getattr(self, name) <= 0:
                raise ConfigError("%s must be positive, got %r" % (name, getattr(self, name)))
        for n in ("hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                  "num_key_value_heads", "head_dim", "vocab_size", "max_position_embeddings", "rms_norm_eps",
                  "rope_theta"):
            positive(n)
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError("num_attention_heads %d is no multiple of num_key_value_heads %d"
                              % (self.num_attention_heads, self.num_key_value_heads))
        if self.hidden_act not in ("silu", "gelu"):       # the two of the reference (convert.py:51-52)
            raise ConfigError("hidden_act %r is not supported ('silu' or 'gelu')" % (self.hidden_act,))
        if self.head_dim % 2 != 0:
            raise ConfigError("head_dim %d must be even" % self.head_dim)
        if self.rotary_dim % 2 != 0 or not 0 <= self.rotary_dim <= self.head_dim:
            raise ConfigError("partial_rotary_factor %r gives a rotary_dim of %d for head_dim %d"
                              % (self.partial_rotary_factor, self.rotary_dim, self.head_dim))
        if self.sliding_window < 0:
            raise ConfigError("sliding_window must not be negative")
        if self.attention_sinks < 0 or (self.attention_sinks and self.sliding_window < self.attention_sinks):
            raise ConfigError("attention_sinks (%d) must not be negative and needs a sliding_window at least as wide"
                              % self.attention_sinks)

    @property
    def rotary_dim(self):
        return int(self.head_dim * self.partial_rotary_factor)                           # convert.py:43

    def with_window(self, window, sinks=0):
        """Attend over the last `window` positions only, and over the first `sinks` beside them."""
        import dataclasses
        if not window:
            return self
        cfg = dataclasses.replace(self, sliding_window=int(window), attention_sinks=int(sinks))
        cfg.validate()
        return cfg

    def with_context(self, n):
        """The reference's `-T <n>` (src/main.cpp:437-439, src/infer.cpp:484-488): a context of n
        positions.  Up to position n - 1 every key is visible; from there on the first KV_SINKS
        positions and the last n - KV_SINKS."""
        if not n:
            return self
        if int(n) < 2 * KV_SINKS:
            raise ConfigError("a context of %d positions leaves no window beside the %d attention sinks"
                              % (int(n), KV_SINKS))
        return self.with_window(int(n) - KV_SINKS, KV_SINKS)

    # ------------------------------------------------------------------ writing
    def to_dict(self):
        d = {
            "architectures": [self.architecture], "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size, "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads, "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim, "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings, "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta, "hidden_act": self.hidden_act,
            "tie_word_embeddings": bool(self.tie_word_embeddings),
        }
        if self.partial_rotary_factor != 1.0:
            d["partial_rotary_factor"] = self.partial_rotary_factor
        if self.rope_scaling is not None:
            d["rope_scaling"] = self.rope_scaling.to_dict()
        if self.sliding_window:
            d["sliding_window"] = self.sliding_window
        if self.attention_sinks:
            d["attention_sinks"] = self.attention_sinks
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return d

    # ------------------------------------------------------------------ the model as data
    def to_spec(self):
        """Every layer: RMSNorm -> grouped-query attention with RoPE -> residual,
        RMSNorm -> SwiGLU -> residual (src/infer.cpp:256-386); then the final norm
        and the head, tied to the embedding unless the folder has a head of its own
        (model.cpp:389-398)."""
        pos = PartSpec("rope", {
            "head_dim": self.head_dim, "rotary_dim": self.rotary_dim, "theta": self.rope_theta,
            "scaling": self.rope_scaling.to_dict() if self.rope_scaling else None,
            "weight_rows": "half_split",          # q/k rows of the folder are in Hugging Face order
        })
        norm = {"eps": self.rms_norm_eps}
        layers = []
        for i in range(self.num_hidden_layers):
            layers.append(LayerSpec(
                block="prenorm_residual",
                mixer=PartSpec("gqa_attention", {
                    "n_heads": self.num_attention_heads, "n_kv_heads": self.num_key_value_heads,
                    "head_dim": self.head_dim, "window": self.sliding_window, "sinks": self.attention_sinks,
                    "position": pos,
                }, prefix="self_attn."),
                feed_forward=PartSpec("swiglu", {"hidden": self.intermediate_size, "activation": self.hidden_act},
                                      prefix="mlp."),
                mixer_norm=PartSpec("rmsnorm", norm, prefix="input_layernorm."),
                feed_forward_norm=PartSpec("rmsnorm", norm, prefix="post_attention_layernorm."),
                prefix="model.layers.%d." % i))
        return ModelSpec(
            architecture=self.architecture, dim=self.hidden_size, vocab_size=self.vocab_size,
            max_positions=self.max_position_embeddings,
            embedding=PartSpec("token_embedding", {"vocab_size": self.vocab_size}, prefix="model.embed_tokens."),
            layers=layers,
            final_norm=PartSpec("rmsnorm", norm, prefix="model.norm."),
            head=PartSpec("lm_head", {"vocab_size": self.vocab_size, "tied": self.tie_word_embeddings},
                          prefix="lm_head."),
            bos_token_id=self.bos_token_id, eos_token_ids=list(self.eos_token_ids))
