"""LLaMA: the dense pre-norm decoder (RMSNorm, rotary positions, SwiGLU, MHA or GQA).

This file is the whole of what is specific to the architecture: the keys of its
config.json, their checks, and the translation into a `ModelSpec` that names
generic parts.  The network is the one of the reference's LLaMA-2 graph
(src/graph/llama_like.cpp:54-109): embedding, N x (norm, attention, add, norm,
feed-forward, add), norm, head; tensor names are the checkpoint's own
(the right-hand sides of src/graph/llama_like.cpp:10-21).  Constants that the
reference fixes in code (eps src/graph/llama_like.cpp:78,96 and
src/core/graph.h:163, rotary base src/kern/naive/naive.cpp:396) come from the
configuration here, one eps for every norm.
"""
from __future__ import annotations

import warnings
from dataclasses import asdict, dataclass, field
from typing import List, Optional

from ..config.registry import ConfigError, register_architecture
from ..config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

_REQUIRED = ("hidden_size", "intermediate_size", "num_hidden_layers",
             "num_attention_heads", "vocab_size")
# keys that describe training, the file or the tokenizer and change no result here
_IGNORED = {"architectures", "model_type", "torch_dtype", "dtype", "transformers_version",
            "use_cache", "initializer_range", "pad_token_id", "attention_dropout",
            "pretraining_tp", "_name_or_path"}


@register_architecture("LlamaForCausalLM")
@dataclass
class LlamaConfig:
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    vocab_size: int
    num_key_value_heads: int = 0          # 0: same as num_attention_heads
    head_dim: int = 0                     # 0: hidden_size / num_attention_heads
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    max_position_embeddings: int = 2048
    tie_word_embeddings: bool = False
    bos_token_id: Optional[int] = 1
    eos_token_id: List[int] = field(default_factory=lambda: [2])
    hidden_act: str = "silu"
    attention_bias: bool = False
    mlp_bias: bool = False
    rope_scaling: Optional[dict] = None

    architecture = "LlamaForCausalLM"
    # what the command line's --type may name for this architecture (the reference's model-type
    # strings, src/graph/graph_imp.cpp:6-21: "llama" and "llama2" are its two LLaMA graphs)
    cli_type_names = ("llama", "llama2")

    # ------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d: dict) -> "LlamaConfig":
        missing = [k for k in _REQUIRED if k not in d]
        if missing:
            raise ConfigError(f"config.json of {cls.architecture} lacks required keys: {missing}")
        known = set(cls.__dataclass_fields__) | _IGNORED
        unknown = sorted(k for k in d if k not in known)
        if unknown:
            warnings.warn(f"config.json keys not used by {cls.architecture}: {unknown}")
        kw = {k: d[k] for k in cls.__dataclass_fields__ if k in d}
        eos = kw.get("eos_token_id", [2])
        if eos is None:
            eos = []
        elif isinstance(eos, int):
            eos = [eos]
        kw["eos_token_id"] = [int(e) for e in eos]
        cfg = cls(**kw)
        cfg.validate()
        return cfg

    def validate(self) -> None:
        def positive_int(name):
            v = getattr(self, name)
            if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
                raise ConfigError(f"{name} must be a positive integer, got {v!r}")
        for name in _REQUIRED + ("max_position_embeddings",):
            positive_int(name)
        if self.num_key_value_heads in (0, None):
            self.num_key_value_heads = self.num_attention_heads
        positive_int("num_key_value_heads")
        if self.head_dim in (0, None):
            if self.hidden_size % self.num_attention_heads:
                raise ConfigError(
                    f"hidden_size {self.hidden_size} is not a multiple of num_attention_heads "
                    f"{self.num_attention_heads} and no head_dim is given")
            self.head_dim = self.hidden_size // self.num_attention_heads
        positive_int("head_dim")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even (rotary pairs)")
        if not (isinstance(self.rms_norm_eps, float) and self.rms_norm_eps > 0):
            raise ConfigError(f"rms_norm_eps must be a positive float, got {self.rms_norm_eps!r}")
        self.rope_theta = float(self.rope_theta)
        if not self.rope_theta > 0:
            raise ConfigError(f"rope_theta must be positive, got {self.rope_theta!r}")
        if self.hidden_act != "silu":
            raise ConfigError(f"unsupported hidden_act {self.hidden_act!r} (only 'silu')")
        if self.attention_bias or self.mlp_bias:
            raise ConfigError("unsupported: attention_bias / mlp_bias (LLaMA has no biases)")
        if self.rope_scaling not in (None, {}):
            raise ConfigError(f"unsupported rope_scaling {self.rope_scaling!r}")
        for t in [self.bos_token_id] + list(self.eos_token_id):
            if t is not None and not (0 <= int(t) < self.vocab_size):
                raise ConfigError(f"token id {t} outside the vocabulary of {self.vocab_size}")

    def to_dict(self) -> dict:
        d = asdict(self)
        d["architectures"] = [self.architecture]
        d["model_type"] = "llama"
        if len(d["eos_token_id"]) == 1:
            d["eos_token_id"] = d["eos_token_id"][0]
        return d

    # ------------------------------------------------------------ translation
    def to_spec(self) -> ModelSpec:
        E, F, V = self.hidden_size, self.intermediate_size, self.vocab_size
        nh, nkv, hd = self.num_attention_heads, self.num_key_value_heads, self.head_dim
        norm = lambda name: PartSpec("rms_norm", {"size": E, "eps": self.rms_norm_eps},
                                     {"weight": name})
        layers = []
        for i in range(self.num_hidden_layers):
            p = f"model.layers.{i}."
            layers.append(LayerSpec(
                block="pre_norm",
                mixer=PartSpec(
                    "attention",
                    {"hidden_size": E, "num_heads": nh, "num_kv_heads": nkv, "head_dim": hd,
                     "window": None, "softmax_scale": None},
                    {"q": p + "self_attn.q_proj.weight", "k": p + "self_attn.k_proj.weight",
                     "v": p + "self_attn.v_proj.weight", "o": p + "self_attn.o_proj.weight"}),
                feed_forward=PartSpec(
                    "swiglu", {"hidden_size": E, "intermediate_size": F},
                    {"gate": p + "mlp.gate_proj.weight", "up": p + "mlp.up_proj.weight",
                     "down": p + "mlp.down_proj.weight"}),
                mixer_norm=norm(p + "input_layernorm.weight"),
                feed_forward_norm=norm(p + "post_attention_layernorm.weight"),
                position=PartSpec(
                    "rotary", {"head_dim": hd, "rotary_dim": hd, "theta": self.rope_theta,
                               "pairing": "half", "max_positions": self.max_position_embeddings}),
            ))
        head_tensors = {"weight": "lm_head.weight"}
        head_params = {"hidden_size": E, "vocab_size": V}
        if self.tie_word_embeddings:
            head_params["tied_fallback"] = "model.embed_tokens.weight"
        return ModelSpec(
            architecture=self.architecture,
            vocab_size=V, hidden_size=E, max_positions=self.max_position_embeddings,
            embedding=PartSpec("token_embedding", {"vocab_size": V, "hidden_size": E},
                               {"weight": "model.embed_tokens.weight"}),
            layers=layers,
            schedule=[ScheduleEntry(layer=i, cache_line=i) for i in range(self.num_hidden_layers)],
            final_norm=norm("model.norm.weight"),
            head=PartSpec("lm_head", head_params, head_tensors),
            bos_token_id=self.bos_token_id,
            eos_token_ids=list(self.eos_token_id),
            ignored_tensor_suffixes=[".rotary_emb.inv_freq"],
        )
