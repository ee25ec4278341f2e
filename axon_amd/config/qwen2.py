"""The Qwen2.5 dense decoder's configuration: config.json keys to typed fields to a ModelSpec.

Keys, defaults and refusals follow the reference's reading of a Hugging Face checkpoint
(src/safetensors.rs:609-727 for the keys, src/model.rs:1283-1328 for the checks):
rms_norm_eps defaults to 1e-6 (src/model.rs:1784), rope_theta to 10000 (src/model.rs:639),
head_dim to hidden_size / heads (src/model.rs:1782-1783), tie_word_embeddings to false
(src/safetensors.rs:1608-1609); num_key_value_heads has no default (src/model.rs:1283-1296).
"""
from __future__ import annotations

import struct
from dataclasses import dataclass
from typing import Any, Dict, Optional

from .base import (ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec, Run, get_flag, get_number,
                   get_whole)


def _as_float32(x: float) -> float:
    return struct.unpack("<f", struct.pack("<f", x))[0]


@dataclass(frozen=True)
class Qwen2Config(ModelConfig):
    num_hidden_layers: int
    hidden_size: int
    intermediate_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: Optional[int]
    max_position_embeddings: int
    rope_theta: float
    rms_norm_eps: float
    tie_word_embeddings: bool
    head_dim_given: bool = False

    architecture = "Qwen2ForCausalLM"
    model_type = "qwen2"

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, cfg: Dict[str, Any]) -> "Qwen2Config":
        if not isinstance(cfg, dict):
            raise ConfigError("config.json is not a JSON object")
        act = cfg.get("hidden_act")
        if act is not None and act != "silu":
            # src/safetensors.rs:618-622
            raise ConfigError(f"hidden_act {act} is not supported (silu)")
        if cfg.get("use_sliding_window") is True:
            # src/safetensors.rs:623-625
            raise ConfigError("use_sliding_window true is not supported")
        if cfg.get("quantization_config") is not None:
            raise ConfigError("quantization_config is not supported: quantized weights are out of scope")
        # rope_theta may live under rope_parameters (src/safetensors.rs:647-651); a scaling type
        # other than "default" is refused (only the plain frequencies are built).
        rp = dict(cfg.get("rope_parameters") or {}) if isinstance(cfg.get("rope_parameters"), dict) else {}
        scaling = cfg.get("rope_scaling")
        if isinstance(scaling, dict):
            rp = {**scaling, **rp}
        elif scaling is not None:
            raise ConfigError(f"rope_scaling = {scaling!r} is not an object")
        rope_type = rp.get("rope_type", rp.get("type"))
        if rope_type is not None and str(rope_type).lower() != "default":
            raise ConfigError(f"RoPE scaling type {rope_type} is not supported")
        theta_src = rp if "rope_theta" in rp else cfg

        nh = get_whole(cfg, "num_attention_heads")
        dim = get_whole(cfg, "hidden_size")
        hd = get_whole(cfg, "head_dim", None)
        given = hd is not None
        if hd is None:
            if dim % nh:
                raise ConfigError(f"hidden_size {dim} is not a multiple of num_attention_heads {nh}")
            hd = dim // nh
        nkv = get_whole(cfg, "num_key_value_heads")
        if nh % nkv:
            # src/model.rs:1313-1320
            raise ConfigError(f"num_attention_heads {nh} is not a multiple of num_key_value_heads {nkv}")
        if hd % 2:
            raise ConfigError(f"head_dim {hd} is odd: rotary pairs need an even size")
        return cls(
            num_hidden_layers=get_whole(cfg, "num_hidden_layers"),
            hidden_size=dim,
            intermediate_size=get_whole(cfg, "intermediate_size"),
            num_attention_heads=nh,
            num_key_value_heads=nkv,
            head_dim=hd,
            vocab_size=get_whole(cfg, "vocab_size", None),
            max_position_embeddings=get_whole(cfg, "max_position_embeddings"),
            # kept as the 32-bit float nearest to the file's value, then widened (src/safetensors.rs:649-651)
            rope_theta=_as_float32(get_number(theta_src, "rope_theta", 10000.0)),
            rms_norm_eps=get_number(cfg, "rms_norm_eps", 1e-6),
            tie_word_embeddings=get_flag(cfg, "tie_word_embeddings", False),
            head_dim_given=given,
        )

    def to_dict(self) -> Dict[str, Any]:
        d = {
            "architectures": [self.architecture],
            "model_type": self.model_type,
            "num_hidden_layers": self.num_hidden_layers,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rope_theta": self.rope_theta,
            "rms_norm_eps": self.rms_norm_eps,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "use_sliding_window": False,
        }
        if self.head_dim_given or self.head_dim * self.num_attention_heads != self.hidden_size:
            d["head_dim"] = self.head_dim
        return d

    embedding_tensor = "model.embed_tokens.weight"

    def vocab_tensor(self):
        # the reference takes the vocabulary from the embedding's rows, not from vocab_size (src/model.rs:1797-1798)
        return self.embedding_tensor if self.vocab_size is None else None

    def with_vocab(self, vocab_size: int) -> "Qwen2Config":
        from dataclasses import replace
        return replace(self, vocab_size=vocab_size)

    def ignores_tensor(self, name: str) -> bool:
        return name.endswith("rotary_emb.inv_freq")          # src/safetensors.rs:1157-1159

    # ------------------------------------------------------------------ the model as data
    def model_spec(self) -> ModelSpec:
        if self.vocab_size is None:
            raise ConfigError("vocab_size is not known yet: it comes from config.json or the embedding tensor")
        norm = PartSpec("rmsnorm", {"size": self.hidden_size, "eps": self.rms_norm_eps})
        position = PartSpec("rope", {"head_dim": self.head_dim, "rotary_dim": self.head_dim,
                                     "theta": self.rope_theta})
        mixer = PartSpec("gqa_attention", {
            "hidden_size": self.hidden_size,
            "num_heads": self.num_attention_heads,
            "num_kv_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            # a bias is used iff its tensor exists (src/model.rs:2984-2991); an output bias is
            # refused for this architecture (src/model.rs:1596-1598)
            "qkv_bias": "optional",
            "out_bias": False,
            "window": 0,
            "position": position,
        })
        ffn = PartSpec("swiglu_mlp", {"hidden_size": self.hidden_size,
                                      "intermediate_size": self.intermediate_size})
        layers = [LayerSpec(block="prenorm", mixer=mixer, feed_forward=ffn, norm=norm,
                            prefix=f"model.layers.{i}.") for i in range(self.num_hidden_layers)]
        return ModelSpec(
            hidden_size=self.hidden_size,
            vocab_size=self.vocab_size,
            embedding=PartSpec("token_embedding", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                                                   "tensor": self.embedding_tensor}),
            layers=layers,
            order=[Run(layer=i, cache=i) for i in range(self.num_hidden_layers)],
            final_norm=PartSpec("rmsnorm", {"size": self.hidden_size, "eps": self.rms_norm_eps,
                                            "tensor": "model.norm.weight"}),
            # the head is lm_head.weight if the tensor exists, else the embedding matrix; untied
            # and missing is an error (src/model.rs:1800-1803, src/safetensors.rs:1608-1614)
            head=PartSpec("lm_head", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                                      "tensor": "lm_head.weight", "tied_to": self.embedding_tensor,
                                      "tied": self.tie_word_embeddings}),
            max_positions=self.max_position_embeddings,
        )
