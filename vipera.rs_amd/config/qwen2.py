"""Configuration of the Qwen2 dense decoder, read from its own ``config.json`` keys.

Block layout as the reference runs it: "pre-norm residual blocks, RMSNorm,
grouped-query attention with NeoX-style rotary embeddings, SwiGLU feed-forward,
and a final norm before the output projection"
(crates/vipera-backend-cpu/src/model.rs:3-4).  Defaults and checks follow
``ModelConfig::from_gguf`` (model.rs:1343-1398): KV heads default to the head
count (1352), the head width defaults to hidden/heads and must divide (1367-1377)
and be even (1378), heads must be a multiple of KV heads (1383), eps defaults to
1e-6 (1397) and the rotary base to 10,000 (1398).
"""
from __future__ import annotations

from dataclasses import asdict, dataclass, field
from typing import Any, Dict, List, Optional, Tuple

from ..errors import InvalidArgumentError, UnsupportedError
from .base import KeyReader, LayerSpec, ModelConfig, PartSpec


@dataclass
class Qwen2Config(ModelConfig):
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    tie_word_embeddings: bool = False
    max_position_embeddings: int = 32768
    hidden_act: str = "silu"
    use_sliding_window: bool = False
    sliding_window: Optional[int] = None
    max_window_layers: Optional[int] = None
    eos_token_ids: Tuple[int, ...] = ()
    torch_dtype: str = "bfloat16"
    # head_dim was given in the file (and is written back) rather than derived
    explicit_head_dim: bool = field(default=False, repr=False)

    architecture = "Qwen2ForCausalLM"

    # --- reading ----------------------------------------------------------------------
    @classmethod
    def from_dict(cls, data: Dict[str, Any]) -> "Qwen2Config":
        r = KeyReader(data)
        hidden = r.integer("hidden_size", minimum=1)
        heads = r.integer("num_attention_heads", minimum=1)
        kv_heads = r.integer("num_key_value_heads", default=heads, minimum=1)
        explicit = r.has("head_dim")
        if explicit:
            head_dim = r.integer("head_dim", minimum=1)
        else:
            if hidden % heads != 0:
                raise InvalidArgumentError(
                    f"config.json: \"hidden_size\" {hidden} is not a multiple of "
                    f"\"num_attention_heads\" {heads} and no \"head_dim\" is given"
                )
            head_dim = hidden // heads
        if r.has("rope_scaling"):
            raise UnsupportedError(
                f"config.json: \"rope_scaling\" is {data['rope_scaling']!r}; scaled rotary "
                "embeddings are not implemented"
            )
        eos = data.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, int) and not isinstance(eos, bool):
            eos_ids = (eos,)
        elif isinstance(eos, list) and all(isinstance(e, int) and not isinstance(e, bool) for e in eos):
            eos_ids = tuple(eos)
        else:
            raise InvalidArgumentError(
                f"config.json: key \"eos_token_id\" is {eos!r}, expected an integer or a list of integers"
            )
        config = cls(
            vocab_size=r.integer("vocab_size", minimum=1),
            hidden_size=hidden,
            intermediate_size=r.integer("intermediate_size", minimum=1),
            num_hidden_layers=r.integer("num_hidden_layers", minimum=0),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            rms_norm_eps=r.number("rms_norm_eps", default=1e-6),
            rope_theta=r.number("rope_theta", default=10000.0),
            tie_word_embeddings=r.boolean("tie_word_embeddings", False),
            max_position_embeddings=r.integer("max_position_embeddings", default=32768, minimum=1),
            hidden_act=r.string("hidden_act", default="silu"),
            use_sliding_window=r.boolean("use_sliding_window", False),
            sliding_window=r.integer("sliding_window", minimum=1) if r.has("sliding_window") else None,
            max_window_layers=r.integer("max_window_layers", minimum=0) if r.has("max_window_layers") else None,
            eos_token_ids=eos_ids,
            torch_dtype=r.string("torch_dtype", default="bfloat16"),
            explicit_head_dim=explicit,
        )
        config.validate()
        return config

    def validate(self) -> None:
        if self.head_dim % 2 != 0:
            raise InvalidArgumentError(
                f"config.json: \"head_dim\" is {self.head_dim}; rotary embeddings need an even head width"
            )
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise InvalidArgumentError(
                f"config.json: \"num_attention_heads\" {self.num_attention_heads} is not a multiple of "
                f"\"num_key_value_heads\" {self.num_key_value_heads}"
            )
        if self.hidden_act != "silu":
            raise UnsupportedError(
                f"config.json: \"hidden_act\" is {self.hidden_act!r}; only \"silu\" is implemented"
            )
        if not self.rms_norm_eps >= 0.0:
            raise InvalidArgumentError(
                f"config.json: key \"rms_norm_eps\" is {self.rms_norm_eps!r}, expected a number at or above 0"
            )
        if not self.rope_theta > 0.0:
            raise InvalidArgumentError(
                f"config.json: key \"rope_theta\" is {self.rope_theta!r}, expected a number above 0"
            )
        if self.use_sliding_window and self.sliding_window is None:
            raise InvalidArgumentError(
                "config.json: \"use_sliding_window\" is true but \"sliding_window\" is missing"
            )

    def to_dict(self) -> Dict[str, Any]:
        data: Dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "qwen2",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "max_position_embeddings": self.max_position_embeddings,
            "hidden_act": self.hidden_act,
            "use_sliding_window": self.use_sliding_window,
            "torch_dtype": self.torch_dtype,
        }
        if self.explicit_head_dim or self.head_dim * self.num_attention_heads != self.hidden_size:
            data["head_dim"] = self.head_dim
        if self.sliding_window is not None:
            data["sliding_window"] = self.sliding_window
        if self.max_window_layers is not None:
            data["max_window_layers"] = self.max_window_layers
        if self.eos_token_ids:
            data["eos_token_id"] = (
                self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
            )
        return data

    # --- the description the generic decoder consumes ---------------------------------------
    def window_of_layer(self, index: int) -> int:
        """Positions a layer attends to, counting its own; 0 means all of them.

        With ``use_sliding_window`` the first ``max_window_layers`` layers see the
        whole history and every later layer sees the last ``sliding_window``
        positions: ``[pos + 1 - window, pos]``, the range the reference keeps for a
        window with no sink tokens (model.rs:2509).
        """
        if not self.use_sliding_window or self.sliding_window is None:
            return 0
        first_windowed = self.max_window_layers if self.max_window_layers is not None else 0
        return int(self.sliding_window) if index >= first_windowed else 0

    def layer_specs(self) -> List[LayerSpec]:
        specs = []
        norm = {"width": self.hidden_size, "eps": self.rms_norm_eps}
        for index in range(self.num_hidden_layers):
            prefix = f"model.layers.{index}."
            specs.append(
                LayerSpec(
                    block="prenorm",
                    mixer=PartSpec(
                        "attention",
                        {
                            "hidden": self.hidden_size,
                            "heads": self.num_attention_heads,
                            "kv_heads": self.num_key_value_heads,
                            "head_dim": self.head_dim,
                            "qkv_bias": True,
                            "out_bias": False,
                            "window": self.window_of_layer(index),
                            "scale": None,  # 1/sqrt(head_dim), model.rs:1816
                            "name": "self_attn",
                        },
                    ),
                    ffn=PartSpec(
                        "gated_mlp",
                        {
                            "hidden": self.hidden_size,
                            "intermediate": self.intermediate_size,
                            "activation": self.hidden_act,
                            "name": "mlp",
                        },
                    ),
                    mixer_norm=PartSpec("rmsnorm", dict(norm, name="input_layernorm")),
                    ffn_norm=PartSpec("rmsnorm", dict(norm, name="post_attention_layernorm")),
                    position=PartSpec(
                        "rotary_neox",
                        {"head_dim": self.head_dim, "rotary_dim": self.head_dim, "base": self.rope_theta},
                    ),
                    prefix=prefix,
                )
            )
        return specs

    def embedding_spec(self) -> PartSpec:
        return PartSpec(
            "embedding",
            {"vocab": self.vocab_size, "width": self.hidden_size, "name": "model.embed_tokens"},
        )

    def final_norm_spec(self) -> PartSpec:
        return PartSpec("rmsnorm", {"width": self.hidden_size, "eps": self.rms_norm_eps, "name": "model.norm"})

    def head_spec(self) -> PartSpec:
        return PartSpec(
            "lm_head",
            {
                "vocab": self.vocab_size,
                "width": self.hidden_size,
                "name": "lm_head",
                "tied_to": "model.embed_tokens" if self.tie_word_embeddings else None,
            },
        )
