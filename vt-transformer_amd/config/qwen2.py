"""Qwen2: typed configuration read from the keys of its config.json.

The reference runs this architecture from constants typed into the head of
v1/models/qwen2-7b/inference_fp16.dag:1-15 (RMS_EPS, ROTARY_BASE, VOCAB_SIZE,
HIDDEN_SIZE, KV_PROJ, INTERMEDIATE_SIZE, HEADS_NUM, KV_HEADS_NUM, HEAD_HIDDEN,
MAX_CONTEXT) and the literal 28 of its layer loop (:355-357, :377-379).  The
key names are those of the checkpoint's config.json (the reference lists the
ones it copies from in vt-transformer/models/qwen3-0.6b/qwen3.hpp:12-15).

Fixed by the architecture, as in the reference's layer program (:287-345):
bias on the Q, K and V projections and none on the output projection or in
the feed-forward; rotation of the whole head in half-split pairs; score
scale 1/sqrt(head_dim); norm before mixer and before feed-forward; SiLU gate.
"""
from __future__ import annotations

from dataclasses import dataclass, field, asdict
from typing import Any, Dict, List, Optional

from .base import (ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec,
                   ScheduleEntry, read_key, require_positive)


@dataclass
class Qwen2Config(ModelConfig):
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool
    hidden_act: str = "silu"
    use_sliding_window: bool = False
    sliding_window: Optional[int] = None
    max_window_layers: Optional[int] = None
    eos_token_id: List[int] = field(default_factory=list)
    bos_token_id: Optional[int] = None
    torch_dtype: str = "bfloat16"

    architecture = "Qwen2ForCausalLM"

    # ------------------------------------------------------------------
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "Qwen2Config":
        hidden = read_key(d, "hidden_size", int)
        heads = read_key(d, "num_attention_heads", int)
        require_positive("hidden_size", hidden)
        require_positive("num_attention_heads", heads)
        kv_heads = read_key(d, "num_key_value_heads", int, heads)
        if "head_dim" in d and d["head_dim"] is not None:
            head_dim = read_key(d, "head_dim", int)
        else:
            if hidden % heads:
                raise ConfigError(
                    f"config.json: no 'head_dim' given and hidden_size {hidden} is not a multiple of "
                    f"num_attention_heads {heads}")
            head_dim = hidden // heads
        eos = d.get("eos_token_id")
        if eos is None:
            eos_list: List[int] = []
        elif isinstance(eos, int):
            eos_list = [eos]
        elif isinstance(eos, list) and all(isinstance(e, int) for e in eos):
            eos_list = list(eos)
        else:
            raise ConfigError(f"config.json: 'eos_token_id' must be an integer or a list of integers, got {eos!r}")
        scaling = d.get("rope_scaling")
        if scaling is not None:
            kind = scaling.get("rope_type", scaling.get("type")) if isinstance(scaling, dict) else scaling
            if kind not in (None, "default"):
                raise ConfigError(f"config.json: 'rope_scaling' {scaling!r} is not supported")
        cfg = cls(
            vocab_size=read_key(d, "vocab_size", int),
            hidden_size=hidden,
            intermediate_size=read_key(d, "intermediate_size", int),
            num_hidden_layers=read_key(d, "num_hidden_layers", int),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            # defaults of absent keys are the reference's constants (inference_fp16.dag:1-2,14)
            rms_norm_eps=read_key(d, "rms_norm_eps", float, 1e-6),
            rope_theta=read_key(d, "rope_theta", float, 1000000.0),
            max_position_embeddings=read_key(d, "max_position_embeddings", int, 32768),
            tie_word_embeddings=read_key(d, "tie_word_embeddings", bool, False),
            hidden_act=read_key(d, "hidden_act", str, "silu"),
            use_sliding_window=read_key(d, "use_sliding_window", bool, False),
            sliding_window=read_key(d, "sliding_window", int, None),
            max_window_layers=read_key(d, "max_window_layers", int, None),
            eos_token_id=eos_list,
            bos_token_id=read_key(d, "bos_token_id", int, None),
            torch_dtype=read_key(d, "torch_dtype", str, d.get("dtype") or "bfloat16"),
        )
        cfg.check()
        return cfg

    def check(self) -> None:
        for name in ("vocab_size", "intermediate_size", "num_hidden_layers", "num_key_value_heads",
                     "head_dim", "rms_norm_eps", "rope_theta", "max_position_embeddings"):
            require_positive(name, getattr(self, name))
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"config.json: num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"config.json: head_dim {self.head_dim} must be even for rotary pairs")
        if self.hidden_act != "silu":
            raise ConfigError(f"config.json: hidden_act '{self.hidden_act}' is not supported (only 'silu')")
        if self.use_sliding_window:
            if self.sliding_window is None or self.sliding_window <= 0:
                raise ConfigError("config.json: use_sliding_window is true but 'sliding_window' is not a positive integer")

    def to_dict(self) -> Dict[str, Any]:
        d = asdict(self)
        d["architectures"] = [self.architecture]
        d["model_type"] = "qwen2"
        eos = d["eos_token_id"]
        d["eos_token_id"] = None if not eos else (eos[0] if len(eos) == 1 else eos)
        return d

    # ------------------------------------------------------------------
    def window_of_layer(self, i: int) -> int:
        """0 = all earlier keys.  With use_sliding_window, layers from index
        max_window_layers on see only the last `sliding_window` keys (the
        reference has no window anywhere, v1/tensortype/hip_kernels/causal_mask.cpp:57-83;
        this follows the documented meaning of the checkpoint's keys: parity unpinned)."""
        if not self.use_sliding_window:
            return 0
        first = self.max_window_layers if self.max_window_layers is not None else self.num_hidden_layers
        return int(self.sliding_window) if i >= first else 0

    def to_spec(self) -> ModelSpec:
        rotary = PartSpec("rotary", {"theta": self.rope_theta, "dim": self.head_dim})
        norm = PartSpec("rmsnorm", {"eps": self.rms_norm_eps})
        layers = []
        for i in range(self.num_hidden_layers):
            mixer = PartSpec("attention", {
                "num_heads": self.num_attention_heads,
                "num_kv_heads": self.num_key_value_heads,
                "head_dim": self.head_dim,
                "qkv_bias": True,
                "out_bias": False,
                "window": self.window_of_layer(i),
                "position": rotary,
                "prefix": "self_attn.",
            })
            ffn = PartSpec("gated_mlp", {
                "intermediate_size": self.intermediate_size,
                "activation": self.hidden_act,
                "prefix": "mlp.",
            })
            layers.append(LayerSpec(
                block=PartSpec("prenorm", {}),
                mixer=mixer,
                feed_forward=ffn,
                norms={"input": PartSpec("rmsnorm", {"eps": self.rms_norm_eps, "name": "input_layernorm.weight"}),
                       "post_mixer": PartSpec("rmsnorm", {"eps": self.rms_norm_eps,
                                                          "name": "post_attention_layernorm.weight"})},
                prefix=f"model.layers.{i}.",
            ))
        spec = ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab_size,
            hidden_size=self.hidden_size,
            embedding=PartSpec("embedding", {"name": "model.embed_tokens.weight"}),
            layers=layers,
            schedule=[ScheduleEntry(i) for i in range(self.num_hidden_layers)],
            final_norm=PartSpec("rmsnorm", {"eps": self.rms_norm_eps, "name": "model.norm.weight"}),
            head=PartSpec("linear_head", {"name": "lm_head.weight",
                                          "tied_to": "model.embed_tokens.weight" if self.tie_word_embeddings else None}),
            max_positions=self.max_position_embeddings,
            eos_token_ids=list(self.eos_token_id),
            bos_token_id=self.bos_token_id,
        )
        spec.validate()
        return spec
