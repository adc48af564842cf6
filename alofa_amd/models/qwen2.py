"""Qwen2ForCausalLM: a dense decoder of pre-norm blocks, grouped-query attention
with q/k/v bias and half-split rotary positions, a SwiGLU feed-forward, RMSNorm,
and an output matrix that may be tied to the embedding
(src/alofa/model/arch/qwen.mojo:915-998 for the keys and their rules,
:1176-1189 for the tensor names)."""
from __future__ import annotations

from dataclasses import dataclass, asdict
from typing import Optional

from ..config.base import LayerSpec, ModelConfig, ModelSpec, PartSpec, RunEntry
from ..errors import AlofaError


def _need(raw: dict, key: str, kind, where: str):
    if key not in raw:
        raise AlofaError("invalid_argument", "config.json lacks a required key", f"key={key} config={where}")
    v = raw[key]
    if kind is bool:
        if not isinstance(v, bool):
            raise AlofaError("parse", "config value must be true or false", f"key={key} config={where}")
        return v
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise AlofaError("parse", "config value must be a number", f"key={key} config={where}")
    if kind is int:
        if int(v) != v:
            raise AlofaError("parse", "config value must be a whole number", f"key={key} config={where}")
        return int(v)
    return float(v)


@dataclass(frozen=True)
class Qwen2Config(ModelConfig):
    num_hidden_layers: int
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    max_position_embeddings: int
    use_sliding_window: bool = False
    sliding_window: Optional[int] = None
    max_window_layers: Optional[int] = None

    architecture = "Qwen2ForCausalLM"

    @classmethod
    def from_dict(cls, raw: dict, where: str = "<dict>") -> "Qwen2Config":
        # keys the reference does not read (qwen.mojo:939-954) but whose other values would change the
        # model: refused by name rather than computed wrongly
        if raw.get("rope_scaling") is not None:
            raise AlofaError("unsupported", "scaled rotary positions are not built", f"key=rope_scaling value={raw['rope_scaling']!r} config={where}")
        if raw.get("hidden_act", "silu") != "silu":
            raise AlofaError("unsupported", "the feed-forward's activation is SiLU", f"key=hidden_act value={raw['hidden_act']!r} config={where}")
        if raw.get("use_mrope", False) not in (False, None):
            raise AlofaError("unsupported", "multi-axis rotary positions are not built", f"key=use_mrope value={raw['use_mrope']!r} config={where}")
        hidden = _need(raw, "hidden_size", int, where)
        heads = _need(raw, "num_attention_heads", int, where)
        if heads <= 0:
            raise AlofaError("parse", "num_attention_heads must be positive", f"config={where}")
        # head_dim is optional and falls back to hidden // heads (qwen.mojo:946-949)
        head_dim = _need(raw, "head_dim", int, where) if "head_dim" in raw else hidden // heads
        use_window = _need(raw, "use_sliding_window", bool, where) if "use_sliding_window" in raw else False
        layers = _need(raw, "num_hidden_layers", int, where)
        cfg = cls(
            num_hidden_layers=layers,
            hidden_size=hidden,
            num_attention_heads=heads,
            num_key_value_heads=_need(raw, "num_key_value_heads", int, where),
            head_dim=head_dim,
            intermediate_size=_need(raw, "intermediate_size", int, where),
            vocab_size=_need(raw, "vocab_size", int, where),
            rms_norm_eps=_need(raw, "rms_norm_eps", float, where),
            rope_theta=_need(raw, "rope_theta", float, where),
            tie_word_embeddings=_need(raw, "tie_word_embeddings", bool, where),
            max_position_embeddings=(_need(raw, "max_position_embeddings", int, where)
                                     if "max_position_embeddings" in raw else 32768),
            use_sliding_window=use_window,
            sliding_window=_need(raw, "sliding_window", int, where) if use_window else None,
            max_window_layers=(_need(raw, "max_window_layers", int, where)
                               if use_window and "max_window_layers" in raw else (layers if use_window else None)),
        )
        cfg.validate(where)
        return cfg

    def validate(self, where: str) -> None:
        """The reference's checks (qwen.mojo:977-994, :852-857) and the bounds
        of the keys this engine reads in addition."""
        if self.num_attention_heads * self.head_dim != self.hidden_size:
            raise AlofaError("parse", "heads * head_dim must equal hidden", f"config={where}")
        if self.num_key_value_heads <= 0 or self.num_attention_heads % self.num_key_value_heads != 0:
            raise AlofaError("parse", "n_kv_heads must be positive and divide n_heads", f"config={where}")
        if self.num_hidden_layers <= 0 or self.intermediate_size <= 0 or self.vocab_size <= 0:
            raise AlofaError("parse", "layer, feed-forward and vocabulary sizes must be positive", f"config={where}")
        if not self.rms_norm_eps > 0:
            raise AlofaError("parse", "rms norm eps must be positive", f"config={where}")
        if not self.rope_theta > 0:
            raise AlofaError("parse", "rope_theta must be positive", f"config={where}")
        if self.head_dim <= 0 or self.head_dim % 2 != 0:
            raise AlofaError("unsupported", "head dimension must be positive and even", f"head_dim={self.head_dim}")
        if self.max_position_embeddings <= 0:
            raise AlofaError("parse", "max_position_embeddings must be positive", f"config={where}")
        if self.use_sliding_window:
            if self.sliding_window is None or self.sliding_window <= 0:
                raise AlofaError("parse", "sliding_window must be positive when use_sliding_window is set", f"config={where}")
            if not 0 <= self.max_window_layers <= self.num_hidden_layers:
                raise AlofaError("parse", "max_window_layers must lie within the layers", f"config={where}")

    def to_dict(self) -> dict:
        d = {k: v for k, v in asdict(self).items() if v is not None}
        d["architectures"] = [self.architecture]
        d["model_type"] = "qwen2"
        return d

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    def window_of(self, layer: int) -> Optional[int]:
        """Layers from ``max_window_layers`` upward see only the last
        ``sliding_window`` keys when ``use_sliding_window`` is set. The
        reference does not read these keys; this rule is the engine's own."""
        if self.use_sliding_window and layer >= self.max_window_layers:
            return self.sliding_window
        return None

    def spec(self) -> ModelSpec:
        h, d = self.hidden_size, self.head_dim
        position = PartSpec("rotary", {"theta": self.rope_theta, "head_dim": d, "pairing": "half"})
        layers = []
        for i in range(self.num_hidden_layers):
            p = f"model.layers.{i}."
            layers.append(LayerSpec(prefix=p, block=PartSpec("prenorm"), parts=dict(
                mixer=PartSpec("gqa_attention", {
                    "prefix": p + "self_attn.", "hidden": h, "heads": self.num_attention_heads,
                    "kv_heads": self.num_key_value_heads, "head_dim": d, "qkv_bias": True,
                    "out_bias": False, "window": self.window_of(i), "position": position}),
                feed_forward=PartSpec("swiglu", {
                    "prefix": p + "mlp.", "hidden": h, "intermediate": self.intermediate_size}),
                norms=(PartSpec("rmsnorm", {"name": p + "input_layernorm.weight", "width": h, "eps": self.rms_norm_eps}),
                       PartSpec("rmsnorm", {"name": p + "post_attention_layernorm.weight", "width": h, "eps": self.rms_norm_eps})),
            )))
        return ModelSpec(
            hidden_size=h, vocab_size=self.vocab_size, max_positions=self.max_position_embeddings,
            embedding=PartSpec("token_embedding", {"name": "model.embed_tokens.weight", "vocab": self.vocab_size, "width": h}),
            layers=tuple(layers),
            order=tuple(RunEntry(i) for i in range(self.num_hidden_layers)),
            final_norm=PartSpec("rmsnorm", {"name": "model.norm.weight", "width": h, "eps": self.rms_norm_eps}),
            head=PartSpec("lm_head", {"name": "lm_head.weight", "tied_to": "model.embed_tokens.weight" if self.tie_word_embeddings else None,
                                      "vocab": self.vocab_size, "width": h}),
        )
