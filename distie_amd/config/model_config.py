"""Typed model configuration and the description of a model as a list of parts.

Two levels:

* an *architecture config* (here `Qwen2Config`) is read from the architecture's own
  `config.json` keys and validates them;
* a `ModelSpec` is what the engine builds from: one `LayerSpec` per layer, each naming
  its mixer, feed-forward, norms and arrangement as `PartSpec`s with every size and
  constant as a parameter, plus the order in which layers run. Nothing below the
  architecture config knows the word "Qwen2".
"""

from __future__ import annotations

import json
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Mapping, Optional, Sequence


class ConfigError(ValueError):
    """config.json does not describe a model this engine can build."""


@dataclass(frozen=True)
class PartSpec:
    """One part of a layer: which implementation (`kind`, a key of the part registry),
    where its tensors live in the checkpoint (`prefix`), and its sizes and constants."""

    kind: str
    prefix: str = ""
    params: Mapping[str, Any] = field(default_factory=dict)

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)


@dataclass(frozen=True)
class LayerSpec:
    """A layer = an arrangement (`block`) and the parts it arranges, under the names that the block's
    class gives them (the pre-norm block of this package: `mixer`, `feed_forward`, `mixer_norm`,
    `feed_forward_norm`; another block may arrange four norms, two mixers, or no feed-forward)."""

    block: PartSpec
    parts: Mapping[str, PartSpec] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order: run layer `layer`; `cache_of` names the layer whose
    cache it uses (itself by default). A layer that reads another layer's cache writes
    nothing into it."""

    layer: int
    cache_of: Optional[int] = None

    @property
    def cache_layer(self) -> int:
        return self.layer if self.cache_of is None else self.cache_of

    @property
    def writes_cache(self) -> bool:
        return self.cache_of is None or self.cache_of == self.layer


@dataclass(frozen=True)
class ModelSpec:
    """Everything the builder needs; produced by an architecture's config."""

    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding: PartSpec
    layers: Sequence[LayerSpec]
    order: Sequence[LayerCall]
    final_norm: PartSpec
    head: PartSpec
    eos_token_ids: Sequence[int] = ()
    # A position encoding that acts on the embeddings (learned or computed absolute positions); encodings
    # that act inside a mixer (rotation) are named in that mixer's params instead.
    position: Optional[PartSpec] = None


def read_config_json(model_dir) -> dict:
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise ConfigError(f"no config.json in {model_dir}")
    try:
        data = json.loads(path.read_text())
    except json.JSONDecodeError as exc:
        raise ConfigError(f"{path}: not valid JSON ({exc})") from exc
    if not isinstance(data, dict):
        raise ConfigError(f"{path}: expected a JSON object")
    return data


def _require(data: Mapping[str, Any], key: str, kind=int):
    if key not in data or data[key] is None:
        raise ConfigError(f"config.json lacks required key '{key}'")
    try:
        return kind(data[key])
    except (TypeError, ValueError) as exc:
        raise ConfigError(f"config.json key '{key}' = {data[key]!r} is not {kind.__name__}") from exc


@dataclass(frozen=True)
class Qwen2Config:
    """The keys of a Qwen2 `config.json`.

    Required keys have no default, as in the reference's reader
    (worker/src/inference/qwen2/model.py:41-74); its validation errors are kept.
    Keys the reference never reads but this engine needs: `max_position_embeddings`,
    `sliding_window`, `use_sliding_window`, `max_window_layers`, `eos_token_id`.
    """

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    max_position_embeddings: int
    layer_windows: tuple  # per layer: window length or None
    hidden_act: str = "silu"
    eos_token_ids: tuple = ()

    architecture = "Qwen2ForCausalLM"

    @property
    def num_key_value_groups(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "Qwen2Config":
        heads = _require(data, "num_attention_heads")
        kv_heads = int(data.get("num_key_value_heads") or heads)
        hidden = _require(data, "hidden_size")
        if heads < 1 or kv_heads < 1 or heads % kv_heads != 0:
            raise ConfigError("num_attention_heads must be a positive multiple of num_key_value_heads")
        explicit = data.get("head_dim")
        head_dim = int(explicit) if explicit else hidden // heads
        if head_dim < 1 or hidden != heads * head_dim:
            raise ConfigError("hidden_size must equal num_attention_heads * head_dim")
        if head_dim % 2 != 0:
            raise ConfigError("head_dim must be even for rotate-half RoPE")
        act = data.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"only silu MLP is supported, got {act}")
        layers = _require(data, "num_hidden_layers")
        vocab = _require(data, "vocab_size")
        inter = _require(data, "intermediate_size")
        if layers < 1 or vocab < 1 or inter < 1:
            raise ConfigError("num_hidden_layers, vocab_size and intermediate_size must be >= 1")
        eps = _require(data, "rms_norm_eps", float)
        theta = cls._rope_theta(data)
        max_pos = int(data.get("max_position_embeddings") or 0)
        if max_pos < 1:
            raise ConfigError("config.json lacks required key 'max_position_embeddings'")
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        return cls(
            vocab_size=vocab, hidden_size=hidden, intermediate_size=inter, num_hidden_layers=layers,
            num_attention_heads=heads, num_key_value_heads=kv_heads, head_dim=head_dim,
            rms_norm_eps=eps, rope_theta=theta,
            tie_word_embeddings=bool(data.get("tie_word_embeddings", False)),
            max_position_embeddings=max_pos,
            layer_windows=cls._layer_windows(data, layers),
            hidden_act=act, eos_token_ids=eos_ids,
        )

    @staticmethod
    def _rope_theta(data: Mapping[str, Any]) -> float:
        """`rope_parameters.rope_theta` wins; any rope type but "default" is an error
        (worker/src/inference/qwen2/model.py:413-419)."""
        params = data.get("rope_parameters") or {}
        scaling = data.get("rope_scaling") or {}
        for source in (params, scaling):
            if isinstance(source, dict):
                kind = source.get("rope_type", source.get("type", "default"))
                if kind != "default":
                    raise ConfigError(f"unsupported RoPE type {kind}")
        if isinstance(params, dict) and "rope_theta" in params:
            return float(params["rope_theta"])
        return _require(data, "rope_theta", float)

    @staticmethod
    def _layer_windows(data: Mapping[str, Any], layers: int) -> tuple:
        """Which layers see only the last `sliding_window` keys.

        The reference rejects every windowed layer (model.py:58-60); here `layer_types`
        wins when present ("full_attention" / "sliding_attention", the strings of
        worker/tests/test_qwen2.py:67), otherwise layer l is windowed iff
        `use_sliding_window` and l >= `max_window_layers`."""
        window = data.get("sliding_window")
        types = data.get("layer_types")
        if types:
            types = list(types)
            if len(types) != layers:
                raise ConfigError(f"layer_types has {len(types)} entries for {layers} layers")
            out = []
            for kind in types:
                if kind == "full_attention":
                    out.append(None)
                elif kind == "sliding_attention":
                    if window is None or int(window) < 1:
                        raise ConfigError("sliding_attention layers need sliding_window >= 1")
                    out.append(int(window))
                else:
                    raise ConfigError(f"unknown layer type {kind!r}")
            return tuple(out)
        if not data.get("use_sliding_window", False) or window is None:
            return (None,) * layers
        if int(window) < 1:
            raise ConfigError("sliding_window must be >= 1")
        first = int(data.get("max_window_layers", layers))
        return tuple(int(window) if l >= first else None for l in range(layers))

    def to_dict(self) -> dict:
        """The config.json that reads back as this configuration."""
        windows = [w for w in self.layer_windows if w is not None]
        out = {
            "architectures": [self.architecture],
            "model_type": "qwen2",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "max_position_embeddings": self.max_position_embeddings,
            "hidden_act": self.hidden_act,
        }
        if windows:
            out["sliding_window"] = windows[0]
            out["layer_types"] = ["full_attention" if w is None else "sliding_attention"
                                  for w in self.layer_windows]
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out

    def model_spec(self) -> ModelSpec:
        """Qwen2 as parts: pre-norm blocks of grouped-query attention with q/k/v bias and
        rotary positions, a SwiGLU feed-forward and RMS norms
        (worker/src/inference/qwen2/model.py:138-152, 228-249, 293-303)."""
        layers = []
        for l in range(self.num_hidden_layers):
            base = f"model.layers.{l}."
            norm = {"eps": self.rms_norm_eps, "size": self.hidden_size}
            layers.append(LayerSpec(PartSpec("prenorm_residual"), {
                "mixer": PartSpec("attention", base + "self_attn.", {
                    "hidden_size": self.hidden_size,
                    "num_heads": self.num_attention_heads,
                    "num_kv_heads": self.num_key_value_heads,
                    "head_dim": self.head_dim,
                    "qkv_bias": True,
                    "out_bias": False,
                    "window": self.layer_windows[l],
                    "scale": self.head_dim ** -0.5,
                    "position": PartSpec("rope", "", {"dim": self.head_dim, "theta": self.rope_theta}),
                }),
                "feed_forward": PartSpec("swiglu", base + "mlp.", {
                    "hidden_size": self.hidden_size,
                    "intermediate_size": self.intermediate_size,
                }),
                "mixer_norm": PartSpec("rmsnorm", base + "input_layernorm.", norm),
                "feed_forward_norm": PartSpec("rmsnorm", base + "post_attention_layernorm.", norm),
            }))
        return ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab_size,
            hidden_size=self.hidden_size,
            max_positions=self.max_position_embeddings,
            embedding=PartSpec("token_embedding", "model.embed_tokens.",
                               {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size}),
            layers=tuple(layers),
            order=tuple(LayerCall(l) for l in range(self.num_hidden_layers)),
            final_norm=PartSpec("rmsnorm", "model.norm.", {"eps": self.rms_norm_eps, "size": self.hidden_size}),
            head=PartSpec("lm_head", "lm_head.", {
                "vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                "tied_to": "model.embed_tokens.weight" if self.tie_word_embeddings else None}),
            eos_token_ids=self.eos_token_ids,
        )
