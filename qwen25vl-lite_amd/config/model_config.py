"""Typed model configuration, read from a model folder's ``config.json``.

Every size and constant of the decoder comes from the file.  Sizes have no default: a
``config.json`` that leaves one out is refused.  The few optional keys follow the rules the
reference applies when a key is absent (reference src/qwen25vl_lite/config.py:77-134 for the
decoder fields, :163-201 for where they are looked up).
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, fields
from typing import Any, Dict, Optional, Tuple

__all__ = ["ConfigError", "TextConfig", "Qwen25VLConfig", "read_config_json"]


class ConfigError(ValueError):
    """A ``config.json`` that cannot describe a model this engine builds."""


_REQUIRED_SIZES = (
    "hidden_size",
    "intermediate_size",
    "num_hidden_layers",
    "num_attention_heads",
    "vocab_size",
)

FULL_ATTENTION = "full_attention"
SLIDING_ATTENTION = "sliding_attention"


@dataclass(frozen=True)
class TextConfig:
    """Sizes and constants of the text decoder (``text_config`` in config.json).

    Field names are the keys of ``config.json`` (reference config.py:81-95).  Added keys:
    ``max_window_layers`` and ``layer_types`` decide which layers use the sliding window,
    ``head_dim`` may be given instead of derived, and ``layer_schedule`` gives the order in
    which layers run.
    """

    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    vocab_size: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int = 128000
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1_000_000.0
    mrope_section: Tuple[int, ...] = ()
    hidden_act: str = "silu"
    attention_dropout: float = 0.0
    sliding_window: Optional[int] = None
    use_sliding_window: bool = False
    max_window_layers: Optional[int] = None
    layer_types: Tuple[str, ...] = ()
    layer_schedule: Tuple[Any, ...] = ()
    tie_word_embeddings: bool = True

    # ------------------------------------------------------------------ derived
    @property
    def num_key_value_groups(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    def layer_window(self, layer: int) -> Optional[int]:
        """The sliding window of a layer, or None if it sees every earlier key."""
        if self.layer_types[layer] == SLIDING_ATTENTION:
            return int(self.sliding_window)
        return None

    def num_params(self) -> int:
        """Parameter count (reference config.py:120-134)."""
        h, hd, inter = self.hidden_size, self.head_dim, self.intermediate_size
        nh, nkv = self.num_attention_heads, self.num_key_value_heads
        per_layer = h * nh * hd + nh * hd
        per_layer += 2 * (h * nkv * hd + nkv * hd)
        per_layer += nh * hd * h
        per_layer += 3 * h * inter
        per_layer += 2 * h
        total = self.vocab_size * h + per_layer * self.num_hidden_layers + h
        if not self.tie_word_embeddings:
            total += self.vocab_size * h
        return total

    def kv_bytes_per_token(self, bytes_per_value: int) -> int:
        """Bytes of keys and values one token holds in all layers (reference planner.py:39-41)."""
        return 2 * self.num_hidden_layers * self.num_key_value_heads * self.head_dim * bytes_per_value

    # ------------------------------------------------------------------ parsing
    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "TextConfig":
        raw = dict(raw)
        missing = [k for k in _REQUIRED_SIZES if k not in raw]
        if missing:
            raise ConfigError(f"config.json lacks the size(s) {missing}; no size has a default")
        nh = int(raw["num_attention_heads"])
        hidden = int(raw["hidden_size"])
        layers = int(raw["num_hidden_layers"])
        if nh <= 0 or hidden <= 0 or layers <= 0:
            raise ConfigError("hidden_size, num_attention_heads and num_hidden_layers must be positive")
        nkv = int(raw.get("num_key_value_heads") or nh)
        if raw.get("head_dim") is not None:
            head_dim = int(raw["head_dim"])
        else:
            # reference config.py:97-99: the head size is hidden_size // heads
            if hidden % nh:
                raise ConfigError(
                    f"hidden_size {hidden} is not a multiple of num_attention_heads {nh} and no head_dim is given")
            head_dim = hidden // nh
        if nh % nkv:
            raise ConfigError(f"num_attention_heads {nh} is not a multiple of num_key_value_heads {nkv}")
        if head_dim % 2:
            raise ConfigError(f"head_dim {head_dim} must be even for the rotation")

        section = raw.get("mrope_section")
        if section is None:
            raise ConfigError("config.json gives no mrope_section (looked in rope_scaling, rope_parameters, "
                              "text_config and the top level)")
        section = tuple(int(s) for s in section)
        if len(section) != 3 or sum(section) != head_dim // 2 or min(section) < 0:
            raise ConfigError(
                f"mrope_section {section} must be three counts that add up to head_dim/2 = {head_dim // 2}")

        act = str(raw.get("hidden_act", "silu"))
        if act != "silu":
            raise ConfigError(f"hidden_act {act!r} is not built; the decoder's feed-forward uses 'silu'")

        use_window = bool(raw.get("use_sliding_window", False))
        window = raw.get("sliding_window")
        window = None if window is None else int(window)
        max_window_layers = raw.get("max_window_layers")
        max_window_layers = None if max_window_layers is None else int(max_window_layers)
        layer_types = raw.get("layer_types")
        if layer_types is not None:
            layer_types = tuple(str(t) for t in layer_types)
            if len(layer_types) != layers:
                raise ConfigError(f"layer_types has {len(layer_types)} entries for {layers} layers")
            bad = sorted(set(layer_types) - {FULL_ATTENTION, SLIDING_ATTENTION})
            if bad:
                raise ConfigError(f"unknown layer type(s) {bad}")
        elif use_window:
            # Layers with index >= max_window_layers use the window; the others see everything.
            first = layers if max_window_layers is None else max_window_layers
            layer_types = tuple(SLIDING_ATTENTION if i >= first else FULL_ATTENTION for i in range(layers))
        else:
            layer_types = tuple(FULL_ATTENTION for _ in range(layers))
        if SLIDING_ATTENTION in layer_types and (window is None or window <= 0):
            raise ConfigError("a layer uses sliding attention but sliding_window is not a positive number")

        schedule = raw.get("layer_schedule")
        schedule = tuple(schedule) if schedule is not None else ()

        kwargs: Dict[str, Any] = dict(
            hidden_size=hidden,
            intermediate_size=int(raw["intermediate_size"]),
            num_hidden_layers=layers,
            num_attention_heads=nh,
            vocab_size=int(raw["vocab_size"]),
            num_key_value_heads=nkv,
            head_dim=head_dim,
            mrope_section=section,
            hidden_act=act,
            sliding_window=window,
            use_sliding_window=use_window,
            max_window_layers=max_window_layers,
            layer_types=layer_types,
            layer_schedule=schedule,
        )
        for key, cast in (("max_position_embeddings", int), ("rms_norm_eps", float), ("rope_theta", float),
                          ("attention_dropout", float), ("tie_word_embeddings", bool)):
            if raw.get(key) is not None:
                kwargs[key] = cast(raw[key])
        if kwargs["intermediate_size"] <= 0 or kwargs["vocab_size"] <= 0:
            raise ConfigError("intermediate_size and vocab_size must be positive")
        return cls(**kwargs)

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {}
        for f in fields(self):
            v = getattr(self, f.name)
            if isinstance(v, tuple):
                v = list(v)
            out[f.name] = v
        if not out["layer_schedule"]:
            out.pop("layer_schedule")
        return out


@dataclass(frozen=True)
class Qwen25VLConfig:
    """Top level of ``config.json`` (reference config.py:137-201).

    Only what the text decoder and the scheduler use is kept: the decoder's fields, the
    architecture name that picks the model class, the end-of-sequence id, and the stored
    dtype.  Vision fields are ignored.
    """

    text_config: TextConfig
    architectures: Tuple[str, ...] = ()
    model_type: str = ""
    eos_token_id: Optional[int] = None
    bos_token_id: Optional[int] = None
    pad_token_id: Optional[int] = None
    torch_dtype: str = "bfloat16"
    name_or_path: str = field(default="", compare=False)

    @property
    def vocab_size(self) -> int:
        return self.text_config.vocab_size

    @property
    def hidden_size(self) -> int:
        return self.text_config.hidden_size

    @property
    def tie_word_embeddings(self) -> bool:
        return self.text_config.tie_word_embeddings

    @property
    def architecture(self) -> str:
        """The key into the architecture registry."""
        if self.architectures:
            return self.architectures[0]
        return self.model_type

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "Qwen25VLConfig":
        # The decoder's fields live in text_config; a file without one gives them at the top.
        if isinstance(raw.get("text_config"), dict):
            text_raw = dict(raw["text_config"])
        else:
            text_raw = {k: v for k, v in raw.items() if k in _TEXT_KEYS}
        # reference config.py:165-177: rope constants may sit in rope_scaling (released
        # checkpoints) or rope_parameters, at the top level or in text_config; the decoder's
        # own key wins, then those blocks, then a top-level key.
        for key in ("rope_scaling", "rope_parameters"):
            for holder in (raw, raw.get("text_config") or {}):
                block = holder.get(key)
                if isinstance(block, dict):
                    for name in ("mrope_section", "rope_theta"):
                        if name in block and text_raw.get(name) is None:
                            text_raw[name] = block[name]
        for name in ("rope_theta", "mrope_section", "sliding_window", "use_sliding_window",
                     "max_window_layers", "layer_types"):
            if name in raw and text_raw.get(name) is None:
                text_raw[name] = raw[name]
        if text_raw.get("tie_word_embeddings") is None:
            # reference config.py:178
            text_raw["tie_word_embeddings"] = raw.get("tie_word_embeddings", True)
        text = TextConfig.from_dict(text_raw)

        def opt_int(key):
            v = raw.get(key)
            if isinstance(v, (list, tuple)):
                v = v[0] if v else None
            return None if v is None else int(v)

        return cls(
            text_config=text,
            architectures=tuple(raw.get("architectures") or ()),
            model_type=str(raw.get("model_type", "")),
            eos_token_id=opt_int("eos_token_id"),
            bos_token_id=opt_int("bos_token_id"),
            pad_token_id=opt_int("pad_token_id"),
            torch_dtype=str(raw.get("torch_dtype", raw.get("dtype", "bfloat16"))),
            name_or_path=str(raw.get("_name_or_path", "")),
        )

    def to_dict(self) -> Dict[str, Any]:
        text = self.text_config.to_dict()
        out: Dict[str, Any] = {
            "architectures": list(self.architectures),
            "model_type": self.model_type,
            "torch_dtype": self.torch_dtype,
            "tie_word_embeddings": self.text_config.tie_word_embeddings,
            "rope_scaling": {"type": "mrope", "mrope_section": list(self.text_config.mrope_section)},
            "text_config": text,
        }
        for key in ("eos_token_id", "bos_token_id", "pad_token_id"):
            if getattr(self, key) is not None:
                out[key] = getattr(self, key)
        return out

    @classmethod
    def from_json(cls, path: str) -> "Qwen25VLConfig":
        return cls.from_dict(read_config_json(path))

    @classmethod
    def from_pretrained(cls, model_dir: str) -> "Qwen25VLConfig":
        """Read ``<model_dir>/config.json``; a path to a ``.json`` file is taken as is
        (reference config.py:203-211)."""
        path = model_dir if str(model_dir).endswith(".json") else os.path.join(model_dir, "config.json")
        if not os.path.isfile(path):
            raise FileNotFoundError(
                f"no config.json under {model_dir!r}; point --model at a folder that holds config.json "
                "and model.safetensors")
        cfg = cls.from_json(path)
        object.__setattr__(cfg, "name_or_path", os.path.abspath(os.path.dirname(path)))
        return cfg


_TEXT_KEYS = {f.name for f in fields(TextConfig)}


def read_config_json(path: str) -> Dict[str, Any]:
    with open(path, "r", encoding="utf-8") as fh:
        raw = json.load(fh)
    if not isinstance(raw, dict):
        raise ConfigError(f"{path} does not hold a JSON object")
    return raw
