"""The Qwen2.5-VL text decoder as a model spec (reference src/qwen25vl_lite/text.py).

Per layer: RMSNorm, attention with biased q/k/v projections, MRoPE and grouped key/value
heads, an unbiased output projection, RMSNorm, a SwiGLU feed-forward; then a final RMSNorm
and an output head that may be the embedding table.  Layers the configuration marks as
``sliding_attention`` see only the last ``sliding_window`` keys.
"""

from __future__ import annotations

from typing import List, Optional

from ..config.model_config import Qwen25VLConfig
from ..config.registry import register_architecture
from ..parts.base import PartSpec
from .spec import LayerSpec, ModelSpec, RunEntry

__all__ = ["qwen25vl_text_spec", "map_checkpoint_name", "store_checkpoint_name"]

_ROOTS = ("embed_tokens", "layers", "norm")


def store_checkpoint_name(name: str) -> str:
    """Canonical name -> the released checkpoints' name (the inverse of :func:`map_checkpoint_name`
    for the layout a written model folder uses)."""
    return name if name.startswith("lm_head.") else "model.language_model." + name


def map_checkpoint_name(name: str) -> Optional[str]:
    """Checkpoint name -> canonical name (``layers.0.self_attn.q_proj.weight``, ``lm_head.weight`` ...).

    Both layouts in the wild are taken (reference model.py:52-73): ``model.language_model.*``
    of the released checkpoints and ``model.*`` of newer writers.  The vision tower's tensors
    (``visual.*``, ``model.visual.*``) are not part of this model and are skipped.
    """
    if name.startswith("lm_head."):
        return name
    rest = name[len("model."):] if name.startswith("model.") else name
    if rest.startswith("visual."):
        return None
    if rest.startswith("language_model."):
        rest = rest[len("language_model."):]
    if rest.split(".")[0] in _ROOTS:
        return rest
    return name  # unknown: reported by the loader as unexpected


def qwen25vl_text_spec(config: Qwen25VLConfig) -> ModelSpec:
    t = config.text_config
    position = PartSpec("mrope", {"theta": t.rope_theta, "sections": tuple(t.mrope_section)})

    # layer_schedule: entries are layer indices, or {"layer": i, "cache_from": j} where j is an
    # earlier position of the list whose keys and values the entry reads.
    run: List[RunEntry] = []
    if t.layer_schedule:
        for e in t.layer_schedule:
            if isinstance(e, dict):
                run.append(RunEntry(int(e["layer"]), None if e.get("cache_from") is None else int(e["cache_from"])))
            else:
                run.append(RunEntry(int(e)))
    else:
        run = [RunEntry(i) for i in range(t.num_hidden_layers)]
    reads_only = {e.layer for e in run if e.cache_from is not None}
    writes = {e.layer for e in run if e.cache_from is None}
    if reads_only & writes:
        raise ValueError(f"layers {sorted(reads_only & writes)} appear both with and without cache_from")

    layers: List[LayerSpec] = []
    for i in range(t.num_hidden_layers):
        norm = PartSpec("rms_norm", {"size": t.hidden_size, "eps": t.rms_norm_eps})
        mixer = PartSpec("paged_attention", {
            "hidden_size": t.hidden_size,
            "num_heads": t.num_attention_heads,
            "num_kv_heads": t.num_key_value_heads,
            "head_dim": t.head_dim,
            "qkv_bias": True,            # always on in this architecture (reference text.py:79-82)
            "window": t.layer_window(i),
            "scale": None,
            "position": position,
            "kv_shared": i in reads_only,
        })
        ffn = PartSpec("swiglu", {"hidden_size": t.hidden_size, "intermediate_size": t.intermediate_size})
        block = PartSpec("pre_norm", {
            "norm1": norm, "mixer": mixer, "norm2": norm, "ffn": ffn,
            "names": {"norm1": "input_layernorm", "mixer": "self_attn",
                      "norm2": "post_attention_layernorm", "ffn": "mlp"},
        })
        layers.append(LayerSpec(block, f"layers.{i}."))

    return ModelSpec(
        hidden_size=t.hidden_size,
        vocab_size=t.vocab_size,
        layers=layers,
        run=run,
        final_norm=PartSpec("rms_norm", {"size": t.hidden_size, "eps": t.rms_norm_eps}),
        tie_word_embeddings=t.tie_word_embeddings,
        position_rows=3,
        map_name=map_checkpoint_name,
        store_name=store_checkpoint_name,
        eos_token_id=config.eos_token_id,
    )


register_architecture("Qwen2_5_VLForConditionalGeneration", qwen25vl_text_spec, Qwen25VLConfig.from_dict)
# model_type, for a config.json without architectures, and that of a bare text_config
register_architecture("qwen2_5_vl", qwen25vl_text_spec, Qwen25VLConfig.from_dict)
register_architecture("qwen2_5_vl_text", qwen25vl_text_spec, Qwen25VLConfig.from_dict)
