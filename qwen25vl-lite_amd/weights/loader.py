"""Loading a model's tensors from safetensors, by name
(reference src/qwen25vl_lite/model.py:351-442).

The model says which tensors it expects (canonical name, shape, role).  The checkpoint's
names are mapped by the architecture (both ``model.language_model.*`` and ``model.*`` are
taken, ``visual.*`` is skipped).  Everything wrong with a checkpoint is collected and raised
as one :class:`WeightsError` that lists the missing tensors, the unexpected ones and the
wrong shapes.  Tensors are copied to the device part by part, so the host never holds a
second copy of the model.

How tensors are kept: matrices and tables in the run dtype (bfloat16 stays bfloat16; for a
float32 run everything becomes float32); vectors (norm weights, biases) in float32, which is
where they enter the arithmetic, so a vector stored in 32-bit keeps all its bits; integer
tables as int32.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from .safetensors_io import SafetensorsFile, checkpoint_shards

__all__ = ["WeightsError", "load_weights", "kept_dtype"]


class WeightsError(RuntimeError):
    """The checkpoint does not fit the model.  ``missing``, ``unexpected`` and ``wrong_shape``
    hold the details that the message lists."""

    def __init__(self, missing: List[str], unexpected: List[str], wrong_shape: List[Tuple[str, tuple, tuple]],
                 wrong_dtype: List[Tuple[str, str]] = ()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        lines = ["the checkpoint does not fit the model:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + ", ".join(
                f"{n}: checkpoint {tuple(got)} != model {tuple(want)}" for n, got, want in self.wrong_shape))
        if self.wrong_dtype:
            lines.append(f"  wrong dtype ({len(self.wrong_dtype)}): " + ", ".join(
                f"{n}: {d}" for n, d in self.wrong_dtype))
        super().__init__("\n".join(lines))


def kept_dtype(role: str, run_dtype: torch.dtype) -> torch.dtype:
    if role == "int":
        return torch.int32
    if role == "vector":
        return torch.float32
    return run_dtype


def load_weights(model_dir: str, model, *, strict: bool = True, progress=None) -> Dict[str, int]:
    """Fill ``model`` (a :class:`DecoderModel`) from the safetensors files of ``model_dir``.

    Returns counters ``{"loaded", "skipped", "tied"}``.  With ``strict`` (the default) any
    missing or unexpected tensor or wrong shape raises :class:`WeightsError`; without it
    unexpected tensors are ignored, the rest still raises.
    """
    expected = model.expected_tensors()
    spec = model.spec
    files = [SafetensorsFile(p) for p in checkpoint_shards(model_dir)]
    try:
        where: Dict[str, Tuple[SafetensorsFile, str]] = {}
        unexpected: List[str] = []
        skipped = 0
        for f in files:
            for raw in f.keys():
                name = spec.map_name(raw)
                if name is None:
                    skipped += 1
                elif name in expected:
                    where[name] = (f, raw)
                else:
                    unexpected.append(raw)

        tied = False
        missing = [n for n in expected if n not in where]
        if spec.head_name in missing and spec.tie_word_embeddings:
            # reference model.py:381-388, 416-418: a stored head wins; else a tied head is the table
            missing.remove(spec.head_name)
            tied = True
        wrong_shape, wrong_dtype = [], []
        for name, (f, raw) in where.items():
            if f.shape(raw) != tuple(expected[name].shape):
                wrong_shape.append((raw, f.shape(raw), tuple(expected[name].shape)))
            is_float = f.dtype(raw).is_floating_point
            if is_float != (expected[name].role != "int"):
                wrong_dtype.append((raw, f"stored as {f.dtype(raw)}"))
        if missing or wrong_shape or wrong_dtype or (strict and unexpected):
            raise WeightsError(sorted(missing), sorted(unexpected) if strict else [], wrong_shape, wrong_dtype)

        loaded = 0
        for part, names in model.part_groups():
            tensors = {}
            for local, name in names.items():
                if name not in where:
                    continue  # the tied head
                f, raw = where[name]
                dtype = kept_dtype(expected[name].role, model.dtype)
                tensors[local] = f.tensor(raw).to(device=model.device, dtype=dtype).contiguous()
                loaded += 1
                if progress is not None:
                    progress(name)
            if tensors:
                model.load_part(part, tensors)
        if tied:
            model.tie_head()
        return {"loaded": loaded, "skipped": skipped, "tied": int(tied)}
    finally:
        for f in files:
            f.close()
