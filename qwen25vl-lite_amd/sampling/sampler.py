"""The device sampler: one token per logits row, chosen by a HIP kernel.

The reference samples on the host, one request at a time (reference
src/qwen25vl_lite/sampling.py:67-121, engine.py:802-829).  Here a step's rows are sampled
together on the GPU; the only host work is the uniform random number of each row, which comes
from the reference's per-token generator rule (seed + number of tokens generated so far).
"""

from __future__ import annotations

import ctypes
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..ops.kernels import KernelError, _check, _fn, _stream
from .params import SamplingParams

__all__ = ["sample_rows", "sample_rows_begin", "sample_slots_begin", "PendingSample", "uniform_for", "uniform_from"]

_ROW = np.dtype([("temperature", "<f4"), ("top_p", "<f4"), ("min_p", "<f4"), ("u", "<f4"),
                 ("repetition", "<f4"), ("presence", "<f4"), ("frequency", "<f4"), ("top_k", "<i4"),
                 ("prev_begin", "<i4"), ("prev_end", "<i4")])


def uniform_from(seed: Optional[int], step: int) -> float:
    """The uniform number in [0, 1) for output token number ``step`` of a request with this seed
    (None: from the global generator): a generator seeded with ``seed + step`` draws it
    (the rule of reference engine.py:823-829)."""
    if seed is None:
        return float(torch.rand(1).item())
    gen = torch.Generator()
    gen.manual_seed(int(seed) + int(step))
    return float(torch.rand(1, generator=gen).item())


def uniform_for(params: SamplingParams, step: int) -> float:
    """The uniform number in [0, 1) for a request's output token number ``step``."""
    return 0.0 if params.temperature <= 0 else uniform_from(params.seed, step)


class _Staging:
    """Pinned host buffers that take turns carrying the sampler's per-row settings to the device:
    a copy from pinned memory does not make the host wait for the work queued before it."""

    _rings = {}

    @classmethod
    def to_device(cls, packed: np.ndarray, device: torch.device) -> torch.Tensor:
        key = device.index or 0
        ring = cls._rings.setdefault(key, {"turn": -1, "slots": [None] * 4})
        turn = ring["turn"] = (ring["turn"] + 1) % len(ring["slots"])
        slot = ring["slots"][turn]
        if slot is None or slot[0].numel() < packed.size:
            slot = ring["slots"][turn] = (torch.empty(max(1024, 2 * packed.size), dtype=torch.int32, pin_memory=True),
                                         torch.cuda.Event())
        else:
            slot[1].synchronize()       # the copy that last read this buffer is done
        host, copied = slot
        host.numpy()[:packed.size] = packed
        buf = torch.empty(packed.size, dtype=torch.int32, device=device)
        buf.copy_(host[:packed.size], non_blocking=True)
        copied.record()
        return buf


class PendingSample:
    """Sampled ids that are on their way: ``device_ids`` (int32 ``[M]``, valid for kernels queued
    after the sampler on the same stream) and a copy to pinned host memory whose end an event
    marks.  :meth:`result` waits for that copy only, not for work queued after it."""

    _pinned = {}     # device index -> ring of pinned int32 buffers, so that two samples can be pending
    _turn = {}

    def __init__(self, device_ids: torch.Tensor):
        m = device_ids.numel()
        key = device_ids.device.index or 0
        ring = self._pinned.setdefault(key, [None] * 4)
        turn = self._turn[key] = (self._turn.get(key, -1) + 1) % len(ring)
        if ring[turn] is None or ring[turn].numel() < m:
            ring[turn] = torch.empty(max(256, m), dtype=torch.int32, pin_memory=True)
        self.device_ids = device_ids
        self._host = ring[turn][:m]
        self._host.copy_(device_ids, non_blocking=True)
        self._event = torch.cuda.Event()
        self._event.record()
        self._ids: Optional[List[int]] = None

    def result(self) -> List[int]:
        if self._ids is None:
            self._event.synchronize()
            self._ids = self._host.tolist()
        return self._ids


def sample_rows(logits: torch.Tensor, params: Sequence[SamplingParams], prev_ids: Sequence[Sequence[int]],
                steps: Sequence[int], uniforms: Optional[Sequence[float]] = None) -> List[int]:
    """Sample a token for each row of float32 ``logits [M, vocab]`` on the GPU.

    ``prev_ids[m]`` are the tokens request ``m`` has generated so far (for the penalties) and
    ``steps[m]`` their number (for the seed rule).  ``uniforms`` overrides the random numbers.
    """
    pending = sample_rows_begin(logits, params, prev_ids, steps, uniforms)
    return pending.result() if pending is not None else []


def sample_rows_begin(logits: torch.Tensor, params: Sequence[SamplingParams], prev_ids: Sequence[Sequence[int]],
                      steps: Sequence[int], uniforms: Optional[Sequence[float]] = None) -> Optional[PendingSample]:
    """Queue the sampling of :func:`sample_rows` and the copy of its ids to the host; nothing is
    waited for.  None for no rows."""
    if not logits.is_cuda:
        raise KernelError("sampling has no CPU path: logits must be on the GPU")
    if logits.dtype != torch.float32 or logits.dim() != 2 or not logits.is_contiguous():
        raise KernelError("logits must be contiguous float32 [M, vocab]")
    m, vocab = logits.shape
    if not (len(params) == len(prev_ids) == len(steps) == m):
        raise ValueError("one SamplingParams, token list and step per logits row is needed")
    if m == 0:
        return None
    rows = np.zeros(m, _ROW)
    flat: List[int] = []
    first = params[0]
    if (uniforms is None and first.temperature <= 0 and first.repetition_penalty == 1.0 and first.presence_penalty == 0.0
            and first.frequency_penalty == 0.0 and all(p is first or p == first for p in params)):
        # one greedy setting for the whole batch (the usual decode step): fill the rows at once
        rows[:] = (first.temperature, first.top_p, first.min_p, 0.0, 1.0, 0.0, 0.0, first.top_k if first.top_k else -1, 0, 0)
        params_iter = ()
    else:
        params_iter = enumerate(params)
    for i, p in params_iter:
        need_prev = p.repetition_penalty != 1.0 or p.presence_penalty != 0.0 or p.frequency_penalty != 0.0
        begin = len(flat)
        if need_prev:
            flat.extend(int(t) for t in prev_ids[i])
        u = uniforms[i] if uniforms is not None else uniform_for(p, steps[i])
        rows[i] = (p.temperature, p.top_p, p.min_p, u, p.repetition_penalty, p.presence_penalty,
                   p.frequency_penalty, p.top_k if p.top_k else -1, begin, len(flat))
    need_scores = any(p.temperature > 0 or len(flat) for p in params)
    plain = any(p.temperature <= 0 and p.repetition_penalty == 1.0 and p.presence_penalty == 0.0
                and p.frequency_penalty == 0.0 for p in params)
    return _launch(logits, rows, flat, need_scores, plain)


def sample_slots_begin(logits: torch.Tensor, records, slots: Sequence[int], prev_ids: Sequence[Sequence[int]],
                       uniforms: Optional[Sequence[float]] = None) -> Optional[PendingSample]:
    """:func:`sample_rows_begin` for requests whose settings and sampler state lie in their slots
    (``records``: :class:`~qwen25vl_lite_amd.cache.slots.SlotRecords`): row ``m`` of the logits belongs to the
    request in slot ``slots[m]``.  The rows' settings are gathered by slot index; only rows with
    penalties (their generated tokens, ``prev_ids[m]``) and rows that draw (one generator each, by
    the seed rule) are visited one by one."""
    if not logits.is_cuda:
        raise KernelError("sampling has no CPU path: logits must be on the GPU")
    if logits.dtype != torch.float32 or logits.dim() != 2 or not logits.is_contiguous():
        raise KernelError("logits must be contiguous float32 [M, vocab]")
    m = logits.shape[0]
    at = np.asarray(slots, np.int64)
    if at.shape != (m,) or len(prev_ids) != m:
        raise ValueError("one slot and token list per logits row is needed")
    if m == 0:
        return None
    rows = np.zeros(m, _ROW)
    for name in ("temperature", "top_p", "min_p", "top_k", "repetition", "presence", "frequency"):
        rows[name] = getattr(records, name)[at]
    flat: List[int] = []
    draws = rows["temperature"] > 0
    penal = (rows["repetition"] != 1.0) | (rows["presence"] != 0.0) | (rows["frequency"] != 0.0)
    for i in np.nonzero(penal)[0]:
        rows["prev_begin"][i] = len(flat)
        flat.extend(int(t) for t in prev_ids[i])
        rows["prev_end"][i] = len(flat)
    for i in np.nonzero(draws)[0]:
        seed = int(records.seed[at[i]])
        rows["u"][i] = uniforms[i] if uniforms is not None else uniform_from(None if seed < 0 else seed,
                                                                             int(records.generated[at[i]]))
    return _launch(logits, rows, flat, bool(draws.any() or flat), bool((~draws & ~penal).any()))


def _launch(logits: torch.Tensor, rows: np.ndarray, flat: List[int], need_scores: bool, plain: bool) -> PendingSample:
    """Send the rows' settings to the device and queue the sampler.  ``need_scores``: some row scales
    or penalises its logits (into a copy); ``plain``: some row is a plain argmax."""
    m, vocab = logits.shape
    fn = _fn("sample", "qvl_sample_rows",
             [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
              ctypes.c_int, ctypes.c_int, ctypes.c_void_p])
    dev = logits.device
    with torch.cuda.device(dev):
        packed = np.concatenate([rows.view(np.int32), np.asarray(flat or [0], np.int32)])
        buf = _Staging.to_device(packed, dev)
        n_row_words = rows.view(np.int32).size
        scores = torch.empty_like(logits) if need_scores else logits
        out = torch.empty(m, dtype=torch.int32, device=dev)
        # a greedy row without penalties is a plain argmax: several blocks scan it side by side
        parts = None
        if plain:
            part_bytes = int(_fn("sample", "qvl_sample_argmax_part_bytes", [])())
            parts = torch.empty(m * part_bytes, dtype=torch.uint8, device=dev)
        _check(fn(logits.data_ptr(), scores.data_ptr(), buf.data_ptr(), buf[n_row_words:].data_ptr(),
                  parts.data_ptr() if parts is not None else None, out.data_ptr(), m, vocab, _stream()),
               "sample_rows")
        return PendingSample(out)
