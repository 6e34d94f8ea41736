"""The step function: runs a batch of (request, its next tokens) through the model from the
cache and returns the logits at the wanted places.

Reference counterpart: ``ModelRunner`` (reference src/qwen25vl_lite/engine.py:204-486), which
runs a prompt portion of one request or single tokens of several, never both.  Here both
share one batch: only the tokens brought are run, as one flat batch, against the keys and
values earlier steps left in the pages.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from ..cache import CacheManager, KVStorage
from ..config.engine_config import EngineConfig
from ..models.decoder import DecoderModel
from .batch import StepEntry, build_step

__all__ = ["ModelRunner"]


class ModelRunner:
    """Owns the cache (manager and tensors) and the per-request state, and steps the model."""

    def __init__(self, model: DecoderModel, engine_cfg: EngineConfig, *, max_prefix_nodes: int = 4096):
        if model.device.type != "cuda":
            raise RuntimeError("the model runs on the GPU only; build it with device='cuda:0'")
        if model.dtype != engine_cfg.dtype:
            raise ValueError(f"the model holds {model.dtype} weights but the engine is set to {engine_cfg.dtype}")
        self.model = model
        self.ecfg = engine_cfg
        self.device = model.device
        self.dtype = model.dtype
        self.vocab_size = model.spec.vocab_size
        self.eos_token_id = model.spec.eos_token_id
        groups = model.cache_groups()
        # A cached prefix holds keys and values only.  A mixer with a state of its own would start
        # a request that adopted one from a cleared state, not from the state after the prefix:
        # with such a mixer in the model the prefix cache stays off.
        has_state = any(need is not None for need in model.entry_state)
        self.cache = CacheManager(groups, engine_cfg.num_blocks, engine_cfg.block_size, engine_cfg.max_num_seqs,
                                  enable_prefix_cache=engine_cfg.enable_prefix_cache and not has_state,
                                  max_prefix_nodes=max_prefix_nodes)
        self.storage = KVStorage(groups, engine_cfg.num_blocks, engine_cfg.block_size, self.dtype, self.device)
        # one state row per request slot, and a spare one that the padding rows of a captured
        # decode step read and write
        self.pad_state_slot = engine_cfg.max_num_seqs
        self.states: List[Optional[torch.Tensor]] = [
            None if need is None else torch.zeros((engine_cfg.max_num_seqs + 1, *need.shape), dtype=need.dtype,
                                                  device=self.device)
            for need in model.entry_state
        ]
        self.slots = model.make_slots(self.storage, self.states)
        self.position_rows = model.spec.position_rows
        self.steps = 0
        if engine_cfg.tune_library_products:
            from ..ops.linear import tune_library_products
            tune_library_products(True)
        # decode steps from HIP graphs, if asked for and every part can be captured
        self.graphs = None
        if engine_cfg.hip_graph and model.graph_safe:
            from .graph import DecodeGraphs
            self.graphs = DecodeGraphs(self)

    def close(self) -> None:
        """Drop the captured decode graphs now (after a device synchronization) instead of when the
        runner goes away.  The runner keeps working: graphs are captured again when needed."""
        if self.graphs is not None:
            self.graphs.close()

    # ------------------------------------------------------------------ requests
    def admit(self, req_id, params=None, rope_delta: int = 0) -> int:
        return self.cache.admit(req_id, params, rope_delta)

    def release(self, req_id) -> None:
        self.cache.release(req_id)

    def fork(self, src_id, dst_id) -> None:
        """``dst_id`` continues from where ``src_id`` stands: full pages shared, the page being
        filled copied, per-request state rows copied."""
        for group, src_page, dst_page in self.cache.fork(src_id, dst_id):
            self.storage.copy_pages(group, [src_page], [dst_page])
        a, b = self.cache.slot_of(src_id), self.cache.slot_of(dst_id)
        for state in self.states:
            if state is not None:
                state[b].copy_(state[a])
        self.cache.take_fresh(dst_id)      # the copied state must not be cleared

    def _clear_state(self, entries: Sequence[StepEntry]) -> None:
        for e in entries:
            if self.cache.take_fresh(e.req_id):
                slot = self.cache.slot_of(e.req_id)
                for state in self.states:
                    if state is not None:
                        state[slot].zero_()

    # ------------------------------------------------------------------ the step
    @torch.no_grad()
    def execute(self, entries: Sequence[StepEntry], device_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Run one step.  Pages for the new tokens are reserved here if the caller has not done
        so (:class:`~qwen25vl_lite_amd.cache.OutOfPages` if they cannot be).  Returns float32 logits
        ``[wanted, vocab]`` in the order of the entries and of each entry's ``want``.

        ``device_tokens`` (int32 ``[len(entries)]`` on the device): the entries' single tokens, for
        a step that :meth:`decodes_from_graph` and is queued before the host has seen the ids the
        step before it sampled; the entries' own token ids are placeholders then."""
        for e in entries:
            self.cache.reserve(e.req_id, e.start + len(e.tokens))
        self._clear_state(entries)
        with torch.cuda.device(self.device):
            if self.graphs is not None and self.graphs.takes(entries):
                for e in entries:
                    if not 0 <= e.tokens[0] < self.vocab_size:
                        raise ValueError(f"request {e.req_id!r}: token id outside [0, {self.vocab_size})")
                    if self.cache.num_tokens(e.req_id) != e.start:
                        raise ValueError(f"request {e.req_id!r}: the step does not continue where the cache ends")
                    if self.cache.records.rope_delta[self.cache.slot_of(e.req_id)] != e.rope_delta:
                        raise ValueError(f"request {e.req_id!r}: the entry's rope delta is not the one in its slot's "
                                         "record (set at admission)")
                logits = self.graphs.run(entries, device_tokens)
            elif device_tokens is not None:
                raise ValueError("token ids on the device are taken by decode steps that run from a graph only")
            else:
                step = build_step(entries, self.cache, self.position_rows, self.dtype, self.device, self.vocab_size)
                logits = self.model.forward(step, self.slots)
        for e in entries:
            self.cache.commit(e.req_id, e.start + len(e.tokens))
        self.steps += 1
        return logits

    def decodes_from_graph(self, entries: Sequence[StepEntry]) -> bool:
        """Whether :meth:`execute` would replay these entries from a decode graph."""
        return self.graphs is not None and self.graphs.takes(entries)

    def sample_begin(self, logits: torch.Tensor, params: Sequence, prev_ids: Sequence[Sequence[int]],
                     steps: Sequence[int]):
        """Queue the sampling; the returned object has ``device_ids`` and ``result()`` (see
        :class:`~qwen25vl_lite_amd.sampling.sampler.PendingSample`)."""
        from ..sampling.sampler import sample_rows_begin
        with torch.cuda.device(self.device):
            return sample_rows_begin(logits, params, prev_ids, steps)

    def sample_slots_begin(self, logits: torch.Tensor, slots: Sequence[int], prev_ids: Sequence[Sequence[int]]):
        """Queue the sampling of one token per logits row for the requests in ``slots``, whose
        settings and sampler state lie in the cache manager's slot records; ``prev_ids`` are the
        tokens each has generated (read for rows with penalties only).  Returns what
        :meth:`sample_begin` returns."""
        from ..sampling.sampler import sample_slots_begin
        with torch.cuda.device(self.device):
            return sample_slots_begin(logits, self.cache.records, slots, prev_ids)

    def sample(self, logits: torch.Tensor, params: Sequence, prev_ids: Sequence[Sequence[int]],
               steps: Sequence[int]) -> List[int]:
        """One token per logits row, on the device (see :mod:`qwen25vl_lite_amd.sampling`)."""
        from ..sampling.sampler import sample_rows
        return sample_rows(logits, params, prev_ids, steps)
