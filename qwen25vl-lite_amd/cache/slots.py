"""The fixed-size record every live request keeps in its slot.

A request's slot (an index below ``max_num_seqs``) names a row in each of these arrays: how many
of its tokens are in the cache, the offset of its text positions (the rope delta of a prompt with
explicit position rows, reference src/qwen25vl_lite/cache.py:584-610), and its sampler's state
(the seed and the number of tokens generated so far, from which the reference draws token by
token, engine.py:823-829, and the settings of sampling.py:16-41).  The scheduler fills a row when
it admits a request and moves it on as tokens are computed and sampled; a step then gathers what
it needs for all its requests with one index operation per field instead of a loop over requests.
"""

from __future__ import annotations

import numpy as np

__all__ = ["SlotRecords", "NO_SEED"]

NO_SEED = -1     # draws come from the global generator


class SlotRecords:
    FIELDS = (("num_tokens", np.int32), ("rope_delta", np.int32), ("seed", np.int64), ("generated", np.int32),
              ("temperature", np.float32), ("top_p", np.float32), ("min_p", np.float32), ("top_k", np.int32),
              ("repetition", np.float32), ("presence", np.float32), ("frequency", np.float32))

    def __init__(self, max_num_seqs: int):
        self.size = int(max_num_seqs)
        for name, dtype in self.FIELDS:
            setattr(self, name, np.zeros(self.size, dtype))
        self.clear_all()

    def clear_all(self) -> None:
        for slot in range(self.size):
            self.clear(slot)

    def clear(self, slot: int) -> None:
        """The record of a slot nobody holds: greedy, no penalties, nothing computed."""
        self.num_tokens[slot] = self.rope_delta[slot] = self.generated[slot] = 0
        self.seed[slot] = NO_SEED
        self.temperature[slot] = self.min_p[slot] = self.presence[slot] = self.frequency[slot] = 0.0
        self.top_p[slot] = self.repetition[slot] = 1.0
        self.top_k[slot] = -1

    def assign(self, slot: int, params=None, rope_delta: int = 0, generated: int = 0) -> None:
        """Fill a slot's record at admission.  ``params``: the request's sampling settings (an
        object with the fields of ``SamplingParams``), None for a request that is not sampled."""
        self.clear(slot)
        self.rope_delta[slot] = int(rope_delta)
        self.generated[slot] = int(generated)
        if params is not None:
            self.seed[slot] = NO_SEED if params.seed is None else int(params.seed)
            self.temperature[slot] = params.temperature
            self.top_p[slot] = params.top_p
            self.min_p[slot] = params.min_p
            self.top_k[slot] = params.top_k if params.top_k else -1
            self.repetition[slot] = params.repetition_penalty
            self.presence[slot] = params.presence_penalty
            self.frequency[slot] = params.frequency_penalty

    def copy(self, src: int, dst: int) -> None:
        for name, _ in self.FIELDS:
            getattr(self, name)[dst] = getattr(self, name)[src]

    def plain_greedy(self, slots: np.ndarray) -> bool:
        """Whether all these requests take the largest logit as it is (no temperature, no penalties)."""
        return bool((self.temperature[slots] <= 0).all() and (self.repetition[slots] == 1.0).all()
                    and (self.presence[slots] == 0.0).all() and (self.frequency[slots] == 0.0).all())
