"""Decoding options of a request (reference src/qwen25vl_lite/sampling.py:16-41)."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Sequence

__all__ = ["SamplingParams"]


@dataclass
class SamplingParams:
    """``temperature == 0`` means greedy.  Names, defaults and meanings are the reference's:

    * ``top_k > 0`` keeps the scores that reach the k-th largest; ``min_p`` drops tokens whose
      probability is below ``min_p`` times the largest; ``top_p`` keeps the smallest set of the
      most likely tokens whose mass reaches ``top_p`` (the token that crosses it stays);
      they apply in this order, after the division by ``temperature``.
    * the penalties act on the tokens generated so far: logits of seen tokens are divided by
      ``repetition_penalty`` if positive, else multiplied; then ``presence_penalty`` and
      ``frequency_penalty`` times the count are subtracted.
    * ``seed``: the random number of output token ``i`` comes from a generator seeded with
      ``seed + i`` (reference engine.py:823-829), so a request's stream does not depend on what it
      is batched with; ``None`` draws from the global generator.
    * ``stop`` (strings) is refused by the engine, which has no tokenizer; ``stop_token_ids``
      ends the request with reason ``"stop"``.
    """

    temperature: float = 0.0
    top_p: float = 1.0
    top_k: int = -1
    max_tokens: int = 512
    repetition_penalty: float = 1.0
    presence_penalty: float = 0.0
    frequency_penalty: float = 0.0
    min_p: float = 0.0
    seed: Optional[int] = None
    stop: Sequence[str] = field(default_factory=tuple)
    stop_token_ids: Sequence[int] = field(default_factory=tuple)
    ignore_eos: bool = False

    def validate(self) -> None:
        """Raise ValueError for a value outside its range, naming the field and the value."""
        ranges = (
            ("temperature", self.temperature >= 0, "zero (greedy) or more"),
            ("top_p", 0.0 < self.top_p <= 1.0, "above 0 and at most 1"),
            ("min_p", 0.0 <= self.min_p <= 1.0, "between 0 and 1"),
            ("max_tokens", self.max_tokens >= 1, "at least one token"),
            ("repetition_penalty", self.repetition_penalty > 0, "above 0 (1 switches it off)"),
        )
        for name, ok, wanted in ranges:
            if not ok:
                raise ValueError(f"SamplingParams.{name} = {getattr(self, name)!r}: expected {wanted}")
