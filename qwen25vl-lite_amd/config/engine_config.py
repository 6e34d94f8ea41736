"""Scheduling and memory settings of the engine (reference src/qwen25vl_lite/engine.py:43-66).

The names and meanings are the reference's; the settings of parts this engine does not have
(quantised cache, vision tiers, pruning, swap to host memory, graph buckets) are left out.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

__all__ = ["EngineConfig", "DTYPES", "dtype_from_name"]

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def dtype_from_name(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in DTYPES.values():
            raise ValueError(f"dtype {name} is not built; use one of {sorted(DTYPES)}")
        return name
    try:
        return DTYPES[str(name)]
    except KeyError:
        raise ValueError(f"dtype {name!r} is not built; use one of {sorted(DTYPES)}") from None


@dataclass
class EngineConfig:
    """Knobs of the scheduler and the cache.

    ``num_blocks`` pages of ``block_size`` tokens are made for every cache group;
    ``max_num_seqs`` requests may be live at once; a step runs at most
    ``max_num_batched_tokens`` tokens, decoded tokens included; ``max_model_len`` bounds a
    request's prompt plus output.  ``preemption`` is what happens when pages run out:
    only ``"recompute"`` is built (the victim gives its pages back and is prefilled again,
    prompt and tokens generated so far).  ``hip_graph`` replays decode steps from captured HIP graphs;
    with ``decode_lookahead`` (off unless asked for) the scheduler then queues the decode step after the running one before
    the host has seen the running one's tokens (the ids go from the sampler to the next step on the
    device), so that the GPU does not wait for the host between steps.
    ``tune_library_products`` lets PyTorch's TunableOp choose the library kernel of each product shape
    (seconds per new shape, once): for runs with few distinct step sizes.
    """

    num_blocks: int = 2048
    block_size: int = 16
    max_num_seqs: int = 8
    max_num_batched_tokens: int = 4096
    max_model_len: int = 32768
    enable_prefix_cache: bool = True
    enable_chunked_prefill: bool = True
    preemption: str = "recompute"
    device: str = "cuda:0"
    dtype: torch.dtype = torch.float32
    hip_graph: bool = False
    decode_lookahead: bool = False
    tune_library_products: bool = False

    def __post_init__(self) -> None:
        self.dtype = dtype_from_name(self.dtype)
        if self.block_size <= 0 or self.num_blocks <= 0:
            raise ValueError("block_size and num_blocks must be positive")
        if self.block_size % 16:
            raise ValueError("block_size must be a multiple of 16 (the attention kernels walk keys 16 at a time)")
        if self.max_num_seqs <= 0:
            raise ValueError("max_num_seqs must be positive")
        if self.max_num_batched_tokens <= 0:
            raise ValueError("max_num_batched_tokens must be positive")
        if self.max_model_len <= 0:
            raise ValueError("max_model_len must be positive")
        if self.preemption != "recompute":
            raise ValueError("preemption must be 'recompute' (swapping pages to host memory is not built)")

    @property
    def max_blocks_per_seq(self) -> int:
        return (self.max_model_len + self.block_size - 1) // self.block_size
