"""A small front end: model folder in, generated token ids out.

The reference has no such class; its tests and CLI wire the pieces by hand (reference
tests/test_engine.py:21-33, cli.py:106-118, 210-241).  ``LLM`` does that wiring:
configuration, model from the registry, weights, runner, scheduler.
"""

from __future__ import annotations

from typing import List, Optional, Sequence, Union

from ..config import EngineConfig, dtype_from_name, load_config
from ..models import build_model
from ..sampling.params import SamplingParams
from ..weights import fill_random, load_weights
from .runner import ModelRunner
from .scheduler import LLMEngine, RequestOutput

__all__ = ["LLM"]


class LLM:
    """``LLM(model_dir, dtype="bfloat16", **engine options).generate(prompts, params)``.

    ``model`` is a folder with ``config.json`` and ``model.safetensors``, or a configuration
    object (of any registered architecture) together with ``random_seed`` for random weights
    drawn on the GPU.  The architecture named in ``config.json`` decides how the rest of the
    file is read and which model is built.  Engine options are the fields of :class:`EngineConfig`.
    """

    def __init__(self, model, dtype="bfloat16", *, random_seed: Optional[int] = None,
                 device: str = "cuda:0", **engine_options):
        run_dtype = dtype_from_name(dtype)
        from_folder = isinstance(model, (str, bytes)) or hasattr(model, "__fspath__")
        if from_folder:
            self.config = load_config(model)
        else:
            self.config = model
            if random_seed is None:
                raise ValueError("a configuration without a model folder needs random_seed")
        self.model = build_model(self.config, run_dtype, device)
        if random_seed is not None:
            fill_random(self.model, int(random_seed))
        else:
            load_weights(model, self.model)
        self.engine_config = EngineConfig(dtype=run_dtype, device=device, **engine_options)
        self.runner = ModelRunner(self.model, self.engine_config)
        self.engine = LLMEngine(self.runner, self.engine_config)

    def close(self) -> None:
        """Give the captured decode graphs back now; ``with LLM(...) as llm:`` does it on leaving."""
        self.runner.close()

    def __enter__(self) -> "LLM":
        return self

    def __exit__(self, *exc) -> None:
        self.close()

    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Union[SamplingParams, Sequence[SamplingParams], None] = None) -> List[RequestOutput]:
        """Generate for every prompt (lists of token ids); results in the order of the prompts."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        if len(params) != len(prompts):
            raise ValueError("one SamplingParams per prompt is needed")
        ids = [self.engine.add_request(p, sp) for p, sp in zip(prompts, params)]
        by_id = {o.seq_id: o for o in self.engine.run_until_complete()}
        return [by_id[i] for i in ids]
