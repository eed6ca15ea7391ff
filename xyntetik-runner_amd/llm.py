"""The Python entry point: load a model folder and generate.

    from xyntetik_runner_amd import LLM, SamplingParams
    llm = LLM("/path/to/model", dtype="bfloat16")
    tokens = llm.generate([[1, 2, 3]], SamplingParams(temperature=0.8, seed=7, max_new_tokens=32))

The reference's Python package is a client of its HTTP server
(python/src/xyntetik_runner/__init__.py:1-35); this one binds the
engine directly and works on token ids.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Union

from .engine import Engine, ModelRunner
from .sampling import SamplingParams


class LLM:
    def __init__(self, model: str, dtype: str = "bfloat16", max_tokens: Optional[int] = None,
                 page_size: int = 64, max_batched_tokens: int = 2048, max_running: int = 64,
                 max_model_len: Optional[int] = None, device: str = "cuda:0", gpu_memory_fraction: float = 0.9):
        """``max_tokens``: cache positions over all live requests.  By default the cache takes what
        ``gpu_memory_fraction`` of the card leaves once the weights are loaded (at most what
        ``max_running`` requests of ``max_model_len`` tokens need), and ``CacheTooSmall`` is raised
        if that does not hold one request of ``max_model_len`` (default: the model's context)."""
        from .config import load_config
        arch, cfg = load_config(model)
        spec = arch.build_spec(cfg)
        ctx = max_model_len or spec.max_position
        self.runner = ModelRunner.from_folder(model, dtype=dtype, max_tokens=max_tokens, max_model_len=ctx,
                                              gpu_memory_fraction=gpu_memory_fraction,
                                              max_step_tokens=max_batched_tokens,
                                              page_size=page_size, max_requests=max_running, device=device)
        self.engine = Engine(self.runner, max_batched_tokens=max_batched_tokens, max_running=max_running,
                             max_model_len=ctx)

    @property
    def spec(self):
        return self.runner.spec

    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Union[SamplingParams, Sequence[SamplingParams], None] = None) -> List[List[int]]:
        return self.engine.generate(prompts, params)

    def add_request(self, prompt: Sequence[int], params: Optional[SamplingParams] = None, req_id=None):
        return self.engine.add_request(prompt, params, req_id)

    def step(self):
        return self.engine.step()

    def has_work(self) -> bool:
        return self.engine.has_work()
