"""The Python entry point: load a model folder once, generate for lists of token ids.

The blocking loop of the reference (``generate_with_prefill_token_quantum``,
src/generation.rs:1412-1533) is the scheduler run with one or many requests.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence, Union

from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .engine import Engine
from .scheduler import EngineConfig, Request, Scheduler


@dataclass
class GenerationResult:
    """Tokens and the reference's metrics of one request (src/generation.rs:35-99)."""
    token_ids: List[int]
    finish_reason: str
    prompt_tokens: int
    time_to_first_token: Optional[float]
    total_time: float
    prefill_time: Optional[float] = None       # from the request's admission to its first token

    @property
    def generated_tokens(self) -> int:
        return len(self.token_ids)

    @property
    def prefill_tokens_per_second(self) -> Optional[float]:
        """Prompt tokens over the time from admission to the first token (src/generation.rs:76-79)."""
        if not self.prefill_time or self.prefill_time <= 0:
            return None
        return self.prompt_tokens / self.prefill_time

    @property
    def output_tokens_per_second(self) -> Optional[float]:
        """Emitted tokens over the whole time of the request (src/generation.rs:93-98)."""
        return len(self.token_ids) / self.total_time if self.total_time > 0 else None

    @property
    def decode_tokens_per_second(self) -> Optional[float]:
        if self.time_to_first_token is None or len(self.token_ids) < 2:
            return None
        decode_time = self.total_time - self.time_to_first_token
        return (len(self.token_ids) - 1) / decode_time if decode_time > 0 else None


class LLM:
    """A loaded model with its cache, sampler and scheduler settings."""

    def __init__(self, model: Union[str, Engine], dtype: str = "bfloat16", device: str = "cuda:0",
                 kv_cache_block_tokens: int = 16, kv_cache_capacity_tokens: Optional[int] = None,
                 engine_config: Optional[EngineConfig] = None, measured_paths: bool = True):
        """``model``: a folder with config.json and model.safetensors, or an ``Engine`` that is
        already built (its own dtype and cache sizes then hold; it needs a state slot for each of
        ``engine_config.max_active_sequences``).  ``measured_paths``: as for ``Engine``."""
        self.engine_config = engine_config or EngineConfig()
        if isinstance(model, Engine):
            self.engine = model
            if self.engine.cache.slots.total < self.engine_config.max_active_sequences:
                raise ValueError(f"the engine has {self.engine.cache.slots.total} state slots, fewer than "
                                 f"max_active_sequences = {self.engine_config.max_active_sequences}")
        else:
            self.engine = Engine(model, dtype=dtype, device=device, kv_cache_block_tokens=kv_cache_block_tokens,
                                 kv_cache_capacity_tokens=kv_cache_capacity_tokens,
                                 max_active_sequences=self.engine_config.max_active_sequences,
                                 measured_paths=measured_paths)
        self.sampler = Sampler(self.engine.vocab_size, self.engine.device)
        eos = getattr(self.engine.config, "eos_token_id", None)
        self.stop_token_ids = () if eos is None else (eos,)
        self._next_id = 0

    def generate(self, prompts: Sequence[Sequence[int]],
                 sampling_params: Union[SamplingParams, Sequence[SamplingParams], None] = None,
                 on_token=None, on_round=None) -> List[GenerationResult]:
        """``prompts``: token ids of each request.  One ``SamplingParams`` for all, or one per
        prompt; with a single one, request i samples with ``seed + i`` (the reference offsets
        its seed per request the same way, src/main.rs:188-197).  ``on_token(request, token)`` is
        called for every emitted token, ``on_round(seconds)`` after every round of the scheduler."""
        if sampling_params is None:
            sampling_params = SamplingParams()
        if isinstance(sampling_params, SamplingParams):
            base = sampling_params
            per_request = [SamplingParams(**{**base.__dict__, "seed": base.seed + index})
                           for index in range(len(prompts))]
        else:
            per_request = list(sampling_params)
            if len(per_request) != len(prompts):
                raise ValueError("one SamplingParams per prompt is needed")
        scheduler = Scheduler(self.engine, self.sampler, self.engine_config, self.stop_token_ids, on_token)
        ids = []
        for prompt, params in zip(prompts, per_request):
            request_id = f"gen-{self._next_id}"
            self._next_id += 1
            ids.append(request_id)
            scheduler.submit(request_id, prompt, params)
        finished = scheduler.run(on_round)
        results = []
        for request_id in ids:
            request: Request = finished[request_id]
            ttft = None if request.first_token_at is None else request.first_token_at - request.submitted_at
            prefill = None
            if request.first_token_at is not None and request.started_at is not None:
                prefill = request.first_token_at - request.started_at
            results.append(GenerationResult(list(request.generated), request.finish_reason, len(request.prompt),
                                            ttft, request.finished_at - request.submitted_at, prefill))
        return results


def generate(model: Union[str, LLM], prompts: Sequence[Sequence[int]],
             sampling_params: Union[SamplingParams, Sequence[SamplingParams], None] = None,
             **llm_options) -> List[List[int]]:
    """Generated token ids for each prompt.  ``model``: a folder with config.json and
    model.safetensors, or an ``LLM`` that is already loaded."""
    llm = model if isinstance(model, LLM) else LLM(model, **llm_options)
    return [result.token_ids for result in llm.generate(prompts, sampling_params)]
