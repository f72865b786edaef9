"""The Python entry point: load a model folder, generate from token ids or text.

Mirrors the reference's ``Runtime::load`` + ``generate`` / ``generate_tokens``
(crates/leone/src/runtime.rs:1305, 3524-3540) and its ``GenerateOptions``
(crates/leone/src/runtime.rs:251-287): ``max_tokens`` there is ``max_new_tokens``
here, the sampler options keep their command-line names.
"""
from __future__ import annotations

import os
from typing import Callable, Hashable, List, Optional, Sequence, Union

import torch

from .engine.engine import Engine
from .engine.generate import GenerationResult, GenerationStats, generate_tokens
from .engine.scheduler import SchedulerPolicy
from .ops.profile import Recorder, StepProfile
from .runtime import load_model, random_model
from .sampling.sampler import SamplingParams


def sampling_params(temperature: Optional[float] = None, seed: int = 0, top_k: Optional[int] = None,
                    top_p: Optional[float] = None, min_p: Optional[float] = None,
                    truncations: Optional[Sequence[tuple]] = None, repeat_penalty: float = 1.0,
                    presence_penalty: float = 0.0, frequency_penalty: float = 0.0,
                    penalty_window: int = 64, dry_multiplier: float = 0.0, dry_base: float = 1.75,
                    dry_allowed_length: int = 2, dry_window: int = 64, dry_breakers: Sequence[int] = (),
                    mirostat: Optional[tuple] = None) -> SamplingParams:
    """``temperature`` None is greedy.  ``truncations`` gives stages in order; the named
    shortcuts are appended as top-k, top-p, min-p.  ``dry_multiplier`` above zero turns the
    repeated-suffix penalty on; ``mirostat`` is (target surprise in nats, learning rate)."""
    stages = list(truncations or [])
    if top_k is not None:
        stages.append(("top_k", top_k))
    if top_p is not None:
        stages.append(("top_p", top_p))
    if min_p is not None:
        stages.append(("min_p", min_p))
    params = SamplingParams(temperature, stages, seed, repeat_penalty, presence_penalty, frequency_penalty,
                            penalty_window, dry_multiplier, dry_base, dry_allowed_length, dry_window,
                            tuple(int(t) for t in dry_breakers), mirostat)
    if stages and temperature is None:
        raise ValueError("truncation stages need a temperature; greedy takes the highest logit")
    params.validate()
    return params


def cache_bytes_per_token(model) -> int:
    """Bytes one cached token takes over all cache slots of the model: every paged need says its own
    (``bytes_per_token(element size)``), whatever kind of cache it is."""
    size = torch.empty((), dtype=model.dtype).element_size()
    return sum(need.bytes_per_token(size) for need in model.cache_needs().values() if getattr(need, "paged", False))


def default_num_pages(model, page_tokens: int, max_requests: int, max_context: int, bytes_per_token: int) -> int:
    wanted = max_requests * ((max_context + page_tokens - 1) // page_tokens)
    free, _ = torch.cuda.mem_get_info(model.device)
    affordable = int(free * 0.8) // max(1, bytes_per_token * page_tokens)
    return max(1, min(wanted, affordable))


class Runtime:
    """A loaded model with its cache, ready to generate."""

    def __init__(self, model, *, num_pages: Optional[int] = None, max_tokens: Optional[int] = None,
                 page_tokens: int = 64, max_requests: int = 64, max_context: Optional[int] = None,
                 policy: Optional[SchedulerPolicy] = None, tokenizer=None, graphs: bool = True,
                 poison_freed: bool = False, streamed_weights: Optional[bool] = None, tune_products: bool = False):
        """``tune_products``: let the vendor library's products of a full prompt portion (the policy's
        ``prefill_chunk_tokens``) run with the fastest of the library's algorithms, measured now (a few
        seconds; ``Engine.tune_products``)."""
        self.model = model
        model.keep_streamed_copies(streamed_weights)       # before the cache is sized by what is free
        self.config = getattr(model, "config", None)
        context = min(max_context or model.spec.max_positions, model.spec.max_positions)
        if num_pages is None and max_tokens is None:
            num_pages = default_num_pages(model, page_tokens, max_requests, context, cache_bytes_per_token(model))
        self.engine = Engine(model, num_pages=num_pages, max_tokens=max_tokens, page_tokens=page_tokens,
                             max_requests=max_requests, max_context=context, graphs=graphs,
                             poison_freed=poison_freed, streamed_weights=streamed_weights)
        self.policy = policy or SchedulerPolicy(max_live_requests=max_requests)
        self.tuned_products = []
        if tune_products and model.dtype == torch.bfloat16:
            portion = min(self.policy.prefill_chunk_tokens, self.policy.max_step_tokens, context)
            if portion <= self.engine.cache.free_pages(0) * page_tokens:      # the trial step needs that room for a moment
                self.tuned_products = self.engine.tune_products(portion)
        self.tokenizer = tokenizer
        self.last_stats: Optional[GenerationStats] = None
        self.last_decode_profile: Optional[StepProfile] = None

    @classmethod
    def load(cls, model_dir: str, dtype: Union[str, torch.dtype] = "bfloat16", device: Optional[str] = None,
             **engine_options) -> "Runtime":
        model = load_model(model_dir, dtype, device)
        tokenizer = None
        tokenizer_file = os.path.join(model_dir, "tokenizer.json")
        if os.path.exists(tokenizer_file):
            from tokenizers import Tokenizer
            tokenizer = Tokenizer.from_file(tokenizer_file)
        return cls(model, tokenizer=tokenizer, **engine_options)

    @classmethod
    def random(cls, config, seed: int = 0, dtype: Union[str, torch.dtype] = "bfloat16",
               device: Optional[str] = None, **engine_options) -> "Runtime":
        return cls(random_model(config, seed, dtype, device), **engine_options)

    @property
    def eos_token_id(self) -> Optional[int]:
        return getattr(self.config, "eos_token_id", None)

    def generate_tokens(self, prompts: Sequence[Sequence[int]], max_new_tokens: int,
                        sampling: Union[SamplingParams, Sequence[Optional[SamplingParams]], None] = None,
                        eos_token_id: Union[int, None, str] = "config",
                        on_token: Optional[Callable[[Hashable, int], None]] = None,
                        logit_observer: Optional[Callable] = None,
                        profile_decode_steps: int = 0,
                        cancelled: Optional[Callable[[], bool]] = None, look_ahead: bool = True) -> List[GenerationResult]:
        """Token ids in, token ids out, one result per prompt in order.  ``sampling``: one policy for all prompts,
        or a list with one for each (None: greedy).  ``profile_decode_steps``: time
        that many decode steps operation by operation (they run without graph replay); the result is
        left in ``last_decode_profile``.  ``cancelled``: asked before every step; a yes ends every request
        with the tokens it has (the reference's cancellation flag, crates/leone-cli/src/main.rs:1600-1602).
        ``look_ahead`` False: every step waits for the tokens of the one before (``engine.generate.Generator``);
        the tokens are the same."""
        eos = self.eos_token_id if eos_token_id == "config" else eos_token_id
        recorder = Recorder(profile_decode_steps) if profile_decode_steps > 0 else None
        results, stats = generate_tokens(self.engine, prompts, max_new_tokens, sampling, eos, self.policy, on_token,
                                         logit_observer, recorder, cancelled, look_ahead)
        self.last_stats = stats
        self.last_decode_profile = recorder.profile if recorder is not None else None
        return results

    def encode(self, text: str) -> List[int]:
        if self.tokenizer is None:
            raise ValueError("the model folder has no tokenizer.json; give token ids instead of text")
        return list(self.tokenizer.encode(text).ids)

    def decode(self, tokens: Sequence[int]) -> str:
        if self.tokenizer is None:
            raise ValueError("the model folder has no tokenizer.json")
        return self.tokenizer.decode(list(tokens))

    def generate(self, prompts: Sequence[str], max_new_tokens: int, sampling: Optional[SamplingParams] = None,
                 **options) -> List[str]:
        results = self.generate_tokens([self.encode(p) for p in prompts], max_new_tokens, sampling, **options)
        return [self.decode(r.tokens) for r in results]


def generate(model: Union[str, dict, Runtime], prompts: Sequence[Sequence[int]], max_new_tokens: int,
             temperature: Optional[float] = None, seed: int = 0, top_k: Optional[int] = None,
             top_p: Optional[float] = None, eos_token_id: Union[int, None, str] = "config",
             dtype: str = "bfloat16", **engine_options) -> List[GenerationResult]:
    """One call: ``model`` is a model folder, a config.json mapping (random weights from ``seed``) or a Runtime."""
    if isinstance(model, Runtime):
        runtime = model
    elif isinstance(model, dict):
        runtime = Runtime.random(model, seed, dtype, **engine_options)
    else:
        runtime = Runtime.load(model, dtype, **engine_options)
    return runtime.generate_tokens(prompts, max_new_tokens, sampling_params(temperature, seed, top_k, top_p),
                                   eos_token_id)
