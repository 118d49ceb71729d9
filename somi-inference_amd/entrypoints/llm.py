"""The Python entry point, in the reference's manner.

Reference: ``LLM`` (somi_inference/entrypoints/llm.py:55-170): constructor
options ``num_blocks=256``, ``block_size=16``, ``max_concurrent=16``, ``device``,
``dtype=float32``; ``generate(prompt, *, max_new_tokens, temperature=1.0,
top_k=-1, top_p=1.0, repetition_penalty=1.0)`` returns only the newly generated
text; ``generate_stream`` raises ``NotImplementedError``.  Those names, defaults
and meanings are kept.  The three backend strings of the reference are gone (one
kernel path per dtype), and the reference's one-prompt-at-a-time ``generate`` also
takes token ids and lists of prompts, which run together under continuous batching.
"""

from __future__ import annotations

import os
from collections import deque
from dataclasses import replace
from typing import Iterator, Sequence

import torch

from ..config.base import ModelConfig, read_config_json
from ..config.engine import DEFAULT_BLOCK_SIZE, DEFAULT_MAX_CONCURRENT, DEFAULT_NUM_BLOCKS, EngineConfig
from ..engine.engine import Engine
from ..engine.request import Request
from ..engine.scheduler import Scheduler
from ..models.loader import load_model, make_runner, random_model
from ..sampling.params import SamplingParams
from ..sampling.rng import _mix
from ..sampling.sampler import Sampler
from .tokenizer import Tokenizer, has_tokenizer_files

Prompt = "str | Sequence[int]"


class LLM:
    def __init__(
        self,
        model_name: str | ModelConfig,
        *,
        num_blocks: int | None = DEFAULT_NUM_BLOCKS,
        block_size: int = DEFAULT_BLOCK_SIZE,
        max_concurrent: int = DEFAULT_MAX_CONCURRENT,
        device: torch.device | str | None = None,
        dtype: torch.dtype | str = torch.float32,
        max_num_batched_tokens: int = 2048,
        max_chunk: int | None = None,
        seed: int = 0,
        random_seed: int | None = None,
        eos_token_id: int | None = None,
        memory_fraction: float = 0.9,
    ) -> None:
        """``model_name``: a model folder (config.json + model.safetensors), or a typed
        configuration together with ``random_seed`` for seeded random weights.  ``num_blocks=None``
        (not in the reference): as many cache pages as fit into ``memory_fraction`` of the device memory that
        is free once the weights are loaded."""
        device = torch.device(device) if device is not None else torch.device("cuda:0")
        if device.type == "cuda" and device.index is None:
            device = torch.device("cuda:0")
        self.options = EngineConfig(dtype=str(dtype).replace("torch.", ""), block_size=block_size,
                                    num_blocks=1 if num_blocks is None else num_blocks, max_concurrent=max_concurrent,
                                    max_num_batched_tokens=max_num_batched_tokens, max_chunk=max_chunk,
                                    device=str(device))
        self.device, self.dtype, self.seed = device, self.options.dtype, int(seed)
        self.tokenizer: Tokenizer | None = None
        if isinstance(model_name, ModelConfig):
            if random_seed is None:
                raise ValueError("a configuration instead of a model folder needs random_seed")
            self.config = model_name
            self.model = random_model(self.config, random_seed, dtype=self.dtype, device=device)
        else:
            model_dir = os.fspath(model_name)
            self.model, self.config = load_model(model_dir, dtype=self.dtype, device=device)
            if has_tokenizer_files(model_dir):
                self.tokenizer = Tokenizer(model_dir)
        self.runner = make_runner(self.model, block_size=block_size, num_blocks=num_blocks,
                                  max_requests=max_concurrent, memory_fraction=memory_fraction)
        if num_blocks is None:
            self.options = replace(self.options, num_blocks=self.runner.cache.num_blocks)
        self.kv_manager = self.runner.cache
        self.sampler = Sampler()
        self.scheduler = Scheduler(self.runner.cache, max_concurrent=max_concurrent,
                                   max_num_batched_tokens=max_num_batched_tokens, chunk=self.options.chunk,
                                   vocab_size=self.model.vocab_size, max_positions=self.model.plan.max_positions,
                                   granule=self.model.portion_granule())
        if eos_token_id is None:
            eos_token_id = self.tokenizer.eos_token_id if self.tokenizer else getattr(self.config, "eos_token_id", None)
        self.engine = Engine(self.runner, self.scheduler, self.sampler, eos_token_id)
        self._next_seq_id = 0

    # ----------------------------------------------------------------- warm-up
    def warm_up(self, max_context: int | None = None) -> int:
        """Optional work before requests are served; not in the reference.

        The decode steps of up to ``max_concurrent`` requests with contexts of up to ``max_context`` tokens
        (default: 4,096, or what the pool holds if that is less) are captured as graphs, so that serving never
        stops to capture one.  Returns the number of graphs captured.
        """
        pool_tokens = self.options.num_blocks * self.options.block_size
        return self.runner.capture_decode_graphs(self.options.max_concurrent, min(max_context or 4096, pool_tokens))

    # ---------------------------------------------------------------- generate
    def _encode(self, prompt) -> tuple[list[int], bool]:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("the model folder has no tokenizer files: pass token ids instead of text")
            return self.tokenizer.encode(prompt), True
        return [int(t) for t in prompt], False

    def generate(
        self,
        prompt,
        *,
        max_new_tokens: int,
        temperature: float = 1.0,
        top_k: int = -1,
        top_p: float = 1.0,
        repetition_penalty: float = 1.0,
        seed: int | None = None,
    ):
        """Generate for one prompt or a list of prompts; returns only what was newly generated.

        A text prompt gives text, a prompt of token ids gives token ids; a list of
        prompts gives a list of results in the same order.  ``seed`` fixes the random
        stream of temperature sampling (per prompt: ``seed + index``).
        """
        many = isinstance(prompt, (list, tuple)) and len(prompt) > 0 and not isinstance(prompt[0], int)
        prompts = list(prompt) if many else [prompt]
        requests, as_text = [], []
        for index, item in enumerate(prompts):
            tokens, is_text = self._encode(item)
            as_text.append(is_text)
            request_seed = (seed + index) if seed is not None else _mix(self.seed ^ _mix(self._next_seq_id))
            params = SamplingParams(temperature=temperature, top_k=top_k, top_p=top_p,
                                    repetition_penalty=repetition_penalty, seed=request_seed)
            requests.append(Request(self._next_seq_id, tokens, max_new_tokens, params, seed=request_seed))
            self._next_seq_id += 1
        finished = self.engine.run(deque((0, r) for r in requests))
        if len(finished) != len(requests):
            raise RuntimeError(f"{len(requests)} requests were run and {len(finished)} finished")
        results = []
        for request, is_text in zip(requests, as_text):
            results.append(self.tokenizer.decode(request.output_tokens) if is_text else list(request.output_tokens))
        return results if many else results[0]

    def generate_stream(self, prompt: str, *, max_new_tokens: int) -> Iterator[str]:
        """Streaming generation is deferred, as in the reference (entrypoints/llm.py:166-170)."""
        del prompt, max_new_tokens
        raise NotImplementedError("Streaming not yet implemented")
