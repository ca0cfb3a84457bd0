"""Text-in / text-out entry point, in the manner of the reference's ``engine.llm``
(python/engine/llm.py:33-77)."""

from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path
from typing import List, Optional, Sequence

from ..config.base import generation_end_token
from ..sampling.params import SamplingParams
from .engine import Engine
from .model import Model


@dataclass
class GenerationConfig:
    max_tokens: int = 64
    temperature: float = 0.0  # <= 0 is greedy
    top_k: int = 0
    top_p: float = 1.0


class LLM:
    """Load a model folder and generate through the engine.

    Options of the reference keep their names and meanings: ``block_size`` (tokens per cache
    page), ``num_blocks`` (pages in the pool; 0: as many as the free device memory holds), ``seed`` (sampling), ``max_batch`` (most requests
    running at once), ``eos_id`` (default: read from the folder).  ``dtype`` ('bfloat16' or
    'float32'), ``max_tokens_per_step``, ``prefill_chunk``, ``tune_gemms`` and ``weight_copies`` (keep
    the large matrices a second time in the order the decode kernels read them: twice the memory,
    decode steps some 8 % faster) are this engine's.
    ``enable_prefix_cache`` is accepted and has no effect (no prefix cache here); ``quantize``
    is refused (no quantized weights here)."""

    def __init__(self, model_dir, *, block_size: int = 16, num_blocks: int = 2048, seed: int = 0,
                 max_batch: int = 256, eos_id: Optional[int] = None, enable_prefix_cache: bool = True,
                 quantize: bool = False, dtype: str = "bfloat16", device: str = "cuda:0",
                 max_tokens_per_step: int = 2048, prefill_chunk: Optional[int] = None, tune_gemms: bool = False,
                 weight_copies: bool = True):
        if quantize:
            raise NotImplementedError("LLM: quantized weights are not part of this engine")
        model_dir = Path(model_dir)
        self.model = Model.from_pretrained(model_dir, dtype=dtype, device=device, weight_copies=weight_copies)
        self.engine = Engine(self.model, block_size, num_blocks, seed, max_batch, enable_prefix_cache,
                             max_tokens_per_step=max_tokens_per_step, prefill_chunk=prefill_chunk,
                             fill_rows=self._tuned_rows(tune_gemms, self.model))
        if eos_id is None:
            # the folder's generation_config.json, then the model's typed configuration
            eos_id = generation_end_token(model_dir)
            if eos_id < 0:
                eos_id = self.model.config.end_token
        self.eos_id = eos_id
        self._model_dir = model_dir
        self._tokenizer = None

    @staticmethod
    def _tuned_rows(tune_gemms: bool, model):
        """``tune_gemms``: let torch time the library's kernels for the product shapes of a few row
        counts (seconds, once per shape) instead of trusting its heuristic, and fill the steps that are
        not decode steps up to those counts.  Only the bfloat16 path calls the library."""
        import torch

        if not tune_gemms or model.dtype != torch.bfloat16:
            return None
        from ..ops import enable_library_tuning
        from .context import padded_tokens

        enable_library_tuning()
        return padded_tokens

    @classmethod
    def from_config(cls, config, weight_seed: int = 0, *, block_size: int = 16, num_blocks: int = 2048, seed: int = 0,
                    max_batch: int = 256, eos_id: int = -1, dtype: str = "bfloat16", device: str = "cuda:0",
                    max_tokens_per_step: int = 2048, prefill_chunk: Optional[int] = None,
                    weight_copies: bool = True, tune_gemms: bool = False) -> "LLM":
        """An engine over random weights made from ``config`` (the dictionary of a config.json, or a
        typed configuration) and ``weight_seed``: no folder, no tokenizer, token ids in and out.
        The weights are those that ``write_random_model`` writes for the same seed (as float32)."""
        from ..models import parse_config

        typed = parse_config(config) if isinstance(config, dict) else config
        llm = cls.__new__(cls)
        llm.model = Model.from_random(typed, weight_seed, dtype=dtype, device=device, weight_copies=weight_copies)
        llm.engine = Engine(llm.model, block_size, num_blocks, seed, max_batch,
                            max_tokens_per_step=max_tokens_per_step, prefill_chunk=prefill_chunk,
                            fill_rows=cls._tuned_rows(tune_gemms, llm.model))
        llm.eos_id = eos_id
        llm._model_dir = None
        llm._tokenizer = None
        return llm

    @property
    def tokenizer(self):
        if self._tokenizer is None and self._model_dir is None:
            raise RuntimeError("LLM: a model made from a configuration has no tokenizer; use generate_ids")
        if self._tokenizer is None:
            from .tokenizer import EngineTokenizer

            self._tokenizer = EngineTokenizer.from_model_dir(self._model_dir)
        return self._tokenizer

    def _params(self, config: GenerationConfig) -> SamplingParams:
        return SamplingParams(config.temperature, config.top_k, config.top_p)

    def generate_ids(self, prompt_ids: Sequence[int], config: Optional[GenerationConfig] = None) -> List[int]:
        config = config or GenerationConfig()
        return self.engine.generate(list(prompt_ids), self._params(config), config.max_tokens, self.eos_id)

    def generate_ids_batch(self, prompts: Sequence[Sequence[int]],
                           config: Optional[GenerationConfig] = None) -> List[List[int]]:
        config = config or GenerationConfig()
        return self.engine.generate_batch(prompts, self._params(config), config.max_tokens, self.eos_id)

    def generate(self, prompt: str, config: Optional[GenerationConfig] = None) -> str:
        ids = self.tokenizer.encode(prompt)
        return self.tokenizer.decode(self.generate_ids(ids, config))
