"""The reference's programmatic interface, in Python's spelling: `NewEngine(path, cfg)`, `Infer`,
`InferWithCallback`, `InferWithLogits`, `Close`, `GetEmbedding(s)`, `EmbeddingDim`
(internal/engine/engine.go:380, 1273-1296, 1809-1858) and
`SamplerConfig{Temperature, TopK, TopP, RepPenalty, Seed}` (internal/engine/types_base.go:7-15).
One sequence a call, as there; batches go through `generate`."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, List, Optional, Sequence, Tuple

import torch

from .engine.generate import EngineBackend, GenerationLoop
from .loading import load_engine
from .sampling import SamplingParams


@dataclass(frozen=True)
class SamplerConfig:
    """Zero values mean what they mean in the reference: temperature 0 is greedy
    (internal/engine/sampler.go:81-84), top_k <= 0 and top_p <= 0 or >= 1 are off (:309-339),
    rep_penalty acts above 1 (:77-79).  Only the seed differs: 0 is a seed like any other here,
    the reference takes the clock for it (:18-26).  `debug_activations` and `quality_mode` are the
    reference's remaining two fields (internal/engine/types_base.go:13-14): the first makes it log
    statistics of activations, which `Engine.step(observe=...)` and `trace_run --dump-activations` give
    as tensors here, the second is never read there; both are accepted and change nothing."""

    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 0.0
    rep_penalty: float = 0.0
    seed: int = 0
    debug_activations: bool = False
    quality_mode: bool = False

    def params(self) -> SamplingParams:
        return SamplingParams(temperature=self.temperature, top_k=max(0, self.top_k),
                              top_p=self.top_p if 0.0 < self.top_p < 1.0 else 1.0,
                              repetition_penalty=self.rep_penalty if self.rep_penalty > 1.0 else 1.0,
                              seed=self.seed)


class QuarrelEngine:
    def __init__(self, path: str, dtype: str = "bfloat16", kv_cache_size: int = 2048,
                 device: str = "cuda:0") -> None:
        """`kv_cache_size`: tokens the cache holds (the reference's `KVCacheSize`, engine.go:388); an
        explicit size is also the longest a sequence may get, whatever the configuration's context
        length says (internal/engine/kv_cache_sliding_window.go:38-60)."""
        self.engine = load_engine(path, dtype=dtype, max_tokens=kv_cache_size, max_slots=1, device=device,
                                  max_sequence_tokens=kv_cache_size)

    def _run(self, tokens: Sequence[int], n: int, cfg: Optional[SamplerConfig],
             callback: Optional[Callable[[int], None]], keep_logits: bool) -> Tuple[List[int], Optional[torch.Tensor]]:
        backend = EngineBackend(self.engine, (cfg or SamplerConfig()).params(), use_graphs=not keep_logits)
        backend.keep_logits = keep_logits
        try:
            cb = (lambda _request, token: callback(token)) if callback is not None else None
            out = GenerationLoop(backend, max_batch=1).run([list(tokens)], n, tuple(self.engine.model.spec.stop_ids),
                                                           False, cb)
            return out.tokens[0], backend.last_logits
        finally:
            backend.close()

    def infer(self, tokens: Sequence[int], n: int, sampler_config: Optional[SamplerConfig] = None) -> List[int]:
        """Up to n new ids after the prompt; the prompt is not returned (engine.go:1273-1276)."""
        return self._run(tokens, n, sampler_config, None, False)[0]

    def infer_with_callback(self, tokens: Sequence[int], n: int, sampler_config: Optional[SamplerConfig],
                            callback: Callable[[int], None]) -> List[int]:
        """`callback(id)` for every generated id as it is made (engine.go:1287-1296)."""
        return self._run(tokens, n, sampler_config, callback, False)[0]

    def infer_with_logits(self, tokens: Sequence[int], n: int,
                          sampler_config: Optional[SamplerConfig] = None) -> Tuple[List[int], torch.Tensor]:
        """The ids, and the float32 logits [vocab] that the last of them was drawn from, as the model
        gave them (before the repetition penalty) (engine.go:1278-1285)."""
        ids, logits = self._run(tokens, n, sampler_config, None, True)
        return ids, logits[0]

    def embedding_dim(self) -> int:
        """Width of the embedding vectors (engine.go:1852-1858)."""
        return int(self.engine.model.spec.width)

    def get_embeddings(self, tokens: Sequence[int]) -> torch.Tensor:
        """The rows of the embedding table for these ids, float32 [len(tokens), width], looked up by
        the kernel the model itself starts with (engine.go:1809-1836)."""
        e = self.engine
        vocab = int(e.model.spec.vocab_size)
        for i, t in enumerate(tokens):
            if not 0 <= int(t) < vocab:
                raise ValueError(f"token {t} (place {i}) out of vocab range [0, {vocab})")  # engine.go:1814-1816
        ids = torch.tensor([int(t) for t in tokens], dtype=torch.int32, device=e.device)
        out = torch.empty((len(tokens), self.embedding_dim()), dtype=torch.float32, device=e.device)
        if len(tokens):
            e.run_on_stream(lambda: e.kernels.embed(e.model.embedding.table, ids, out))
        return out

    def get_embedding(self, token: int) -> torch.Tensor:
        """One id's embedding vector, float32 [width] (engine.go:1809-1822)."""
        return self.get_embeddings([token])[0]

    def close(self) -> None:
        self.engine = None


def new_engine(path: str, **options) -> QuarrelEngine:
    return QuarrelEngine(path, **options)
