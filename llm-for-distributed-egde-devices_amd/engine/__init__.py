from .kv_cache import KVCache, KVView
from .generate import Generator, GenerationResult, SamplingParams, needs_host_sampler
from .paged import PagedCache
from .ragged import RaggedEngine, RaggedGenerator, RaggedScheduler

__all__ = ["KVCache", "KVView", "Generator", "GenerationResult", "SamplingParams", "needs_host_sampler", "PagedCache",
           "RaggedEngine", "RaggedGenerator", "RaggedScheduler"]
