"""Engine options.  Names, meanings and defaults follow the reference's
``Config`` (src/config.hpp:17-30) and the keys its engine accepts
(src/engine/llm_engine.cpp:11-16); unlike there, every field is enforced."""
from __future__ import annotations

import dataclasses
from typing import Optional


@dataclasses.dataclass
class EngineConfig:
    model: str = ""
    #: "bfloat16" (serving kernels) or "float32" (everything in true 32-bit)
    dtype: str = "bfloat16"
    #: most tokens in one step, prompt portions and decoded tokens together (config.hpp:19)
    max_num_batched_tokens: int = 16384
    #: most tokens of ONE request in one step: longer prompts are cut into portions of this size, so that the requests
    #: decoding beside them get a token every step (the reference runs every prompt whole, scheduler.cpp:59-71)
    prefill_chunk: int = 2048
    #: most requests running at once (config.hpp:20)
    max_num_seqs: int = 512
    #: most tokens of one request, clamped to max_position_embeddings (config.hpp:12, 21)
    max_model_len: int = 4096
    #: share of the free device memory that the cache pool may take when
    #: num_kvcache_blocks is not given (config.hpp:22)
    gpu_memory_utilization: float = 0.9
    #: True: launch every step kernel by kernel; False: replay decode steps from HIP graphs (config.hpp:24)
    enforce_eager: bool = False
    #: tokens in a cache page (config.hpp:26; the reference's default is 4).  Values lie transposed inside a page, and the
    #: decode attention reads 32 keys at a time: whole memory lines with pages of 8 to 32 tokens, half lines with larger
    #: ones (64 requests of 8337 keys: 397 us a layer with pages of 64 or 128 against 355 with pages of 16).  A size that
    #: is no multiple of 8 (the reference's 4) is taken too, by the plain attention kernel, which is built for checking
    kvcache_block_size: int = 16
    #: pages in the pool of every cache group; None = from free memory (config.hpp:27)
    num_kvcache_blocks: Optional[int] = None
    #: base seed of temperature sampling
    seed: int = 0
    #: True: a finished request keeps its pages and slot for a further turn (append_to_request), as the reference's do
    #: until they are removed (llm_engine.cpp:40-73); they are the first to go when pages or slots are short
    keep_finished_cache: bool = False
    #: "both": every bfloat16 matrix is held as rows (for the library's products of many rows) and in tiles (for the
    #: products of few rows).  "tiled": in tiles only, which halves the weights' memory; a step of more than 64 rows
    #: then restores each matrix's rows into a scratch tensor ahead of its product (a prompt portion of 2048 tokens
    #: takes about a sixth longer).  Matrices without a tiled form (float32, odd shapes) keep their rows either way.
    weight_copies: str = "both"

    def validate(self) -> None:
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError("dtype must be 'bfloat16' or 'float32', got %r" % (self.dtype,))
        for name in ("max_num_batched_tokens", "prefill_chunk", "max_num_seqs", "max_model_len", "kvcache_block_size"):
            if getattr(self, name) <= 0:
                raise ValueError("%s must be positive" % name)
        if self.num_kvcache_blocks is not None and self.num_kvcache_blocks <= 0:
            raise ValueError("num_kvcache_blocks must be positive")
        if self.weight_copies not in ("both", "tiled"):
            raise ValueError("weight_copies must be 'both' or 'tiled', got %r" % (self.weight_copies,))
        if not (0.0 < self.gpu_memory_utilization <= 1.0):
            raise ValueError("gpu_memory_utilization must be in (0, 1]")
