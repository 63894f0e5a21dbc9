"""Engine options: the names, meanings and defaults of the reference's command line
(bins/dinfer/src/main.rs:30-131) and of its SchedulerConfig / CacheConfig
(crates/core/src/config.rs:25-92), as far as they concern one GPU.
"""
from __future__ import annotations

from dataclasses import dataclass


@dataclass
class EngineOptions:
    dtype: str = "bfloat16"             # "bfloat16" or "float32"
    max_model_len: int = 4096           # prompt + output per request; width of the block table
    max_num_seqs: int = 16              # live requests; also the most logits rows of a serving step
    max_num_batched_tokens: int = 2048  # per-step token budget
    num_blocks: int | None = None       # cache pages per group; None: sized from free memory
    block_size: int = 16                # tokens per page
    gpu_memory_utilization: float = 0.9
    decode_exempt_from_budget: bool = True   # a decode row does not consume the token budget
    long_prefill_token_threshold: int = 0    # per-request cap on a prompt portion (0: none)
    prefill_tokens_per_step: int = 0         # cap on all prompt tokens of a step (0: none)
    enable_chunked_prefill: bool = True
    # a prompt portion that does not end its request ends at a multiple of this many tokens (1: anywhere). The engine
    # raises it to what the model's layers ask for (a layer that works in chunks of its own), never lowers it
    prefill_chunk_alignment: int = 1
    # pages keep the tokens they hold and a later request with the same start reuses them; None: on where every
    # layer keeps all its keys (a window layer gives pages back while the request lives), as --no-prefix-caching
    # of the reference implies (bins/dinfer/src/main.rs:30-131: the cache is on unless switched off)
    enable_prefix_caching: bool | None = None
    hip_graph: bool = True              # replay decode steps from captured HIP graphs
    # while a step of single decode rows runs, the next one is planned and launched already (its input tokens stay on
    # the device), and only then the running step's tokens are read: the host's work between two steps is hidden
    # (the reference's engine does so by default too: crates/core/src/engine.rs:153-154,209)
    async_scheduling: bool = True
    # "measured": the engine's warm-up times the library's candidates once per shape, keeps the choices in
    # gemm_plan_file and later processes reuse them; "heuristic": the library's first suggestion, nothing timed
    gemm_tuning: str = "measured"
    gemm_plan_file: str | None = None   # None: beside the built libraries; "": choices are not kept between processes
    device: int = 0
    max_logits_rows: int | None = None  # None: max_num_seqs; replay and tests ask for more

    def check(self) -> None:
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {self.dtype!r}")
        for name in ("max_model_len", "max_num_seqs", "max_num_batched_tokens", "block_size", "prefill_chunk_alignment"):
            if getattr(self, name) <= 0:
                raise ValueError(f"{name} must be positive, got {getattr(self, name)}")
        if self.gemm_tuning not in ("measured", "heuristic"):
            raise ValueError(f"gemm_tuning must be 'measured' or 'heuristic', got {self.gemm_tuning!r}")
        if self.num_blocks is not None and self.num_blocks <= 0:
            raise ValueError(f"num_blocks must be positive, got {self.num_blocks}")
        if not (0.0 < self.gpu_memory_utilization <= 1.0):
            raise ValueError(f"gpu_memory_utilization must be in (0, 1], got {self.gpu_memory_utilization}")
