"""Configuration of the engine around a model: precision, cache geometry, step budget.

The reference's counterparts: ``CacheConfig{block_size, num_gpu_blocks}``
(include/block_manager.h:8-12), ``AsyncEngine(model_path, max_blocks=0, block_size=16)``
(include/async_engine.h:24-25), the cache sized to 90 % of free memory less 500 MiB
(src/qwen.cc:527-543) and ``MAX_TOKENS_PER_STEP = 512 + 64`` (src/scheduler.cc:48).
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

_DTYPES = {
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"engine dtype must be bfloat16 or float32, got {name}")
        return name
    try:
        return _DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"engine dtype must be bfloat16 or float32, got '{name}'") from None


@dataclass
class EngineConfig:
    dtype: torch.dtype = torch.bfloat16
    block_size: int = 16            # tokens in a page
    max_blocks: int = 0             # pages in each pool; 0: size from free memory
    memory_fraction: float = 0.90   # of free device memory, when max_blocks == 0
    memory_reserve: int = 500 << 20
    # tokens a step may run: decode tokens and portions of prompts together.  The reference cuts
    # prompts at 576 (src/scheduler.cc:48); 256 CUs want more rows to a product (an 8B-shaped
    # 2,048-token prompt runs at 68 k tokens a second whole and at 46 k in portions of 576)
    max_tokens_per_step: int = 2048
    max_seqs: int = 256             # live requests (also the number of state slots)
    device: str = "cuda:0"
    use_graphs: bool = True         # replay decode steps from HIP graphs (bfloat16 on the GPU)
    graph_max_batch: int = 256      # largest decode batch that is captured
    graph_cache_size: int = 32      # captured steps kept (one per number of rows, table width and planners' hint)
    run_ahead: bool = True          # queue a step before the host has the tokens of the one before
    time_steps: bool = False        # bracket every step with two events: LLMEngine.stats() gives its GPU time

    def __post_init__(self) -> None:
        self.dtype = parse_dtype(self.dtype)
        if self.block_size <= 0:
            raise ValueError("block_size must be positive")
        if self.max_tokens_per_step <= 0:
            raise ValueError("max_tokens_per_step must be positive")
        if self.max_seqs <= 0:
            raise ValueError("max_seqs must be positive")
