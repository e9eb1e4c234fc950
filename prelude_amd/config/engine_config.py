"""Runtime settings of the engine, apart from the model's own config.json.

Names and defaults follow the reference where it has them
(crates/prelude-core/src/config.rs:33-51, crates/prelude-core/src/scheduler/state.rs:224-243,
crates/prelude-server/src/main.rs:15-183); the page size default is the
benchmark's 16 (the reference's scheduler default, state.rs:240).
"""
from __future__ import annotations

import dataclasses
from typing import Optional


@dataclasses.dataclass
class EngineConfig:
    dtype: str = "bfloat16"                 # "bfloat16" | "float32"
    device: str = "cuda:0"
    page_size: int = 16                     # tokens per cache page
    max_cache_tokens: Optional[int] = None  # tokens the page pool holds; None = from free memory
    gpu_memory_utilization: float = 0.9
    max_state_slots: int = 256              # slots for per-request state (used by stateful mixers only)
    # scheduler
    max_num_batched_tokens: int = 8192
    long_prefill_token_threshold: int = 0
    max_running_requests: int = 256
    max_total_tokens: int = 0
    decode_reservation_cap: int = 0         # 0 = max_position_embeddings
    decode_priority_max_remaining_tokens: int = 4
    # decode steps replayed from HIP graphs
    hip_graph: bool = True
    hip_graph_max_bs: int = 64
    hip_graph_cache_size: int = 32          # captured graphs kept (one per batch size and table width); the least recently used goes
    # steps that bring prompt portions are replayed from a graph too when they are small (at most this many tokens:
    # there the host's launches take longer than the kernels) and their shape has been met before; 0: never
    hip_graph_portion_tokens: int = 1024
    # a second copy of every bfloat16 weight matrix, in the tiles the few-row product streams fastest
    # (decode steps run about a tenth faster for twice the weight memory)
    weight_tiles: bool = True
    # launch a step before the previous step's token ids have reached the host (they are handed on
    # on the device); a request that ends on a token value then runs one step too many, which is dropped
    overlap_steps: bool = True

    def torch_dtype(self):
        import torch
        try:
            return {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32,
                    "f32": torch.float32, "fp32": torch.float32}[self.dtype]
        except KeyError:
            raise ValueError(f"dtype {self.dtype!r} is not one of bfloat16, float32") from None
