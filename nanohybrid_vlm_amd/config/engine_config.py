"""Engine options: names and meanings follow the reference's ``Config``
(nanovllm/config.py:11-75), minus what belongs to other architectures or to
several GPUs. Values are checked in the manner of nanovllm/config.py:156-273:
each bad value raises ``ValueError`` and names the field.
"""
from __future__ import annotations

from dataclasses import dataclass, fields

_DTYPES = {
    "bfloat16": "bfloat16", "bf16": "bfloat16",
    "float32": "float32", "fp32": "float32",
}


@dataclass
class EngineConfig:
    model: str                                  # folder with config.json and model.safetensors
    max_num_batched_tokens: int = 16384         # tokens in one step (decode tokens and prompt portions together)
    max_prefill_wait_ms: float = 50.0           # a waiting prompt older than this gets room reserved
    scheduler_policy: str = "decode_first"      # or "prefill_first"
    max_num_seqs: int = 512                     # live requests
    max_model_len: int = 4096                   # capped by max_position_embeddings
    gpu_memory_utilization: float = 0.9
    enforce_eager: bool = False                 # True: no HIP graphs for decode
    max_graph_batch: int = 256                  # decode steps of up to this many requests replay a graph
    max_graph_tokens: int = 256                 # so do other steps (prompt portions, alone or beside decoded tokens) of up to this many tokens; 0: none
    warm_up: bool = False                       # True: every size of step that replays a graph is met once when the engine starts
    run_ahead: bool = True                      # a decode step that is bound to follow is issued before the host knows the tokens it feeds
    eos: int = -1                               # filled from config.json when -1
    kvcache_block_size: int = 256               # tokens in a page (any positive number)
    num_kvcache_blocks: int = -1                # -1: sized from free memory
    num_state_slots: int = -1                   # -1: max_num_seqs
    enable_prefix_cache: bool = False           # requests with a common start share its full pages
    # bfloat16 matrix products are done the fastest way measured (own kernel or one of the library's algorithms), timed
    # once per shape and process; which way wins can differ from start to start, and with it the last bits of the logits.
    measure_gemms: bool = True                  # False: nothing is timed; shapes follow gemm_choices, else the fixed rule
    gemm_choices: str | None = None             # a JSON file of choices: read if it exists (and then nothing is timed), see LLM.save_gemm_choices
    fuse_norms: bool = True                     # bfloat16 products of up to 16 rows make the residual addition after them and the norm before them in their own kernels
    dtype: str = "bfloat16"                     # "bfloat16" or "float32" (true 32-bit everywhere)
    # the residual stream between layers in a bfloat16 run: "float32" keeps the unrounded sum; "model" rounds it to
    # bfloat16 after every addition, as the reference does (and reads and writes a third fewer bytes in every norm)
    residual_dtype: str = "float32"
    seed: int = 0                               # default seed of temperature sampling
    device: str = "cuda:0"                      # the one GPU

    def __post_init__(self):
        if self.dtype not in _DTYPES:
            raise ValueError(f"dtype must be one of {sorted(_DTYPES)}, got {self.dtype!r}")
        self.dtype = _DTYPES[self.dtype]
        if self.residual_dtype not in ("float32", "model"):
            raise ValueError("residual_dtype must be 'float32' or 'model'")
        if self.scheduler_policy not in ("decode_first", "prefill_first"):
            raise ValueError("scheduler_policy must be 'decode_first' or 'prefill_first'")
        if self.max_prefill_wait_ms < 0:
            raise ValueError("max_prefill_wait_ms must be non-negative")
        if self.max_num_batched_tokens <= 0:
            raise ValueError("max_num_batched_tokens must be positive")
        if self.max_num_seqs <= 0:
            raise ValueError("max_num_seqs must be positive")
        if self.max_model_len <= 0:
            raise ValueError("max_model_len must be positive")
        if not (0 < self.gpu_memory_utilization <= 1):
            raise ValueError("gpu_memory_utilization must be in (0, 1]")
        if self.kvcache_block_size <= 0:
            raise ValueError("kvcache_block_size must be positive")
        if self.num_kvcache_blocks != -1 and self.num_kvcache_blocks <= 0:
            raise ValueError("num_kvcache_blocks must be -1 or positive")
        if self.num_state_slots != -1 and self.num_state_slots <= 0:
            raise ValueError("num_state_slots must be -1 or positive")
        if self.max_graph_batch <= 0:
            raise ValueError("max_graph_batch must be positive")
        if self.max_graph_tokens < 0:
            raise ValueError("max_graph_tokens must not be negative")

    @classmethod
    def field_names(cls) -> set[str]:
        return {f.name for f in fields(cls)}
