"""Engine-level settings: everything that is not a property of the model.

The reference scatters these over constructor arguments (`pyre/scheduler.py:28`)
and a module constant for the page size (`pyre/paged_cache.py:37`).
"""

from __future__ import annotations

from dataclasses import dataclass

DTYPE_NAMES = {
    "bfloat16": "bfloat16", "bf16": "bfloat16",
    "float32": "float32", "fp32": "float32", "f32": "float32",
}


@dataclass
class EngineConfig:
    dtype: str = "bfloat16"          #: "bfloat16" or "float32" (true 32-bit everywhere)
    device: str = "cuda:0"
    page_size: int = 16              #: tokens per cache page
    num_pages: int | None = None     #: pages per cache group; None: from max_cached_tokens
    max_cached_tokens: int | None = None  #: tokens the page pool holds; None: from free memory
    memory_fraction: float = 0.85    #: of free device memory, when neither of the above is set
    max_num_seqs: int = 64           #: requests live at a time (slots)
    max_num_batched_tokens: int = 2048  #: tokens in one step
    prefill_chunk: int = 512         #: largest portion of one prompt in a step
    max_model_len: int | None = None  #: longest request; None: the model's max positions
    use_graphs: bool = True          #: capture decode-only steps in HIP graphs
    #: row counts (tokens in a step) for which the BLAS library is asked, once at start-up,
    #: to time its kernels for this model's many-row 16-bit products and keep the fastest
    tune_gemm_rows: tuple = ()
    #: debugging aid: fill every cache page and state slot with NaN when it goes back to its
    #: pool (and all of them at the start), so that a read of freed memory shows in the logits
    debug_poison: bool = False

    def __post_init__(self) -> None:
        if self.dtype not in DTYPE_NAMES:
            raise ValueError(f"dtype must be one of {sorted(set(DTYPE_NAMES))}, got {self.dtype!r}")
        self.dtype = DTYPE_NAMES[self.dtype]
        for name in ("page_size", "max_num_seqs", "max_num_batched_tokens", "prefill_chunk"):
            if getattr(self, name) <= 0:
                raise ValueError(f"{name} must be positive")
