"""MI355X (gfx950) mode of llama2j's per-token forward pass.

The product is `libllama2j_hip.so` (C ABI in include/llama2j_hip.h).  This package is the thin
host-side mirror of the reference's Java entry points over that ABI via ctypes: `Config`, `Quant`,
`Transformer` (weights + run state + forward), `Sampler`.  It never falls back to a CPU path.
"""
from .binding import (Config, Quant, Sampler, Tokenizer, Transformer, L2JError, lib, lib_path, build_library,  # noqa: F401
                      TENSOR, BUFFER, KERNEL, F_EXACT_SILU)
