"""MI355X (gfx950) attention path for llm_simple.

The product is ``libllmhip.so`` (hand-written HIP kernels behind the C ABI of
``include/llmhip.h``) plus the C++ device layer in ``csrc/``.  This package is
the thin Python binding used by the tests and the benchmark: it loads the
shared library with ctypes and mirrors the reference's operator names
(prebuild/npu_ops.h) as ``hip_*_layer`` functions.  There is no CPU fallback:
importing :mod:`llm_simple_amd.ops` raises when the library is missing.
"""
from . import ops  # noqa: F401
from .ops import (  # noqa: F401
    DT_BFLOAT16,
    DT_FLOAT16,
    LlmHipError,
    hip_flash_attn_gqa_layer,
    hip_flash_attn_layer,
    hip_flash_attn_opt_prefill_layer,
    hip_flash_decode_gqa_layer,
    hip_rope_kv_append_layer,
    hip_rope_layer,
    hip_rope_single_layer,
    init_freq_cis,
    lib,
)
