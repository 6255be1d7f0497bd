"""MI355X-native LLaMA3 token loop: hand-written gfx950 kernels behind a C-ABI
(csrc/, include/llmcu_hip.h) and a C++ host layer that mirrors the reference's
own structure (src/safetensor, src/llama3, src/inference, src/main.cpp).

The directory name carries a dot, so import it through
`__graft_entry__.load_package()` (registers it as module `llm_cu_amd`).
"""
from . import capi, engine, ops  # noqa: F401
from .capi import LIB_PATH, LlmError, ModelConfig, device_count, init, lib  # noqa: F401
