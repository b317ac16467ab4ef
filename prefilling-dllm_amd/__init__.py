"""MI355X-native hot path of Prefilling-dLLM: hand-written HIP kernels (gfx950) behind a C ABI
(libpdllm_hip.so, include/pdllm.h) and a thin Python operator layer mirroring the reference
engine's operator interface.  Importing `ops` loads the shared library and fails loudly when it
has not been built -- there is no CPU fallback in the product path."""

__all__ = ["ops", "engine_ops", "context", "attention"]
