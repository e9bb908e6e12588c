"""slai_amd -- MI355X-native implementation of slai's per-token decode path.

``runtime`` wraps the C ABI of ``lib/libslai_hip.so`` (HIP kernels for gfx950 + the host
mirror of slai's operator API); ``gguf_writer`` / ``synth`` build synthetic model files.
"""
__all__ = ["build", "runtime", "gguf_writer", "synth"]
