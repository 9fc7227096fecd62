"""lumen_amd: Lumen's batch-1 inference path on one MI355X (gfx950).

Host-side mirror of the reference's operator interface (Tensor, matmul,
Linear, RMSNorm, SiLU, Embedding, RotaryEmbedding, SelfAttention,
KVCacheInner, LlamaKVCache, LlamaModel) over the C ABI in
include/lumen_hip.h.  Importing a submodule that computes loads
lumen_amd/lib/liblumen_hip.so and raises if it is missing; nothing here
falls back to the CPU.
"""
__all__ = ["autograd", "ops", "layers", "kv_cache", "models", "synth"]
