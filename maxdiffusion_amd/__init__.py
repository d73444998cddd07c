"""MI355X-native DiT attention hot path: fused q/k RMSNorm + RoPE, flash-attention forward with
LSE, chunk merge -- hand-written HIP for gfx950 behind a C ABI (include/mdattn.h)."""

__version__ = "0.1.0"
