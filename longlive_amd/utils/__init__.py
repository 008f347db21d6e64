"""LongLive-level host helpers of the NVFP4 path: quantized-Linear swap with module filter,
NVFP4 KV-cache interface, RoPE and adaLN entry points."""
