"""Causal Wan2.2-TI2V-5B-shaped DiT on the NVFP4 kernels: block, model and streaming generator."""
from .model import CausalDiT, DiTBlock, DiTConfig
from .generator import StreamingGenerator

__all__ = ["CausalDiT", "DiTBlock", "DiTConfig", "StreamingGenerator"]
