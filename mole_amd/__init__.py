"""MI355X-native implementation of MOLE's single-GPU MoE-layer hot path (HIP for gfx950 behind a C ABI)."""
__version__ = "0.1.0"
