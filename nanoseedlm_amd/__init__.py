"""MI355X-native SeedLM decode-in-matmul backend (hand-written HIP for gfx950 behind the reference's kc_* C entry points)."""
__all__ = ["packs"]
