"""Lowering passes: fuse (kernel boundaries) → schedule (knobs) → lower (HIP source)."""
