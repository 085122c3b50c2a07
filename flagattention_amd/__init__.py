"""flag_attn operators on hand-written gfx950 (MI355X) HIP kernels."""
