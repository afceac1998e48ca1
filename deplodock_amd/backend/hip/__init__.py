"""HIP backend for gfx950: hipRTC compile cache, C-ABI launcher binding, program runtime."""
