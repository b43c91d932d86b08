"""Backends of the kernel layer. `hip` is the hand-written gfx950 backend."""
