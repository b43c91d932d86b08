"""Kernel layer: per-op dispatch (`registry`), the shape tuning table (`tuning`), the op
modules (`fp8`, `quant`) and the backends that implement them (`backends.hip`: hand-written
HIP for gfx950 behind the C ABI; the torch-eager reference launchers live in the op modules).
Mirrors the layering of reference `src/kohakumoss_kernels`."""
