"""The `hip` backend: hand-written HIP kernels for gfx950 behind the C ABI
(`kohakumosstrainer_amd.native`). Importing it registers its launchers and ops; it raises when
the kernel library is not built, and the registry then marks the backend unavailable with that
reason (a GPU op on gfx950 has no other backend to go to, so `resolve` reports it)."""

from kohakumosstrainer_amd import native

_why = native.available()
if _why is not None:
    raise RuntimeError(_why)

from kohakumosstrainer_amd.kernels.backends.hip import fp8_linear, int8, quant  # noqa: E402,F401
