"""HIP backend of the weight-only `quant_linear` on gfx950: forward y = (x @ q^T) * scale + bias
with the int8 / e4m3 codes widened in registers ahead of the 16-bit MFMA, and the input
gradient dx = dy @ round16(q * scale). Host-side counterpart of reference
`backends/triton/quant.py` (candidates :144-149, launchers :213-263, registration :270-276).
"""

from kohakumosstrainer_amd import native
from kohakumosstrainer_amd.kernels import registry, tuning
from kohakumosstrainer_amd.kernels.constraints import requires
from kohakumosstrainer_amd.kernels.hadamard import HALF
from kohakumosstrainer_amd.kernels.hadamard import rotate_2d
from kohakumosstrainer_amd.kernels.quant import fmt_supported, make_quant_linear, register_launchers
from kohakumosstrainer_amd.kernels.rotated import compose, group_supported, make_quant_linear_rotated, register_rotated_launchers
from kohakumosstrainer_amd.kernels.tuning import pow2

_RESOLVED: dict[tuple, dict] = {}
tuning.on_reset(_RESOLVED.clear)


def candidates(m: int) -> list[dict]:
    cfgs = native.configs(native.KERNEL_WO_FWD)
    fits = [c for c in cfgs if c["bm"] <= max(64, pow2(m, 32))] or cfgs
    return sorted(fits, key=lambda c: -(c["bm"] * c["bn"]) if m >= 1024 else c["bm"])


def _key(m, n, k, x, q, bias) -> str:
    return f"m{pow2(m, 32)}_n{n}_k{k}_{x.dtype}_{q.dtype}_b{bias is not None}"


def _pick(kernel, which, m, n, k, x, q, bias, launch, in_backward):
    key = (which, x.device.index, pow2(m, 32), n, k, x.dtype, q.dtype, bias is None)
    cfg = _RESOLVED.get(key)
    if cfg is None:
        table_key = _key(m, n, k, x, q, bias)
        cfg = tuning.select(kernel, x.device, table_key, lambda: candidates(m), launch, shortlist=8, in_backward=in_backward)
        if tuning.decided(kernel, x.device, table_key):
            _RESOLVED[key] = cfg
    return cfg


def fwd(x, q, scale, bias):
    m, (n, k) = x.shape[0], q.shape
    cfg = _pick("quant_fwd", "fwd", m, n, k, x, q, bias, lambda c: lambda: native.wo_gemm_fwd(x, q, scale, bias, c["id"]), False)
    return native.wo_gemm_fwd(x, q, scale, bias, cfg["id"])


def dgrad(g, q, scale):
    m, (n, k) = g.shape[0], q.shape
    cfg = _pick("quant_dgrad", "dgrad", m, n, k, g, q, None, lambda c: lambda: native.wo_gemm_dgrad(g, q, scale, c["id"]), True)
    return native.wo_gemm_dgrad(g, q, scale, cfg["id"])


def _format_supported(query):
    return fmt_supported(query.get("fmt", "int8"), query.arch)


register_launchers("hip", fwd, dgrad)
registry.register("quant_linear", "hip", make_quant_linear("hip"), supports=requires(kinds=("hip",), archs=("gfx950",), dtypes=HALF, extra=_format_supported))


def _rotated_supported(query):
    return _format_supported(query) or group_supported(query)


# the rotated base: one pass of the HIP butterfly kernel around the plain launchers (reference
# backends/triton/quant_rotated.py registers its fused and separate-pass pairs the same way)
register_rotated_launchers("hip", *compose(fwd, dgrad, rotate_2d))
registry.register("quant_linear_rotated", "hip", make_quant_linear_rotated("hip"), supports=requires(kinds=("hip",), archs=("gfx950",), dtypes=HALF, extra=_rotated_supported))
