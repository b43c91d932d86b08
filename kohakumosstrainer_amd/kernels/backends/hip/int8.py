"""HIP backend of `int8_linear` on gfx950: per-row int8 activation quantizer, int8 GEMM on the
int32 MFMA with both scales and the bias applied to the accumulator in the eager path's order of
roundings (outputs equal the eager reference bit for bit), and the two input-gradient modes.
Host-side counterpart of reference `backends/triton/int8.py` (launchers :234-270, registration
:273-281). A rotated base (`group` > 0) has its activations rotated inside the quantizer kernel
(rows of up to 4096 elements; longer rows get a pass of the butterfly kernel first) and one pass of
the butterfly kernel over dx. The int8 input gradient contracts over N, so it reads a `[K, N]` copy
of the codes; the reference makes its column-major copy per call (`int8/formats.py:55-58`), here it
is made once per frozen code tensor and kept for as long as that tensor lives.
"""

import weakref

from kohakumosstrainer_amd import native
from kohakumosstrainer_amd.kernels import registry, tuning
from kohakumosstrainer_amd.kernels.backends.hip import quant as wo
from kohakumosstrainer_amd.kernels.constraints import requires
from kohakumosstrainer_amd.kernels.hadamard import HALF
from kohakumosstrainer_amd.kernels.hadamard import rotate_2d
from kohakumosstrainer_amd.kernels.int8.op import int8_supported, make_int8_linear, register_launchers
from kohakumosstrainer_amd.kernels.tuning import pow2

ALIGN_K = 128
_RESOLVED: dict[tuple, dict] = {}
tuning.on_reset(_RESOLVED.clear)


def candidates(m: int) -> list[dict]:
    cfgs = [{"gemm": "hip", **c} for c in native.configs(native.KERNEL_GEMM_FP8)]
    limit = max(pow2(m, 16), min(c["bm"] for c in cfgs))
    fits = [c for c in cfgs if c["bm"] <= limit] or cfgs
    return sorted(fits, key=lambda c: -(c["bm"] * c["bn"]) if m >= 1024 else c["bm"])


def _check(kind, contraction):
    if contraction % ALIGN_K:
        raise ValueError(f"int8_{kind}: contraction length {contraction} must be a multiple of {ALIGN_K}")


def _pick(kernel, kind, m, n, k, a, bias, launch, in_backward):
    key = (kind, a.device.index, pow2(m, 32), n, k, a.dtype, bias is None)
    cfg = _RESOLVED.get(key)
    if cfg is None:
        table_key = f"m{pow2(m, 32)}_n{n}_k{k}_{a.dtype}_b{bias is not None}"
        cfg = tuning.select(kernel, a.device, table_key, lambda: candidates(m), launch, shortlist=8, in_backward=in_backward)
        if tuning.decided(kernel, a.device, table_key):
            _RESOLVED[key] = cfg
    return cfg


# `[K, N]` copies of frozen `[N, K]` code tensors, by the identity of the tensor object. An entry goes
# when its tensor is collected and is remade when the tensor has been written to since.
_TRANSPOSED: dict[int, tuple] = {}


def transposed_codes(q):
    key = id(q)
    hit = _TRANSPOSED.get(key)
    if hit is not None and hit[0]() is q and hit[1] == q._version:
        return hit[2]
    q_t = q.t().contiguous()
    _TRANSPOSED[key] = (weakref.ref(q, lambda _ref, key=key: _TRANSPOSED.pop(key, None)), q._version, q_t)
    return q_t


def fwd(x, q, scale, bias, group):
    m, k = x.shape
    n = q.shape[0]
    _check("fwd", k)
    q, scale = q.contiguous(), scale.float().contiguous()
    xq, xs = native.quant_rows_i8_rotated(x, group) if group else native.quant_rows_i8(x)
    cfg = _pick("int8_fwd", "fwd", m, n, k, x, bias, lambda c: lambda: native.gemm_i8_rows(xq, xs, q, scale, bias, x.dtype, c["id"]), False)
    return native.gemm_i8_rows(xq, xs, q, scale, bias, x.dtype, cfg["id"])


def dgrad(dy, q, scale, group, mode):
    m, n = dy.shape
    k = q.shape[1]
    if mode == "16bit":
        dx = wo.dgrad(dy, q.contiguous(), scale)  # the weight-only kernel over the stored codes, its tuned tile
        return rotate_2d(dx, group) if group else dx
    _check("dgrad", n)
    gq, gs = native.quant_rows_i8(dy, scale)
    q_t = transposed_codes(q)
    cfg = _pick("int8_dgrad", "dgrad", m, k, n, dy, None, lambda c: lambda: native.gemm_i8_rows(gq, gs, q_t, None, None, dy.dtype, c["id"]), True)
    dx = native.gemm_i8_rows(gq, gs, q_t, None, None, dy.dtype, cfg["id"])
    return rotate_2d(dx, group) if group else dx


register_launchers("hip", fwd, dgrad)
registry.register("int8_linear", "hip", make_int8_linear("hip"), supports=requires(kinds=("hip",), archs=("gfx950",), dtypes=HALF, extra=int8_supported))
