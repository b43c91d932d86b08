"""HIP backend of `fp8_linear` on gfx950: the GEMM paths of the form c = Q(a) B^T (forward:
a = x, B = W; fp8 input gradient: a = dy, B = W^T, the dgrad copy), one tile configuration per
problem picked by the tuner and bound once settled. Each path includes its activation
quantizer. Host-side counterpart of reference `backends/triton/fp8/linear.py` (candidates
:88-118, runner :162-196, `_select` :254-286, launchers :289-301, registration :309-320).

Recipes served on the GPU: `mx` (block-scaled MFMA; the activation quantizer writes the
MFMA-packed scales directly, the weight's packed copy comes in `aux` or is packed per call),
`tensor` (plain fp8 MFMA, scalar scales on the accumulator), `row` (the same GEMM with one
scale per output row and one per output column on the accumulator) and `block` (per K block of
128 the MFMA's partial sum is scaled by the row's and the 128 x 128 weight block's fp32 scales
and added to the running sum on the vector ALU). The 16-bit input gradient of a base stored
without a dgrad copy (`dy @ dequantize(W)`, the reference's `w16` path, `linear.py:152-153`) is one
kernel too: the codes are widened, scaled and rounded in registers on their way to the 16-bit
MFMA, for every scale layout; no 16-bit copy of the weight is ever written.
"""

import torch

from kohakumosstrainer_amd import native
from kohakumosstrainer_amd.kernels import registry, tuning
from kohakumosstrainer_amd.kernels.constraints import requires
from kohakumosstrainer_amd.kernels.hadamard import HALF
from kohakumosstrainer_amd.kernels.errors import BackendUnavailable
from kohakumosstrainer_amd.kernels.fp8.formats import packed_numel
from kohakumosstrainer_amd.kernels.fp8.op import OPS, register_launchers
from kohakumosstrainer_amd.kernels.tuning import pow2

GPU_RECIPES = ("mx", "tensor", "row", "block")
ALIGN_K = 128
_RESOLVED: dict[tuple, dict] = {}
tuning.on_reset(_RESOLVED.clear)


def candidates(recipe: str, m: int, n: int | None = None, k: int | None = None) -> list[dict]:
    """GEMM paths of `recipe` for M rows, the planner's first pick first: the library's tile
    configurations (large tiles for large M: fewest bytes fetched per flop; smaller ones when M is
    short or the grid would not fill 256 CUs) and, for `mx`, `row` and `block` at short M, the one-launch
    kernel that quantizes x inside the GEMM (reference `fused` candidates, `linear.py:97,102-104,113`)."""
    kernel = {"mx": native.KERNEL_GEMM_MX, "block": native.KERNEL_GEMM_BLOCKS}.get(recipe, native.KERNEL_GEMM_FP8)
    cfgs = [{"gemm": "hip", **c} for c in native.configs(kernel)]
    limit = max(pow2(m, 16), min(c["bm"] for c in cfgs))
    fits = [c for c in cfgs if c["bm"] <= limit] or cfgs
    ranked = sorted(fits, key=lambda c: -(c["bm"] * c["bn"]) if m >= 1024 else c["bm"])
    if recipe == "block":
        # measured at M16384 K3072 N9216: the 256 x 256 tile with two wavefronts per SIMD 0.42 ms, the
        # 128 x 128 tile (two workgroups per compute unit) 0.47 ms, the 256 x 128 tile 0.50 ms with eight
        # wavefronts and 0.54 ms with four. Short M and narrow N keep the small tile first.
        big = m >= 1024 and (n is None or n >= 512)
        ranked = sorted(fits, key=lambda c: (not (big and c["bn"] == 256), c["bm"], -c.get("waves", 4)))
    if recipe in ("mx", "row", "block") and m <= native.FUSED_MAX_M and (n is None or n % 32 == 0) and (k is None or k % 128 == 0):
        # measured at K3072 N9216, one launch against quantizer + GEMM. mx: 9.1 against 19 us at M = 1,
        # 11.0 against 21 at M = 16, 15.4 against 21 at M = 32 (even at 48); block: 10.6 against 21.4, 12.2
        # against 22.7, 19.2 against 23.0: first pick up to 16 rows, a timed candidate up to 32. row (a
        # second pass over x for the row maxima): 10.8 against 14.6 us at M = 1, even at M = 16: only
        # ever a timed candidate, up to 16 rows.
        fused = {"gemm": "fused", "id": -1, "bm": 16 * -(-max(m, 1) // 16), "bn": 64 if (n or 64) % 64 == 0 else 32}
        if recipe in ("mx", "block"):
            ranked.insert(0 if m <= 16 else len(ranked), fused)
        elif m <= 16:
            ranked.append(fused)
    return ranked


def _table_key(kind, m, n, k, a, recipe, bias) -> str:
    return f"{kind}_m{pow2(m, 16)}_n{n}_k{k}_{a.dtype}_{recipe}_{'x' if bias is None else 'b'}"


def _check_shapes(kind, a, bq, recipe):
    if recipe not in GPU_RECIPES:
        raise BackendUnavailable(f"fp8_{kind}", {"hip": f"recipe {recipe!r} is not built for gfx950 yet"}, persist=False)
    if a.shape[1] % ALIGN_K or bq.shape[1] != a.shape[1]:
        raise ValueError(f"fp8_{kind}: contraction length {a.shape[1]} (weight {tuple(bq.shape)}) must match and be a multiple of {ALIGN_K}")


def _run(cfg, recipe, a, bq, bs, baux, bias):
    """(a16 [M, K], bq [N, K], bs, baux, bias) -> Q(a) bq^T in a's dtype with tile config `cfg`."""
    if recipe == "mx":
        if baux is None or baux.numel() != packed_numel(bq.shape[0], bq.shape[1]) or baux.dtype != torch.uint8:
            baux = native.pack_scales(bs)
        if cfg["gemm"] == "fused":
            return native.gemm_mx_fused(a, bq, baux, bias)
        aq, _, a_packed = native.quant_mx(a, natural=False, packed=True)
        return native.gemm_mx(aq, a_packed, bq, baux, bias, a.dtype, cfg["id"], packed=True)
    if recipe == "block":
        if cfg["gemm"] == "fused":
            return native.gemm_fp8_blocks_fused(a, bq, bs.float(), bias)
        aq, _, sa_t = native.quant_blocks(a, "act", natural=False, kmajor=True)
        return native.gemm_fp8_blocks(aq, sa_t, bq, bs.float(), bias, a.dtype, cfg["id"], kmajor=True)
    if recipe == "row":
        if cfg["gemm"] == "fused":
            return native.gemm_fp8_rows_fused(a, bq, bs.float(), bias)
        aq, sa = native.quant_rows(a)
        return native.gemm_fp8_rows(aq, sa, bq, bs.float(), bias, a.dtype, cfg["id"])
    aq, sa = native.quant_tensor(a)
    return native.gemm_fp8_tensor(aq, sa, bq, bs.reshape(1).float(), bias, a.dtype, cfg["id"])


def _select(kind, a, bq, bs, baux, bias, recipe, in_backward):
    m, k = a.shape
    n = bq.shape[0]
    key = (kind, a.device.index, pow2(m, 16), n, k, a.dtype, recipe, bias is None)
    cfg = _RESOLVED.get(key)
    if cfg is not None:
        return cfg
    table_key = _table_key(kind, m, n, k, a, recipe, bias)
    cfg = tuning.select(
        f"fp8_{kind}",
        a.device,
        table_key,
        lambda: candidates(recipe, m, n, k),
        lambda c: lambda: _run(c, recipe, a, bq, bs, baux, bias),
        shortlist=8,
        in_backward=in_backward,
    )
    if tuning.decided(f"fp8_{kind}", a.device, table_key):
        _RESOLVED[key] = cfg
    return cfg


def fwd(x, q, scale, aux, bias, recipe):
    _check_shapes("fwd", x, q, recipe)
    cfg = _select("fwd", x, q, scale, aux, bias, recipe, False)
    return _run(cfg, recipe, x, q, scale, aux, bias)


def w16_candidates(m: int) -> list[dict]:
    """Tile configurations of the 16-bit input gradient, largest first for long M."""
    cfgs = native.configs(native.KERNEL_WO_DGRAD)
    fits = [c for c in cfgs if c["bm"] <= max(64, pow2(m, 32))] or cfgs
    return sorted(fits, key=lambda c: -(c["bm"] * c["bn"]) if m >= 1024 else c["bm"])


def _dgrad_16bit(dy, q, scale, recipe):
    """dx = dy @ round16(q * scale) over the stored codes `q [N, K]`; `scale` in `recipe`'s layout."""
    if recipe not in GPU_RECIPES:
        raise BackendUnavailable("fp8_dgrad", {"hip": f"recipe {recipe!r} is not built for gfx950 yet"}, persist=False)
    m, (n, k) = dy.shape[0], q.shape
    key = ("w16", dy.device.index, pow2(m, 32), n, k, dy.dtype, recipe)
    cfg = _RESOLVED.get(key)
    if cfg is None:
        table_key = f"w16_m{pow2(m, 32)}_n{n}_k{k}_{dy.dtype}_{recipe}"
        cfg = tuning.select(
            "fp8_dgrad_w16",
            dy.device,
            table_key,
            lambda: w16_candidates(m),
            lambda c: lambda: native.wo_gemm_dgrad(dy, q, scale, c["id"], recipe),
            shortlist=4,
            in_backward=True,
        )
        if tuning.decided("fp8_dgrad_w16", dy.device, table_key):
            _RESOLVED[key] = cfg
    return native.wo_gemm_dgrad(dy, q, scale, cfg["id"], recipe)


def dgrad(dy, q, scale, q_t, scale_t, aux_t, recipe):
    if q_t is None:
        return _dgrad_16bit(dy, q, scale, recipe)
    _check_shapes("dgrad", dy, q_t, recipe)
    cfg = _select("dgrad", dy, q_t, scale_t, aux_t, None, recipe, True)
    return _run(cfg, recipe, dy, q_t, scale_t, aux_t, None)


def _gpu_recipe(query):
    recipe = query.get("recipe", "row")
    return None if recipe in GPU_RECIPES else f"fp8 recipe {recipe!r} is not built for gfx950 (have {GPU_RECIPES})"


register_launchers("hip", fwd, dgrad)
for _op, _make in OPS.items():
    registry.register(_op, "hip", _make("hip"), supports=requires(kinds=("hip",), archs=("gfx950",), dtypes=HALF, extra=_gpu_recipe))
