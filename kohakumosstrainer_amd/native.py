"""ctypes binding of libkm_kernels.so (hand-written HIP for gfx950) and thin tensor-level
wrappers. torch is used for device memory and the current stream only.

Every wrapper validates shapes / dtypes / devices on the host before a launch, allocates
its outputs, launches on torch's current stream of the operand's device and never
synchronizes. A missing or unloadable library raises `KernelLibraryMissing` (a
RuntimeError): there is no CPU or torch fallback behind these functions.
"""

import ctypes
import threading
from pathlib import Path

import torch
from torch import Tensor

LIB_PATH = Path(__file__).resolve().parent / "_lib" / "libkm_kernels.so"
E4M3 = torch.float8_e4m3fn
KM_BF16, KM_F16 = 0, 1
QUANT_TENSOR_WORKSPACE_BYTES = 2048  # KM_QUANT_TENSOR_WORKSPACE_BYTES of include/km_kernels.h
KM_OK, KM_ERR_ARG, KM_ERR_LAUNCH, KM_ERR_UNSUPPORTED = 0, -1, -2, -3  # return codes of every entry point
KM_Q_INT8, KM_Q_E4M3 = 0, 1
KERNEL_GEMM_MX, KERNEL_GEMM_FP8, KERNEL_WO_FWD, KERNEL_WO_DGRAD, KERNEL_GEMM_BLOCKS = 0, 1, 2, 3, 4
ROLE_ACT, ROLE_WEIGHT = 0, 1
BLOCK = 128
SCALES_ROWMAJOR, SCALES_PACKED, SCALES_KMAJOR = 0, 1, 2
_DTYPES = {torch.bfloat16: KM_BF16, torch.float16: KM_F16}
_QFORMATS = {torch.int8: KM_Q_INT8, E4M3: KM_Q_E4M3}

EXPORTS = (
    "km_abi_version",
    "km_last_error",
    "km_quant_mx",
    "km_scales_packed_bytes",
    "km_scales_pack",
    "km_quant_tensor",
    "km_quant_rows",
    "km_quant_blocks",
    "km_quant_rows_i8",
    "km_quant_rows_i8_rotated",
    "km_gemm_mx",
    "km_gemm_mx_fused",
    "km_gemm_fp8_rows_fused",
    "km_gemm_fp8_blocks_fused",
    "km_gemm_fp8_tensor",
    "km_gemm_fp8_rows",
    "km_gemm_fp8_blocks",
    "km_gemm_i8_rows",
    "km_wo_gemm_fwd",
    "km_wo_gemm_dgrad",
    "km_wo_gemm_dgrad_w16",
    "km_wo_gemm_dgrad_static",
    "km_wo_gemm_path",
    "km_group_hadamard",
    "km_probe_mfma_ceiling",
    "km_num_configs",
    "km_config_desc",
)

_lock = threading.Lock()
_lib: ctypes.CDLL | None = None


class KernelLibraryMissing(RuntimeError):
    """libkm_kernels.so is not built or cannot be loaded."""


class KernelError(RuntimeError):
    """A kernel entry point returned an error code (bad arguments or a failed launch)."""


def _declare(lib: ctypes.CDLL) -> None:
    c = ctypes
    p, i64, i32 = c.c_void_p, c.c_int64, c.c_int
    lib.km_abi_version.restype = i32
    lib.km_last_error.restype = c.c_char_p
    lib.km_quant_mx.argtypes = [p, i64, i64, i64, i64, i32, p, p, p, p]
    lib.km_scales_packed_bytes.argtypes = [i64, i64]
    lib.km_scales_pack.argtypes = [p, i64, i64, p, p]
    lib.km_quant_tensor.argtypes = [p, i64, i64, i64, i64, i32, p, p, p, p]
    lib.km_quant_rows.argtypes = [p, i64, i64, i64, i64, i32, p, p, p]
    lib.km_quant_blocks.argtypes = [p, i64, i64, i64, i64, i32, i32, p, p, p, p]
    lib.km_quant_rows_i8.argtypes = [p, i64, i64, i64, i64, i32, p, p, p, p]
    lib.km_quant_rows_i8_rotated.argtypes = [p, i64, i64, i64, i32, i32, p, p, p]
    lib.km_gemm_mx.argtypes = [p, p, p, p, p, p, i64, i64, i64, i32, i32, i32, p]
    lib.km_gemm_mx_fused.argtypes = [p, i64, p, p, p, p, i64, i64, i64, i32, p]
    lib.km_gemm_fp8_rows_fused.argtypes = [p, i64, p, p, p, p, i64, i64, i64, i32, p]
    lib.km_gemm_fp8_blocks_fused.argtypes = [p, i64, p, p, p, p, i64, i64, i64, i32, p]
    lib.km_gemm_fp8_tensor.argtypes = [p, p, p, p, p, p, i64, i64, i64, i32, i32, p]
    lib.km_gemm_fp8_rows.argtypes = [p, p, p, p, p, p, i64, i64, i64, i32, i32, p]
    lib.km_gemm_fp8_blocks.argtypes = [p, p, p, p, p, p, i64, i64, i64, i32, i32, i32, p]
    lib.km_gemm_i8_rows.argtypes = [p, p, p, p, p, p, i64, i64, i64, i32, i32, p]
    lib.km_wo_gemm_fwd.argtypes = [p, p, p, p, p, i64, i64, i64, i32, i32, i32, p]
    lib.km_wo_gemm_dgrad.argtypes = [p, p, p, p, p, i64, i64, i64, i32, i32, i32, p]
    lib.km_wo_gemm_dgrad_w16.argtypes = [p, p, p, i32, i64, p, i64, i64, i64, i32, i32, i32, p]
    lib.km_wo_gemm_dgrad_static.argtypes = [p, p, p, p, i64, i64, i64, i32, i32, i32, p]
    lib.km_wo_gemm_path.argtypes = [i32, p, p, p, p, i64, i64, i64]
    lib.km_group_hadamard.argtypes = [p, i64, i64, i32, i32, p, p]
    lib.km_probe_mfma_ceiling.argtypes = [p, p, p, i64, i32, c.POINTER(c.c_int64), p]
    lib.km_num_configs.argtypes = [i32]
    lib.km_config_desc.argtypes = [i32, i32, c.c_char_p, i32]
    for name in EXPORTS:
        if name not in ("km_last_error", "km_scales_packed_bytes"):
            getattr(lib, name).restype = i32
    lib.km_scales_packed_bytes.restype = i64


def load() -> ctypes.CDLL:
    """The loaded library (cached). Raises KernelLibraryMissing when it is not there."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not LIB_PATH.exists():
                raise KernelLibraryMissing(
                    f"{LIB_PATH} is not built; run `python -m kohakumosstrainer_amd.build` (needs hipcc)"
                )
            try:
                lib = ctypes.CDLL(str(LIB_PATH))
            except OSError as err:
                raise KernelLibraryMissing(f"cannot load {LIB_PATH}: {err}") from err
            missing = [n for n in EXPORTS if not hasattr(lib, n)]
            if missing:
                raise KernelLibraryMissing(f"{LIB_PATH} lacks {missing}")
            _declare(lib)
            _lib = lib
    return _lib


def available() -> str | None:
    """None when the library loads, else why not."""
    try:
        load()
    except KernelLibraryMissing as err:
        return str(err)
    return None


def _check(code: int) -> None:
    if code != 0:
        raise KernelError(load().km_last_error().decode(errors="replace") or f"error {code}")


def _stream(t: Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _on_gpu(*tensors: Tensor | None) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if t.device.type != "cuda":
            raise ValueError(f"HIP kernels need device tensors, got {t.device}")
        if dev is not None and t.device != dev:
            raise ValueError(f"operands on different devices: {dev} and {t.device}")
        dev = t.device
    return dev


def _dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError(f"activation dtype {dtype} not in (bfloat16, float16)") from None


# ---- quantizers -------------------------------------------------------------------------


def packed_scale_bytes(rows: int, k: int) -> int:
    """Size in bytes of the MFMA-packed scale copy of a [rows, k] operand (k % 128 == 0)."""
    n = load().km_scales_packed_bytes(rows, k)
    if n < 0:
        raise ValueError(f"packed mx scales need K % 128 == 0, got K={k}")
    return n


def _new_packed(rows: int, k: int, device) -> Tensor:
    n = packed_scale_bytes(rows, k)
    # rows past the end of the last group of 128 are padding the GEMM may read: keep them zero
    return (torch.zeros if rows % 128 else torch.empty)(n, device=device, dtype=torch.uint8)


def quant_mx(x: Tensor, natural: bool = True, packed: bool = False):
    """MXFP8 quantization of a 2-D bf16 / fp16 operand with any strides; blocks of 32 run
    along the last axis (a transposed view `w.t()` takes the transposing kernel: column-wise
    quantization). Returns `(q e4m3 [rows, K], scale uint8 [rows, K/32])`; with `packed`
    the MFMA-packed scale copy (flat uint8, K % 128 == 0) is appended, and `natural=False`
    returns None in place of the natural scales."""
    if x.dim() != 2:
        raise ValueError(f"fp8 operand must be 2-D, got {tuple(x.shape)}")
    rows, k = x.shape
    if k % 32:
        raise ValueError(f"fp8 mx: K={k} is not a multiple of 32")
    if not (natural or packed):
        raise ValueError("quant_mx: ask for at least one scale layout")
    _on_gpu(x)
    q = torch.empty(rows, k, device=x.device, dtype=torch.uint8)
    s = torch.empty(rows, k // 32, device=x.device, dtype=torch.uint8) if natural else None
    sp = _new_packed(rows, k, x.device) if packed else None
    with torch.cuda.device(x.device):
        _check(
            load().km_quant_mx(
                x.data_ptr(), rows, k, x.stride(0), x.stride(1), _dtype_code(x.dtype), q.data_ptr(),
                None if s is None else s.data_ptr(), None if sp is None else sp.data_ptr(), _stream(x),
            )
        )
    return (q.view(E4M3), s, sp) if packed else (q.view(E4M3), s)


def pack_scales(scale: Tensor) -> Tensor:
    """The MFMA-packed copy of natural mx scales `[rows, K/32]` (K % 128 == 0)."""
    if scale.dim() != 2 or scale.dtype != torch.uint8:
        raise ValueError("mx scales must be a 2-D uint8 tensor")
    _on_gpu(scale)
    rows, blocks = scale.shape
    scale = scale.contiguous()
    out = _new_packed(rows, blocks * 32, scale.device)
    with torch.cuda.device(scale.device):
        _check(load().km_scales_pack(scale.data_ptr(), rows, blocks * 32, out.data_ptr(), _stream(scale)))
    return out


def quant_tensor(x: Tensor) -> tuple[Tensor, Tensor]:
    """`(q e4m3 [rows, K], scale fp32 [1])` under the per-tensor recipe."""
    if x.dim() != 2:
        raise ValueError(f"fp8 operand must be 2-D, got {tuple(x.shape)}")
    _on_gpu(x)
    rows, k = x.shape
    q = torch.empty(rows, k, device=x.device, dtype=torch.uint8)
    s = torch.empty(1, device=x.device, dtype=torch.float32)
    work = torch.empty(QUANT_TENSOR_WORKSPACE_BYTES // 4, device=x.device, dtype=torch.int32)
    with torch.cuda.device(x.device):
        _check(load().km_quant_tensor(x.data_ptr(), rows, k, x.stride(0), x.stride(1), _dtype_code(x.dtype), q.data_ptr(), s.data_ptr(), work.data_ptr(), _stream(x)))
    return q.view(E4M3), s


def quant_rows(x: Tensor) -> tuple[Tensor, Tensor]:
    """`(q e4m3 [rows, K], scale fp32 [rows])` under the per-row recipe; any strides."""
    if x.dim() != 2:
        raise ValueError(f"fp8 operand must be 2-D, got {tuple(x.shape)}")
    _on_gpu(x)
    rows, k = x.shape
    q = torch.empty(rows, k, device=x.device, dtype=torch.uint8)
    s = torch.empty(rows, device=x.device, dtype=torch.float32)
    with torch.cuda.device(x.device):
        _check(load().km_quant_rows(x.data_ptr(), rows, k, x.stride(0), x.stride(1), _dtype_code(x.dtype), q.data_ptr(), s.data_ptr(), _stream(x)))
    return q.view(E4M3), s


def quant_blocks(x: Tensor, role: str = "act", natural: bool = True, kmajor: bool = False):
    """`(q e4m3 [rows, K], scale fp32)` under the block recipe; any strides, K % 128 == 0.
    `role="act"`: one scale per row and 128 columns, `[rows, K/128]`; with `kmajor` its
    `[K/128, rows]` copy (the layout the GEMM reads fastest) is appended, and `natural=False`
    returns None in place of the natural scales. `role="weight"`: one scale per 128 x 128 block,
    `[ceil(rows/128), K/128]`."""
    if x.dim() != 2:
        raise ValueError(f"fp8 operand must be 2-D, got {tuple(x.shape)}")
    if role not in ("act", "weight"):
        raise ValueError(f"fp8 role {role!r} not in ('act', 'weight')")
    if role == "weight" and (kmajor or not natural):
        raise ValueError("weight blocks have the one scale layout")
    if not (natural or kmajor):
        raise ValueError("quant_blocks: ask for at least one scale layout")
    rows, k = x.shape
    if k % BLOCK:
        raise ValueError(f"fp8 block: K={k} is not a multiple of {BLOCK}")
    _on_gpu(x)
    if role == "weight" and rows % BLOCK == 0 and rows > 1 and x.stride(0) == 1 and x.stride(1) >= rows:
        # A transposed view (the W^T copy of the input gradient): its 128 x 128 blocks are the
        # transposed blocks of the memory-order matrix, so codes and scales are the transposes of
        # that matrix's, which the vector kernel quantizes at full bandwidth.
        q, s = quant_blocks(x.t(), "weight")
        return q.view(torch.uint8).t().contiguous().view(E4M3), s.t().contiguous()
    q = torch.empty(rows, k, device=x.device, dtype=torch.uint8)
    srows = rows if role == "act" else -(-rows // BLOCK)
    s = torch.empty(srows, k // BLOCK, device=x.device, dtype=torch.float32) if natural else None
    st = torch.empty(k // BLOCK, rows, device=x.device, dtype=torch.float32) if kmajor else None
    with torch.cuda.device(x.device):
        _check(load().km_quant_blocks(x.data_ptr(), rows, k, x.stride(0), x.stride(1), _dtype_code(x.dtype), ROLE_ACT if role == "act" else ROLE_WEIGHT, q.data_ptr(), None if s is None else s.data_ptr(), None if st is None else st.data_ptr(), _stream(x)))
    return (q.view(E4M3), s, st) if kmajor else (q.view(E4M3), s)


def quant_rows_i8(x: Tensor, col_scale: Tensor | None = None) -> tuple[Tensor, Tensor]:
    """`(q int8 [rows, K], scale fp32 [rows])` of the int8 compute linear, the columns of x times
    `col_scale` [K] (fp32) first when given."""
    if x.dim() != 2:
        raise ValueError(f"int8 operand must be 2-D, got {tuple(x.shape)}")
    _on_gpu(x, col_scale)
    rows, k = x.shape
    if col_scale is not None:
        if tuple(col_scale.shape) != (k,):
            raise ValueError(f"col_scale must be [{k}], got {tuple(col_scale.shape)}")
        col_scale = col_scale.to(torch.float32).contiguous()
    q = torch.empty(rows, k, device=x.device, dtype=torch.int8)
    s = torch.empty(rows, device=x.device, dtype=torch.float32)
    with torch.cuda.device(x.device):
        _check(load().km_quant_rows_i8(x.data_ptr(), rows, k, x.stride(0), x.stride(1), _dtype_code(x.dtype), None if col_scale is None else col_scale.data_ptr(), q.data_ptr(), s.data_ptr(), _stream(x)))
    return q, s


ROTATED_QUANT_MAX_COLS = 4096  # longest row the rotating int8 quantizer holds in LDS (four rows of fp32)


def quant_rows_i8_rotated(x: Tensor, group: int) -> tuple[Tensor, Tensor]:
    """`quant_rows_i8(group_hadamard(x, group))`, bit for bit: one kernel that rotates the rows in
    LDS on their way to the quantizer where the rows fit (groups of 16 and more, unit-stride rows of
    up to `ROTATED_QUANT_MAX_COLS` elements), the two kernels one after the other elsewhere."""
    if x.dim() != 2:
        raise ValueError(f"int8 operand must be 2-D, got {tuple(x.shape)}")
    _on_gpu(x)
    rows, k = x.shape
    fits = group >= 16 and x.stride(1) == 1 and k <= ROTATED_QUANT_MAX_COLS and x.stride(0) % 8 == 0 and x.stride(0) >= k and x.data_ptr() % 16 == 0
    if not fits or rows == 0:
        return quant_rows_i8(group_hadamard(x, group))
    q = torch.empty(rows, k, device=x.device, dtype=torch.int8)
    s = torch.empty(rows, device=x.device, dtype=torch.float32)
    with torch.cuda.device(x.device):
        _check(load().km_quant_rows_i8_rotated(x.data_ptr(), rows, k, x.stride(0), _dtype_code(x.dtype), int(group), q.data_ptr(), s.data_ptr(), _stream(x)))
    return q, s


def group_hadamard(x: Tensor, group: int) -> Tensor:
    """`x [rows, K]` (bf16 / fp16) times blockdiag(H_group) over K, a new contiguous tensor."""
    if x.dim() != 2:
        raise ValueError(f"rotation operand must be 2-D, got {tuple(x.shape)}")
    _on_gpu(x)
    x = x.contiguous()
    y = torch.empty_like(x)
    with torch.cuda.device(x.device):
        _check(load().km_group_hadamard(x.data_ptr(), x.shape[0], x.shape[1], _dtype_code(x.dtype), int(group), y.data_ptr(), _stream(x)))
    return y


def mfma_ceiling_probe(a_codes: Tensor, b_codes: Tensor, trips: int) -> int:
    """Launch the registers-only block-scaled fp8 MFMA loop (`km_probe_mfma_ceiling`) on the current
    stream with the first 16 KiB of `a_codes` / `b_codes` (e4m3 codes of real operands) as its
    fragments; returns the launch's flop count. A measurement aid: time it with events."""
    dev = _on_gpu(a_codes, b_codes)
    frags = []
    for t in (a_codes, b_codes):
        flat = t.contiguous().view(torch.uint8).reshape(-1)
        if flat.numel() < 16384:
            raise ValueError("the probe takes at least 16 KiB of codes per operand")
        frags.append(flat[:16384])
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    sink = torch.empty(cus * 256, dtype=torch.float32, device=dev)
    flop = ctypes.c_int64(0)
    with torch.cuda.device(dev):
        _check(load().km_probe_mfma_ceiling(frags[0].data_ptr(), frags[1].data_ptr(), sink.data_ptr(), sink.numel(), int(trips), ctypes.byref(flop), _stream(a_codes)))
    return flop.value


# ---- GEMMs --------------------------------------------------------------------------------


def _gemm_operands(a: Tensor, b: Tensor, bias: Tensor | None, out_dtype: torch.dtype):
    if a.dim() != 2 or b.dim() != 2 or a.shape[1] != b.shape[1]:
        raise ValueError(f"GEMM operands must be [M, K] and [N, K], got {tuple(a.shape)} and {tuple(b.shape)}")
    if a.dtype != E4M3 or b.dtype != E4M3:
        raise ValueError(f"fp8 GEMM operands must be float8_e4m3fn, got {a.dtype} and {b.dtype}")
    dev = _on_gpu(a, b, bias)
    a, b = a.contiguous(), b.contiguous()
    if bias is not None:
        if bias.shape != (b.shape[0],):
            raise ValueError(f"bias must be [{b.shape[0]}], got {tuple(bias.shape)}")
        bias = bias.to(out_dtype).contiguous()
    m, k = a.shape
    c = torch.empty(m, b.shape[0], device=dev, dtype=out_dtype)
    return a, b, bias, c, m, b.shape[0], k


def gemm_mx(a: Tensor, a_scale: Tensor, b: Tensor, b_scale: Tensor, bias: Tensor | None, out_dtype: torch.dtype, config: int = 0, packed: bool = False) -> Tensor:
    """`(a * 2^(a_scale-127)) (b * 2^(b_scale-127))^T + bias` -> `[M, N]` in `out_dtype`;
    a `[M, K]`, b `[N, K]` e4m3, K a multiple of 128. Scales are uint8: natural
    `[*, K/32]`, or with `packed` the flat MFMA-packed copies (`quant_mx(packed=True)`,
    `pack_scales`)."""
    a, b, bias, c, m, n, k = _gemm_operands(a, b, bias, out_dtype)
    if a_scale.dtype != torch.uint8 or b_scale.dtype != torch.uint8:
        raise ValueError("mx scales must be uint8 (biased E8M0)")
    if packed:
        if k % 128:
            raise ValueError(f"packed mx scales need K % 128 == 0, got K={k}")
        want = (packed_scale_bytes(m, k), packed_scale_bytes(n, k))
        if (a_scale.numel(), b_scale.numel()) != want:
            raise ValueError(f"packed mx scales must hold {want} bytes, got ({a_scale.numel()}, {b_scale.numel()})")
    elif tuple(a_scale.shape) != (m, k // 32) or tuple(b_scale.shape) != (n, k // 32):
        raise ValueError(f"mx scales must be [{m}, {k // 32}] and [{n}, {k // 32}], got {tuple(a_scale.shape)} and {tuple(b_scale.shape)}")
    _on_gpu(a, a_scale, b_scale)
    a_scale, b_scale = a_scale.contiguous(), b_scale.contiguous()
    with torch.cuda.device(a.device):
        _check(
            load().km_gemm_mx(
                a.data_ptr(), a_scale.data_ptr(), b.data_ptr(), b_scale.data_ptr(), None if bias is None else bias.data_ptr(),
                c.data_ptr(), m, n, k, _dtype_code(out_dtype), SCALES_PACKED if packed else SCALES_ROWMAJOR, config, _stream(a),
            )
        )
    return c


FUSED_MAX_M = 32  # beyond this the redundant activation quantization costs more than the launch it saves


def gemm_mx_fused(x: Tensor, b: Tensor, b_scale_packed: Tensor, bias: Tensor | None) -> Tensor:
    """`Q(x) (b * 2^(b_scale-127))^T + bias` in one launch: x `[M, K]` bf16 / fp16 is quantized to
    MXFP8 inside the GEMM (same codes as `quant_mx`), b `[N, K]` e4m3 with its MFMA-packed scales
    (`pack_scales`); K % 128 == 0, N % 32 == 0. Meant for M up to `FUSED_MAX_M`."""
    if x.dim() != 2 or b.dim() != 2 or x.shape[1] != b.shape[1]:
        raise ValueError(f"operands must be [M, K] and [N, K], got {tuple(x.shape)} and {tuple(b.shape)}")
    if b.dtype != E4M3 or b_scale_packed.dtype != torch.uint8:
        raise ValueError("the weight must be float8_e4m3fn with uint8 packed scales")
    dev = _on_gpu(x, b, b_scale_packed, bias)
    m, k = x.shape
    n = b.shape[0]
    if k % 128 or n % 32:
        raise ValueError(f"the fused mx linear needs K % 128 == 0 and N % 32 == 0, got K={k}, N={n}")
    if b_scale_packed.numel() != packed_scale_bytes(n, k):
        raise ValueError(f"packed mx scales must hold {packed_scale_bytes(n, k)} bytes, got {b_scale_packed.numel()}")
    if x.stride(1) != 1 or x.stride(0) % 8 or x.stride(0) < k or x.data_ptr() % 16:
        x = x.contiguous()
    b, b_scale_packed = b.contiguous(), b_scale_packed.contiguous()
    if bias is not None:
        if bias.shape != (n,):
            raise ValueError(f"bias must be [{n}], got {tuple(bias.shape)}")
        bias = bias.to(x.dtype).contiguous()
    c = torch.empty(m, n, device=dev, dtype=x.dtype)
    with torch.cuda.device(dev):
        _check(load().km_gemm_mx_fused(x.data_ptr(), x.stride(0) if m else k, b.data_ptr(), b_scale_packed.data_ptr(), None if bias is None else bias.data_ptr(), c.data_ptr(), m, n, k, _dtype_code(x.dtype), _stream(x)))
    return c


def gemm_fp8_rows_fused(x: Tensor, b: Tensor, b_scale: Tensor, bias: Tensor | None) -> Tensor:
    """`(Q(x) b^T) * s[:, None] * b_scale[None, :] + bias` in one launch under the per-row recipe:
    x `[M, K]` bf16 / fp16 is quantized inside the GEMM (same codes and scales as `quant_rows`),
    b `[N, K]` e4m3, b_scale `[N]` fp32; K % 128 == 0, N % 32 == 0. Meant for M up to `FUSED_MAX_M`."""
    if x.dim() != 2 or b.dim() != 2 or x.shape[1] != b.shape[1]:
        raise ValueError(f"operands must be [M, K] and [N, K], got {tuple(x.shape)} and {tuple(b.shape)}")
    m, k = x.shape
    n = b.shape[0]
    if b.dtype != E4M3 or tuple(b_scale.shape) != (n,) or b_scale.dtype != torch.float32:
        raise ValueError(f"the weight must be float8_e4m3fn with fp32 row scales [{n}]")
    dev = _on_gpu(x, b, b_scale, bias)
    if k % 128 or n % 32:
        raise ValueError(f"the fused row linear needs K % 128 == 0 and N % 32 == 0, got K={k}, N={n}")
    if x.stride(1) != 1 or x.stride(0) % 8 or x.stride(0) < k or x.data_ptr() % 16:
        x = x.contiguous()
    b, b_scale = b.contiguous(), b_scale.contiguous()
    if bias is not None:
        if bias.shape != (n,):
            raise ValueError(f"bias must be [{n}], got {tuple(bias.shape)}")
        bias = bias.to(x.dtype).contiguous()
    c = torch.empty(m, n, device=dev, dtype=x.dtype)
    with torch.cuda.device(dev):
        _check(load().km_gemm_fp8_rows_fused(x.data_ptr(), x.stride(0) if m else k, b.data_ptr(), b_scale.data_ptr(), None if bias is None else bias.data_ptr(), c.data_ptr(), m, n, k, _dtype_code(x.dtype), _stream(x)))
    return c


def gemm_fp8_blocks_fused(x: Tensor, b: Tensor, b_scale: Tensor, bias: Tensor | None) -> Tensor:
    """The block-recipe linear in one launch: x `[M, K]` bf16 / fp16 is quantized per row and 128
    columns inside the GEMM (same codes and scales as `quant_blocks(x, "act")`), b `[N, K]` e4m3,
    b_scale `[ceil(N/128), K/128]` fp32; K % 128 == 0, N % 32 == 0. Meant for M up to `FUSED_MAX_M`."""
    if x.dim() != 2 or b.dim() != 2 or x.shape[1] != b.shape[1]:
        raise ValueError(f"operands must be [M, K] and [N, K], got {tuple(x.shape)} and {tuple(b.shape)}")
    m, k = x.shape
    n = b.shape[0]
    if k % 128 or n % 32:
        raise ValueError(f"the fused block linear needs K % 128 == 0 and N % 32 == 0, got K={k}, N={n}")
    if b.dtype != E4M3 or tuple(b_scale.shape) != (-(-n // BLOCK), k // BLOCK) or b_scale.dtype != torch.float32:
        raise ValueError(f"the weight must be float8_e4m3fn with fp32 block scales [{-(-n // BLOCK)}, {k // BLOCK}]")
    dev = _on_gpu(x, b, b_scale, bias)
    if x.stride(1) != 1 or x.stride(0) % 8 or x.stride(0) < k or x.data_ptr() % 16:
        x = x.contiguous()
    b, b_scale = b.contiguous(), b_scale.contiguous()
    if bias is not None:
        if bias.shape != (n,):
            raise ValueError(f"bias must be [{n}], got {tuple(bias.shape)}")
        bias = bias.to(x.dtype).contiguous()
    c = torch.empty(m, n, device=dev, dtype=x.dtype)
    with torch.cuda.device(dev):
        _check(load().km_gemm_fp8_blocks_fused(x.data_ptr(), x.stride(0) if m else k, b.data_ptr(), b_scale.data_ptr(), None if bias is None else bias.data_ptr(), c.data_ptr(), m, n, k, _dtype_code(x.dtype), _stream(x)))
    return c


def gemm_fp8_tensor(a: Tensor, sa: Tensor, b: Tensor, sb: Tensor, bias: Tensor | None, out_dtype: torch.dtype, config: int = 0) -> Tensor:
    """`(a b^T) * sa * sb + bias`, sa / sb one-element fp32 device tensors."""
    a, b, bias, c, m, n, k = _gemm_operands(a, b, bias, out_dtype)
    if sa.numel() != 1 or sb.numel() != 1 or sa.dtype != torch.float32 or sb.dtype != torch.float32:
        raise ValueError("per-tensor scales must be one-element fp32 tensors")
    _on_gpu(a, sa, sb)
    with torch.cuda.device(a.device):
        _check(load().km_gemm_fp8_tensor(a.data_ptr(), sa.data_ptr(), b.data_ptr(), sb.data_ptr(), None if bias is None else bias.data_ptr(), c.data_ptr(), m, n, k, _dtype_code(out_dtype), config, _stream(a)))
    return c


def gemm_fp8_rows(a: Tensor, sa: Tensor, b: Tensor, sb: Tensor, bias: Tensor | None, out_dtype: torch.dtype, config: int = 0) -> Tensor:
    """`(a b^T) * sa[:, None] * sb[None, :] + bias`, sa `[M]` and sb `[N]` fp32 device vectors."""
    a, b, bias, c, m, n, k = _gemm_operands(a, b, bias, out_dtype)
    if tuple(sa.shape) != (m,) or tuple(sb.shape) != (n,) or sa.dtype != torch.float32 or sb.dtype != torch.float32:
        raise ValueError(f"per-row scales must be fp32 vectors [{m}] and [{n}], got {tuple(sa.shape)} {sa.dtype} and {tuple(sb.shape)} {sb.dtype}")
    _on_gpu(a, sa, sb)
    sa, sb = sa.contiguous(), sb.contiguous()
    with torch.cuda.device(a.device):
        _check(load().km_gemm_fp8_rows(a.data_ptr(), sa.data_ptr(), b.data_ptr(), sb.data_ptr(), None if bias is None else bias.data_ptr(), c.data_ptr(), m, n, k, _dtype_code(out_dtype), config, _stream(a)))
    return c


def gemm_fp8_blocks(a: Tensor, sa: Tensor, b: Tensor, sb: Tensor, bias: Tensor | None, out_dtype: torch.dtype, config: int = 0, kmajor: bool = False) -> Tensor:
    """`sum_kb (a_kb b_kb^T) * sa[:, kb, None] * sb[n // 128, kb] + bias`; sa `[M, K/128]` (with
    `kmajor`: its `[K/128, M]` copy from `quant_blocks(kmajor=True)`), sb `[ceil(N/128), K/128]`
    fp32 device tensors (the block recipe's activation and weight scales)."""
    a, b, bias, c, m, n, k = _gemm_operands(a, b, bias, out_dtype)
    if k % BLOCK:
        raise ValueError(f"fp8 block: K={k} is not a multiple of {BLOCK}")
    want = ((k // BLOCK, m) if kmajor else (m, k // BLOCK), (-(-n // BLOCK), k // BLOCK))
    if (tuple(sa.shape), tuple(sb.shape)) != want or sa.dtype != torch.float32 or sb.dtype != torch.float32:
        raise ValueError(f"block scales must be fp32 {want[0]} and {want[1]}, got {tuple(sa.shape)} {sa.dtype} and {tuple(sb.shape)} {sb.dtype}")
    _on_gpu(a, sa, sb)
    sa, sb = sa.contiguous(), sb.contiguous()
    with torch.cuda.device(a.device):
        _check(load().km_gemm_fp8_blocks(a.data_ptr(), sa.data_ptr(), b.data_ptr(), sb.data_ptr(), None if bias is None else bias.data_ptr(), c.data_ptr(), m, n, k, _dtype_code(out_dtype), SCALES_KMAJOR if kmajor else SCALES_ROWMAJOR, config, _stream(a)))
    return c


def gemm_i8_rows(a: Tensor, sa: Tensor, b: Tensor, sb: Tensor | None, bias: Tensor | None, out_dtype: torch.dtype, config: int = 0) -> Tensor:
    """`((int32(a b^T) * sa[:, None]) * sb[None, :]) + bias` rounded once to `out_dtype`; a `[M, K]`
    and b `[N, K]` int8, sa `[M]` fp32, sb `[N]` fp32 or None (ones)."""
    if a.dim() != 2 or b.dim() != 2 or a.shape[1] != b.shape[1]:
        raise ValueError(f"GEMM operands must be [M, K] and [N, K], got {tuple(a.shape)} and {tuple(b.shape)}")
    if a.dtype != torch.int8 or b.dtype != torch.int8:
        raise ValueError(f"int8 GEMM operands must be int8, got {a.dtype} and {b.dtype}")
    m, k = a.shape
    n = b.shape[0]
    if tuple(sa.shape) != (m,) or sa.dtype != torch.float32 or (sb is not None and (tuple(sb.shape) != (n,) or sb.dtype != torch.float32)):
        raise ValueError(f"int8 GEMM scales must be fp32 vectors [{m}] and [{n}]")
    if bias is not None and (tuple(bias.shape) != (n,) or bias.dtype != out_dtype):
        raise ValueError(f"bias must be [{n}] {out_dtype}, got {tuple(bias.shape)} {bias.dtype}")
    dev = _on_gpu(a, b, sa, sb, bias)
    a, b, sa = a.contiguous(), b.contiguous(), sa.contiguous()
    sb = None if sb is None else sb.contiguous()
    bias = None if bias is None else bias.contiguous()
    c = torch.empty(m, n, device=dev, dtype=out_dtype)
    with torch.cuda.device(dev):
        _check(load().km_gemm_i8_rows(a.data_ptr(), sa.data_ptr(), b.data_ptr(), None if sb is None else sb.data_ptr(), None if bias is None else bias.data_ptr(), c.data_ptr(), m, n, k, _dtype_code(out_dtype), config, _stream(a)))
    return c


def _wo_operands(x: Tensor, q: Tensor, scale: Tensor):
    if x.dim() != 2 or q.dim() != 2:
        raise ValueError(f"weight-only operands must be 2-D, got {tuple(x.shape)} and {tuple(q.shape)}")
    if q.dtype not in _QFORMATS:
        raise ValueError(f"weight codes must be int8 or float8_e4m3fn, got {q.dtype}")
    if tuple(scale.shape) != (q.shape[0],):
        raise ValueError(f"scale must be [{q.shape[0]}], got {tuple(scale.shape)}")
    _on_gpu(x, q, scale)
    return x.contiguous(), q.contiguous(), scale.to(torch.float32).contiguous()


class SlowPathWarning(UserWarning):
    """A problem left the tiled kernels for the one-thread-per-element kernel (ragged K or N, or operands
    that are not 16-byte aligned): correct, and slower by orders of magnitude."""


WO_FWD, WO_DGRAD_W16, WO_DGRAD_TRANSPOSED = 0, 1, 2
_SLOW_SEEN: set[tuple] = set()


def _note_path(direction: int, a: Tensor, q: Tensor, scale: Tensor, c: Tensor, m: int, n: int, k: int) -> None:
    """Warn, once per direction and shape, when the library will serve this problem with its
    element-wise kernel."""
    key = (direction, m, n, k)
    if key in _SLOW_SEEN:
        return
    if load().km_wo_gemm_path(direction, a.data_ptr(), q.data_ptr(), scale.data_ptr(), c.data_ptr(), m, n, k) == 1:
        _SLOW_SEEN.add(key)
        import warnings

        what = ("forward", "input gradient", "input gradient (transposed codes)")[direction]
        warnings.warn(f"weight-only {what} M={m} N={n} K={k}: shape or alignment outside the tiled kernels, the element-wise kernel serves it", SlowPathWarning, stacklevel=3)


def wo_gemm_fwd(x: Tensor, q: Tensor, scale: Tensor, bias: Tensor | None, config: int = 0) -> Tensor:
    """`(x @ q^T) * scale + bias` -> `[M, N]` in x's dtype; q `[N, K]` int8 / e4m3."""
    x, q, scale = _wo_operands(x, q, scale)
    if x.shape[1] != q.shape[1]:
        raise ValueError(f"x is [M, {x.shape[1]}] but q is [N, {q.shape[1]}]")
    m, k = x.shape
    n = q.shape[0]
    if bias is not None:
        if bias.shape != (n,):
            raise ValueError(f"bias must be [{n}], got {tuple(bias.shape)}")
        _on_gpu(x, bias)
        bias = bias.to(x.dtype).contiguous()
    y = torch.empty(m, n, device=x.device, dtype=x.dtype)
    _note_path(WO_FWD, x, q, scale, y, m, n, k)
    with torch.cuda.device(x.device):
        _check(load().km_wo_gemm_fwd(x.data_ptr(), q.data_ptr(), scale.data_ptr(), None if bias is None else bias.data_ptr(), y.data_ptr(), m, n, k, _QFORMATS[q.dtype], _dtype_code(x.dtype), config, _stream(x)))
    return y


WSCALE_ROWS, WSCALE_E8M0, WSCALE_BLOCKS = 0, 1, 2  # weight scale layouts of km_wo_gemm_dgrad_w16


def wo_gemm_dgrad(dy: Tensor, q: Tensor, scale: Tensor, config: int = 0, recipe: str = "row") -> Tensor:
    """`dy @ round(q * scale)` -> `[M, K]` in dy's dtype, over the codes `q [N, K]` as they are
    stored (no transposed copy, no workspace). `recipe` names the scale layout: "row" fp32 `[N]`,
    "tensor" one fp32, "mx" uint8 `[N, K/32]` biased exponents, "block" fp32 `[ceil(N/128), K/128]`
    (the last three for e4m3 codes)."""
    if dy.dim() != 2 or q.dim() != 2 or dy.shape[1] != q.shape[0]:
        raise ValueError(f"dy must be [M, N] and q [N, K], got {tuple(dy.shape)} and {tuple(q.shape)}")
    if q.dtype not in _QFORMATS:
        raise ValueError(f"codes must be int8 or float8_e4m3fn, got {q.dtype}")
    m, n = dy.shape
    k = q.shape[1]
    _on_gpu(dy, q, scale)
    dy, q = dy.contiguous(), q.contiguous()
    if recipe == "row":
        kind, ld, scale = WSCALE_ROWS, 1, scale.float().reshape(-1).contiguous()
        want = n
    elif recipe == "tensor":
        kind, ld, scale = WSCALE_ROWS, 0, scale.float().reshape(-1).contiguous()
        want = 1
    elif recipe == "mx":
        scale = scale.contiguous()
        if scale.dtype != torch.uint8 or scale.dim() != 2 or scale.shape[0] != n:
            raise ValueError(f"mx scales must be uint8 [N, K/32], got {scale.dtype} {tuple(scale.shape)}")
        kind, ld, want = WSCALE_E8M0, scale.shape[1], n * ((k + 31) // 32)
    elif recipe == "block":
        scale = scale.float().contiguous()
        if scale.dim() != 2 or scale.shape[0] != (n + 127) // 128:
            raise ValueError(f"block scales must be [ceil(N/128), K/128], got {tuple(scale.shape)}")
        kind, ld, want = WSCALE_BLOCKS, scale.shape[1], ((n + 127) // 128) * ((k + 127) // 128)
    else:
        raise ValueError(f"unknown scale layout {recipe!r}")
    if scale.numel() < want:
        raise ValueError(f"{recipe} scales of q {tuple(q.shape)} need {want} values, got {scale.numel()}")
    if q.dtype == torch.int8 and kind != WSCALE_ROWS:
        raise ValueError("int8 codes take one scale per row")
    dx = torch.empty(m, k, device=dy.device, dtype=dy.dtype)
    _note_path(WO_DGRAD_W16, dy, q, scale, dx, m, n, k)
    with torch.cuda.device(dy.device):
        _check(load().km_wo_gemm_dgrad_w16(dy.data_ptr(), q.data_ptr(), scale.data_ptr(), kind, ld, dx.data_ptr(), m, n, k, _QFORMATS[q.dtype], _dtype_code(dy.dtype), config, _stream(dy)))
    return dx


def wo_gemm_dgrad_workspace(dy: Tensor, q: Tensor, scale: Tensor, config: int = 0) -> Tensor:
    """The same input gradient through `km_wo_gemm_dgrad`: the codes are first transposed into an
    N * K byte workspace that this wrapper allocates."""
    dy, q, scale = _wo_operands(dy, q, scale)
    if dy.shape[1] != q.shape[0]:
        raise ValueError(f"dy is [M, {dy.shape[1]}] but q is [{q.shape[0]}, K]")
    m, n = dy.shape
    k = q.shape[1]
    dx = torch.empty(m, k, device=dy.device, dtype=dy.dtype)
    work = torch.empty(max(n * k, 1), device=dy.device, dtype=torch.uint8)  # codes transposed to [K, N]
    with torch.cuda.device(dy.device):
        _check(load().km_wo_gemm_dgrad(dy.data_ptr(), q.data_ptr(), scale.data_ptr(), dx.data_ptr(), work.data_ptr(), m, n, k, _QFORMATS[q.dtype], _dtype_code(dy.dtype), config, _stream(dy)))
    return dx


WO_DGRAD_STATIC_MAX_CODES = 64 << 20  # bytes of the library's static transpose workspace per GPU


def wo_gemm_dgrad_static(dy: Tensor, q: Tensor, scale: Tensor, out: Tensor, config: int = 0) -> Tensor:
    """`wo_gemm_dgrad` into the caller's `out` `[M, K]` through the entry point that allocates
    nothing: the transposed codes live in a static device array of the library (N * K up to
    `WO_DGRAD_STATIC_MAX_CODES`). Operands must already be contiguous (fp32 scale); calls that
    overlap on one GPU share that array and race."""
    if dy.dim() != 2 or q.dim() != 2 or dy.shape[1] != q.shape[0]:
        raise ValueError(f"dy must be [M, N] and q [N, K], got {tuple(dy.shape)} and {tuple(q.shape)}")
    m, n = dy.shape
    k = q.shape[1]
    if q.dtype not in _QFORMATS or scale.dtype != torch.float32 or tuple(scale.shape) != (n,):
        raise ValueError("codes must be int8 / float8_e4m3fn with an fp32 scale per row")
    if tuple(out.shape) != (m, k) or out.dtype != dy.dtype:
        raise ValueError(f"out must be [{m}, {k}] {dy.dtype}")
    if not all(t.is_contiguous() for t in (dy, q, scale, out)):
        raise ValueError("the no-allocation entry point takes contiguous operands")
    _on_gpu(dy, q, scale, out)
    with torch.cuda.device(dy.device):
        _check(load().km_wo_gemm_dgrad_static(dy.data_ptr(), q.data_ptr(), scale.data_ptr(), out.data_ptr(), m, n, k, _QFORMATS[q.dtype], _dtype_code(dy.dtype), config, _stream(dy)))
    return out


def configs(kernel: int) -> list[dict]:
    """The tile configurations of one kernel family as dicts (`id` is the ABI config)."""
    lib = load()
    out = []
    buf = ctypes.create_string_buffer(128)
    for i in range(lib.km_num_configs(kernel)):
        _check(lib.km_config_desc(kernel, i, buf, len(buf)))
        row: dict = {"id": i}
        for part in buf.value.decode().split(","):
            key, _, val = part.partition("=")
            row[key] = int(val) if val.lstrip("-").isdigit() else val
        out.append(row)
    return out
