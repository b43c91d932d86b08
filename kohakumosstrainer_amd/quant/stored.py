"""Pre-quantized fp8-compute checkpoints: a model state in which every fp8-compute linear is
`<path>.weight` (its e4m3 codes) plus `<path>.weight_scale` (the scale in its recipe's layout),
with the recipe and the list of layers as a JSON record under the safetensors metadata key
`kohakumoss_fp8`. A base is attached from such a file without ever holding a 16-bit copy of the
weight; on a GPU the attached `ComputeWeight` binds straight to the HIP `fp8_linear`.

Mirrors reference `src/kohakumoss/quant/stored.py:16-94` (same key names, record layout and
function names, so files written by either side load in the other) and adds the two file-level
helpers `save_quantized` / `load_quantized` over safetensors.
"""

import json
import struct
from dataclasses import dataclass
from pathlib import Path

import torch
from torch import Tensor, nn

from kohakumosstrainer_amd.model.linear import MossLinear
from kohakumosstrainer_amd.quant.compute import ComputeWeight

FP8_KEY = "kohakumoss_fp8"
SCALE = ".weight_scale"
KEEP_FP32 = ("rope.bands",)


@dataclass(frozen=True)
class StoredRecord:
    """What the `kohakumoss_fp8` metadata entry says: one recipe, the module paths stored as codes."""

    recipe: str
    layers: tuple[str, ...]

    @classmethod
    def parse(cls, raw: dict) -> "StoredRecord":
        return cls(str(raw["recipe"]), tuple(raw["layers"]))

    def as_dict(self) -> dict:
        return {"recipe": self.recipe, "layers": list(self.layers)}

    def metadata(self) -> dict[str, str]:
        return {FP8_KEY: json.dumps(self.as_dict())}

    @property
    def weight_keys(self) -> set[str]:
        return {path + ".weight" for path in self.layers}

    @property
    def scale_keys(self) -> set[str]:
        return {path + SCALE for path in self.layers}


def compute_bases(model: nn.Module) -> dict[str, ComputeWeight]:
    """{module path: ComputeWeight} of every fp8-compute MossLinear of `model`."""
    found = {}
    for path, module in model.named_modules():
        if isinstance(module, MossLinear) and isinstance(module.base, ComputeWeight):
            found[path] = module.base
    return found


def _host(t: Tensor) -> Tensor:
    return t.detach().contiguous().cpu()


def quantized_state(model: nn.Module, keys: list[str], dtype: torch.dtype) -> tuple[dict[str, Tensor], dict[str, str]]:
    """`(state, metadata)` of `model` over its state `keys`, on the host: an fp8-compute layer
    contributes its codes under `<path>.weight` and its scale under `<path>.weight_scale`, every
    other floating-point tensor is cast to `dtype` (the KEEP_FP32 names stay as they are). A
    checkpoint holds one recipe; a model with folded scales has no fp8 bases to export."""
    if getattr(model, "fold_scales", None) is not None:
        raise ValueError("a folded (fp16-fix) model is exported without fp8 bases")
    bases = compute_bases(model)
    recipes = sorted({base.recipe for base in bases.values()})
    if len(recipes) != 1:
        raise ValueError(f"one fp8 recipe per checkpoint, found {recipes}")
    tensors = dict(model.named_buffers())
    tensors.update(model.named_parameters())
    state: dict[str, Tensor] = {}
    for key in keys:
        owner = key.removesuffix(".weight") if key.endswith(".weight") else None
        base = bases.get(owner) if owner is not None else None
        if base is not None:
            state[key], state[owner + SCALE] = _host(base.q), _host(base.scale)
        else:
            value = tensors[key]
            cast = value.is_floating_point() and key not in KEEP_FP32
            state[key] = _host(value.to(dtype) if cast else value)
    return state, StoredRecord(recipes[0], tuple(sorted(bases))).metadata()


def read_safetensors_metadata(path: str | Path) -> dict[str, str]:
    """The `__metadata__` string map of a safetensors file (empty when it has none). Only the
    header is read: an 8-byte little-endian length, then that many bytes of JSON."""
    with open(path, "rb") as f:
        (length,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(length))
    meta = header.get("__metadata__")
    return dict(meta) if meta else {}


def read_meta_record(path: str | Path, key: str) -> dict | None:
    """The JSON record under metadata `key` of a single safetensors file, or None when the path
    is not a file or the key is absent."""
    if not Path(path).is_file():
        return None
    raw = read_safetensors_metadata(path).get(key)
    return None if raw is None else json.loads(raw)


def read_record(path: str | Path) -> dict | None:
    """The fp8 record of a single-file checkpoint, if it carries one."""
    return read_meta_record(path, FP8_KEY)


def stored_keys(record: dict) -> tuple[set[str], set[str]]:
    """(the `.weight` keys of stored layers, their scale keys)."""
    parsed = StoredRecord.parse(record)
    return parsed.weight_keys, parsed.scale_keys


def _reader(view):
    """`view` is anything that hands out tensors by key: a dict, an open safetensors file."""
    return view.get if hasattr(view, "get") else view.get_tensor


@torch.no_grad()
def attach_stored(model: nn.Module, view, record: dict, device, dtype: torch.dtype) -> int:
    """Give every recorded layer a ComputeWeight built from the codes and scale in `view`, replace
    its dense parameter by an empty placeholder and bind the base for `(device, dtype)`. No 16-bit
    copy of a stored weight is made at any point. Returns the number of layers attached."""
    parsed = StoredRecord.parse(record)
    read = _reader(view)
    for path in parsed.layers:
        layer = model.get_submodule(path)
        if not isinstance(layer, MossLinear):
            raise TypeError(f"{path} is {type(layer).__name__}, not a MossLinear")
        codes = read(path + ".weight").to(device)
        want = (layer.out_features, layer.in_features)
        if tuple(codes.shape) != want:
            raise ValueError(f"{path}: stored codes are {tuple(codes.shape)}, the layer is {want}")
        base = ComputeWeight.from_stored(parsed.recipe, codes, read(path + SCALE).to(device))
        layer.weight = nn.Parameter(torch.empty(0, dtype=dtype, device=device), requires_grad=False)
        layer.set_base(base)
        base.bind(dtype, device)
    return len(parsed.layers)


def save_quantized(model: nn.Module, path: str | Path, dtype: torch.dtype = torch.bfloat16) -> dict:
    """Write `model` (every parameter and persistent buffer) as one safetensors file in the
    stored layout; returns the record written under `kohakumoss_fp8`."""
    from safetensors.torch import save_file

    bases = compute_bases(model)
    keys = list(model.state_dict().keys())
    # a stored layer's dense parameter is gone (numel 0): its `.weight` key stands for the codes
    keys = [k for k in keys if not any(k.startswith(p + ".base.") for p in bases)]
    for p in bases:
        if f"{p}.weight" not in keys:
            keys.append(f"{p}.weight")
    state, meta = quantized_state(model, keys, dtype)
    # the codes keep their float8_e4m3fn dtype in the file: a reader that hands `<path>.weight`
    # straight to its fp8 GEMM (the reference's `attach_stored`) must not see bytes
    save_file(state, str(path), metadata=meta)
    return json.loads(meta[FP8_KEY])


@torch.no_grad()
def load_quantized(model: nn.Module, path: str | Path, device, dtype: torch.dtype) -> int:
    """Load a file written by `save_quantized` (or by the reference's exporter) into `model`:
    recorded layers get their fp8 bases from the file, every other tensor is loaded as usual.
    Returns the number of attached layers (0 for a file without a record: plain load).

    The dense parameter of a recorded layer is replaced by an empty placeholder before anything
    moves to `device`, so its 16-bit weight is never materialised there (and a model built on the
    meta device loads). Every other parameter and persistent buffer of the model must be in the
    file and the file must hold nothing else: a missing or misspelt tensor raises KeyError instead
    of leaving an initial value in place. Codes stored as bytes by an earlier version of this
    package are reinterpreted as e4m3."""
    from safetensors import safe_open

    record = read_record(path)
    device = torch.device(device)
    with safe_open(str(path), framework="pt", device="cpu") as f:
        names = set(f.keys())
        weights, scales = stored_keys(record) if record else (set(), set())
        absent = (weights | scales) - names
        if absent:
            raise KeyError(f"{path}: the record names tensors the file lacks: {sorted(absent)[:4]}")
        for key in sorted(weights):
            layer = model.get_submodule(key.removesuffix(".weight"))
            if not isinstance(layer, MossLinear):
                raise TypeError(f"{key}: {type(layer).__name__} is not a MossLinear")
            layer.weight = nn.Parameter(torch.empty(0, dtype=dtype, device=device), requires_grad=False)
        plain = {k: f.get_tensor(k) for k in names - weights - scales}
        on_meta = any(t.is_meta for t in list(model.parameters()) + list(model.buffers()))
        result = model.load_state_dict(plain, strict=False, assign=on_meta)
        missing = sorted(set(result.missing_keys) - weights)
        if missing or result.unexpected_keys:
            raise KeyError(f"{path} does not match the model: missing {missing[:4]}, unexpected {sorted(result.unexpected_keys)[:4]}")
        model.to(device)
        if not record:
            return 0

        class _View:
            @staticmethod
            def get(key):
                t = f.get_tensor(key)
                return t.view(torch.float8_e4m3fn) if key in weights and t.dtype == torch.uint8 else t

        return attach_stored(model, _View, record, device, dtype)
