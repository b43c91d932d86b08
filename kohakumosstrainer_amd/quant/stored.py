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
from pathlib import Path

import torch
from torch import Tensor, nn

from kohakumosstrainer_amd.model.linear import MossLinear
from kohakumosstrainer_amd.quant.compute import ComputeWeight

FP8_KEY = "kohakumoss_fp8"
SCALE = ".weight_scale"
KEEP_FP32 = ("rope.bands",)


def compute_bases(model: nn.Module) -> dict[str, ComputeWeight]:
    """{module path: ComputeWeight} of every fp8-compute MossLinear of `model`."""
    return {path: lin.base for path, lin in model.named_modules() if isinstance(lin, MossLinear) and isinstance(lin.base, ComputeWeight)}


def quantized_state(model: nn.Module, keys: list[str], dtype: torch.dtype) -> tuple[dict[str, Tensor], dict[str, str]]:
    """`(state, metadata)` of `model` over its state `keys`, on the host: fp8-compute layers as
    codes and scale, every other floating-point tensor cast to `dtype` (the KEEP_FP32 names
    stay fp32). One recipe per checkpoint."""
    if getattr(model, "fold_scales", None) is not None:
        raise ValueError("a folded (fp16-fix) model is exported without fp8 bases")
    bases = compute_bases(model)
    recipes = {b.recipe for b in bases.values()}
    if len(recipes) != 1:
        raise ValueError(f"one fp8 recipe per checkpoint, found {sorted(recipes)}")
    live = {**dict(model.named_buffers()), **dict(model.named_parameters())}
    state: dict[str, Tensor] = {}
    for key in keys:
        path = key[: -len(".weight")] if key.endswith(".weight") else None
        if path in bases:
            state[key] = bases[path].q.contiguous().cpu()
            state[path + SCALE] = bases[path].scale.contiguous().cpu()
            continue
        t = live[key].detach()
        if key not in KEEP_FP32 and t.is_floating_point():
            t = t.to(dtype)
        state[key] = t.contiguous().cpu()
    record = {"recipe": recipes.pop(), "layers": sorted(bases)}
    return state, {FP8_KEY: json.dumps(record)}


def read_safetensors_metadata(path: str | Path) -> dict[str, str]:
    """The `__metadata__` string map of a safetensors file (empty when it has none); reads the
    header only."""
    with open(path, "rb") as f:
        size = int.from_bytes(f.read(8), "little")
        header = json.loads(f.read(size))
    return dict(header.get("__metadata__") or {})


def read_meta_record(path: str | Path, key: str) -> dict | None:
    """The JSON record under metadata `key` of a single safetensors file, if it carries one."""
    path = Path(path)
    if not path.is_file():
        return None
    meta = read_safetensors_metadata(path)
    return json.loads(meta[key]) if key in meta else None


def read_record(path: str | Path) -> dict | None:
    """The fp8 record of a single-file checkpoint, if it carries one."""
    return read_meta_record(path, FP8_KEY)


def stored_keys(record: dict) -> tuple[set[str], set[str]]:
    """(the `.weight` keys of stored layers, their scale keys)."""
    layers = record["layers"]
    return {f"{p}.weight" for p in layers}, {p + SCALE for p in layers}


@torch.no_grad()
def attach_stored(model: nn.Module, view, record: dict, device, dtype: torch.dtype) -> int:
    """Attach a ComputeWeight read from `view` (anything with `.get(key) -> Tensor`: a dict, an
    open safetensors file) to every recorded layer, drop the layer's dense parameter and bind the
    base for `(device, dtype)`; returns how many layers were attached."""
    recipe = record["recipe"]
    get = view.get if hasattr(view, "get") else view.get_tensor
    for path in record["layers"]:
        lin = model.get_submodule(path)
        if not isinstance(lin, MossLinear):
            raise TypeError(f"{path} is {type(lin).__name__}, not a MossLinear")
        q = get(f"{path}.weight").to(device)
        scale = get(path + SCALE).to(device)
        if tuple(q.shape) != (lin.out_features, lin.in_features):
            raise ValueError(f"{path}: stored codes are {tuple(q.shape)}, the layer is {(lin.out_features, lin.in_features)}")
        base = ComputeWeight.from_stored(recipe, q, scale)
        lin.weight = nn.Parameter(torch.empty(0, dtype=dtype, device=device), requires_grad=False)
        lin.set_base(base)
        base.bind(dtype, device)
    return len(record["layers"])


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
    save_file({k: (v.view(torch.uint8) if v.dtype == torch.float8_e4m3fn else v) for k, v in state.items()}, str(path), metadata=meta)
    return json.loads(meta[FP8_KEY])


@torch.no_grad()
def load_quantized(model: nn.Module, path: str | Path, device, dtype: torch.dtype) -> int:
    """Load a file written by `save_quantized` (or by the reference's exporter) into `model`:
    recorded layers get their fp8 bases from the file, every other tensor is loaded as usual.
    Returns the number of attached layers (0 for a file without a record: plain load)."""
    from safetensors import safe_open

    record = read_record(path)
    with safe_open(str(path), framework="pt", device="cpu") as f:
        names = set(f.keys())
        weights, scales = stored_keys(record) if record else (set(), set())
        missing = (weights | scales) - names
        if missing:
            raise KeyError(f"{path}: the record names tensors the file lacks: {sorted(missing)[:4]}")
        plain = {k: f.get_tensor(k) for k in names - weights - scales}
        model.load_state_dict(plain, strict=False)
        model.to(device)
        if not record:
            return 0

        class _View:
            @staticmethod
            def get(key):
                t = f.get_tensor(key)
                return t.view(torch.float8_e4m3fn) if key in weights and t.dtype == torch.uint8 else t

        return attach_stored(model, _View, record, device, dtype)
