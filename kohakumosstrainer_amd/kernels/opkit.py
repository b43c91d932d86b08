"""One builder for every quantized linear op of this package.

All of them have the same shape: `y = FWD(x, frozen parts..., bias, options...)` over the last
axis of `x`, an input gradient `dx = DGRAD(dy, frozen parts..., options...)`, a bias gradient that
is the fp32 column sum of `dy`, and (one op) a dense weight gradient. What differs is the list
of frozen parts, which of them each launcher takes, and the options. An `OpSpec` states that;
`LinearOp` turns it into

  * a table of `(fwd, dgrad)` launcher pairs per backend (`register_launchers`), the seam a
    backend plugs into (reference `src/kohakumoss_kernels/fp8/op.py:43-46`,
    `quant/__init__.py:66-68`),
  * a pair of `torch.library` ops (`<name>` with autograd, `<name>_dgrad`) with shape-only fakes,
    so the op traces under `torch.compile(fullgraph=True)`,
  * an `autograd.Function` doing the same outside a trace, where the dispatcher's per-call
    cost of a library op is not worth paying,
  * `make(backend, autograd=True)`: the callable the registry hands out. It flattens leading
    axes, makes `x` contiguous and restores the shape.

Only the parts the input gradient reads are saved for backward: no 16-bit copy of a frozen
weight lives from forward to backward.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Sequence

import torch
from torch import Tensor

NAMESPACE = "kohakumoss_amd"
_LIBRARY = torch.library.Library(NAMESPACE, "FRAGMENT")


@dataclass(frozen=True)
class OpSpec:
    """name      public op name (`fp8_linear`); the library ops are `<ns>::<name>` and `<ns>::<name>_dgrad`
    parts     tensor operands between x and bias, in call order; a trailing `?` marks one that may be None
    options   `(name, python type)` of the trailing non-tensor operands
    fwd_takes / dgrad_takes   operand names each launcher receives after x / dy (`bias` allowed in fwd)
    out_rows  the part whose row count is the output width N; in_cols the part whose column count is K
              (`name.T` reads the other axis, for transposed copies)
    weight    a dense trainable operand that gets a gradient `dy^T x` (None for frozen bases)"""

    name: str
    parts: tuple[str, ...]
    options: tuple[tuple[str, type], ...]
    fwd_takes: tuple[str, ...]
    dgrad_takes: tuple[str, ...]
    out_rows: str = "q"
    in_cols: str = "q"
    weight: str | None = None
    library_names: tuple[str, str] | None = None  # names of the two library ops; default `<name>`, `<name>_dgrad`
    doc: str = ""

    @property
    def part_names(self) -> tuple[str, ...]:
        return tuple(p.rstrip("?") for p in self.parts)

    @property
    def option_names(self) -> tuple[str, ...]:
        return tuple(n for n, _ in self.options)

    def operands(self) -> tuple[str, ...]:
        """Call order of the public op, without the backend."""
        return ("x", *self.part_names, "bias", *self.option_names)


_SCHEMA_TYPES = {str: "str", int: "int", bool: "bool", float: "float"}


def _schema(spec: OpSpec, first: str, names: Sequence[str]) -> str:
    optional = {p.rstrip("?") for p in spec.parts if p.endswith("?")} | {"bias"}
    types = dict(spec.options)
    args = [f"Tensor {first}"]
    for n in names:
        if n in types:
            args.append(f"{_SCHEMA_TYPES[types[n]]} {n}")
        else:
            args.append(f"Tensor{'?' if n in optional else ''} {n}")
    args.append("str backend")
    return "(" + ", ".join(args) + ") -> Tensor"


def bias_gradient(dy2d: Tensor, dtype: torch.dtype) -> Tensor:
    """Column sum of the incoming gradient in fp32, stored in the bias dtype (reference
    `src/kohakumoss_kernels/fp8/op.py:116-118`)."""
    return dy2d.to(torch.float32).sum(dim=0).to(dtype)


def weight_gradient(dy2d: Tensor, x2d: Tensor, dtype: torch.dtype) -> Tensor:
    """`dy^T x` accumulated in fp32 and stored in the weight's dtype (reference
    `src/kohakumoss_kernels/backends/_master.py:35-38`). The library GEMM with an fp32 result
    where the device has one for the operand type, the fp32 product of the widened operands
    elsewhere."""
    if dy2d.is_cuda and dy2d.dtype in (torch.bfloat16, torch.float16):
        return torch.mm(dy2d.t(), x2d, out_dtype=torch.float32).to(dtype)
    return (dy2d.to(torch.float32).t() @ x2d.to(torch.float32)).to(dtype)


class LinearOp:
    """The launcher table, library ops and factories of one `OpSpec`."""

    def __init__(self, spec: OpSpec):
        self.spec = spec
        self.launchers: dict[str, tuple[Callable, Callable]] = {}
        self._fwd_order = tuple(spec.operands()[1:])  # everything after x
        self._dgrad_order = tuple(spec.dgrad_takes)
        self._define()

    # ---- the seam -----------------------------------------------------------------------
    def register_launchers(self, backend: str, fwd: Callable, dgrad: Callable) -> None:
        self.launchers[backend] = (fwd, dgrad)

    def _pair(self, backend: str) -> tuple[Callable, Callable]:
        try:
            return self.launchers[backend]
        except KeyError:
            raise RuntimeError(f"{self.spec.name}: backend {backend!r} registered no launchers") from None

    def forward(self, x2d: Tensor, named: dict, backend: str) -> Tensor:
        with _device_of(x2d):
            return self._pair(backend)[0](x2d, *(named[n] for n in self.spec.fwd_takes))

    def input_grad(self, dy2d: Tensor, named: dict, backend: str) -> Tensor:
        with _device_of(dy2d):
            return self._pair(backend)[1](dy2d, *(named[n] for n in self.spec.dgrad_takes))

    # ---- shapes -------------------------------------------------------------------------
    @staticmethod
    def _extent(named: dict, ref: str, axis: int) -> int:
        name, _, flip = ref.partition(".")
        return named[name].shape[1 - axis if flip == "T" else axis]

    def out_width(self, named: dict) -> int:
        return self._extent(named, self.spec.out_rows, 0)

    def in_width(self, named: dict) -> int:
        return self._extent(named, self.spec.in_cols, 1)

    # ---- torch.library ops ----------------------------------------------------------------
    def _define(self) -> None:
        spec = self.spec
        short_fwd, short_dgrad = spec.library_names or (spec.name, spec.name + "_dgrad")
        fwd_name, dgrad_name = f"{NAMESPACE}::{short_fwd}", f"{NAMESPACE}::{short_dgrad}"
        _LIBRARY.define(short_fwd + _schema(spec, "x", self._fwd_order))
        _LIBRARY.define(short_dgrad + _schema(spec, "dy", self._dgrad_order))
        self._fwd_op = getattr(getattr(torch.ops, NAMESPACE), short_fwd)
        self._dgrad_op = getattr(getattr(torch.ops, NAMESPACE), short_dgrad)

        def fwd_impl(x, *rest):
            *vals, backend = rest
            return self.forward(x, dict(zip(self._fwd_order, vals)), backend)

        def dgrad_impl(dy, *rest):
            *vals, backend = rest
            return self.input_grad(dy, dict(zip(self._dgrad_order, vals)), backend)

        def fwd_fake(x, *rest):
            named = dict(zip(self._fwd_order, rest[:-1]))
            return x.new_empty(x.shape[0], self.out_width(named))

        def dgrad_fake(dy, *rest):
            named = dict(zip(self._dgrad_order, rest[:-1]))
            return dy.new_empty(dy.shape[0], self.in_width(named))

        torch.library.impl(fwd_name, "CompositeExplicitAutograd", lib=_LIBRARY)(fwd_impl)
        torch.library.impl(dgrad_name, "CompositeExplicitAutograd", lib=_LIBRARY)(dgrad_impl)
        torch.library.register_fake(fwd_name, lib=_LIBRARY)(fwd_fake)
        torch.library.register_fake(dgrad_name, lib=_LIBRARY)(dgrad_fake)

        def setup(ctx, inputs, output):
            x, *rest = inputs
            self._remember(ctx, x, dict(zip(self._fwd_order, rest[:-1])), rest[-1])

        def backward(ctx, grad):
            return self._gradients(ctx, grad, lambda g, named, backend: self._dgrad_op(g, *(named[n] for n in self._dgrad_order), backend))

        torch.library.register_autograd(fwd_name, backward, setup_context=setup, lib=_LIBRARY)

        outer = self

        class Eager(torch.autograd.Function):
            """The same op outside a trace: launchers called directly."""

            @staticmethod
            def forward(ctx, x, *rest):
                *vals, backend = rest
                named = dict(zip(outer._fwd_order, vals))
                outer._remember(ctx, x, named, backend)
                return outer.forward(x, named, backend)

            @staticmethod
            def backward(ctx, grad):
                return outer._gradients(ctx, grad, outer.input_grad)

        self._eager = Eager

    # what backward needs: the parts the input gradient reads (+ x and the dense weight for a
    # weight gradient), the options, and which inputs want a gradient
    def _remember(self, ctx, x: Tensor, named: dict, backend: str) -> None:
        spec = self.spec
        keep = [n for n in spec.dgrad_takes if n in spec.part_names]
        ctx.kept_names = keep
        ctx.kept_none = [named[n] is None for n in keep]
        tensors = [named[n] for n in keep if named[n] is not None]
        ctx.with_weight = spec.weight is not None
        if ctx.with_weight:
            tensors.append(x)
        ctx.save_for_backward(*tensors)
        ctx.static = {n: named[n] for n in spec.dgrad_takes if n not in spec.part_names}
        ctx.backend = backend
        bias = named.get("bias")
        ctx.bias_dtype = None if bias is None else bias.dtype
        ctx.weight_dtype = named[spec.weight].dtype if ctx.with_weight else None

    def _gradients(self, ctx, grad: Tensor, dgrad_call: Callable):
        spec = self.spec
        saved = list(ctx.saved_tensors)
        x_saved = saved.pop() if ctx.with_weight else None
        it = iter(saved)
        named = {n: (None if gone else next(it)) for n, gone in zip(ctx.kept_names, ctx.kept_none)}
        named.update(ctx.static)
        g = grad.contiguous()
        needs = ctx.needs_input_grad  # x, then the operands in call order, then the backend
        grads: list[Tensor | None] = [None] * (len(self._fwd_order) + 2)
        if needs[0]:
            grads[0] = dgrad_call(g, named, ctx.backend)
        position = {n: i + 1 for i, n in enumerate(self._fwd_order)}
        if ctx.bias_dtype is not None and needs[position["bias"]]:
            grads[position["bias"]] = bias_gradient(g, ctx.bias_dtype)
        if ctx.with_weight and needs[position[spec.weight]]:
            grads[position[spec.weight]] = weight_gradient(g, x_saved, ctx.weight_dtype)
        return tuple(grads)

    # ---- factories ------------------------------------------------------------------------
    def make(self, backend: str, autograd: bool = True) -> Callable:
        """The callable for one backend: operands in the spec's call order (`x, parts..., bias,
        options...`). `autograd=False` gives the gradient-free op (same forward, bit for bit)."""
        order = self._fwd_order
        spec = self.spec

        def op(x: Tensor, *operands):
            if len(operands) != len(order):
                raise TypeError(f"{spec.name} takes {('x',) + order}, got {len(operands) + 1} operands")
            lead = x.shape[:-1]
            x2d = x.reshape(-1, x.shape[-1]).contiguous()
            if not autograd:
                with torch.no_grad():
                    y = self.forward(x2d.detach(), dict(zip(order, operands)), backend)
            elif torch.compiler.is_compiling():
                y = self._fwd_op(x2d, *operands, backend)
            else:
                y = self._eager.apply(x2d, *operands, backend)
            return y.reshape(*lead, y.shape[-1])

        op.__name__ = spec.name if autograd else spec.name + "_infer"
        op.__doc__ = spec.doc
        op.backend = backend
        return op


class _device_of:
    """Make the operand's device current for the launch (kernels go to its current stream)."""

    def __init__(self, t: Tensor):
        self.guard = torch.cuda.device(t.device) if t.is_cuda else None

    def __enter__(self):
        if self.guard is not None:
            self.guard.__enter__()

    def __exit__(self, *exc):
        if self.guard is not None:
            self.guard.__exit__(*exc)
        return False
