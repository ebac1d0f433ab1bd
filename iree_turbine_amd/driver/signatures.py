"""Operation signatures parsed from driver commands.

Two command families of the reference driver reach the dense-kernel path:
  * MIOpen-style GEMM: ``gemm`` (fp32) / ``gemmfp16`` with ``--a_w/-k --a_h/-m --b_w/-n --transA/-u --transB/-v
    --forw/-F`` (iree/turbine/kernel/boo/op_exports/gemm.py:103-214).  The flag names are MIOpen's and are
    kept with their quirk: ``--a_w`` is the number of ROWS of A (M) and ``--a_h`` the contraction size (K):
    a_shape = [a_w, a_h], b_shape = [a_h, b_w].
  * profiler-style ``aten::<op>`` commands with four list literals: input dims, input types, input strides,
    concrete inputs (iree/turbine/kernel/boo/op_exports/aten.py:21-198).
Anything else is reported as unparseable (``parse_command`` returns None), as in the reference registry.
"""

from __future__ import annotations

import argparse
import ast
import base64
from dataclasses import dataclass
from typing import Any, Iterable, Sequence

import torch


class OpSignature:
    """What the driver needs from an operation: a name, seeded inputs, and the eager torch form."""

    main_result_index = 0

    @property
    def func_name(self) -> str:
        raise NotImplementedError

    def get_sample_args(self, *, device=None, splat_value=None, seed=None) -> tuple[torch.Tensor, ...]:
        raise NotImplementedError

    def get_nn_module(self) -> torch.nn.Module:
        raise NotImplementedError


_GEMM_COMMANDS = {"gemm": torch.float32, "gemmfp16": torch.float16}
_ATEN_DTYPES = {"float": torch.float32, "double": torch.float64, "c10::Half": torch.float16, "c10::BFloat16": torch.bfloat16}


class _GemmForward(torch.nn.Module):
    def __init__(self, sig: "GEMMSignature"):
        super().__init__()
        self.sig = sig

    def forward(self, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        if self.sig.transpose_a:
            a = a.t()
        if self.sig.transpose_b:
            b = b.t()
        return torch.mm(a, b)


class GEMMSignature(OpSignature):
    """C[m, n] = A[m, k] . B[k, n]; with transpose_a / transpose_b the operand is STORED transposed
    ([k, m] / [n, k]) and transposed back inside the op (gemm.py:26-136).  Only the forward mode exists here."""

    def __init__(self, *, a_shape: Sequence[int], b_shape: Sequence[int], transpose_a: bool = False,
                 transpose_b: bool = False, dtype: torch.dtype = torch.float32):
        if len(a_shape) != 2 or len(b_shape) != 2:
            raise ValueError("expected shapes to be of rank 2")
        if a_shape[1] != b_shape[0]:
            raise ValueError(f"contraction sizes differ: a_shape={list(a_shape)} b_shape={list(b_shape)}")
        self.a_shape = list(a_shape)
        self.b_shape = list(b_shape)
        self.transpose_a = bool(transpose_a)
        self.transpose_b = bool(transpose_b)
        self.dtype = dtype

    @property
    def func_name(self) -> str:
        m, k = self.a_shape
        n = self.b_shape[1]
        items = ["gemm", str(self.dtype).removeprefix("torch."), "forward", f"{m}x{k}x{n}"]
        if self.transpose_a:
            items.append("transA")
        if self.transpose_b:
            items.append("transB")
        return "_".join(items)

    def get_sample_args(self, *, device=None, splat_value=None, seed=None):
        gen = torch.Generator(device=device)
        if seed is not None:
            gen = gen.manual_seed(seed)

        def get(shape):
            if splat_value is not None:
                return torch.ones(shape, dtype=self.dtype, device=device) * splat_value
            return torch.randn(shape, generator=gen, dtype=self.dtype, device=device)

        a_shape = self.a_shape[::-1] if self.transpose_a else self.a_shape
        b_shape = self.b_shape[::-1] if self.transpose_b else self.b_shape
        return get(a_shape), get(b_shape)

    def get_nn_module(self) -> torch.nn.Module:
        return _GemmForward(self)


@dataclass
class AtenSignature(OpSignature):
    """One ATen call as torch.profiler records it: per argument its dims, type string, strides and -- for
    non-tensor arguments -- the literal value (aten.py:21-99)."""

    name: str
    input_dims: Sequence[Sequence[int]]
    input_type: Sequence[str]
    input_strides: Sequence[Sequence[int]]
    concrete_inputs: Sequence[str]

    def __post_init__(self):
        n = len(self.input_dims)
        if not (len(self.input_type) == len(self.input_strides) == len(self.concrete_inputs) == n):
            raise ValueError("aten command: the four argument lists must have the same length")

    @property
    def torch_op(self):
        namespace, op = self.name.split("::")
        return getattr(getattr(torch.ops, namespace), op).default

    def get_concrete_args(self) -> Iterable[tuple[Any, object]]:
        """(schema argument, value) for every argument given as a literal."""
        schema_args = self.torch_op._schema.arguments
        if len(schema_args) < len(self.input_dims):
            raise ValueError(f"{self.name}: {len(self.input_dims)} arguments given, schema has {len(schema_args)}")
        for dims, typ, strides, concrete, schema in zip(self.input_dims, self.input_type, self.input_strides,
                                                        self.concrete_inputs, schema_args):
            if concrete == "":
                continue
            if len(dims) or len(strides):
                raise ValueError(f"{self.name}: concrete argument '{schema.name}' carries dims/strides")
            if typ not in ("Scalar", ""):
                raise ValueError(f"Unsupported concrete argument type: {typ}")
            yield schema, ast.literal_eval(concrete)

    def get_non_concrete_args(self):
        return [(d, t, s) for d, t, s, c in zip(self.input_dims, self.input_type, self.input_strides, self.concrete_inputs)
                if c == ""]

    def concrete_kwargs(self) -> dict[str, object]:
        return {schema.name: val for schema, val in self.get_concrete_args()}

    def get_sample_args(self, *, device=None, splat_value=None, seed=None):
        gen = torch.Generator(device=device)
        if seed is not None:
            gen = gen.manual_seed(seed)

        def get(dims, typ, strides):
            if typ not in _ATEN_DTYPES:
                raise ValueError(f"Unsupported input type: {typ}")
            dtype = _ATEN_DTYPES[typ]
            # non-contiguous strides may address beyond prod(dims) elements
            storage = sum((d - 1) * s for d, s in zip(dims, strides)) + 1 if dims else 1
            if splat_value is not None:
                val = torch.full((storage,), splat_value, dtype=dtype, device=device)
            else:
                val = torch.randn(storage, generator=gen, dtype=dtype, device=device)
            return torch.as_strided(val, list(dims), list(strides))

        return tuple(get(*a) for a in self.get_non_concrete_args())

    def get_nn_module(self) -> torch.nn.Module:
        func, kwargs = self.torch_op, self.concrete_kwargs()

        class FuncModule(torch.nn.Module):
            def forward(self, *args):
                return func(*args, **kwargs)

        return FuncModule()

    @property
    def func_name(self) -> str:
        text = self.name + str(self.input_dims) + str(self.input_type) + str(self.input_strides) + str(self.concrete_inputs)
        return base64.urlsafe_b64encode(text.encode()).decode()


class _QuietParser(argparse.ArgumentParser):
    def error(self, message):  # argparse would print usage and exit the process
        raise ValueError(message)


def _gemm_parser() -> argparse.ArgumentParser:
    p = _QuietParser(add_help=False)
    p.add_argument("command", choices=list(_GEMM_COMMANDS))
    p.add_argument("--a_w", "-k", type=int, default=256)
    p.add_argument("--a_h", "-m", type=int, default=256)
    p.add_argument("--b_w", "-n", type=int, default=256)
    p.add_argument("--transA", "-u", type=int, default=0)
    p.add_argument("--transB", "-v", type=int, default=0)
    p.add_argument("--forw", "-F", type=int, default=1)
    return p


def _aten_parser() -> argparse.ArgumentParser:
    p = _QuietParser(add_help=False)
    for name in ("name", "input_dims", "input_type", "input_strides", "concrete_inputs"):
        p.add_argument(name)
    return p


def parse_command(args: Sequence[str]) -> OpSignature | None:
    """Signature of a driver command (already split into words), or None if no parser accepts it."""
    if not args:
        return None
    try:
        if args[0] in _GEMM_COMMANDS:
            ns = _gemm_parser().parse_args(list(args))
            if min(ns.a_w, ns.a_h, ns.b_w) <= 0:
                raise ValueError("matrix sizes must be positive")
            if ns.forw != 1:
                raise ValueError(f"Unsupported mode {ns.forw}.")  # backward GEMMs are outside the kernel path
            return GEMMSignature(a_shape=[ns.a_w, ns.a_h], b_shape=[ns.a_h, ns.b_w], transpose_a=bool(ns.transA),
                                 transpose_b=bool(ns.transB), dtype=_GEMM_COMMANDS[ns.command])
        if args[0].startswith("aten::"):
            ns = _aten_parser().parse_args(list(args))
            sig = AtenSignature(name=ns.name, input_dims=ast.literal_eval(ns.input_dims),
                                input_type=ast.literal_eval(ns.input_type),
                                input_strides=ast.literal_eval(ns.input_strides),
                                concrete_inputs=ast.literal_eval(ns.concrete_inputs))
            sig.torch_op  # unknown ops fail here
            return sig
    except (ValueError, SyntaxError, AttributeError, TypeError):
        return None
    return None
