"""Operator boundary: a `CustomOp` registered with `torch.library`, mirroring the reference's
interface (iree/turbine/runtime/op_reg/base.py:97-247) for ops whose device implementation is
a pre-built HIP kernel instead of JIT-compiled IR.

Same moving parts, same names:
  * `CustomOp.register` class decorator -> replaces the class by the callable `torch.ops.<ns>.<op>`;
  * `signature` (schema string), `select(ksel)` (shape/dtype transfer function; the Meta kernel
    is derived from it, base.py:1041-1051), `eager_execute(*args)` (the device implementation;
    in the reference returning anything but NotImplemented short-circuits compilation,
    base.py:1061-1064);
  * `KernelSelection` with `arg_tensor / arg_optional_tensor / arg_int / attr_* / return_new_tensor`
    and a `spec_key` of the form ``ns.DEF::name::variant(tensor[rank:dtype]<dims>,...)->(...)``.
There is no IR generator here: `generate` raises, and an `eager_execute` that returns
NotImplemented is an error.  Implementations are registered for the CUDA (HIP) dispatch key
only -- calling an op with CPU tensors fails in the dispatcher; nothing falls back.
"""

from __future__ import annotations

import functools
import threading
from abc import ABC, abstractmethod
from typing import Any, Callable, Optional, Sequence, Type, Union

import torch
from torch import Tensor

_CONFIG_LOCK = threading.Lock()

DEFINED_OP_NAMES: set[tuple[str, str]] = set()
ALL_CUSTOM_OP_REGS: dict[str, "CustomOp"] = {}


def def_library(ns: str) -> torch.library.Library:
    return torch.library.Library(ns, "DEF")


MI355_LIBRARY = def_library("mi355")


class ArgDescriptor:
    __slots__ = ["v", "spec_value"]

    def __init__(self, v, spec_value=None):
        self.v = v
        self.spec_value = spec_value

    @property
    def spec_key(self) -> str:
        return f"attr({self.spec_value})" if self.spec_value is not None else "arg"


class TensorArg(ArgDescriptor):
    """A tensor argument or result: specialised on rank and dtype, and on the dims marked so."""

    __slots__ = ["t", "spec_dims"]

    def __init__(self, t: Tensor):
        super().__init__(t)
        self.t = t
        self.spec_dims: list[Optional[int]] = [None] * t.dim()

    def specialize_all_dims(self):
        self.spec_dims = list(self.t.shape)

    def specialize_dims(self, *indices: int):
        for i in indices:
            self.spec_dims[i] = self.t.size(i)

    def generate_meta(self) -> Tensor:
        return self.t.to(device="meta") if self.t.device.type != "meta" else self.t

    @property
    def spec_key(self) -> str:
        dims = ", ".join("?" if d is None else str(d) for d in self.spec_dims)
        return f"tensor[{self.t.dim()}:{self.t.dtype}]<[{dims}]>"


class KernelSelection:
    """What `CustomOp.select` fills in for one call: checked arguments and result descriptors."""

    def __init__(self, op: "CustomOp", args: Sequence[Any]):
        self.op = op
        self.args = list(args)
        self.arg_descs: list[Optional[ArgDescriptor]] = [None] * len(args)
        self.result_descs: list[TensorArg] = []
        self.variant = "default"

    def arg_tensor(self, arg: int) -> TensorArg:
        t = self.args[arg]
        assert isinstance(t, Tensor), f"Argument type mismatch from Torch for {arg}: Expected tensor, got {type(t)}"
        desc = TensorArg(t)
        self.arg_descs[arg] = desc
        return desc

    def arg_optional_tensor(self, arg: int) -> Optional[TensorArg]:
        if self.args[arg] is None:
            self.arg_descs[arg] = ArgDescriptor(None, "none")
            return None
        return self.arg_tensor(arg)

    def _scalar(self, arg: int, ty, specialise: bool) -> ArgDescriptor:
        v = self.args[arg]
        if ty is float and isinstance(v, int) and not isinstance(v, bool):
            v = float(v)
        assert isinstance(v, ty), f"Argument type mismatch from Torch for {arg}: Expected {ty.__name__}, got {type(v)}"
        desc = ArgDescriptor(v, v if specialise else None)
        self.arg_descs[arg] = desc
        return desc

    def arg_int(self, arg: int) -> ArgDescriptor:
        return self._scalar(arg, int, False)

    def attr_int(self, arg: int) -> ArgDescriptor:
        return self._scalar(arg, int, True)

    def attr_float(self, arg: int) -> ArgDescriptor:
        return self._scalar(arg, float, True)

    def attr_str(self, arg: int) -> ArgDescriptor:
        return self._scalar(arg, str, True)

    def attr_bool(self, arg: int) -> ArgDescriptor:
        return self._scalar(arg, bool, True)

    def return_tensor(self, t: Tensor) -> TensorArg:
        desc = TensorArg(t)
        self.result_descs.append(desc)
        return desc

    def return_new_tensor(self, size: Sequence[int], dtype: torch.dtype) -> TensorArg:
        return self.return_tensor(torch.empty(list(size), dtype=dtype, device="meta"))

    def generate_meta_returns(self):
        results = [d.generate_meta() for d in self.result_descs]
        if len(results) == 1:
            return results[0]
        return None if not results else tuple(results)

    @property
    def spec_key(self) -> str:
        arg_keys = ",".join(d.spec_key if d is not None else "None" for d in self.arg_descs)
        ret_keys = ",".join(d.spec_key for d in self.result_descs)
        return f"{self.op.cache_key_base}::{self.variant}({arg_keys})->({ret_keys})"


class CustomOp(ABC):
    """Subclass, decorate with `@CustomOp.register`, and the class name becomes the op callable."""

    @staticmethod
    def register(op_class: Optional[Type["CustomOp"]] = None, *, library: torch.library.Library = MI355_LIBRARY,
                 dispatch_key: Union[str, Sequence[str], None] = None, register_meta: bool = True,
                 register_impl: bool = True) -> Callable:
        if not op_class:
            return functools.partial(CustomOp.register, library=library, dispatch_key=dispatch_key,
                                     register_meta=register_meta, register_impl=register_impl)
        instance = op_class(library=library, dispatch_key=dispatch_key, register_meta=register_meta,
                            register_impl=register_impl)
        return instance.op

    def __init__(self, *, library, dispatch_key, register_meta: bool, register_impl: bool):
        self.name = name = _define_signature_in_library(library, self.signature)
        self.library = library
        self.cache_key_base = f"{library.ns}.{library.kind}::{name}"
        self.op = getattr(getattr(torch.ops, library.ns), name)
        if register_meta:
            library.impl(name, _get_meta_impl(self), "Meta")
        if register_impl:
            keys = ["CUDA"] if dispatch_key is None else ([dispatch_key] if isinstance(dispatch_key, str) else dispatch_key)
            for k in keys:
                library.impl(name, _create_impl_trampoline(self), k)
        ALL_CUSTOM_OP_REGS[f"{library.ns}.{name}"] = self

    @property
    @abstractmethod
    def signature(self) -> str: ...

    @abstractmethod
    def select(self, sel: KernelSelection): ...

    def eager_execute(self, *args):
        return NotImplemented

    def generate(self, ksel: KernelSelection, kb: Any):
        raise NotImplementedError(f"{self.name}: kernels are pre-built HIP; there is no IR generator")


def _define_signature_in_library(lib: torch.library.Library, signature: str) -> str:
    name = signature.split("(", 1)[0].strip()
    with _CONFIG_LOCK:
        key = (lib.ns, name)
        if key in DEFINED_OP_NAMES:
            raise RuntimeError(f"Duplicate turbine custom op registration: library={lib.ns}, name={name}")
        lib.define(signature)
        DEFINED_OP_NAMES.add(key)
    return name


def _get_meta_impl(op: CustomOp):
    def meta(*args):
        sel = KernelSelection(op, args)
        op.select(sel)
        return sel.generate_meta_returns()

    return meta


def _create_impl_trampoline(op: CustomOp):
    def handler(*args):
        sel = KernelSelection(op, args)
        op.select(sel)  # validates shapes / dtypes before anything is launched
        result = op.eager_execute(*args)
        if result is NotImplemented:
            raise NotImplementedError(f"{op.name}: no device implementation (eager_execute returned NotImplemented)")
        return result

    return handler
