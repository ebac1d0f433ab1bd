"""Symbols, dtypes and hyperparameter binding for the template getters.

`sym.NAME` is a sympy integer symbol exactly as in the reference
(iree/turbine/kernel/_support/indexing.py:45-60); hyperparameters are `{symbol: int}` dicts
(tests/kernel/fused_attention_test.py:84-89); binding a symbol twice with different values is an
error with the reference's wording (indexing.py:160-167, tests/kernel/indexing_test.py:85-92).
Dtype names and bit widths follow iree/turbine/kernel/_support/dtype.py:68-79,113-119.
"""

from __future__ import annotations

from dataclasses import dataclass

import sympy
import torch


class _IndexSymbolExpando:
    def __getattr__(self, n: str):
        return sympy.Symbol(n, integer=True, nonnegative=True)


sym = _IndexSymbolExpando()


@dataclass(frozen=True)
class DataType:
    name: str
    ir_type_asm: str
    bits: int
    torch_dtype: object = None

    def bitwidth(self) -> int:
        return self.bits

    def __repr__(self) -> str:
        return f"DataType({self.ir_type_asm})"

    def __str__(self) -> str:
        return self.name

    def is_int_asm(self) -> bool:
        return self.name in ("i1", "i4", "i8", "i16", "i32", "i64")

    def is_float_asm(self) -> bool:
        return self.name[0] == "f" or self.name == "bf16"

    def is_index_asm(self) -> bool:
        return self.name == "index"


def _t(name: str):
    return getattr(torch, name, None)


# Names, MLIR spellings and bit widths of iree/turbine/kernel/_support/dtype.py:68-79,99-120: `bool` is 1 bit,
# `index` 64, f4* 4, f8* 8, otherwise the number in the name.  (The reference's rule cannot parse "f6E2M3FN";
# here it is 6, the width of the element the MXFP6 kernels unpack.)
bf16 = DataType("bf16", "bf16", 16, torch.bfloat16)
bool = DataType("bool", "i1", 1, torch.bool)  # noqa: A001  (the reference's name)
i1 = bool
i4 = DataType("i4", "i4", 4, None)
i8 = DataType("i8", "i8", 8, torch.int8)
i16 = DataType("i16", "i16", 16, torch.int16)
i32 = DataType("i32", "i32", 32, torch.int32)
i64 = DataType("i64", "i64", 64, torch.int64)
f16 = DataType("f16", "f16", 16, torch.float16)
f32 = DataType("f32", "f32", 32, torch.float32)
f64 = DataType("f64", "f64", 64, torch.float64)
f8e5m2 = DataType("f8E5M2", "f8E5M2", 8, _t("float8_e5m2"))
f8e5m2fnuz = DataType("f8E5M2FNUZ", "f8E5M2FNUZ", 8, _t("float8_e5m2fnuz"))
f8e4m3fn = DataType("f8E4M3FN", "f8E4M3FN", 8, _t("float8_e4m3fn"))
f8e4m3fnuz = DataType("f8E4M3FNUZ", "f8E4M3FNUZ", 8, _t("float8_e4m3fnuz"))
f8e8m0fnu = DataType("f8E8M0FNU", "f8E8M0FNU", 8, _t("float8_e8m0fnu"))
f6e2m3fn = DataType("f6E2M3FN", "f6E2M3FN", 6, None)
f4e2m1fn = DataType("f4E2M1FN", "f4E2M1FN", 4, _t("float4_e2m1fn_x2"))
index = DataType("index", "index", 64, torch.int64)

ALL_DTYPES = (bf16, bool, i4, i8, i16, i32, i64, f16, f32, f64, f8e5m2, f8e5m2fnuz, f8e4m3fn, f8e4m3fnuz, f8e8m0fnu,
              f6e2m3fn, f4e2m1fn, index)


class SymbolBindings:
    """A `{symbol: int}` store with conflict detection."""

    def __init__(self, subs: dict | None = None):
        self.subs: dict[sympy.Symbol, int] = {}
        for k, v in (subs or {}).items():
            self.bind_constant(k, v)

    def bind_constant(self, s, value: int) -> None:
        s = s if isinstance(s, sympy.Basic) else sympy.Symbol(str(s), integer=True, nonnegative=True)
        existing = self.subs.get(s)
        if existing is not None and existing != value:
            raise ValueError(f"Attempt to bind symbol {s}={value} conflicts with previous {existing}")
        self.subs[s] = int(value)

    def get_static_value(self, expr):
        expr = sympy.sympify(expr).subs(self.subs)
        try:
            return int(expr)
        except TypeError:
            return None

    def __getitem__(self, s) -> int:
        v = self.get_static_value(s)
        if v is None:
            raise KeyError(f"{s} did not resolve to a known value")
        return v

    # -- tensors with symbolic shapes (iree/turbine/kernel/_support/indexing.py:146-266) --------------------
    def bind_shaped(self, instance, shaped_type: "ShapedType", dims) -> None:
        """Records that `instance` (any hashable handle) has the symbolic shape of `shaped_type` and the run-time
        sizes `dims`; an entry of `dims` may be None (to be inferred) or a symbol (dynamic)."""
        if not hasattr(self, "_shaped"):
            self._shaped = {}
        if instance in self._shaped:
            raise ValueError(f"Argument binding {instance} is already bound")
        if len(dims) != shaped_type.rank:
            raise ValueError(f"For {shaped_type} mismatched symbolic shape vs dim arity: {shaped_type.symbolic_shape} vs {dims}")
        self._shaped[instance] = (shaped_type, list(dims))

    def finalize(self) -> None:
        """Forward-only inference: a dimension spelled as a bare symbol binds that symbol to its run-time size;
        every dimension expression must then evaluate to the size it was given (or supply it where none was)."""
        shaped = getattr(self, "_shaped", {})
        for inst, (st, dims) in shaped.items():
            for expr, size in zip(st.symbolic_shape, dims):
                if isinstance(expr, sympy.Symbol) and isinstance(size, int):
                    prev = self.subs.get(expr)
                    if prev is not None and prev != size:
                        raise ValueError(f"For {inst} of {st} attempt to bind dim {expr}={size} conflicts with previous {prev}")
                    self.subs[expr] = size
        problems = []
        for inst, (st, dims) in shaped.items():
            for i, (expr, size) in enumerate(zip(st.symbolic_shape, dims)):
                known = sympy.sympify(expr).subs(self.subs).simplify()
                if not isinstance(known, sympy.Integer):
                    if size is None:
                        problems.append(f"  {inst} of {st}[{i}]={known} did not resolve to a known value")
                elif isinstance(size, int) and int(known) != size:
                    problems.append(f"  {inst} of {st}[{i}]={known} was initialized with a mismatched runtime value of {size}")
                else:
                    dims[i] = int(known)  # inferred, or a dynamic dim that turned out static
        if problems:
            raise ValueError("Indexing mismatches were encountered:\n" + "\n".join(problems))

    def eval_static_dim(self, instance, shaped_type: "ShapedType", pos: int):
        return self.get_static_value(shaped_type.symbolic_shape[pos])


class ShapedType:
    """`KernelBuffer[M, N].of(f32)`-style symbolic tensor types (reprs as pinned by the reference's
    tests/kernel/indexing_test.py:21-76)."""

    def __init__(self, kind: str, symbolic_shape: tuple, dtype: DataType = f32):
        self.kind, self.symbolic_shape, self.dtype = kind, tuple(symbolic_shape), dtype

    @property
    def rank(self) -> int:
        return len(self.symbolic_shape)

    def of(self, dtype: DataType) -> "ShapedType":
        return ShapedType(self.kind, self.symbolic_shape, dtype)

    def __repr__(self) -> str:
        return f"{self.kind}[{', '.join(str(d) for d in self.symbolic_shape)}].of({self.dtype.name})"


class _ShapedKind:
    def __init__(self, kind: str):
        self.kind = kind

    def __getitem__(self, shape) -> ShapedType:
        shape = shape if isinstance(shape, tuple) else (shape,)
        if shape and isinstance(shape[-1], DataType):
            return ShapedType(self.kind, shape[:-1], shape[-1])
        return ShapedType(self.kind, shape)


KernelBuffer = _ShapedKind("KernelBuffer")
InputBuffer = _ShapedKind("InputBuffer")
OutputBuffer = _ShapedKind("OutputBuffer")
