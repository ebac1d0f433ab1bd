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


f16 = DataType("f16", "f16", 16, torch.float16)
bf16 = DataType("bf16", "bf16", 16, torch.bfloat16)
f32 = DataType("f32", "f32", 32, torch.float32)
i32 = DataType("i32", "i32", 32, torch.int32)
i8 = DataType("i8", "i8", 8, torch.int8)
f8e8m0fnu = DataType("f8e8m0fnu", "f8E8M0FNU", 8, getattr(torch, "float8_e8m0fnu", None))
f4e2m1fn = DataType("f4e2m1fn", "f4E2M1FN", 4, getattr(torch, "float4_e2m1fn_x2", None))


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
