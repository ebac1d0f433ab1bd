"""Callable kernel objects.

`Launchable` follows the calling rules of the reference's runtime launchable
(iree/turbine/runtime/launch.py:203-272): tensor arguments are made contiguous, all tensors must
live on one device, a call needs at least one tensor (or an explicit `device=`), and outputs are
passed in and written in place, the way DSL kernels take their `OutputBuffer` arguments
(tests/kernel/fused_attention_test.py:26-31,77-90).  Where the reference resolves a compiled VM
function per device, this one holds a pre-built HIP kernel and its bound hyperparameters.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Optional, Sequence

import torch
from torch import Tensor

from .lang import SymbolBindings


class Launchable:
    def __init__(self, name: str, entry: Callable[..., Any], *, num_outputs: int, hyperparams: dict | None = None,
                 description: str = ""):
        self.name = name
        self._entry = entry
        self.num_outputs = num_outputs
        self.hyperparams = dict(hyperparams or {})
        self.description = description

    def __repr__(self) -> str:
        return f"Launchable<{self.name}>"

    def bind(self, subs: dict) -> "Launchable":
        """Returns a copy with extra / overriding hyperparameters; conflicting re-binds raise."""
        merged = SymbolBindings(self.hyperparams)
        for k, v in subs.items():
            merged.bind_constant(k, v)
        return Launchable(self.name, self._entry, num_outputs=self.num_outputs, hyperparams=merged.subs,
                          description=self.description)

    def __call__(self, *args, device: Optional[torch.device] = None, outputs: Sequence[Tensor] = ()):
        all_args = list(args) + list(outputs)
        fixed = []
        for a in all_args:
            if isinstance(a, Tensor):
                if device is None:
                    device = a.device
                elif a.device != torch.device(device):
                    raise RuntimeError(f"Cannot launch with tensors from multiple devices: {a.device} vs {device}")
                fixed.append(a)
            elif isinstance(a, (int, float, bool)) or a is None:
                fixed.append(a)
            else:
                raise ValueError(f"Unsupported argument type: {type(a)}")
        if device is None:
            raise RuntimeError(f"Cannot invoke Launchable {self} without any Tensor args or an explicit device=")
        n_in = len(fixed) - self.num_outputs
        for o in fixed[n_in:]:
            if not (isinstance(o, Tensor) and o.is_contiguous()):
                raise ValueError("Outputs must be contiguous tensors")
        ins = [a.contiguous() if isinstance(a, Tensor) else a for a in fixed[:n_in]]
        self._entry(self.hyperparams, *ins, *fixed[n_in:])
        results = fixed[n_in:]
        if len(results) == 1:
            return results[0]
        return None if not results else results


@dataclass
class WaveCompileOptions:
    """The subset of the compile options that has a meaning for pre-built kernels: `subs` binds the
    hyperparameter symbols a getter returned (optionally overridden by the caller)."""

    subs: dict = field(default_factory=dict)
    canonicalize: bool = True
    run_bench: bool = False
    schedule: Any = None
    use_scheduling_barriers: bool = False
    dynamic_symbols: Sequence = ()


def wave_compile(options: WaveCompileOptions, kernel: Launchable) -> Launchable:
    """Binds `options.subs` into `kernel` and returns the callable.  Nothing is compiled: the
    kernels are built ahead of time into libturbine_mi355.so."""
    if not isinstance(kernel, Launchable):
        raise TypeError(f"wave_compile expects a kernel returned by a template getter, got {type(kernel)}")
    return kernel.bind(options.subs)
