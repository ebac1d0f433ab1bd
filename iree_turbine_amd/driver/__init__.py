"""MIOpen-driver-style command line for the MI355X kernels: the same commands, CSV schema and numerics
verdict as the reference's `iree-boo-driver` (iree/turbine/kernel/boo/driver/driver.py), with this
library's kernels as the default backend."""

from .signatures import AtenSignature, GEMMSignature, OpSignature, parse_command  # noqa: F401
