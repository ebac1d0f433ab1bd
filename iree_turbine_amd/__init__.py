"""MI355X-native dense kernels (fp16 NT GEMM, flash-attention prefill, paged GQA decode attention,
block-scaled MXFP4 GEMM) behind iree-turbine's operator surface.

Importing the package registers `torch.ops.mi355.*`.  The kernels live in
csrc/libturbine_mi355.so (hand-written HIP for gfx950); there is no other implementation.
"""

from . import _lib, lang, launch, launchable, op_reg, ops, templates  # noqa: F401
from .launchable import Launchable, WaveCompileOptions, wave_compile  # noqa: F401
from .ops import *  # noqa: F401,F403

__version__ = "0.1.0"
