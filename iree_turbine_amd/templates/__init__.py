"""Template getters: `get_*_kernel(shape, ...)` -> (kernel, hyperparams), then
`wave_compile(WaveCompileOptions(subs=hyperparams), kernel)` -> callable taking torch tensors with
outputs passed in.  The directory named by the task, iree/turbine/kernel/wave/templates, is not part
of the reference checkout; names, argument order and tensor layouts follow its callers' conventions
as far as they survive (hyperparameters as {sym: int}: tests/kernel/fused_attention_test.py:84-89)."""

from .attention_common import AttentionShape  # noqa: F401
from .gemm import get_gemm_kernel  # noqa: F401
from .mxfp4_gemm import get_mxfp4_gemm_kernel  # noqa: F401
from .paged_decode_attention import get_paged_decode_attention_kernels, paged_decode_attention_shape  # noqa: F401
from .vanilla_attention import get_vanilla_attention_kernel  # noqa: F401
