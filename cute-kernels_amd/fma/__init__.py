"""MI355X-native implementation of the MoE-layer hot path of cute-kernels (`fma`): same public names and call
signatures for the ops and the module on that path, computed by hand-written HIP kernels (gfx950) behind a C ABI."""

from .kernel_backend import KernelBackend
from .math import ceil_divide, divide_if_divisible
from .modules import MoE
from .ops import continuous_count, fused_residual_add_rmsnorm, grouped_gemm, swiglu, swiglu_packed
from .utils import ensure_contiguous, set_seed
