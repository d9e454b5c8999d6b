from .continuous_count import continuous_count
from .fused_residual_add_rmsnorm import fused_residual_add_rmsnorm
from .grouped_gemm import grouped_gemm
from .swiglu import swiglu, swiglu_packed
