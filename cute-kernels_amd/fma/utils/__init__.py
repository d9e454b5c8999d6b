from .contiguous import ensure_contiguous
from .random import set_seed
