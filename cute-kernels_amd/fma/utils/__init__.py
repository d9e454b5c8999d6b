from .contiguous import ensure_contiguous
from .random import set_seed
from .tensor import get_num_elements_and_hidden_size
