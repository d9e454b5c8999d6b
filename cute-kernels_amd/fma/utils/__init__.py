from .contiguous import ensure_contiguous
from .misc import get_num_elements_and_hidden_size, set_seed
