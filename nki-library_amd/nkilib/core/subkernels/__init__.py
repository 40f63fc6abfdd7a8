from .find_nonzero_indices import find_nonzero_indices
from .indexed_flatten import indexed_flatten

__all__ = ["find_nonzero_indices", "indexed_flatten"]
