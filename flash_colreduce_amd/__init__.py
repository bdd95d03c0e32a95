"""MI355X-native attention column reduction (same package surface as the reference:
flash_colreduce/__init__.py:1-4)."""
from .flash import flash_colreduce, flash_colreduce_multi, row_lse2, topk_keep_mask
from .naive import naive_colreduce

__version__ = "0.1.0"
__all__ = ["flash_colreduce", "flash_colreduce_multi", "naive_colreduce", "row_lse2", "topk_keep_mask",
           "__version__"]
