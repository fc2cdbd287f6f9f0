"""Default operator set (mamtorch/kernel/v4/__init__.py:1-5) plus the weight-layout additions."""
from .fullyconnected import fullyconnected, fullyconnected_wt
from .fullyconnected_fast import fullyconnected_fast, fullyconnected_fast_wt
from .selection_count import selection_count, COUNT_REFERENCE, COUNT_HITS, COUNT_FLAGS
from .module_ops import blend, apply_keep, im2col, col2im, fullyconnected_ranges
