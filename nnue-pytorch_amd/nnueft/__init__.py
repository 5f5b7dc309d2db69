"""MI355X-native sparse feature transformer of nnue-pytorch.

The public names are those of the reference's model/modules/feature_transformer/__init__.py:1-11
(minus ComposedFeatureTransformer, which is the unchanged caller of `double_feature_transform`).
"""
from .double_ft_functions import double_feature_transform
from .fused_ft_functions import FusedDoubleFtFunction
from .sparse_linear_functions import (SparseLinearFunction, get_backward_mode, get_sort_placement,
                                      set_backward_mode, set_sort_placement)

__all__ = [
    "FusedDoubleFtFunction",
    "SparseLinearFunction",
    "double_feature_transform",
    "get_backward_mode",
    "set_backward_mode",
    "get_sort_placement",
    "set_sort_placement",
]
