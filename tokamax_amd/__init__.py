"""MI355X-native `ragged_dot` behind the tokamax operator API.

Public names follow tokamax/__init__.py:18-41 for this operator: `ragged_dot`,
`ragged_dot_general`, `RaggedDotGroupSizes`, `Op`, `BoundArguments`, `autotune`,
`AutotuningResult`, and the config options.
"""

from tokamax_amd import config
from tokamax_amd.autotuning.api import AutotuningResult, autotune, get_bound_args
from tokamax_amd.op import AUTO, BoundArguments, NullConfig, Op
from tokamax_amd.quantization import AsQArray, QArray, pack_int4
from tokamax_amd.gated_linear_unit.api import gated_linear_unit
from tokamax_amd.gated_linear_unit.hip import HipGatedLinearUnit
from tokamax_amd.ragged_gather import ragged_gather, ragged_gather_reduce, ragged_scatter
from tokamax_amd.ragged_dot.api import IMPLEMENTATIONS as RAGGED_DOT_IMPLEMENTATIONS
from tokamax_amd.ragged_dot.api import ragged_dot, ragged_dot_general
from tokamax_amd.ragged_dot.base import (
    DEFAULT_RAGGED_DOT_DIM_NUMS,
    RAGGED_CONTRACTING_DOT_DIM_NUMS,
    TRANS_RHS_RAGGED_DOT_DIM_NUMS,
    GroupSizes as RaggedDotGroupSizes,
    RaggedDotDimensionNumbers,
    generate_group_sizes,
)
from tokamax_amd.ragged_dot.hip import Config as HipRaggedDotConfig
from tokamax_amd.ragged_dot.hip import HipRaggedDot

__all__ = [
    "AUTO", "AsQArray", "AutotuningResult", "BoundArguments", "DEFAULT_RAGGED_DOT_DIM_NUMS", "HipGatedLinearUnit",
    "HipRaggedDot",
    "HipRaggedDotConfig", "NullConfig", "Op", "QArray", "RAGGED_CONTRACTING_DOT_DIM_NUMS", "pack_int4",
    "RAGGED_DOT_IMPLEMENTATIONS", "RaggedDotDimensionNumbers", "RaggedDotGroupSizes",
    "TRANS_RHS_RAGGED_DOT_DIM_NUMS", "autotune", "get_bound_args", "config", "gated_linear_unit", "generate_group_sizes", "ragged_dot",
    "ragged_dot_general", "ragged_gather", "ragged_gather_reduce", "ragged_scatter",
]
