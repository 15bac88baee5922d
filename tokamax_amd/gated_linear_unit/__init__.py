"""`gated_linear_unit`: the dense neighbour of the gate-up fused ragged dot (one group)."""

from tokamax_amd.gated_linear_unit.api import IMPLEMENTATIONS, gated_linear_unit
from tokamax_amd.gated_linear_unit.hip import HipGatedLinearUnit

__all__ = ["IMPLEMENTATIONS", "HipGatedLinearUnit", "gated_linear_unit"]
