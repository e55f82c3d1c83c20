"""hdla_hip: MI355X-native operators for HDLA's rank-2 DPLR delta-rule linear attention.

Exports the two operators of the reference package (HRDPLR/__init__.py:1-12) with the same signatures.
"""
from .chunk import ChunkDPLRDeltaRuleFunction, chunk_hrdplr_delta_rule
from .recurrent import FusedRecurrentDPLRDeltaRuleFunction, fused_recurrent_dplr_delta_rule

__all__ = [
    "fused_recurrent_dplr_delta_rule",
    "chunk_hrdplr_delta_rule",
    "ChunkDPLRDeltaRuleFunction",
    "FusedRecurrentDPLRDeltaRuleFunction",
]
