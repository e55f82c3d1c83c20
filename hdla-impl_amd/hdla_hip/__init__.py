"""hdla_hip: MI355X-native operators for HDLA's rank-2 DPLR delta-rule linear attention.

Exports the two operators of the reference package (HRDPLR/__init__.py:1-12) with the same signatures, and the
operator as the HDLA layer calls it (a, b given by beta, k, log_f: HRDPLR/hdla_custom.py:19-43,290-309), the fused
normalisation the layer applies around it (HRDPLR/normalizations/normalize/normalize/normalize_triton.py), the layer's
elementwise stage between projections and operator, and the layer itself (HRDPLR/hdla_custom.py:45-350).
"""
from .chunk import ChunkDPLRDeltaRuleFunction, chunk_hrdplr_delta_rule
from .hdla import ChunkHDLAFunction, chunk_hdla_delta_rule, fused_recurrent_hdla_delta_rule, parameterize_a_b
from .layer import HDLA_Custom, RecurrentCache, get_activation_fn
from . import layer_pre          # submodule: layer_pre.layer_pre, .logsigmoid, .low_rank_up
from .normalize import (GroupRMSNorm, GroupRMSNormFusedGate, NormalizeFunction, RMSNorm, RMSNormFusedGate, SRMSNorm,
                        get_norm_fn, l2_norm, normalize_fn)
from .recurrent import FusedRecurrentDPLRDeltaRuleFunction, fused_recurrent_dplr_delta_rule

__all__ = [
    "fused_recurrent_dplr_delta_rule",
    "chunk_hrdplr_delta_rule",
    "ChunkDPLRDeltaRuleFunction",
    "FusedRecurrentDPLRDeltaRuleFunction",
    "chunk_hdla_delta_rule",
    "fused_recurrent_hdla_delta_rule",
    "parameterize_a_b",
    "ChunkHDLAFunction",
    "normalize_fn",
    "l2_norm",
    "get_norm_fn",
    "RMSNorm",
    "RMSNormFusedGate",
    "SRMSNorm",
    "GroupRMSNorm",
    "GroupRMSNormFusedGate",
    "NormalizeFunction",
    "HDLA_Custom",
    "RecurrentCache",
    "get_activation_fn",
    "layer_pre",
]
