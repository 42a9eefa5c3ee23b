"""kvquant: ODM-KV mixed-precision KV-cache compression, MI355X build.

Exports what the reference's kvquant/__init__.py:10-17 exports.  The press classes pull in
``transformers`` and are imported on first use so that the kernels and the store can be used
without it.
"""
from kvquant.allocator import (
    scores_to_bits, ratio_scores_to_bits, optimal_scores_to_bits,
    calibrate_epsilon, effective_bits, DEFAULT_BIT_LEVELS,
)
from kvquant.scorer import BaseScorer, ExpectedAttentionScorer, RiskScorer
from kvquant.scorer import WindowRiskScorer          # not in the reference: per-query observation-window variant (opt-in)

_LAZY = {
    "TurboQuantPerTokenBackendPress": "kvquant.adaptive_backend_press",
    "TurboQuantBackendPress": "kvquant.backend_press",
    "TurboQuantPerTokenPress": "kvquant.press",
    "PackedCacheLayer": "kvquant.hf_cache",          # not in the reference: a cache layer without a dense copy
}


def __getattr__(name):
    if name in _LAZY:
        import importlib
        return getattr(importlib.import_module(_LAZY[name]), name)
    raise AttributeError(f"module 'kvquant' has no attribute {name!r}")


__all__ = [
    "scores_to_bits", "ratio_scores_to_bits", "optimal_scores_to_bits",
    "calibrate_epsilon", "effective_bits", "DEFAULT_BIT_LEVELS",
    "BaseScorer", "ExpectedAttentionScorer", "RiskScorer",
    "TurboQuantBackendPress",
    "TurboQuantPerTokenPress",
    "TurboQuantPerTokenBackendPress",
]
