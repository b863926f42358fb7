"""Symmetric power retention on MI355X (gfx950): hand-written HIP kernels behind the reference's API.

    from retention_integration_amd import power_retention, power_retention_inference

Same signatures and tensor layouts as the reference package (ref: retention/__init__.py:1-13): Q, K, V
[b, t, h, d]; log_G [b, t, h]; state [b, h, D, d]; sum_of_keys [b, h, D].  The HIP library must have been
built (``python retention_integration_amd/csrc/build.py``); there is no fallback implementation.

``power_retention`` runs the chunked branch as one fused autograd node; ``power_retention_composed`` is the
same function assembled from the four operators through the reference's plugin boundary.  Likewise
``power_retention_inference`` fuses the single-token step; ``power_retention_inference_composed`` is the
maker-assembled form.
"""
from functools import partial

from .cache import RetentionCache
from .fused import chunked_power_retention
from .inference import make_fused_inference
from .maker import make_power_retention, make_power_retention_inference
from .ops import attention, discumsum, expanded_dim, gate_cumsum_or_none, query_state, update_state

power_retention_composed = make_power_retention(update_state, query_state, partial(discumsum, keep_last=False),
                                                attention, scan_keeps_last=False, full_scan_impl=discumsum)
power_retention = make_power_retention(update_state, query_state, partial(discumsum, keep_last=False), attention,
                                       scan_keeps_last=False, chunked_impl=chunked_power_retention,
                                       full_scan_impl=discumsum, gate_cumsum_impl=gate_cumsum_or_none)
power_retention_inference_composed = make_power_retention_inference(update_state, query_state, attention,
                                                                    fused_normalizer=False)
power_retention_inference = make_fused_inference(power_retention_inference_composed)

__all__ = [
    "power_retention", "power_retention_composed", "power_retention_inference",
    "power_retention_inference_composed", "make_power_retention",
    "make_power_retention_inference", "attention", "update_state", "discumsum", "query_state", "expanded_dim",
    "RetentionCache",
]
