"""`import deep_ep` — the reference's package name, served by the MI355X build.

Exports what deep_ep/__init__.py of the reference exports: Buffer, EventOverlap, Config, topk_idx_t.
"""
from deepep_efa_amd import Buffer, Config, EventOverlap, topk_idx_t  # noqa: F401
