"""MI355X-native MoE token dispatch/combine hot path behind the deep_ep.Buffer API.

Importing the package loads the HIP library and the host module; both must have
been built (`python deepep_efa_amd/build.py`).  There is no CPU fallback.
"""
import torch  # noqa: F401  (its HIP runtime must be the one loaded in this process)

from . import _capi as _capi_module

_capi_module.load()

from .deep_ep_cpp import Config, topk_idx_t  # noqa: E402
from .utils import EventOverlap  # noqa: E402
from .buffer import Buffer  # noqa: E402

__all__ = ["Buffer", "Config", "EventOverlap", "topk_idx_t"]
