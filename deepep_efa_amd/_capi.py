"""ctypes view of the C ABI declared in include/deepep_hip.h.

The library must already be built (``python deepep_efa_amd/build.py`` or
``__graft_entry__.build()``); a missing library is an error, never a fallback.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libdeepep_hip.so")

_c = ctypes
_VP, _I, _I64, _SZ, _U32 = _c.c_void_p, _c.c_int, _c.c_int64, _c.c_size_t, _c.c_uint32

# name -> (restype, argtypes); mirrors include/deepep_hip.h one to one.
PROTOTYPES = {
    "deepep_last_error": (_c.c_char_p, []),
    "deepep_abi_version": (_I, []),
    "deepep_ll_row_data_bytes": (_SZ, [_I, _I]),
    "deepep_ll_row_scale_bytes": (_SZ, [_I, _I]),
    "deepep_ll_row_stride": (_SZ, [_I, _I]),
    "deepep_ll_row_payload_bytes": (_SZ, [_I, _I]),
    "deepep_get_low_latency_rdma_size_hint": (_SZ, [_I, _I, _I, _I]),
    "deepep_layout_workspace_bytes": (_SZ, [_I, _I, _I]),
    "deepep_get_dispatch_layout": (_I, [_VP, _I, _I, _I, _I, _VP, _VP, _VP, _VP, _VP, _SZ, _VP]),
    "deepep_routing_sort_workspace_bytes": (_SZ, [_I, _I]),
    "deepep_moe_routing_sort": (_I, [_VP, _I, _I, _VP, _VP, _VP, _VP, _VP, _SZ, _VP]),
    "deepep_channel_prefix_matrix": (_I, [_VP, _I, _I, _I, _VP, _VP]),
    "deepep_pack_rows": (_I, [_VP, _VP, _VP, _VP, _I64, _I, _I, _I, _VP, _VP, _VP]),
    "deepep_per_token_cast_to_fp8": (_I, [_VP, _I, _I, _I, _VP, _VP, _VP]),
    "deepep_ll_dispatch_workspace_bytes": (_SZ, [_I, _I, _I]),
    "deepep_ll_dispatch_send": (_I, [_VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _VP, _VP, _VP, _VP, _VP, _VP, _SZ, _VP]),
    "deepep_ll_dispatch_send_static": (_I, [_VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _VP, _VP, _VP, _VP, _VP, _VP]),
    "deepep_ll_segment_workspace_bytes": (_SZ, [_I, _I]),
    "deepep_ll_dispatch_recv": (_I, [_VP, _VP, _I, _I, _I, _I, _I, _VP, _VP, _VP, _VP, _VP, _VP, _I64, _VP, _SZ, _VP]),
    "deepep_ll_combine_send": (_I, [_VP, _VP, _I, _I, _I, _I, _I, _VP, _VP, _I64, _VP, _SZ, _VP]),
    "deepep_ll_combine_recv": (_I, [_VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _VP, _VP]),
    "deepep_ll_dispatch_is_single_launch": (_I, [_I, _I, _I, _I, _I64]),
    "deepep_ll_dispatch": (_I, [_VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP,
                                _VP, _I64, _VP, _SZ, _VP, _SZ, _VP]),
    "deepep_ll_combine": (_I, [_VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _VP, _VP, _VP, _I64, _VP, _SZ,
                               _VP]),
    "deepep_topk_remap": (_I, [_VP, _VP, _VP, _VP, _I, _I, _I, _I, _I64, _VP, _VP, _VP]),
    "deepep_build_recv_src_meta": (_I, [_VP, _I, _I, _I64, _VP, _VP]),
    "deepep_ll_exchange_metadata": (_I, [_VP, _I, _I, _I, _I, _I64] + [_VP] * 11),
    "deepep_ll_by_source_workspace_bytes": (_SZ, [_I, _I64]),
    "deepep_ll_dispatch_recv_by_source": (_I, [_VP, _I64, _VP, _VP, _VP, _I64, _I, _I, _I, _I, _I, _VP, _VP, _VP, _VP,
                                               _VP, _VP, _VP, _VP, _I64, _VP, _SZ, _VP]),
    "deepep_ll_dispatch_recv_by_source_ordered": (_I, [_VP, _I64, _VP, _I, _I, _I, _I, _I, _I, _VP, _VP, _VP, _VP, _VP,
                                                       _VP, _VP, _VP, _I64, _I64, _VP, _SZ, _VP]),
    "deepep_ll_dispatch_send_by_dest": (_I, [_VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _VP, _I64, _VP, _VP, _VP, _VP,
                                             _VP, _VP, _SZ, _VP]),
    "deepep_ll_combine_send_by_dest": (_I, [_VP, _VP, _VP, _VP, _VP, _VP, _I64, _I, _I, _I, _I, _VP, _VP, _VP, _VP,
                                            _VP, _I64, _VP]),
    "deepep_ll_combine_recv_flat": (_I, [_VP, _I64, _I64, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _VP, _VP]),
    "deepep_combine_reduce_workspace_bytes": (_SZ, [_I, _I]),
    "deepep_combine_reduce": (_I, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I64, _VP, _VP, _VP, _VP, _SZ,
                                   _VP]),
    "deepep_synth_topk_idx": (_I, [_VP, _VP, _I, _I, _I, _I, _U32, _VP, _VP]),
    "deepep_synth_bf16_rows": (_I, [_VP, _I64, _I, _I64, _VP, _U32, _U32, _I, _VP]),
    "deepep_loopback_dispatch_from_peers": (_I, [_VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _I, _VP, _VP, _VP, _SZ,
                                               _VP]),
    "deepep_loopback_combine_from_peers": (_I, [_VP, _VP, _I, _I, _I, _I, _I, _I, _I, _U32, _VP, _VP]),
}

_lib = None


class DeepEPError(RuntimeError):
    """A failed C-ABI call; the text is the library's EPException-style message."""


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: build it with `python deepep_efa_amd/build.py`")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise DeepEPError(load().deepep_last_error().decode())


def ptr(t):
    """Device (or host) address of a torch tensor, or NULL for None."""
    return None if t is None else ctypes.c_void_p(t.data_ptr())
