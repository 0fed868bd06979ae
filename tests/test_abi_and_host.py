"""CPU-only checks: the C-ABI library exports what include/deepep_hip.h declares, size
arithmetic matches the oracle, and the host module's argument checks raise the reference's
EPException text.  No kernel is launched here."""
import os
import re

import pytest

from oracle import deepep_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "deepep_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(deepep_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from deepep_efa_amd import _capi
    lib = _capi.load()
    declared = _declared_symbols()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/deepep_hip.h but not exported"
        assert name in _capi.PROTOTYPES, f"{name} has no ctypes prototype"
    assert sorted(_capi.PROTOTYPES) == declared


def test_abi_revision_is_the_same_everywhere():
    """The header's revision, what the built library reports and what the integration notes tell a
    maintainer to gate on are one number."""
    from deepep_efa_amd import _capi
    header = open(os.path.join(ROOT, "include", "deepep_hip.h")).read()
    revision = int(re.search(r"#define\s+DEEPEP_HIP_ABI_VERSION\s+(\d+)", header).group(1))
    assert _capi.load().deepep_abi_version() == revision
    notes = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    assert re.search(r"`deepep_abi_version\(\)` is (\d+)", notes).group(1) == str(revision)
    # every *_workspace_bytes function the header declares is named there too
    for name in _declared_symbols():
        if name.endswith("_workspace_bytes"):
            assert name in notes, f"INTEGRATION.md does not mention {name}"


@pytest.mark.parametrize("hidden", [128, 512, 2048, 7168])
def test_row_sizes_match_oracle(hidden):
    from deepep_efa_amd import _capi
    lib = _capi.load()
    for fmt in (O.ROW_BF16, O.ROW_FP8, O.ROW_FP8_POW2, O.ROW_FP8_UE8M0):
        assert lib.deepep_ll_row_data_bytes(hidden, fmt) == O.row_data_bytes(hidden, fmt)
        assert lib.deepep_ll_row_scale_bytes(hidden, fmt) == O.row_scale_bytes(hidden, fmt)
        assert lib.deepep_ll_row_stride(hidden, fmt) == O.row_stride(hidden, fmt)


@pytest.mark.parametrize("m,h,r,e", [(128, 7168, 32, 256), (1, 128, 2, 2), (8192, 7168, 64, 256), (256, 2048, 8, 288)])
def test_size_hint_matches_oracle(m, h, r, e):
    from deepep_efa_amd import _capi
    import deep_ep
    assert _capi.load().deepep_get_low_latency_rdma_size_hint(m, h, r, e) == O.get_low_latency_rdma_size_hint(m, h, r, e)
    assert deep_ep.Buffer.get_low_latency_rdma_size_hint(m, h, r, e) == O.get_low_latency_rdma_size_hint(m, h, r, e)


def test_host_argument_checks_without_a_gpu():
    from deepep_efa_amd import _capi
    lib = _capi.load()
    # shape checks run before anything touches the device
    rc = lib.deepep_per_token_cast_to_fp8(None, 4, 100, 1, None, None, None)
    assert rc != 0
    assert lib.deepep_last_error().decode() == "Failed: Assertion error cast.hip:%d 'num_rows >= 0 && num_cols > 0 && num_cols %% 128 == 0'" % \
        int(re.search(r"cast\.hip:(\d+)", lib.deepep_last_error().decode()).group(1))
    rc = lib.deepep_ll_combine_recv(None, None, None, None, 4, 7168, 0, 256, 128, 0, None, None)
    assert rc != 0 and "num_topk > 0" in lib.deepep_last_error().decode()
    rc = lib.deepep_moe_routing_sort(None, -1, 8, None, None, None, None, None, 0, None)
    assert rc != 0 and lib.deepep_last_error().decode().startswith("Failed: Assertion error layout.hip:")
    with pytest.raises(_capi.DeepEPError):
        _capi.check(rc)


def test_config_follows_reference_rules():
    import deep_ep
    cfg = deep_ep.Config(20, 6, 256, 6, 250)
    assert cfg.num_max_rdma_chunked_recv_tokens == 252  # rounded up to a multiple of the send chunk
    assert cfg.num_sms == 20 and cfg.num_max_nvl_chunked_send_tokens == 6
    # csrc/config.hpp:52-74 by hand for 8 ranks, bf16 hidden 7168: see the arithmetic in the test body
    ch, nvl, recv, hb = 10, 8, 256, 14336
    want = ch * nvl * 5 * 4 + ch * nvl * recv * (hb + 8 + 128 * 8 + 128 * 4 + 128 * 4)
    assert cfg.get_nvl_buffer_size_hint(hb, 8) == (want + 127) // 128 * 128
    assert cfg.get_rdma_buffer_size_hint(hb, 8) == 0
    with pytest.raises(RuntimeError, match=r"Failed: Assertion error deep_ep_cpp.cpp:\d+ 'nvl_send < nvl_recv'"):
        deep_ep.Config(20, 300, 256, 6, 128)
    for n in (2, 8, 32, 160):
        assert deep_ep.Buffer.get_dispatch_config(n).num_sms == deep_ep.Buffer.num_sms
        assert deep_ep.Buffer.get_combine_config(n).num_max_rdma_chunked_recv_tokens >= 128
    assert str(deep_ep.topk_idx_t) == "torch.int64"


def test_buffer_needs_a_world():
    import deep_ep
    with pytest.raises(ValueError, match="Either 'group' or 'comm' must be provided"):
        deep_ep.Buffer(None)


def test_c_abi_library_needs_no_torch():
    """The boundary is plain C over device pointers: the library links the HIP runtime and the C/C++
    runtime, nothing from PyTorch, and exports no C++-mangled entry point a caller would have to use."""
    import subprocess
    so = os.path.join(ROOT, "deepep_efa_amd", "libdeepep_hip.so")
    needed = subprocess.run(["readelf", "-d", so], capture_output=True, text=True, check=True).stdout
    libs = re.findall(r"Shared library: \[([^\]]+)\]", needed)
    assert any(lib.startswith("libamdhip64") for lib in libs)
    assert not [lib for lib in libs if "torch" in lib or "c10" in lib or "python" in lib], libs
    header = open(os.path.join(ROOT, "include", "deepep_hip.h")).read()
    code = re.sub(r"/\*.*?\*/", "", header, flags=re.S)  # declarations only, comments cite the reference
    assert 'extern "C"' in code and "torch" not in code and "at::" not in code and "#include <hip" not in code
