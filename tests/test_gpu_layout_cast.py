"""GPU parity: route counting / layout, routing sort, channel prefix, pack and the FP8 cast.

Every call goes through the C ABI (ctypes on libdeepep_hip.so); the expected
values come from the CPU oracle.  Integer and byte outputs must be bit-exact.
"""
import numpy as np
import pytest
import torch

from oracle import deepep_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def capi():
    from deepep_efa_amd import _capi
    _capi.load()
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return _capi


def stream():
    return torch.cuda.current_stream().cuda_stream


def _topk(t, k, e, seed, drop=0):
    g = torch.Generator().manual_seed(seed)
    if t == 0:
        return torch.zeros((0, k), dtype=torch.int64)
    topk = torch.argsort(torch.rand((t, e), generator=g), dim=1)[:, :k].contiguous()
    for _ in range(drop):
        topk[int(torch.randint(0, t, (1,), generator=g)), int(torch.randint(0, k, (1,), generator=g))] = -1
    return topk


def run_layout(capi, topk, num_experts, num_ranks):
    lib = capi.load()
    t, k = topk.shape
    dev = topk.cuda()
    per_rank = torch.full((num_ranks,), -7, dtype=torch.int32, device="cuda")
    per_expert = torch.full((num_experts,), -7, dtype=torch.int32, device="cuda")
    want_rdma = num_ranks > 8 and num_ranks % 8 == 0
    per_rdma = torch.full((num_ranks // 8,), -7, dtype=torch.int32, device="cuda") if want_rdma else None
    is_in = torch.zeros((t, num_ranks), dtype=torch.bool, device="cuda")
    ws = torch.empty(max(16, lib.deepep_layout_workspace_bytes(t, num_ranks, num_experts)), dtype=torch.uint8,
                     device="cuda")
    capi.check(lib.deepep_get_dispatch_layout(capi.ptr(dev), t, k, num_ranks, num_experts, capi.ptr(per_rank),
                                              capi.ptr(per_rdma), capi.ptr(per_expert), capi.ptr(is_in), capi.ptr(ws),
                                              ws.numel(), stream()))
    torch.cuda.synchronize()
    return per_rank.cpu(), None if per_rdma is None else per_rdma.cpu(), per_expert.cpu(), is_in.cpu()


@pytest.mark.parametrize("t,k,e,r,drop", [
    (128, 8, 256, 16, 0),     # CPU-reference configuration
    (128, 8, 256, 32, 10),    # LL configuration, with -1 entries
    (4096, 8, 256, 8, 25),    # normal-mode configuration
    (8192, 8, 256, 64, 0),
    (1, 1, 2, 2, 0), (0, 4, 8, 8, 0), (257, 6, 48, 6, 7), (1000, 3, 160, 160, 9), (300, 9, 288, 24, 3),
])
def test_get_dispatch_layout(capi, t, k, e, r, drop):
    topk = _topk(t, k, e, seed=t + e + r, drop=drop)
    got = run_layout(capi, topk, e, r)
    want = O.get_dispatch_layout(topk, e, r)
    assert torch.equal(got[0], want[0])
    assert (got[1] is None) == (want[1] is None)
    if want[1] is not None:
        assert torch.equal(got[1], want[1])
    assert torch.equal(got[2], want[2])
    assert torch.equal(got[3], want[3])


def test_layout_rejects_bad_shapes(capi):
    lib = capi.load()
    t = torch.zeros((4, 2), dtype=torch.int64, device="cuda")
    out = torch.zeros(64, dtype=torch.int32, device="cuda")
    rc = lib.deepep_get_dispatch_layout(capi.ptr(t), 4, 2, 3, 8, capi.ptr(out), None, capi.ptr(out), capi.ptr(out),
                                        capi.ptr(out), 256, stream())
    assert rc != 0
    msg = lib.deepep_last_error().decode()
    assert msg.startswith("Failed: Assertion error") and "num_experts % num_ranks == 0" in msg


@pytest.mark.parametrize("t,r,p", [(4096, 8, 0.66), (53, 6, 0.4), (1, 3, 1.0), (0, 4, 0.5), (5000, 64, 0.1),
                                   (2048, 160, 0.05)])
def test_routing_sort_channel_prefix(capi, t, r, p):
    lib = capi.load()
    g = torch.Generator().manual_seed(t + r)
    is_in = torch.rand((t, r), generator=g) < p
    dev = is_in.cuda()
    ids = torch.full((max(1, t * r),), -1, dtype=torch.int64, device="cuda")
    counts = torch.full((r,), -1, dtype=torch.int32, device="cuda")
    cumsum = torch.full((r + 1,), -1, dtype=torch.int64, device="cuda")
    ws = torch.empty(max(16, lib.deepep_routing_sort_workspace_bytes(t, r)), dtype=torch.uint8, device="cuda")
    capi.check(lib.deepep_moe_routing_sort(capi.ptr(dev), t, r, capi.ptr(ids), capi.ptr(counts), capi.ptr(cumsum),
                                           capi.ptr(ws), ws.numel(), stream()))
    torch.cuda.synchronize()
    w_ids, w_counts, w_cumsum, total = O.moe_routing_sort(is_in)
    assert torch.equal(counts.cpu(), w_counts) and torch.equal(cumsum.cpu(), w_cumsum)
    assert torch.equal(ids[:total].cpu(), w_ids)
    for c in (10, 12, 1, 7):
        cpm = torch.full((r, c), -1, dtype=torch.int32, device="cuda")
        capi.check(lib.deepep_channel_prefix_matrix(capi.ptr(dev), t, r, c, capi.ptr(cpm), stream()))
        torch.cuda.synchronize()
        assert torch.equal(cpm.cpu(), O.channel_prefix_matrix(is_in, c))


@pytest.mark.parametrize("rows,row_bytes,scale_bytes", [(4096, 14336, 0), (4096, 7168, 224), (37, 256, 8), (5, 16, 0)])
def test_pack_rows(capi, rows, row_bytes, scale_bytes):
    lib = capi.load()
    g = torch.Generator().manual_seed(rows)
    src = torch.randint(0, 256, (rows, row_bytes), dtype=torch.uint8, generator=g)
    sc = torch.randint(0, 256, (rows, scale_bytes), dtype=torch.uint8, generator=g) if scale_bytes else None
    is_in = torch.rand((rows, 8), generator=g) < 0.66
    ids, _, cumsum, total = O.moe_routing_sort(is_in)
    d_src, d_ids = src.cuda(), ids.cuda()
    d_sc = sc.cuda() if sc is not None else None
    n_dev = torch.tensor([total], dtype=torch.int64, device="cuda")
    cap = rows * 8
    dst = torch.full((cap, row_bytes), 0xEE, dtype=torch.uint8, device="cuda")
    dsc = torch.full((cap, scale_bytes), 0xEE, dtype=torch.uint8, device="cuda") if scale_bytes else None
    ids_full = torch.full((cap,), -1, dtype=torch.int64, device="cuda")
    ids_full[:total] = d_ids
    capi.check(lib.deepep_pack_rows(capi.ptr(d_src), capi.ptr(d_sc), capi.ptr(ids_full), capi.ptr(n_dev), cap, rows,
                                    row_bytes, scale_bytes, capi.ptr(dst), capi.ptr(dsc), stream()))
    torch.cuda.synchronize()
    assert torch.equal(dst[:total].cpu(), src[ids])
    assert (dst[total:] == 0xEE).all()
    if scale_bytes:
        assert torch.equal(dsc[:total].cpu(), sc[ids]) and (dsc[total:] == 0xEE).all()


def run_cast(capi, x, fmt):
    lib = capi.load()
    m, n = x.shape
    d = x.cuda()
    q = torch.empty((m, n), dtype=torch.uint8, device="cuda")
    sb = (n // 128) * (1 if fmt == O.ROW_FP8_UE8M0 else 4)
    s = torch.empty((m, sb), dtype=torch.uint8, device="cuda")
    capi.check(lib.deepep_per_token_cast_to_fp8(capi.ptr(d), m, n, fmt, capi.ptr(q), capi.ptr(s), stream()))
    torch.cuda.synchronize()
    return q.cpu(), s.cpu()


def _check_cast(capi, x, fmt):
    q, s = run_cast(capi, x, fmt)
    wq, ws = O.per_token_cast_to_fp8(x, round_scale=fmt != O.ROW_FP8, use_ue8m0=fmt == O.ROW_FP8_UE8M0)
    assert torch.equal(s, ws.contiguous().view(torch.uint8).view(x.shape[0], -1)), "scales differ"
    wq = wq.view(torch.uint8)
    bad = (q != wq).nonzero()
    assert bad.numel() == 0, f"{bad.shape[0]} fp8 bytes differ, first at {bad[0].tolist()}"


@pytest.mark.parametrize("fmt", [O.ROW_FP8, O.ROW_FP8_POW2, O.ROW_FP8_UE8M0])
def test_cast_every_bf16_value_under_many_amax(capi, fmt):
    # Each group holds 127 consecutive bf16 bit patterns plus one amax-setting value, so every
    # finite bf16 value is quantised under several scales, and every value is also an amax once.
    bits = torch.arange(65536, dtype=torch.int32)
    vals = bits.to(torch.int16).view(torch.bfloat16)
    finite = vals[torch.isfinite(vals.float())]
    n = finite.numel() // 127 * 127
    body = finite[:n].view(-1, 127)
    rows = []
    for amax in (1.0, 3.0, 448.0, 0.007, 1e-5, 7.3e4, 3.0e38):
        cap = torch.full((body.shape[0], 1), amax, dtype=torch.bfloat16)
        clipped = torch.where(body.float().abs() <= amax, body, torch.zeros_like(body))
        rows.append(torch.cat([clipped[:, :64], cap, clipped[:, 64:]], 1))
    own = torch.cat([body[:, :5], body[:, :1].expand(-1, 123) * 0], 1)  # small groups: own amax
    rows.append(own)
    x = torch.cat(rows, 0)
    pad = (-x.shape[0]) % 4
    x = torch.cat([x, torch.zeros((pad, 128), dtype=torch.bfloat16)], 0).view(-1, 512).contiguous()
    _check_cast(capi, x, fmt)


@pytest.mark.parametrize("fmt", [O.ROW_FP8, O.ROW_FP8_POW2, O.ROW_FP8_UE8M0])
@pytest.mark.parametrize("m,n", [(128, 7168), (1, 512), (33, 1536), (7, 4096)])
def test_cast_random_and_outliers(capi, fmt, m, n):
    if fmt == O.ROW_FP8_UE8M0 and (n // 128) % 4:
        pytest.skip("UE8M0 packs 4 exponents per int32")
    g = torch.Generator().manual_seed(m * 7 + n)
    x = torch.randn((m, n), generator=g)
    x[::7] *= 100
    if m > 3:
        x[3] = 0
        x[2, :128] = 1e-7
    x[0, 5] = -0.0
    _check_cast(capi, x.to(torch.bfloat16), fmt)


def test_cast_argument_errors(capi):
    lib = capi.load()
    x = torch.zeros((2, 192), dtype=torch.bfloat16, device="cuda")
    rc = lib.deepep_per_token_cast_to_fp8(capi.ptr(x), 2, 192, 1, capi.ptr(x), capi.ptr(x), stream())
    assert rc != 0 and "num_cols % 128 == 0" in lib.deepep_last_error().decode()
    with pytest.raises(capi.DeepEPError):
        capi.check(lib.deepep_per_token_cast_to_fp8(capi.ptr(x), 2, 128, 3, capi.ptr(x), capi.ptr(x), stream()))
