"""GPU parity: route counting / layout, routing sort, channel prefix, pack and the FP8 cast.

Every call goes through the C ABI (ctypes on libdeepep_hip.so); the expected
values come from the CPU oracle.  Integer and byte outputs must be bit-exact.
"""
import os

import numpy as np
import pytest
import torch

from oracle import deepep_oracle as O
from tiny_world import load_tiny_world

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


def test_hand_derived_world_layout_sort_and_prefix(capi):
    """Layout, routing sort and channel prefix against values worked out on paper
    (tests/golden/ll_tiny_world.json): no oracle involved."""
    g, _, topk_all = load_tiny_world()
    lib = capi.load()
    r, e, t = g["num_ranks"], g["num_experts"], g["num_tokens"]
    per_rank, per_rdma, per_expert, is_in = run_layout(capi, topk_all[0], e, r)
    assert per_rank.tolist() == g["layout_rank0"]["num_tokens_per_rank"] and per_rdma is None
    assert per_expert.tolist() == g["layout_rank0"]["num_tokens_per_expert"]
    assert is_in.tolist() == g["layout_rank0"]["is_token_in_rank"]
    want = g["normal_mode_rank0"]
    dev = is_in.cuda()
    ids = torch.full((t * r,), -1, dtype=torch.int64, device="cuda")
    counts = torch.full((r,), -1, dtype=torch.int32, device="cuda")
    cumsum = torch.full((r + 1,), -1, dtype=torch.int64, device="cuda")
    ws = torch.empty(max(16, lib.deepep_routing_sort_workspace_bytes(t, r)), dtype=torch.uint8, device="cuda")
    inverse = torch.full((max(1, t * r),), -7, dtype=torch.int32, device="cuda")
    capi.check(lib.deepep_moe_routing_sort(capi.ptr(dev), t, r, capi.ptr(ids), capi.ptr(counts), capi.ptr(cumsum),
                                           capi.ptr(inverse), capi.ptr(ws), ws.numel(), stream()))
    torch.cuda.synchronize()
    assert counts.cpu().tolist() == want["send_counts"] and cumsum.cpu().tolist() == want["send_cumsum"]
    assert ids[:4].cpu().tolist() == want["sorted_token_ids"]
    assert inverse[:t * r].view(t, r).cpu().tolist() == want["row_of_pair"]
    for c in (2, 3):
        cpm = torch.full((r, c), -1, dtype=torch.int32, device="cuda")
        capi.check(lib.deepep_channel_prefix_matrix(capi.ptr(dev), t, r, c, capi.ptr(cpm), stream()))
        torch.cuda.synchronize()
        assert cpm.cpu().tolist() == want[f"channel_prefix_matrix_{c}_channels"]


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
    inverse = torch.full((max(1, t * r),), -7, dtype=torch.int32, device="cuda")
    capi.check(lib.deepep_moe_routing_sort(capi.ptr(dev), t, r, capi.ptr(ids), capi.ptr(counts), capi.ptr(cumsum),
                                           capi.ptr(inverse), capi.ptr(ws), ws.numel(), stream()))
    torch.cuda.synchronize()
    w_ids, w_counts, w_cumsum, total = O.moe_routing_sort(is_in)
    assert torch.equal(counts.cpu(), w_counts) and torch.equal(cumsum.cpu(), w_cumsum)
    assert torch.equal(ids[:total].cpu(), w_ids)
    assert torch.equal(inverse[:t * r].view(t, r).cpu(), _want_row_of_pair(is_in, w_ids, w_cumsum))
    for c in (10, 12, 1, 7):
        cpm = torch.full((r, c), -1, dtype=torch.int32, device="cuda")
        capi.check(lib.deepep_channel_prefix_matrix(capi.ptr(dev), t, r, c, capi.ptr(cpm), stream()))
        torch.cuda.synchronize()
        assert torch.equal(cpm.cpu(), O.channel_prefix_matrix(is_in, c))


@pytest.mark.parametrize("seed", range(int(os.environ.get("DEEPEP_TEST_RANDOM_SHAPES", "16"))))
def test_layout_sort_prefix_seeded_random_shapes(capi, seed):
    """Layout, routing sort and channel prefix on shapes nobody picked by hand (both sort paths)."""
    g = np.random.default_rng(500 + seed)
    r = int(g.choice([1, 2, 3, 5, 8, 9, 16, 24, 40, 64, 72, 96]))
    epr = int(g.choice([1, 2, 3, 8]))
    e = r * epr
    k = int(g.integers(1, min(e, 10) + 1))
    t = int(g.choice([0, 1, 5, 63, 64, 65, 255, 256, 257, 1000, 1025, 3000, 4097, 8192, 8193, 9000]))
    topk = _topk(t, k, e, seed=seed, drop=int(g.integers(0, 20)))
    got = run_layout(capi, topk, e, r)
    want = O.get_dispatch_layout(topk, e, r)
    assert torch.equal(got[0], want[0]) and torch.equal(got[2], want[2]) and torch.equal(got[3], want[3])
    assert (got[1] is None) == (want[1] is None) and (want[1] is None or torch.equal(got[1], want[1]))
    lib = capi.load()
    is_in = want[3]
    dev = is_in.cuda()
    ids = torch.full((max(1, t * r),), -1, dtype=torch.int64, device="cuda")
    counts = torch.full((r,), -1, dtype=torch.int32, device="cuda")
    cumsum = torch.full((r + 1,), -1, dtype=torch.int64, device="cuda")
    ws = torch.empty(max(16, lib.deepep_routing_sort_workspace_bytes(t, r)), dtype=torch.uint8, device="cuda")
    inverse = torch.full((max(1, t * r),), -7, dtype=torch.int32, device="cuda")
    capi.check(lib.deepep_moe_routing_sort(capi.ptr(dev), t, r, capi.ptr(ids), capi.ptr(counts), capi.ptr(cumsum),
                                           capi.ptr(inverse), capi.ptr(ws), ws.numel(), stream()))
    torch.cuda.synchronize()
    w_ids, w_counts, w_cumsum, total = O.moe_routing_sort(is_in)
    assert torch.equal(counts.cpu(), w_counts) and torch.equal(cumsum.cpu(), w_cumsum)
    assert torch.equal(ids[:total].cpu(), w_ids) and (ids[total:] == -1).all()
    assert torch.equal(inverse[:t * r].view(t, r).cpu(), _want_row_of_pair(is_in, w_ids, w_cumsum))
    c = int(g.choice([1, 3, 10, 12, 17, 40]))
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
def test_cast_every_bf16_value_as_the_amax_of_a_group(capi, fmt):
    """One group per positive finite bf16 value (and its negative), that value its only non-zero element: the
    scale of every possible amax, power-of-two rounding included, against the oracle."""
    bits = torch.arange(1, 0x7F80, dtype=torch.int32)
    vals = torch.cat([bits, bits | 0x8000]).to(torch.int16).view(torch.bfloat16)
    pad = (-vals.numel()) % 4
    x = torch.zeros((vals.numel() + pad, 128), dtype=torch.bfloat16)
    x[:vals.numel(), 77] = vals
    _check_cast(capi, x.view(-1, 512).contiguous(), fmt)


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


# ---- the steps either side of the normal-mode pack ------------------------------------------------
def _want_row_of_pair(is_in, ids, cumsum):
    """The inverse of the per-rank token list: where (token, rank) stands in it, -1 for non-members."""
    t, r = is_in.shape
    inv = torch.full((t, r), -1, dtype=torch.int32)
    for rank in range(r):
        lo, hi = int(cumsum[rank]), int(cumsum[rank + 1])
        inv[ids[lo:hi], rank] = torch.arange(lo, hi, dtype=torch.int32)
    return inv


def _normal_world(t, k, e, r, seed, drop=3):
    topk = _topk(t, k, e, seed, drop)
    if t > 2:
        topk[0, :] = -1   # sent nowhere
        topk[1, 1:] = -1  # held by exactly one rank
    g = torch.Generator().manual_seed(seed + 1)
    w = torch.rand((t, k), generator=g)
    _, _, _, is_in = O.get_dispatch_layout(topk, e, r)
    ids, counts, cumsum, total = O.moe_routing_sort(is_in)
    return topk, w, is_in, ids, counts, cumsum, total


@pytest.mark.parametrize("t,k,e,r", [(4096, 8, 256, 8), (333, 6, 64, 16), (5, 2, 8, 4), (1200, 8, 288, 72)])
def test_topk_remap(capi, t, k, e, r):
    lib = capi.load()
    topk, w, _, ids, _, cumsum, total = _normal_world(t, k, e, r, seed=t + r)
    want_e, want_w = O.topk_remap(topk, w, ids, cumsum, e // r)
    cap = total + 7  # rows past the device-side total must stay untouched
    out_e = torch.full((cap, k), -99, dtype=torch.int64, device="cuda")
    out_w = torch.full((cap, k), -99.0, dtype=torch.float32, device="cuda")
    ids_dev = torch.cat([ids, torch.zeros(7, dtype=torch.int64)]).cuda()
    topk_dev, w_dev, cumsum_dev = topk.cuda(), w.cuda(), cumsum.cuda()  # named: they must outlive the launch
    capi.check(lib.deepep_topk_remap(capi.ptr(topk_dev), capi.ptr(w_dev), capi.ptr(ids_dev), capi.ptr(cumsum_dev), t, k,
                                     r, e // r, cap, capi.ptr(out_e), capi.ptr(out_w), stream()))
    torch.cuda.synchronize()
    assert torch.equal(out_e[:total].cpu(), want_e)
    assert torch.equal(out_w[:total].cpu(), want_w)
    assert (out_e[total:] == -99).all() and (out_w[total:] == -99.0).all()


@pytest.mark.parametrize("r,local", [(8, 8), (32, 8), (17, 4), (1, 1)])
def test_build_recv_src_meta(capi, r, local):
    lib = capi.load()
    g = torch.Generator().manual_seed(r)
    counts = torch.randint(0, 50, (r,), generator=g)
    counts[r // 2] = 0
    cumsum = torch.zeros(r + 1, dtype=torch.int64)
    cumsum[1:] = torch.cumsum(counts, 0)
    total = int(cumsum[r])
    want = O.build_recv_src_meta(cumsum, local)
    meta = torch.full((total + 3, 8), 0xEE, dtype=torch.uint8, device="cuda")
    cumsum_dev = cumsum.cuda()
    capi.check(lib.deepep_build_recv_src_meta(capi.ptr(cumsum_dev), r, local, total + 3, capi.ptr(meta), stream()))
    torch.cuda.synchronize()
    assert torch.equal(meta[:total].cpu(), want)
    assert (meta[total:] == 0xEE).all()


@pytest.mark.parametrize("t,k,e,r,h,with_bias", [(4096, 8, 256, 8, 7168, False), (333, 6, 64, 16, 512, True),
                                                 (5, 2, 8, 4, 128, True), (700, 8, 288, 72, 1024, False)])
def test_combine_reduce(capi, t, k, e, r, h, with_bias):
    """The per-token sum of the rows that came back: bit-exact against the float32 chain in rank order,
    within 1e-2 relative of the float64 index_add_ of deep_ep/buffer.py:1542-1557."""
    lib = capi.load()
    topk, w, is_in, ids, counts, cumsum, total = _normal_world(t, k, e, r, seed=t + h)
    g = torch.Generator().manual_seed(5)
    rows = torch.randn((total, h), generator=g).to(torch.bfloat16)
    rw = torch.rand((total, k), generator=g)
    b0 = torch.randn((t, h), generator=g).to(torch.bfloat16) if with_bias else None
    b1 = torch.randn((t, h), generator=g).to(torch.bfloat16) if with_bias else None
    out_x = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
    out_x.view(torch.int16).fill_(0x7FC0)
    out_w = torch.full((t, k), float("nan"), dtype=torch.float32, device="cuda")
    ws = torch.full((max(256, lib.deepep_combine_reduce_workspace_bytes(t, r)),), 0x7F, dtype=torch.uint8, device="cuda")
    dev = [None if v is None else v.cuda() for v in (rows, rw, ids, cumsum, is_in, b0, b1)]  # outlive the launch
    capi.check(lib.deepep_combine_reduce(*[capi.ptr(v) for v in dev], t, h, k, r, total, None, capi.ptr(out_x),
                                         capi.ptr(out_w), capi.ptr(ws), ws.numel(), stream()))
    torch.cuda.synchronize()
    chain_x, chain_w = O.combine_reduce_f32_chain(rows, rw, ids, cumsum, t, b0, b1)
    assert torch.equal(out_x.cpu().view(torch.int16), chain_x.view(torch.int16))
    assert torch.equal(out_w.cpu(), chain_w)
    # with the table the routing sort leaves: one launch, no workspace, the same bits
    table = _want_row_of_pair(is_in, ids, cumsum).cuda()
    out_x2 = torch.empty_like(out_x)
    out_x2.view(torch.int16).fill_(0x7FC0)
    out_w2 = torch.full_like(out_w, float("nan"))
    capi.check(lib.deepep_combine_reduce(*[capi.ptr(v) for v in dev], t, h, k, r, total, capi.ptr(table),
                                         capi.ptr(out_x2), capi.ptr(out_w2), None, 0, stream()))
    torch.cuda.synchronize()
    assert torch.equal(out_x2.view(torch.int16), out_x.view(torch.int16)) and torch.equal(out_w2, out_w)
    ref_x, ref_w = O.combine_reduce(rows, rw, ids, t, b0, b1)
    err = (out_x.cpu().double() - ref_x).abs()
    assert (err <= 1e-2 * ref_x.abs() + 1e-2 * ref_x.abs().mean()).all()
    assert torch.allclose(out_w.cpu().double(), ref_w, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("seed", range(int(os.environ.get("DEEPEP_TEST_RANDOM_SHAPES", "16"))))
def test_pack_remap_reduce_seeded_random_shapes(capi, seed):
    """Pack, top-k remap and the combine reduce on shapes nobody picked by hand: odd rank counts, ragged
    hidden sizes, tokens that go nowhere."""
    lib = capi.load()
    g = np.random.default_rng(900 + seed)
    r = int(g.choice([1, 2, 3, 5, 8, 9, 16, 24, 64, 65, 100]))
    epr = int(g.choice([1, 2, 3, 8]))
    e = r * epr
    k = int(g.integers(1, min(e, 10) + 1))
    t = int(g.choice([5, 6, 63, 64, 65, 255, 257, 1000, 1500]))
    h = int(g.choice([8, 64, 128, 136, 512, 520, 1024, 2056]))  # row bytes = 2h: a multiple of 16
    with_bias = bool(g.integers(0, 2))
    topk, w, is_in, ids, counts, cumsum, total = _normal_world(t, k, e, r, seed=3000 + seed)
    topk[:: max(2, t // 3)] = -1  # tokens no rank holds
    _, _, _, is_in = O.get_dispatch_layout(topk, e, r)
    ids, counts, cumsum, total = O.moe_routing_sort(is_in)
    tg = torch.Generator().manual_seed(seed)
    x = torch.randn((t, h), generator=tg).to(torch.bfloat16)
    # pack: rows gathered into per-rank contiguous order
    cap = total + 5
    ids_full = torch.full((cap,), -1, dtype=torch.int64)
    ids_full[:total] = ids
    dev = dict(x=x.cuda(), ids=ids_full.cuda(), n=torch.tensor([total], dtype=torch.int64, device="cuda"))
    packed = torch.full((cap, h), float("nan"), dtype=torch.bfloat16, device="cuda")
    capi.check(lib.deepep_pack_rows(capi.ptr(dev["x"]), None, capi.ptr(dev["ids"]), capi.ptr(dev["n"]), cap, t, h * 2, 0,
                                    capi.ptr(packed), None, stream()))
    torch.cuda.synchronize()
    assert torch.equal(packed[:total].cpu().view(torch.int16), x[ids].view(torch.int16))
    assert packed[total:].isnan().all()
    # remap
    want_e, want_w = O.topk_remap(topk, w, ids, cumsum, epr)
    out_e = torch.full((cap, k), -99, dtype=torch.int64, device="cuda")
    out_w = torch.full((cap, k), -99.0, dtype=torch.float32, device="cuda")
    topk_dev, w_dev, cumsum_dev = topk.cuda(), w.cuda(), cumsum.cuda()
    capi.check(lib.deepep_topk_remap(capi.ptr(topk_dev), capi.ptr(w_dev), capi.ptr(dev["ids"]), capi.ptr(cumsum_dev), t, k,
                                     r, epr, cap, capi.ptr(out_e), capi.ptr(out_w), stream()))
    torch.cuda.synchronize()
    assert torch.equal(out_e[:total].cpu(), want_e) and torch.equal(out_w[:total].cpu(), want_w)
    assert (out_e[total:] == -99).all()
    # reduce of rows that come back changed
    rows = torch.randn((total, h), generator=tg).to(torch.bfloat16)
    b0 = torch.randn((t, h), generator=tg).to(torch.bfloat16) if with_bias else None
    b1 = torch.randn((t, h), generator=tg).to(torch.bfloat16) if with_bias else None
    out_x = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
    out_x.view(torch.int16).fill_(0x7FC0)
    out_cw = torch.full((t, k), float("nan"), dtype=torch.float32, device="cuda")
    ws = torch.full((max(256, lib.deepep_combine_reduce_workspace_bytes(t, r)),), 0x7F, dtype=torch.uint8, device="cuda")
    held = [None if v is None else v.cuda() for v in (rows, want_w, ids, cumsum, is_in, b0, b1)]
    table = _want_row_of_pair(is_in, ids, cumsum).cuda() if seed % 2 else None  # with and without the sort's table
    capi.check(lib.deepep_combine_reduce(*[capi.ptr(v) for v in held], t, h, k, r, total, capi.ptr(table),
                                         capi.ptr(out_x), capi.ptr(out_cw), capi.ptr(ws), ws.numel(), stream()))
    torch.cuda.synchronize()
    chain_x, chain_w = O.combine_reduce_f32_chain(rows, want_w, ids, cumsum, t, b0, b1)
    assert torch.equal(out_x.cpu().view(torch.int16), chain_x.view(torch.int16))
    assert torch.equal(out_cw.cpu(), chain_w)


def test_normal_mode_steps_through_the_host_module():
    """topk_remap / build_recv_src_meta / combine_reduce with the reference's Python-visible signatures."""
    from deepep_efa_amd import normal
    t, k, e, r, h = 257, 4, 32, 8, 256
    topk, w, is_in, ids, counts, cumsum, total = _normal_world(t, k, e, r, seed=12)
    ids_d, counts_d, cumsum_d, total_d = normal.moe_routing_sort(is_in.cuda())
    assert total_d == total and torch.equal(ids_d.cpu(), ids)
    re, rw = normal.topk_remap(topk.cuda(), w.cuda(), ids_d, cumsum_d, total_d, r, e // r)
    want_e, want_w = O.topk_remap(topk, w, ids, cumsum, e // r)
    assert torch.equal(re.cpu(), want_e) and torch.equal(rw.cpu(), want_w)
    meta = normal.build_recv_src_meta(counts_d, cumsum_d, total_d, r, 8)
    assert torch.equal(meta.cpu(), O.build_recv_src_meta(cumsum, 8))
    # the exchange is the identity here: every rank returns the row it was sent
    x = torch.randn((t, h), generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
    send_x, _ = normal.pack_rows(x.cuda(), None, ids_d, cumsum_d)
    cx, cw = normal.combine_reduce(send_x, rw, ids_d, cumsum_d, is_in.cuda())
    ids_p, counts_p, cumsum_p, total_p, row_of_pair = normal.moe_routing_sort_with_positions(is_in.cuda())
    assert total_p == total and torch.equal(ids_p, ids_d) and torch.equal(cumsum_p, cumsum_d)
    assert torch.equal(row_of_pair.cpu(), _want_row_of_pair(is_in, ids, cumsum))
    cx2, cw2 = normal.combine_reduce(send_x, rw, ids_d, cumsum_d, is_in.cuda(), row_of_pair=row_of_pair)
    assert torch.equal(cx2.view(torch.int16), cx.view(torch.int16)) and torch.equal(cw2, cw)
    # remapped weights are zero outside the destination's experts, so their sum is the original weight row
    want_cw = torch.where(topk >= 0, w, torch.zeros_like(w))
    assert torch.allclose(cw.cpu(), want_cw, rtol=1e-6, atol=1e-7)
    chain_x, _ = O.combine_reduce_f32_chain(x[ids], None, ids, cumsum, t)
    assert torch.equal(cx.cpu().view(torch.int16), chain_x.view(torch.int16))
    with pytest.raises(RuntimeError, match="Assertion"):
        normal.topk_remap(topk.cuda(), w.cuda(), ids_d, cumsum_d, total_d + 10 ** 6, r, e // r)


def test_row_scatter_probe(capi):
    """The bare read-rows / store-K-copies kernel bench.py times beside the send side: every named row gets
    the fold of its token's row, every other byte is left alone."""
    import bench
    probe = bench.load_bench_probe()
    t, h, k, rows, stride = 37, 512, 3, 200, 640
    g = torch.Generator().manual_seed(5)
    x = torch.randint(0, 2 ** 16, (t, h), generator=g, dtype=torch.int32).to(torch.uint16)
    dst_rows = torch.randperm(rows, generator=g)[:t * k].view(t, k).to(torch.int32)
    dst_rows[::5, 1] = -1
    dst = torch.full((rows, stride), 0xEE, dtype=torch.uint8, device="cuda")
    x_dev, rows_dev = x.cuda(), dst_rows.cuda()
    assert probe.bench_probe_row_scatter(capi.ptr(x_dev), t, h, capi.ptr(rows_dev), k, capi.ptr(dst), stride,
                                         stream()) == 0
    torch.cuda.synchronize()
    words = x.view(torch.uint8).view(t, h // 16, 2, 16)          # 32 bytes per thread: two 16-byte vectors
    fold = (words[:, :, 0] ^ words[:, :, 1]).reshape(t, h)       # one vector out
    want = torch.full((rows, stride), 0xEE, dtype=torch.uint8)
    for i in range(t):
        for j in range(k):
            if dst_rows[i, j] >= 0:
                want[int(dst_rows[i, j]), :h] = fold[i]
    assert torch.equal(dst.cpu(), want)
