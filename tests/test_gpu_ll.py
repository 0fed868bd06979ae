"""GPU parity of the low-latency dispatch + combine path, through the C ABI.

One GPU plays rank `rank` of an R-rank world; the other ranks' rows are put
in HBM by the loopback entry points.  Expected values come from the CPU
oracle restated from the reference.  Integer outputs, FP8 bytes and scales
must be bit-exact; the combine must match the float32 FMA-chain definition
bit for bit and the float64 sum within 1e-2 relative.
"""
import ctypes
import os

import numpy as np
import pytest
import torch

from oracle import deepep_oracle as O
from tiny_world import load_tiny_world, tiny_world_expected

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rt():
    from deepep_efa_amd import _capi, ll_runtime, loopback
    _capi.load()
    assert torch.cuda.is_available(), "these tests need the MI355X"

    class NS:
        pass

    ns = NS()
    ns.capi, ns.ll, ns.lb = _capi, ll_runtime, loopback
    return ns


def make_world(r, t, h, k, e, seed, drop=10, recipe="randn"):
    g = torch.Generator().manual_seed(seed)
    if recipe == "rank_const":  # tests/test_low_latency.py:59-60
        xs = []
        for rank in range(r):
            x = torch.ones((t, h), dtype=torch.bfloat16) * (rank - 128)
            x[:, -128:] = torch.arange(t).to(torch.bfloat16).view(-1, 1)
            xs.append(x)
        x_all = torch.stack(xs)
    else:
        x_all = torch.randn((r, t, h), generator=g).to(torch.bfloat16)
        x_all[:, ::9] *= 30
    scores = torch.rand((r, t, e), generator=g)
    topk = torch.topk(scores, k, dim=-1)[1].contiguous()
    for _ in range(drop):
        s, i, j = [int(torch.randint(0, n, (1,), generator=g)) for n in (r, t, k)]
        topk[s, i, j] = -1
    w = torch.randn((r, t, k), generator=g).abs()
    return x_all, topk, w


ONE_CALL = pytest.mark.parametrize("one_call", [False, True], ids=["two_calls", "one_call"])


def poison_outputs(st):
    """Fresh tensors may reuse memory that an earlier test left holding the right answer."""
    st.packed_recv_x.view(torch.uint8).fill_(0xEE)
    if st.packed_recv_scales is not None:
        st.packed_recv_scales.view(torch.uint8).fill_(0xEE)
    st.packed_recv_src_info.fill_(-7)
    st.packed_recv_count.fill_(-7)
    st.packed_recv_layout_range.fill_(-7)
    st.pair_slot.fill_(-7)


def run_dispatch(st, world, x, topk, stats=None, one_call=False):
    poison_outputs(st)
    if one_call:
        world.dispatch_from_peers(st)
        st.dispatch(x, topk, stats)
    else:
        st.dispatch_send(x, topk)
        world.dispatch_from_peers(st)
        st.dispatch_recv(stats)
    torch.cuda.synchronize()


def run_combine(st, world, y, topk, w, out, mode, seed=0, one_call=False):
    out.view(torch.int16).fill_(0x7FC0)  # NaN
    if one_call:
        world.combine_from_peers(st, mode=mode, seed=seed)
        st.combine(y, topk, w, out)
    else:
        world.combine_from_peers(st, mode=mode, seed=seed)
        st.combine_send(y)
        st.combine_recv(topk, w, out)
    torch.cuda.synchronize()


def dispatch_on_gpu(rt, x_all, topk_all, rank, e, m, fmt, stats=None, one_call=False):
    r, t, h = x_all.shape
    k = topk_all.shape[2]
    shape = rt.ll.LLShape(num_ranks=r, rank=rank, num_experts=e, max_tokens=m, hidden=h, num_topk=k, fmt=fmt)
    st = rt.ll.LowLatencyState(shape)
    world = rt.lb.LoopbackWorld(r, rank, seed=0)
    world.set_inputs(x_all.cuda(), topk_all.cuda())
    x, topk = world.own_inputs()
    run_dispatch(st, world, x, topk, stats, one_call)
    return st, world


def check_dispatch(st, want, fmt):
    count = st.packed_recv_count.cpu()
    assert torch.equal(count, want["packed_recv_count"])
    assert torch.equal(st.packed_recv_layout_range.cpu(), want["packed_recv_layout_range"])
    px = st.packed_recv_x.view(torch.uint8).view(want["packed_recv_x"].shape).cpu()
    src = st.packed_recv_src_info.cpu()
    ps = None if st.packed_recv_scales is None else \
        st.packed_recv_scales.view(torch.uint8).view(want["packed_recv_scales"].shape).cpu()
    for le in range(count.numel()):
        n = int(count[le])
        assert torch.equal(src[le, :n], want["packed_recv_src_info"][le, :n]), f"src_info expert {le}"
        assert torch.equal(px[le, :n], want["packed_recv_x"][le, :n]), f"payload bytes expert {le}"
        if ps is not None:
            assert torch.equal(ps[le, :n], want["packed_recv_scales"][le, :n]), f"scale bytes expert {le}"


@pytest.mark.parametrize("fmt", [O.ROW_FP8, O.ROW_BF16, O.ROW_FP8_POW2, O.ROW_FP8_UE8M0])
@pytest.mark.parametrize("r,rank,t,h,k,e", [
    (4, 1, 8, 512, 3, 16), (8, 7, 33, 1024, 4, 64), (2, 0, 1, 512, 1, 2),
    (4, 1, 40, 512, 9, 64),    # K > 8
    (2, 1, 600, 512, 8, 16),   # a mid-sized batch: the send side sweeps every earlier entry, in the single launch too
    (4, 3, 300, 512, 11, 32),  # both
    (2, 0, 1100, 512, 8, 16),  # T*K > 8192: chunk histograms under the send kernel's sweep, small receive path
    (8, 5, 4200, 512, 4, 64),  # more than 8192 expected rows: receive runs as index kernel + flat row copy
    (8, 2, 20, 512, 4, 512),   # more than 256 segments: 16 counts per lane in the register segment table
    (16, 9, 12, 512, 6, 1024),  # the most experts the path takes
    (1, 0, 16, 512, 2, 4),     # a world of one rank: every row is the rank's own
    (4, 1, 12, 512, 2, 4),     # one expert per rank
    (2, 1, 9, 512, 64, 128),   # the most selections per token
    (4, 2, 24, 1536, 4, 16),   # hidden not a multiple of 1024: the last row piece is partly empty
    (8, 3, 17, 5120, 8, 64),
    (128, 77, 9, 512, 4, 128),   # many ranks, one expert each
    (256, 3, 5, 512, 2, 512),
    (512, 500, 3, 512, 2, 1024),  # the widest world the path takes
])
@ONE_CALL
def test_dispatch_small_worlds(rt, fmt, r, rank, t, h, k, e, one_call):
    x_all, topk_all, _ = make_world(r, t, h, k, e, seed=r * 100 + t, drop=min(5, t))
    st, _ = dispatch_on_gpu(rt, x_all, topk_all, rank, e, t, fmt, one_call=one_call)
    want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, t, fmt)
    check_dispatch(st, want, fmt)
    send_count, pair_slot = O.route(topk_all[rank], e, t)
    assert torch.equal(st.send_count.cpu(), send_count)
    assert torch.equal(st.pair_slot[:t].cpu(), pair_slot)


@pytest.mark.parametrize("key,rank", [("rank0_ascending", 0), ("rank1_ascending", 1)])
@ONE_CALL
@pytest.mark.parametrize("fmt", [O.ROW_BF16, O.ROW_FP8])
def test_hand_derived_world(rt, key, rank, one_call, fmt):
    """The HIP path against values worked out on paper (tests/golden/ll_tiny_world.json): no oracle involved."""
    g, x_all, topk_all = load_tiny_world()
    e, m, h, t, k = g["num_experts"], g["max_tokens"], g["hidden"], g["num_tokens"], g["num_topk"]
    st, world = dispatch_on_gpu(rt, torch.stack(x_all), torch.stack(topk_all), rank, e, m, fmt, one_call=one_call)
    want, layout = tiny_world_expected(g, key)
    assert st.packed_recv_count.cpu().tolist() == want["count"]
    assert torch.equal(st.packed_recv_layout_range.cpu(), layout)
    for le, n in enumerate(want["count"]):
        assert st.packed_recv_src_info[le, :n].cpu().tolist() == want["src_info"][le]
        values = torch.tensor(want["row_value"][le], dtype=torch.float32)
        if fmt == O.ROW_BF16:
            assert torch.equal(st.packed_recv_x[le, :n].cpu().float(), values.view(-1, 1).expand(-1, h))
        else:
            assert (st.packed_recv_x[le, :n].view(torch.uint8).cpu() == g["fp8"]["payload_byte"]).all()
            assert torch.equal(st.packed_recv_scales[le, :n].cpu().view(-1), values / torch.tensor(448.0))
    if rank != 0:
        return
    assert st.send_count.cpu().tolist() == g["route_rank0"]["send_count"]
    assert st.pair_slot[:t].cpu().tolist() == g["route_rank0"]["pair_slot"]
    if fmt == O.ROW_BF16:  # identity experts: what comes back is what was sent
        y = st.packed_recv_x.clone()
        out = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
        w = torch.tensor(g["topk_weights_rank0"], dtype=torch.float32, device="cuda")
        run_combine(st, world, y, topk_all[0].cuda(), w, out, mode=0, one_call=one_call)
        expect = torch.tensor(g["combine_rank0_identity_experts"]).view(-1, 1).expand(-1, h)
        assert torch.equal(out.cpu().float(), expect)


def check_exchange_metadata(got, want, capacity):
    assert got["send_counts"].cpu().tolist() == want["send_counts"].tolist()
    assert got["recv_counts"].cpu().tolist() == want["recv_counts"].tolist()
    assert got["totals"].cpu().tolist() == [want["total_send"], want["total_recv"], int(want["corrupt"])]
    assert got["combine_remote_recv_offset"].cpu().tolist() == want["combine_remote_recv_offset"].tolist()
    n = min(want["total_recv"], capacity)
    assert got["num_recv_tokens"].cpu().tolist() == [want["total_recv"], n]
    for key in ("source_rank", "source_offset", "padded_index", "combine_send_offset"):
        assert got[key][:n].cpu().tolist() == want[key][:n].tolist(), key
        assert (got[key][n:] == -7).all(), key  # nothing written past the records
    assert (got["tokens_per_expert"] == 0).all()


@pytest.mark.parametrize("r,e,m,k,rank,capacity", [(2, 4, 3, 2, 1, 16), (6, 24, 40, 5, 4, 400), (32, 256, 128, 8, 5, 4096),
                                                   (64, 256, 8192, 8, 63, 70000), (8, 64, 300, 6, 0, 100),
                                                   (1, 4, 9, 2, 0, 32), (160, 160, 20, 3, 77, 64)])
def test_exchange_metadata(rt, r, e, m, k, rank, capacity):
    """Counts, combine offsets and row records from the gathered route counts, against the reference's host loops."""
    g = torch.Generator().manual_seed(r * 7 + e)
    if r * m <= 4096:
        topk_all = [torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(m)]) for _ in range(r)]
        routed = torch.stack([O.route(tk, e, m)[0] for tk in topk_all]).to(torch.int32)
    else:  # any matrix of plausible counts will do
        routed = torch.randint(0, min(m, 60) + 1, (r, e), generator=g, dtype=torch.int32)
    for name, mat in (("clean", routed), ("corrupt", routed.clone())):
        if name == "corrupt":
            mat[r // 2, e // 3] = m + 1
        got = {}
        out = rt.ll.exchange_metadata(mat.cuda(), rank, m, capacity)
        torch.cuda.synchronize()
        want = O.ll_exchange_metadata(mat, rank, m)
        assert want["corrupt"] == (name == "corrupt")
        # poison-free check of "nothing written past the records": run again into pre-filled buffers
        for key in ("source_rank", "source_offset", "padded_index", "combine_send_offset"):
            got[key] = torch.full((capacity,), -7, dtype=torch.int32, device="cuda")
        lib, capi = rt.capi.load(), rt.capi
        for key in ("send_counts", "recv_counts", "totals", "combine_remote_recv_offset", "num_recv_tokens",
                    "tokens_per_expert"):
            got[key] = torch.full_like(out[key], -7)
        capi.check(lib.deepep_ll_exchange_metadata(
            capi.ptr(mat.cuda()), e, r, rank, m, capacity, capi.ptr(got["send_counts"]), capi.ptr(got["recv_counts"]),
            capi.ptr(got["totals"]), capi.ptr(got["combine_remote_recv_offset"]), capi.ptr(got["source_rank"]),
            capi.ptr(got["source_offset"]), capi.ptr(got["padded_index"]), capi.ptr(got["combine_send_offset"]),
            capi.ptr(got["num_recv_tokens"]), capi.ptr(got["tokens_per_expert"]),
            torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        check_exchange_metadata(got, want, capacity)
        for key in got:
            n = min(want["total_recv"], capacity) if got[key].numel() == capacity else got[key].numel()
            assert torch.equal(out[key][:n], got[key][:n]), key


def test_exchange_metadata_hand_derived_world(rt):
    g, _, _ = load_tiny_world()
    routed = torch.tensor(g["all_num_routed"], dtype=torch.int32)
    for rank in (0, 1):
        out = rt.ll.exchange_metadata(routed.cuda(), rank, g["max_tokens"], 8)
        torch.cuda.synchronize()
        want = g["exchange_metadata"][f"rank{rank}"]
        n = want["total_recv"]
        assert out["send_counts"].cpu().tolist() == want["send_counts"]
        assert out["recv_counts"].cpu().tolist() == want["recv_counts"]
        assert out["totals"].cpu().tolist() == [want["total_send"], n, 0]
        assert out["combine_remote_recv_offset"].cpu().tolist() == want["combine_remote_recv_offset"]
        assert out["num_recv_tokens"].cpu().tolist() == [n, n]
        for key in ("source_rank", "source_offset", "padded_index", "combine_send_offset"):
            assert out[key][:n].cpu().tolist() == want[key], key


def rows_by_source(x_all, topk_all, rank, e, m, fmt, slot_rows):
    """What an all-to-all leaves on rank `rank`: for every source s, the rows it sends to this rank's experts,
    in the sender's (token, k) order, at the start of slot s of one buffer (rows past the slot are lost)."""
    r, _, h = x_all.shape
    epr = e // r
    stride = O.row_stride(h, fmt)
    buf = torch.full((r * slot_rows, stride), 0xEE, dtype=torch.uint8)
    for s in range(r):
        _, _, experts, _, rows = O.staged_rows(x_all[s], topk_all[s], s, e, m, fmt, r)
        mine = rows[(experts // epr) == rank][:slot_rows]
        buf[s * slot_rows:s * slot_rows + mine.shape[0]] = mine
    return buf


def recv_by_source_on_gpu(rt, buf, routed, rank, e, m, h, fmt, slot_rows, capacity):
    """The exchange-metadata records for `routed`, then the receive side fed from the per-source buffer."""
    lib, capi = rt.capi.load(), rt.capi
    r = routed.shape[0]
    meta = rt.ll.exchange_metadata(routed.cuda(), rank, slot_rows, capacity)
    shape = rt.ll.LLShape(num_ranks=r, rank=rank, num_experts=e, max_tokens=m, hidden=h, num_topk=1, fmt=fmt)
    st = rt.ll.LowLatencyState(shape, keep_remote_rows=False)
    poison_outputs(st)
    ws = torch.empty(lib.deepep_ll_by_source_workspace_bytes(e, capacity), dtype=torch.uint8, device="cuda")
    tokens_per_expert = torch.full((e // r,), 77, dtype=torch.int32, device="cuda")
    dev = buf.cuda()
    capi.check(lib.deepep_ll_dispatch_recv_by_source(
        capi.ptr(dev), slot_rows, capi.ptr(meta["recv_counts"]), capi.ptr(meta["source_offset"]),
        capi.ptr(meta["num_recv_tokens"]), capacity, h, e, r, m, fmt, capi.ptr(st.packed_recv_x),
        capi.ptr(st.packed_recv_scales), capi.ptr(st.packed_recv_src_info), capi.ptr(st.packed_recv_layout_range),
        capi.ptr(st.packed_recv_count), None, capi.ptr(tokens_per_expert), None, 0, capi.ptr(ws), ws.numel(),
        torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return st, tokens_per_expert, meta


@pytest.mark.parametrize("fmt", [O.ROW_FP8, O.ROW_BF16, O.ROW_FP8_UE8M0])
@pytest.mark.parametrize("r,rank,t,h,k,e", [
    (4, 1, 8, 512, 3, 16), (8, 7, 33, 1024, 4, 64), (2, 0, 1, 512, 1, 2),
    (32, 5, 128, 7168, 8, 256),   # the headline shape
    (8, 3, 700, 512, 8, 256),     # past 4096 records: chunk histograms, sources of two chunks each
    (4, 1, 900, 512, 4, 16),      # up to 4096 records: one workgroup per source walks its two chunks, running counts
    (16, 2, 1200, 512, 8, 64),    # 9600 records in chunks of 512, about 600 per source
    (16, 5, 4096, 512, 8, 64),    # 32768 records: four chunks per source, 80 chunk workgroups
    (1, 0, 16, 512, 2, 4),        # a world of one rank
    (4, 2, 64, 512, 2, 4),        # one expert per rank
    (2, 1, 40, 512, 6, 2048),     # 1024 local experts: ten bits of expert id
])
def test_dispatch_recv_by_source(rt, fmt, r, rank, t, h, k, e):
    """Rows delivered grouped by source rank + the exchange-metadata records give the packed outputs of
    the staged receive, i.e. the same oracle outputs (csrc/kernels/efa_kernels.cu:877-1052,1227-1389)."""
    x_all, topk_all, _ = make_world(r, t, h, k, e, seed=r * 31 + t, drop=min(5, t))
    m = t
    slot_rows = t * min(k, e // r)  # the most one source can send to one rank
    buf = rows_by_source(x_all, topk_all, rank, e, m, fmt, slot_rows)
    routed = torch.stack([O.route(topk_all[s], e, m)[0] for s in range(r)]).to(torch.int32)
    capacity = int(routed[:, rank * (e // r):(rank + 1) * (e // r)].sum()) + 5
    st, tokens_per_expert, meta = recv_by_source_on_gpu(rt, buf, routed, rank, e, m, h, fmt, slot_rows, capacity)
    want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, m, fmt)
    check_dispatch(st, want, fmt)
    assert torch.equal(tokens_per_expert.cpu(), want["packed_recv_count"])
    assert int(meta["num_recv_tokens"][0]) == int(want["packed_recv_count"].sum())


@pytest.mark.parametrize("seed", range(int(os.environ.get("DEEPEP_TEST_RANDOM_SHAPES", "24"))))
def test_dispatch_recv_by_source_seeded_random_shapes(rt, seed):
    """The by-source receive on shapes nobody picked by hand, on both sides of its 4096-record bound."""
    r, rank, t, _, h, k, e, fmt, drop = _random_shape(seed)
    if seed % 3 == 0:
        t = t * 7  # more records: sources of several chunks
    x_all, topk_all, _ = make_world(r, t, h, k, e, seed=2000 + seed, drop=drop)
    m = t
    slot_rows = t * min(k, e // r)
    buf = rows_by_source(x_all, topk_all, rank, e, m, fmt, slot_rows)
    routed = torch.stack([O.route(topk_all[s], e, m)[0] for s in range(r)]).to(torch.int32)
    capacity = int(routed[:, rank * (e // r):(rank + 1) * (e // r)].sum()) + seed % 4
    st, tokens_per_expert, meta = recv_by_source_on_gpu(rt, buf, routed, rank, e, m, h, fmt, slot_rows, capacity)
    want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, m, fmt)
    check_dispatch(st, want, fmt)
    assert torch.equal(tokens_per_expert.cpu(), want["packed_recv_count"])


@pytest.mark.parametrize("t", [24, 1500], ids=["one_workgroup_per_source", "chunked"])
def test_dispatch_recv_by_source_drops_what_does_not_fit(rt, t):
    """A slot of M rows per source, as the reference sizes it (csrc/transport/ll_pipeline.cpp:1527): rows a
    source sends beyond it are lost, the others land as if the lost ones had not been sent; and with fewer
    record slots than rows, only the rows that have a record are received."""
    r, rank, h, k, e, fmt = 2, 0, 512, 4, 8, O.ROW_FP8
    x_all, topk_all, _ = make_world(r, t, h, k, e, seed=3, drop=0)
    topk_all[1, :, :] = torch.tensor([0, 1, 2, 3])  # every token of source 1 names all of rank 0's experts
    slot_rows = t  # source 1 sends 4 * t rows
    buf = rows_by_source(x_all, topk_all, rank, e, t, fmt, slot_rows)
    routed = torch.stack([O.route(topk_all[s], e, t)[0] for s in range(r)]).to(torch.int32)
    for capacity in (4 * t * r, t // 2 + 3):
        st, _, meta = recv_by_source_on_gpu(rt, buf, routed, rank, e, t, h, fmt, slot_rows, capacity)
        recv_counts = meta["recv_counts"].cpu().tolist()
        # expected: walk the records the way the kernel may use them
        epr, n = e // r, 0
        want_rows = [[[] for _ in range(r)] for _ in range(epr)]
        tail_at = O.row_payload(h, fmt) - 16
        tail = buf[:, tail_at:tail_at + 16].contiguous().view(torch.int32)
        for s in range(r):
            for j in range(recv_counts[s]):
                if n < capacity and j < slot_rows:
                    row = s * slot_rows + j
                    want_rows[int(tail[row, 3])][s].append(row)
                n += 1
        count = st.packed_recv_count.cpu().tolist()
        layout = st.packed_recv_layout_range.cpu()
        px = st.packed_recv_x.view(torch.uint8).cpu()
        for le in range(epr):
            begin = 0
            for s in range(r):
                rows = want_rows[le][s]
                assert int(layout[le, s]) == (((begin << 32) | len(rows)) if rows else 0), (capacity, le, s)
                if rows:
                    idx = torch.tensor(rows)
                    assert torch.equal(px[le, begin:begin + len(rows)], buf[idx, :h])
                    assert torch.equal(st.packed_recv_src_info[le, begin:begin + len(rows)].cpu(), tail[idx, 0])
                begin += len(rows)
            assert count[le] == begin


def _random_shape(seed):
    g = np.random.default_rng(seed)
    r = int(g.choice([1, 2, 3, 4, 5, 6, 8, 12, 16, 24]))
    epr = int(g.choice([1, 2, 3, 5, 8, 16]))
    e = r * epr
    k = int(g.integers(1, min(e, 12) + 1))
    t = int(g.choice([1, 2, 7, 31, 64, 100, 129, 257, 300, 1100]))
    m = t + int(g.choice([0, 0, 1, 13, 64]))  # room for more tokens than the batch holds
    h = int(g.choice([128, 256, 384, 640, 1024, 2048, 2176]))
    fmt = int(g.choice([O.ROW_FP8, O.ROW_BF16, O.ROW_FP8_POW2]))
    rank, drop = int(g.integers(0, r)), int(g.integers(0, min(40, t * k) + 1))
    if h % 512 == 0 and int(g.integers(0, 3)) == 0:
        fmt = O.ROW_FP8_UE8M0  # packed exponent bytes need whole groups of four scales
    return r, rank, t, m, h, k, e, fmt, drop


@pytest.mark.parametrize("seed", range(int(os.environ.get("DEEPEP_TEST_RANDOM_SHAPES", "24"))))
@ONE_CALL
def test_dispatch_and_combine_seeded_random_shapes(rt, seed, one_call):
    """Shapes nobody picked by hand: odd world sizes, hidden sizes with a ragged last piece, more slots
    than tokens, many or no dropped selections.  Dispatch bit-exact, combine against the float32 chain."""
    r, rank, t, m, h, k, e, fmt, drop = _random_shape(seed)
    x_all, topk_all, w_all = make_world(r, t, h, k, e, seed=1000 + seed, drop=drop)
    st, world = dispatch_on_gpu(rt, x_all, topk_all, rank, e, m, fmt, one_call=one_call)
    want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, m, fmt)
    check_dispatch(st, want, fmt)
    send_count, pair_slot = O.route(topk_all[rank], e, m)
    assert torch.equal(st.send_count.cpu(), send_count)
    assert torch.equal(st.pair_slot[:t].cpu(), pair_slot)
    # combine with the identity expert: every pair returns the row it was sent, so out = x * sum of weights
    epr = e // r
    y = torch.zeros((epr, r * m, h), dtype=torch.bfloat16)
    count = st.packed_recv_count.cpu()
    for le in range(epr):
        n = int(count[le])
        if fmt == O.ROW_BF16:
            y[le, :n] = st.packed_recv_x[le, :n].cpu()
        else:
            y[le, :n] = O.per_token_cast_back(st.packed_recv_x[le, :n].cpu(), st.packed_recv_scales[le, :n].cpu())
    out = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
    run_combine(st, world, y.cuda(), topk_all[rank].cuda(), w_all[rank].cuda(), out, mode=0, one_call=one_call)
    wsum = w_all[rank].masked_fill(topk_all[rank] == -1, 0).sum(1).view(-1, 1)
    expect = x_all[rank].float() * wsum
    got = out.cpu().float()
    assert torch.isnan(got).sum().item() == 0
    live = wsum.view(-1) > 0
    assert (got[~live] == 0).all()  # a token with no valid selection combines to zero
    if live.any():
        diff = O.calc_diff(expect[live], got[live])
        assert diff < (2e-3 if fmt != O.ROW_BF16 else 1e-4), (diff, (r, rank, t, m, h, k, e, fmt))


def test_dispatch_send_staging_and_send_slots(rt):
    """The send side alone: own rows for own experts land in recv_staging, the rest in send_slots."""
    r, rank, t, h, k, e, m = 4, 2, 20, 512, 4, 32, 24
    x_all, topk_all, _ = make_world(r, t, h, k, e, seed=5, drop=6)
    shape = rt.ll.LLShape(r, rank, e, m, h, k, O.ROW_FP8)
    st = rt.ll.LowLatencyState(shape)
    st.recv_staging.fill_(0xAB)
    st.send_slots.fill_(0xCD)
    st.dispatch_send(x_all[rank].cuda(), topk_all[rank].cuda())
    torch.cuda.synchronize()
    send_count, pair_slot, experts, slots, rows = O.staged_rows(x_all[rank], topk_all[rank], rank, e, m, O.ROW_FP8, r)
    assert torch.equal(st.send_count.cpu(), send_count)
    assert torch.equal(st.pair_slot[:t].cpu(), pair_slot)
    stride = st.stride
    staging = st.recv_staging.cpu().view(e // r, r, m, stride)
    sendbuf = st.send_slots.cpu().view(e, m, stride)
    epr = e // r
    touched_stage = torch.zeros((epr, r, m), dtype=torch.bool)
    touched_send = torch.zeros((e, m), dtype=torch.bool)
    payload = O.row_payload(h, O.ROW_FP8)
    assert stride == O.row_stride(h, O.ROW_FP8) == 640 and payload == 544  # a row takes whole 128-byte lines
    for i in range(rows.shape[0]):
        ex, sl = int(experts[i]), int(slots[i])
        if ex // epr == rank:
            got, fill = staging[ex % epr, rank, sl], 0xAB
            touched_stage[ex % epr, rank, sl] = True
        else:
            got, fill = sendbuf[ex, sl], 0xCD
            touched_send[ex, sl] = True
        assert torch.equal(got[:payload], rows[i, :payload])
        assert (got[payload:] == fill).all()  # nothing is written behind the tail
    assert (staging[~touched_stage] == 0xAB).all() and (sendbuf[~touched_send] == 0xCD).all()
    rc = st.recv_count.cpu().view(epr, r)
    assert torch.equal(rc[:, rank], send_count[rank * epr:(rank + 1) * epr])
    assert (rc[:, [s for s in range(r) if s != rank]] == 0).all()


@ONE_CALL
@pytest.mark.parametrize("use_fp8", [True, False])
def test_reference_recipe_roundtrip(rt, use_fp8, one_call):
    """tests/test_low_latency.py:59-60,113-147,181-184 on one rank of an 8-rank world."""
    r, rank, t, h, k, e = 8, 3, 64, 2048, 6, 64
    fmt = O.ROW_FP8 if use_fp8 else O.ROW_BF16
    x_all, topk_all, w_all = make_world(r, t, h, k, e, seed=77, drop=10, recipe="rank_const")
    stats = torch.zeros(e // r, dtype=torch.int32, device="cuda")
    st, world = dispatch_on_gpu(rt, x_all, topk_all, rank, e, t, fmt, stats, one_call=one_call)
    epr = e // r
    count = st.packed_recv_count.cpu()
    lr_all = st.packed_recv_layout_range.cpu()
    assert torch.equal(stats.cpu(), count)
    for i in range(epr):
        expert = rank * epr + i
        n = int(count[i])
        lr = lr_all[i]
        assert n == int((lr & 0xFFFFFFFF).sum()) == int((topk_all == expert).sum())
        if n == 0:
            continue
        if use_fp8:
            recv = O.per_token_cast_back(st.packed_recv_x[i, :n].cpu(), st.packed_recv_scales[i, :n].cpu()).float()
        else:
            recv = st.packed_recv_x[i, :n].cpu().float()
        src = st.packed_recv_src_info[i, :n].cpu()
        assert torch.equal(recv[:, :-128].amin(-1), recv[:, :-128].amax(-1))
        assert (recv[:, -128:] - src.view(-1, 1) % t).sum().item() == 0
        for j in range(r):
            begin, cnt = int(lr[j] >> 32), int(lr[j] & 0xFFFFFFFF)
            assert int((recv[:, :-128].amin(-1) == j - 128).sum()) == int((topk_all[j] == expert).sum())
            assert (recv[begin:begin + cnt, :-128] - j + 128).sum().item() == 0
    # combine with an identity expert (simulated_gemm_x = dequantised recv)
    if use_fp8:
        el, n_slots = st.packed_recv_x.shape[:2]
        q = st.packed_recv_x.view(-1, h).cpu()
        sc = st.packed_recv_scales.view(-1, h // 128).cpu()
        live = torch.zeros((el, n_slots), dtype=torch.bool)
        for i in range(el):
            live[i, :int(count[i])] = True
        y = torch.zeros((el * n_slots, h), dtype=torch.bfloat16)
        y[live.view(-1)] = O.per_token_cast_back(q[live.view(-1)], sc[live.view(-1)])
        y = y.view(el, n_slots, h).cuda()
    else:
        y = st.packed_recv_x.clone()
    out = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
    topk, w = topk_all[rank].cuda(), w_all[rank].cuda()
    run_combine(st, world, y, topk, w, out, mode=0, one_call=one_call)
    x = x_all[rank]
    wsum = w_all[rank].masked_fill(topk_all[rank] == -1, 0).sum(1).view(-1, 1)
    diff = O.calc_diff(x.float() * wsum, out.cpu())
    assert torch.isnan(out.float()).sum().item() == 0
    assert diff < (9e-4 if use_fp8 else 1e-5), diff


@pytest.mark.parametrize("r,rank,t,h,k,e", [(32, 5, 128, 7168, 8, 256), (4, 0, 16, 512, 3, 8),
                                            (8, 3, 4200, 512, 4, 64),   # large-batch combine-send path
                                            (8, 3, 1024, 4096, 8, 64),  # the largest single launch: moves > 192 MB, so it streams
                                            (4, 2, 40, 512, 11, 64),    # more than eight selections per token
                                            (8, 6, 20, 512, 4, 512),    # more than 256 segments
                                            (4, 1, 33, 1536, 5, 32),    # hidden not a multiple of 512
                                            (128, 77, 9, 512, 4, 128),  # many ranks, one expert each
                                            (512, 500, 3, 512, 2, 1024)])
@ONE_CALL
def test_combine_random_expert_outputs(rt, oracle_c, r, rank, t, h, k, e, one_call):
    """Seeded expert outputs along the dispatch routing; combine vs the float32 chain and the float64 sum."""
    x_all, topk_all, w_all = make_world(r, t, h, k, e, seed=31 + r, drop=10)
    st, world = dispatch_on_gpu(rt, x_all, topk_all, rank, e, t, O.ROW_FP8, one_call=one_call)
    epr, n_slots, lib, capi = e // r, r * t, rt.capi.load(), rt.capi
    seed_local, seed_remote = 1234, 4321
    # local experts' outputs: row key = local_expert * N + slot
    y = torch.zeros((epr, n_slots, h), dtype=torch.bfloat16, device="cuda")
    capi.check(lib.deepep_synth_bf16_rows(capi.ptr(y), epr * n_slots, h, h * 2, None, 0, seed_local, 0,
                                          torch.cuda.current_stream().cuda_stream))
    out = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
    run_combine(st, world, y, topk_all[rank].cuda(), w_all[rank].cuda(), out, mode=1, seed=seed_remote,
                one_call=one_call)
    # oracle: which row does each of this rank's pairs get back?
    topk, w = topk_all[rank], w_all[rank]
    _, pair_slot = O.route(topk, e, t)
    want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, t, O.ROW_FP8)
    keys_local, keys_remote = [], []
    pair_rows = torch.zeros((t, k, h), dtype=torch.bfloat16)
    live = pair_slot >= 0
    idx_local, idx_remote = [], []
    for ti in range(t):
        for ki in range(k):
            if not live[ti, ki]:
                continue
            ex, sl = int(topk[ti, ki]), int(pair_slot[ti, ki])
            if ex // epr == rank:
                begin = int(want["packed_recv_layout_range"][ex % epr, rank] >> 32)
                keys_local.append((ex % epr) * n_slots + begin + sl)
                idx_local.append((ti, ki))
            else:
                keys_remote.append(ex * t + sl)
                idx_remote.append((ti, ki))
    if idx_local:
        rows = O.synth_bf16_rows(np.array(keys_local, dtype=np.uint32), h, seed_local)
        ii = torch.tensor(idx_local)
        pair_rows[ii[:, 0], ii[:, 1]] = rows
    if idx_remote:
        rows = O.synth_bf16_rows(np.array(keys_remote, dtype=np.uint32), h, seed_remote)
        ii = torch.tensor(idx_remote)
        pair_rows[ii[:, 0], ii[:, 1]] = rows
    chain = torch.empty((t, h), dtype=torch.int16)
    live8 = live.to(torch.uint8).contiguous()
    oracle_c.oracle_combine_chain(ctypes.c_void_p(pair_rows.view(torch.int16).data_ptr()),
                                  ctypes.c_void_p(w.contiguous().data_ptr()), ctypes.c_void_p(live8.data_ptr()), t, k,
                                  h, ctypes.c_void_p(chain.data_ptr()))
    got = out.cpu()
    assert torch.equal(got.view(torch.int16), chain), "combine differs from the float32 FMA chain"
    # accumulate: the sum starts from what `out` holds (csrc/kernels/coop_combine_recv.cuh:174-179)
    prev = torch.randn((t, h), generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    out2 = prev.cuda()
    if one_call:
        st.combine(y, topk_all[rank].cuda(), w_all[rank].cuda(), out2, accumulate=True)
    else:
        st.combine_recv(topk_all[rank].cuda(), w_all[rank].cuda(), out2, accumulate=True)
    torch.cuda.synchronize()
    want2 = O.ll_combine_f32_chain(pair_rows, w, live, initial=prev)
    assert torch.equal(out2.cpu().view(torch.int16), want2.view(torch.int16)), "accumulating combine"
    ref = O.ll_combine(pair_rows, topk, w, live)
    err = (got.double() - ref).abs()
    assert (err <= 1e-2 * ref.abs() + 1e-2 * ref.abs().mean()).all()
    assert O.calc_diff(got, ref) < 1e-5


@ONE_CALL
@pytest.mark.parametrize("e,rank", [(256, 11), (288, 7)])  # 288 experts: the reference's own LL test, nine per rank
def test_ll_config_full_size(rt, one_call, e, rank):
    """One GPU's share of EP=32 at 128 tokens x 7168, top-8 of 256 (or 288) experts, seeded world."""
    r, t, h, k = 32, 128, 7168, 8
    shape = rt.ll.LLShape(r, rank, e, t, h, k, O.ROW_FP8)
    st = rt.ll.LowLatencyState(shape)
    world = rt.lb.LoopbackWorld(r, rank, seed=2024)
    world.synthesise(t, h, k, e)
    x, topk = world.own_inputs()
    run_dispatch(st, world, x, topk, one_call=one_call)
    # the oracle regenerates the same world from the seed
    topk_all = O.synth_topk_idx(O.uniform_cdf(e), np.arange(r), t, k, 2024)
    assert torch.equal(world.topk_idx_all.cpu(), topk_all)
    x_all = O.synth_bf16_rows(np.arange(r * t, dtype=np.uint32), h, 2024).view(r, t, h)
    assert torch.equal(world.x_all.cpu().view(torch.int16), x_all.view(torch.int16))
    want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, t, O.ROW_FP8)
    check_dispatch(st, want, O.ROW_FP8)
    assert int(st.packed_recv_count.sum()) == int(((topk_all // (e // r)) == rank).sum())


@ONE_CALL
def test_skewed_routing_roundtrip(rt, one_call):
    """Zipf(1.2) popularity, 1 % outlier rows, EP=64 with 4 local experts, hot experts past half their slots."""
    r, rank, t, h, k, e = 64, 0, 256, 1024, 8, 256
    shape = rt.ll.LLShape(r, rank, e, t, h, k, O.ROW_FP8)
    st = rt.ll.LowLatencyState(shape)
    world = rt.lb.LoopbackWorld(r, rank, seed=99)
    world.synthesise(t, h, k, e, popularity="zipf", outlier_period=100)
    x, topk = world.own_inputs()
    run_dispatch(st, world, x, topk, one_call=one_call)
    topk_all = O.synth_topk_idx(O.zipf_cdf(e), np.arange(r), t, k, 99)
    x_all = O.synth_bf16_rows(np.arange(r * t, dtype=np.uint32), h, 99, outlier_period=100).view(r, t, h)
    assert torch.equal(world.topk_idx_all.cpu(), topk_all)
    assert torch.equal(world.x_all.cpu().view(torch.int16), x_all.view(torch.int16))
    want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, t, O.ROW_FP8)
    check_dispatch(st, want, O.ROW_FP8)
    assert int(st.packed_recv_count[0]) > r * t // 2, "the hottest expert should fill over half its slots"
    # round trip with identity experts: combined == x * sum(w) within FP8 error
    count = st.packed_recv_count.cpu()
    el, n_slots = st.packed_recv_x.shape[:2]
    y = torch.zeros((el, n_slots, h), dtype=torch.bfloat16)
    for i in range(el):
        n = int(count[i])
        y[i, :n] = O.per_token_cast_back(st.packed_recv_x[i, :n].cpu(), st.packed_recv_scales[i, :n].cpu())
    g = torch.Generator().manual_seed(1)
    w = torch.softmax(torch.randn((t, k), generator=g), dim=-1)
    out = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
    run_combine(st, world, y.cuda(), topk, w.cuda(), out, mode=0, one_call=one_call)
    diff = O.calc_diff(x_all[rank].float() * w.sum(1, keepdim=True), out.cpu())
    assert diff < 9e-4, diff


def test_ll_argument_errors(rt):
    lib, capi = rt.capi.load(), rt.capi
    z = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    # tokens beyond num_max_dispatch_tokens_per_rank
    rc = lib.deepep_ll_dispatch_send(capi.ptr(z), capi.ptr(z), 9, 128, 2, 8, 2, 0, 8, 1, capi.ptr(z), capi.ptr(z),
                                     capi.ptr(z), capi.ptr(z), capi.ptr(z), capi.ptr(z), 4096, s)
    assert rc != 0 and "num_tokens <= max_tokens" in lib.deepep_last_error().decode()
    # experts not divisible by ranks
    rc = lib.deepep_ll_dispatch_recv(capi.ptr(z), capi.ptr(z), 128, 9, 2, 8, 1, capi.ptr(z), capi.ptr(z), capi.ptr(z),
                                     capi.ptr(z), capi.ptr(z), None, 0, None, 0, s)
    assert rc != 0 and "num_experts % num_ranks == 0" in lib.deepep_last_error().decode()
    # workspace too small
    rc = lib.deepep_ll_dispatch_send(capi.ptr(z), capi.ptr(z), 8, 128, 2, 8, 2, 0, 8, 1, capi.ptr(z), capi.ptr(z),
                                     capi.ptr(z), capi.ptr(z), capi.ptr(z), capi.ptr(z), 16, s)
    assert rc != 0 and "workspace_bytes" in lib.deepep_last_error().decode()
    torch.cuda.synchronize()


@ONE_CALL
def test_empty_batch(rt, one_call):
    """No tokens on this rank: counts come from the peers alone, combine returns nothing."""
    r, rank, t, h, k, e = 4, 2, 6, 512, 2, 8
    x_all, topk_all, _ = make_world(r, t, h, k, e, seed=8, drop=0)
    shape = rt.ll.LLShape(r, rank, e, t, h, k, O.ROW_FP8)
    st = rt.ll.LowLatencyState(shape)
    world = rt.lb.LoopbackWorld(r, rank)
    world.set_inputs(x_all.cuda(), topk_all.cuda())
    run_dispatch(st, world, x_all[rank, :0].cuda(), topk_all[rank, :0].cuda(), one_call=one_call)
    xs, tks = list(x_all), list(topk_all)
    xs[rank], tks[rank] = xs[rank][:0], tks[rank][:0]
    want = O.ll_dispatch(xs, tks, rank, e, t, O.ROW_FP8)
    check_dispatch(st, want, O.ROW_FP8)
    assert (st.send_count == 0).all()


def test_large_batch_without_the_segment_workspace(rt, oracle_c):
    """A large batch but no workspace for the row index: receive and row return fall back to the
    kernels of the small-batch path and must give the same answers."""
    r, rank, t, h, k, e = 8, 5, 4200, 512, 4, 64
    x_all, topk_all, w_all = make_world(r, t, h, k, e, seed=77, drop=10)
    shape = rt.ll.LLShape(num_ranks=r, rank=rank, num_experts=e, max_tokens=t, hidden=h, num_topk=k, fmt=O.ROW_FP8)
    st = rt.ll.LowLatencyState(shape)
    assert st.segment_workspace is not None
    st.segment_workspace = None
    world = rt.lb.LoopbackWorld(r, rank, seed=0)
    world.set_inputs(x_all.cuda(), topk_all.cuda())
    x, topk = world.own_inputs()
    run_dispatch(st, world, x, topk)
    want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, t, O.ROW_FP8)
    check_dispatch(st, want, O.ROW_FP8)
    # identity experts: the round trip returns x * sum(w) within the FP8 error
    count = st.packed_recv_count.cpu()
    y = torch.zeros((e // r, r * t, h), dtype=torch.bfloat16)
    for le in range(e // r):
        n = int(count[le])
        y[le, :n] = O.per_token_cast_back(st.packed_recv_x[le, :n].cpu(), st.packed_recv_scales[le, :n].cpu())
    out = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
    w = torch.softmax(w_all[rank], dim=-1)
    run_combine(st, world, y.cuda(), topk, w.cuda(), out, mode=0)
    wsum = w.masked_fill(topk_all[rank] == -1, 0).sum(1, keepdim=True)
    assert O.calc_diff(x_all[rank].float() * wsum, out.cpu()) < 9e-4


@pytest.mark.parametrize("zero_copy", [False, True], ids=["rows_returned", "zero_copy"])
@pytest.mark.parametrize("fmt", [O.ROW_FP8, O.ROW_BF16])
def test_every_rank_on_one_gpu_with_a_real_exchange(rt, fmt, zero_copy):
    """All R ranks run on the one GPU, each with its own buffers, and the exchange between them is a
    plain copy of what the send sides produced (send_slots -> the peer's recv_staging, then
    combine_send_slots -> the peer's combine_staging).  Nothing is synthesised "in a peer's name":
    this is the data flow of a multi-GPU run with the transport replaced by device copies.
    zero_copy: the combine returns no rows; the exchange takes each (expert, source) range straight
    from the expert outputs, where layout_range says it lies."""
    r, t, h, k, e = 4, 12, 512, 3, 16
    epr = e // r
    x_all, topk_all, w_all = make_world(r, t, h, k, e, seed=123, drop=4)
    states = []
    for rank in range(r):
        st = rt.ll.LowLatencyState(rt.ll.LLShape(r, rank, e, t, h, k, fmt))
        st.recv_count.zero_()
        st.dispatch_send(x_all[rank].cuda(), topk_all[rank].cuda())
        states.append(st)
    torch.cuda.synchronize()
    # the dispatch exchange: rank s's rows for expert e travel to the rank that owns e
    for s in range(r):
        src = states[s]
        slots = src.send_slots.view(e, t, src.stride)
        counts = src.send_count.cpu()
        for ex in range(e):
            dst_rank, le = ex // epr, ex % epr
            if dst_rank == s:
                continue
            cnt = int(counts[ex])
            dst = states[dst_rank]
            dst.recv_staging.view(epr, r, t, dst.stride)[le, s, :cnt] = slots[ex, :cnt]
            dst.recv_count.view(epr, r)[le, s] = cnt
    outs = []
    for rank in range(r):
        st = states[rank]
        poison_outputs_keep_pair_slot(st)
        st.dispatch_recv()
        torch.cuda.synchronize()
        want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, t, fmt)
        check_dispatch(st, want, fmt)
        # identity experts
        if fmt == O.ROW_BF16:
            y = st.packed_recv_x.clone()
        else:
            q = st.packed_recv_x.float().view(epr, r * t, h // 128, 128)
            y = (q * st.packed_recv_scales.unsqueeze(-1)).view(epr, r * t, h).to(torch.bfloat16)
        y = torch.nan_to_num(y, nan=0.0, posinf=0.0, neginf=0.0)  # rows past the counts hold poison
        if not zero_copy:
            st.combine_send(y)
        outs.append(y)
    torch.cuda.synchronize()
    # the combine exchange: what rank q returns for rank s's pairs goes to s's staging for q's experts
    for q in range(r):
        src = states[q]
        back = src.combine_send_slots  # [E_l, R, M, H]
        lr = src.packed_recv_layout_range.cpu()
        for le in range(epr):
            for s in range(r):
                if s == q:
                    continue
                begin, cnt = int(lr[le, s] >> 32), int(lr[le, s] & 0xFFFFFFFF)
                if zero_copy:
                    states[s].combine_staging[q * epr + le, :cnt] = outs[q][le, begin:begin + cnt]
                else:
                    states[s].combine_staging[q * epr + le, :cnt] = back[le, s, :cnt]
    for rank in range(r):
        st = states[rank]
        out = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
        out.view(torch.int16).fill_(0x7FC0)
        topk, w = topk_all[rank].cuda(), w_all[rank].cuda()
        if zero_copy:
            st.combine_send_slots.view(torch.int16).fill_(0x7FC0)
            st.combine(outs[rank], topk, w, out, zero_copy=True)  # the own experts' rows are read from the outputs
        else:
            st.combine_recv(topk, w, out)
        torch.cuda.synchronize()
        if zero_copy:
            assert (st.combine_send_slots.view(torch.int16) == 0x7FC0).all()
        wsum = w_all[rank].masked_fill(topk_all[rank] == -1, 0).sum(1, keepdim=True)
        diff = O.calc_diff(x_all[rank].float() * wsum, out.cpu())
        assert not torch.isnan(out.float()).any()
        assert diff < (9e-4 if fmt != O.ROW_BF16 else 1e-5), (rank, diff)


def poison_outputs_keep_pair_slot(st):
    st.packed_recv_x.view(torch.uint8).fill_(0xEE)
    if st.packed_recv_scales is not None:
        st.packed_recv_scales.view(torch.uint8).fill_(0xEE)
    st.packed_recv_src_info.fill_(-7)
    st.packed_recv_count.fill_(-7)
    st.packed_recv_layout_range.fill_(-7)


def test_exchange_metadata_through_the_host_module(rt):
    """The pybind11 binding returns the same values as the C-ABI call, and rejects a host tensor."""
    from deepep_efa_amd import deep_ep_cpp
    r, e, m, rank, cap = 8, 64, 50, 3, 512
    g = torch.Generator().manual_seed(77)
    routed = torch.randint(0, m + 1, (r, e), generator=g, dtype=torch.int32)
    send, recv, totals, remote, records, num_recv, per_expert = deep_ep_cpp.ll_exchange_metadata(routed.cuda(), rank, m, cap)
    torch.cuda.synchronize()
    want = O.ll_exchange_metadata(routed, rank, m)
    n = min(want["total_recv"], cap)
    assert send.cpu().tolist() == want["send_counts"].tolist() and recv.cpu().tolist() == want["recv_counts"].tolist()
    assert totals.cpu().tolist() == [want["total_send"], want["total_recv"], 0]
    assert remote.cpu().tolist() == want["combine_remote_recv_offset"].tolist()
    assert num_recv.cpu().tolist() == [want["total_recv"], n] and (per_expert == 0).all()
    for i, key in enumerate(("source_rank", "source_offset", "padded_index", "combine_send_offset")):
        assert records[i, :n].cpu().tolist() == want[key][:n].tolist(), key
    with pytest.raises(RuntimeError, match="Assertion"):
        deep_ep_cpp.ll_exchange_metadata(routed, rank, m, cap)


@pytest.mark.parametrize("hint", ["batch", "unknown", "huge"])
def test_capacity_far_above_the_batch(rt, hint):
    """A caller may size M for its largest batch and dispatch a small one.  The kernels are picked from the
    expected-rows hint, not from the capacity, and every hint gives the same result."""
    r, rank, t, m, h, k, e = 8, 2, 40, 5000, 512, 4, 64
    x_all, topk_all, w_all = make_world(r, t, h, k, e, seed=4242, drop=7)
    shape = rt.ll.LLShape(num_ranks=r, rank=rank, num_experts=e, max_tokens=m, hidden=h, num_topk=k, fmt=O.ROW_FP8)
    st = rt.ll.LowLatencyState(shape)
    st.expected_rows = {"batch": t * k, "unknown": 0, "huge": 10 ** 6}[hint]
    if st.segment_workspace is None:
        st.segment_workspace = torch.empty(rt.capi.load().deepep_ll_segment_workspace_bytes(e, m), dtype=torch.uint8,
                                           device="cuda")
    world = rt.lb.LoopbackWorld(r, rank, seed=0)
    world.set_inputs(x_all.cuda(), topk_all.cuda())
    x, topk = world.own_inputs()
    run_dispatch(st, world, x, topk, None, one_call=True)
    single = rt.capi.load().deepep_ll_dispatch_is_single_launch(t, k, e, m, st.expected_rows) == 1
    assert single == (hint == "batch")
    want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, m, O.ROW_FP8)
    check_dispatch(st, want, O.ROW_FP8)
    # combine with identity experts
    epr = e // r
    y = torch.zeros((epr, r * m, h), dtype=torch.bfloat16)
    count = st.packed_recv_count.cpu()
    for le in range(epr):
        n = int(count[le])
        y[le, :n] = O.per_token_cast_back(st.packed_recv_x[le, :n].cpu(), st.packed_recv_scales[le, :n].cpu())
    out = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
    run_combine(st, world, y.cuda(), topk_all[rank].cuda(), w_all[rank].cuda(), out, mode=0, one_call=True)
    wsum = w_all[rank].masked_fill(topk_all[rank] == -1, 0).sum(1).view(-1, 1)
    live = wsum.view(-1) > 0
    assert O.calc_diff((x_all[rank].float() * wsum)[live], out.cpu().float()[live]) < 2e-3


@ONE_CALL
@pytest.mark.parametrize("fmt", [O.ROW_FP8, O.ROW_BF16])
def test_tokens_naming_an_expert_more_than_once(rt, fmt, one_call):
    """Top-k never does it, but the path defines it: every pair gets its own slot in (token, k) order, and
    pairs beyond the M slots of a (source, expert) segment are dropped (slot -1, not counted, not combined)."""
    r, rank, t, m, h, k, e = 2, 1, 6, 6, 256, 4, 4
    g = torch.Generator().manual_seed(5)
    x_all = torch.randn((r, t, h), generator=g).to(torch.bfloat16)
    topk_all = torch.tensor([[[3, 3, 3, 3]] * t,                       # 24 pairs for expert 3: 6 kept, 18 dropped
                             [[2, 2, 0, -1], [2, 3, 3, 1], [0, 0, 0, 0], [2, 1, 2, 1], [-1, -1, 3, 3], [2, 2, 2, 2]]])
    w_all = torch.rand((r, t, k), generator=g) + 0.1
    st, world = dispatch_on_gpu(rt, x_all, topk_all, rank, e, m, fmt, one_call=one_call)
    want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, m, fmt)
    check_dispatch(st, want, fmt)
    send_count, pair_slot = O.route(topk_all[rank], e, m)
    assert torch.equal(st.send_count.cpu(), send_count) and torch.equal(st.pair_slot[:t].cpu(), pair_slot)
    # what rank 0 sent to expert 3 (on rank 1): exactly M rows, the first M pairs in (token, k) order
    lr = int(st.packed_recv_layout_range[1, 0])
    assert lr & 0xFFFFFFFF == m
    assert st.packed_recv_src_info[1, (lr >> 32):(lr >> 32) + m].cpu().tolist() == [0, 0, 0, 0, 1, 1]
    # combine: identity experts on the received rows; dropped pairs contribute nothing
    epr = e // r
    y = torch.zeros((epr, r * m, h), dtype=torch.bfloat16)
    count = st.packed_recv_count.cpu()
    for le in range(epr):
        n = int(count[le])
        if fmt == O.ROW_BF16:
            y[le, :n] = st.packed_recv_x[le, :n].cpu()
        else:
            y[le, :n] = O.per_token_cast_back(st.packed_recv_x[le, :n].cpu(), st.packed_recv_scales[le, :n].cpu())
    out = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
    run_combine(st, world, y.cuda(), topk_all[rank].cuda(), w_all[rank].cuda(), out, mode=0, one_call=one_call)
    live = pair_slot >= 0
    back = x_all[rank] if fmt == O.ROW_BF16 else O.per_token_cast_back(*O.per_token_cast_to_fp8(x_all[rank]))
    chain = O.ll_combine_f32_chain(back.unsqueeze(1).expand(-1, k, -1).contiguous(), w_all[rank], live)
    assert torch.equal(out.cpu().view(torch.int16), chain.view(torch.int16))


@ONE_CALL
@pytest.mark.parametrize("fmt", [O.ROW_FP8, O.ROW_BF16])
def test_send_past_the_streaming_bound(rt, one_call, fmt):
    """2800 tokens x 7168, top-8: the send moves more than 192 MB, so its payload stores carry the
    non-temporal hint (a different kernel instantiation); every output must be what the oracle says."""
    r, rank, t, h, k, e = 2, 1, 2800, 7168, 8, 16
    x_all, topk_all, _ = make_world(r, t, h, k, e, seed=2800, drop=10)
    assert t * (2 * h + k * O.row_payload(h, fmt)) > 192 * 2 ** 20
    st, _ = dispatch_on_gpu(rt, x_all, topk_all, rank, e, t, fmt, one_call=one_call)
    want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, t, fmt)
    check_dispatch(st, want, fmt)
    send_count, pair_slot = O.route(topk_all[rank], e, t)
    assert torch.equal(st.send_count.cpu(), send_count)
    assert torch.equal(st.pair_slot.cpu(), pair_slot)
    # the rows for the other rank's experts, byte for byte, on a sample of pairs
    _, _, experts, slots, rows = O.staged_rows(x_all[rank][:64], topk_all[rank][:64], rank, e, t, fmt, r)
    payload = O.row_payload(h, fmt)
    sendbuf = st.send_slots.view(e, t, st.stride)
    for i in range(0, rows.shape[0], 7):
        ex, sl = int(experts[i]), int(slots[i])
        if ex // (e // r) != rank:
            assert torch.equal(sendbuf[ex, sl, :payload].cpu(), rows[i, :payload]), (ex, sl)


@pytest.mark.parametrize("fmt", [O.ROW_FP8, O.ROW_BF16])
def test_every_rank_on_one_gpu_through_an_all_to_all(rt, fmt):
    """The data flow of the all_to_all_single fallback (deep_ep/buffer.py:2268,2297) with all R ranks on the
    one GPU: every rank's send side fills its per-expert slots; the "all-gather" of the route counts is the
    stack of the ranks' send_count; each rank's message to rank d is its rows for d's experts, expert by
    expert, copied into slot `source` of d's receive buffer; deepep_ll_exchange_metadata turns the gathered
    counts into the records and deepep_ll_dispatch_recv_by_source unpacks.  The packed outputs must be the
    oracle's (csrc/kernels/efa_kernels.cu:877-1052,1227-1389; csrc/transport/ll_pipeline.cpp:1204-1361)."""
    r, t, h, k, e = 4, 40, 512, 3, 16
    epr = e // r
    x_all, topk_all, _ = make_world(r, t, h, k, e, seed=321, drop=6)
    lib, capi = rt.capi.load(), rt.capi
    states = []
    for rank in range(r):
        st = rt.ll.LowLatencyState(rt.ll.LLShape(r, rank, e, t, h, k, fmt))
        st.dispatch_send(x_all[rank].cuda(), topk_all[rank].cuda())
        states.append(st)
    torch.cuda.synchronize()
    routed = torch.stack([st.send_count for st in states])  # [R, E]: what an all-gather of the counts leaves everywhere
    slot_rows = t * min(k, epr)
    stride = states[0].stride
    for rank in range(r):
        # the messages: source s -> this rank, rows in expert-major order (inside an expert, slot order)
        buf = torch.full((r * slot_rows, stride), 0xEE, dtype=torch.uint8, device="cuda")
        for s in range(r):
            src = states[s]
            counts = src.send_count.cpu()
            if s == rank:  # a rank's rows for its own experts were staged, not put into send slots
                own = src.recv_staging.view(epr, r, t, stride)
                parts = [own[le, rank, :int(counts[rank * epr + le])] for le in range(epr)]
            else:
                slots = src.send_slots.view(e, t, stride)
                parts = [slots[ex, :int(counts[ex])] for ex in range(rank * epr, (rank + 1) * epr)]
            msg = torch.cat(parts)
            buf[s * slot_rows:s * slot_rows + msg.shape[0]] = msg
        capacity = int(routed[:, rank * epr:(rank + 1) * epr].sum())
        meta = rt.ll.exchange_metadata(routed, rank, slot_rows, capacity)
        st = states[rank]
        poison_outputs_keep_pair_slot(st)
        ws = torch.empty(lib.deepep_ll_by_source_workspace_bytes(e, capacity), dtype=torch.uint8, device="cuda")
        capi.check(lib.deepep_ll_dispatch_recv_by_source(
            capi.ptr(buf), slot_rows, capi.ptr(meta["recv_counts"]), capi.ptr(meta["source_offset"]),
            capi.ptr(meta["num_recv_tokens"]), capacity, h, e, r, t, fmt, capi.ptr(st.packed_recv_x),
            capi.ptr(st.packed_recv_scales), capi.ptr(st.packed_recv_src_info), capi.ptr(st.packed_recv_layout_range),
            capi.ptr(st.packed_recv_count), None, None, None, 0, capi.ptr(ws), ws.numel(),
            torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, t, fmt)
        check_dispatch(st, want, fmt)
        assert int(meta["num_recv_tokens"][0]) == int(want["packed_recv_count"].sum())


@pytest.mark.parametrize("fmt", [O.ROW_FP8, O.ROW_BF16])
def test_single_launch_dispatch_past_the_streaming_bound(rt, fmt):
    """700 tokens x 7168, top-8 on two ranks: 5600 entries, so the dispatch is one launch, and more than
    64 MB of traffic, so that launch is the streaming instantiation."""
    r, rank, t, h, k, e = 2, 0, 700, 7168, 8, 16
    x_all, topk_all, _ = make_world(r, t, h, k, e, seed=700, drop=10)
    lib = rt.capi.load()
    assert lib.deepep_ll_dispatch_is_single_launch(t, k, e, t, t * k) == 1
    e_l = e // r
    received = sum(int(((tk >= rank * e_l) & (tk < (rank + 1) * e_l)).sum()) for tk in topk_all)
    assert t * (2 * h + k * O.row_payload(h, fmt)) + 2 * received * O.row_payload(h, fmt) > 64 * 2 ** 20
    st, _ = dispatch_on_gpu(rt, x_all, topk_all, rank, e, t, fmt, one_call=True)
    want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, t, fmt)
    check_dispatch(st, want, fmt)
    send_count, pair_slot = O.route(topk_all[rank], e, t)
    assert torch.equal(st.send_count.cpu(), send_count)
    assert torch.equal(st.pair_slot.cpu(), pair_slot)


@pytest.mark.parametrize("r,rank,t,h,k,e", [(8, 3, 64, 1024, 6, 64), (8, 3, 1500, 512, 8, 64)],
                         ids=["one_launch", "large_batch"])
def test_combine_without_row_return_reduces_the_same(rt, r, rank, t, h, k, e):
    """NULL send slots (zero copy): the call is the reduce alone; `out` is bit-identical to the full call's
    and no returned row is written."""
    x_all, topk_all, w_all = make_world(r, t, h, k, e, seed=91, drop=7)
    st, world = dispatch_on_gpu(rt, x_all, topk_all, rank, e, t, O.ROW_BF16, one_call=True)
    y = torch.randn((e // r, r * t, h), generator=torch.Generator().manual_seed(9)).to(torch.bfloat16).cuda()
    world.combine_from_peers(st, mode=1, seed=5)
    topk, w = topk_all[rank].cuda(), torch.softmax(w_all[rank], dim=-1).cuda()
    outs = []
    for zero_copy in (False, True):
        st.combine_send_slots.view(torch.int16).fill_(0x7FC0)
        out = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
        out.view(torch.int16).fill_(0x7FC0)
        st.combine(y, topk, w, out, zero_copy=zero_copy)
        torch.cuda.synchronize()
        outs.append(out)
        touched = bool((st.combine_send_slots.view(torch.int16) != 0x7FC0).any())
        assert touched != zero_copy
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))


# ---------------------------------------------------------------------------------------------
# The all-to-all shaped transport: one contiguous message per peer in both directions
# ---------------------------------------------------------------------------------------------
def send_by_dest_on_gpu(rt, x, topk, rank, r, e, m, fmt):
    t, h = x.shape
    k = topk.shape[1]
    st = rt.ll.AllToAllState(rt.ll.LLShape(r, rank, e, m, h, k, fmt))
    st.send_rows.fill_(0xEE)
    st.pair_slot.fill_(-7)
    for name in ("send_count", "send_expert_prefix", "send_counts", "send_cumsum"):
        getattr(st, name).fill_(-7)
    st.dispatch_send(x.cuda(), topk.cuda())
    torch.cuda.synchronize()
    return st


def check_send_by_dest(st, want, t):
    payload = st.lib.deepep_ll_row_payload_bytes(st.shape.hidden, st.shape.fmt)
    assert torch.equal(st.send_count.cpu(), want["send_count"])
    assert torch.equal(st.send_expert_prefix.cpu(), want["send_expert_prefix"])
    assert torch.equal(st.send_counts.cpu(), want["send_counts"])
    assert torch.equal(st.send_cumsum.cpu(), want["send_cumsum"])
    assert torch.equal(st.pair_slot[:t].cpu(), want["pair_slot"])
    n = want["rows"].shape[0]
    got = st.send_rows.cpu()
    h, fmt = st.shape.hidden, st.shape.fmt
    db, sb = O.row_data_bytes(h, fmt), O.row_scale_bytes(h, fmt)
    dp, sp = O.align_up(db, 16), O.align_up(sb, 16)
    touched = torch.zeros(got.shape[1], dtype=torch.bool)
    for lo, hi in ((0, db), (dp, dp + sb), (dp + sp, dp + sp + 16)):  # data, scales, tail: the padding is nobody's
        assert torch.equal(got[:n, lo:hi], want["rows"][:, lo:hi]), (lo, hi)
        touched[lo:hi] = True
    assert payload == dp + sp + 16
    assert (got[:n, ~touched] == 0xEE).all() and (got[n:] == 0xEE).all()  # nothing between the parts or behind the rows


@pytest.mark.parametrize("fmt", [O.ROW_FP8, O.ROW_BF16, O.ROW_FP8_UE8M0])
@pytest.mark.parametrize("r,rank,t,h,k,e", [
    (4, 1, 8, 512, 3, 16), (8, 7, 33, 1024, 4, 64), (2, 0, 1, 512, 1, 2),
    (32, 5, 128, 7168, 8, 256),  # the headline shape
    (2, 0, 1100, 512, 8, 16),    # T * K > 8192: the tables come from the chunk histograms
    (8, 5, 4200, 512, 4, 64),
    (16, 9, 12, 512, 6, 1024),   # the most experts
    (1, 0, 16, 512, 2, 4),       # a world of one rank
    (4, 2, 24, 1536, 4, 16),     # hidden not a multiple of 1024
    (512, 500, 3, 512, 2, 1024),
    (4, 3, 256, 512, 8, 32),     # 2048 entries: the last batch whose tables are built inside the send launch
    (4, 3, 257, 512, 8, 32),     # 2056 entries: the first with a launch for them
])
def test_send_by_dest(rt, fmt, r, rank, t, h, k, e):
    """One buffer, contiguous per destination rank, rows by expert and slot; counts, prefixes and every
    row byte against the oracle (csrc/kernels/efa_kernels.cu:2332-2400, row tail :797-800)."""
    x_all, topk_all, _ = make_world(r, t, h, k, e, seed=r * 17 + t, drop=min(5, t))
    st = send_by_dest_on_gpu(rt, x_all[rank], topk_all[rank], rank, r, e, t, fmt)
    check_send_by_dest(st, O.ll_send_by_dest(x_all[rank], topk_all[rank], rank, e, t, fmt, r), t)


@pytest.mark.parametrize("receive", ["from_tails", "ordered"])
def test_all_to_all_with_an_empty_batch(rt, receive):
    """No token anywhere: the tables are zeros, nothing is received, the records stay untouched, and the reduce of
    no tokens is a no-op."""
    r, rank, m, h, k, e = 4, 2, 8, 512, 2, 8
    x = torch.empty((0, h), dtype=torch.bfloat16)
    topk = torch.empty((0, k), dtype=torch.int64)
    st = send_by_dest_on_gpu(rt, x, topk, rank, r, e, m, O.ROW_FP8)
    assert (st.send_count == 0).all() and (st.send_expert_prefix == 0).all()
    assert (st.send_counts == 0).all() and (st.send_cumsum == 0).all()
    assert (st.send_rows == 0xEE).all()
    routed = torch.zeros((r, e), dtype=torch.int32, device="cuda")
    st.exchange_metadata(routed)
    poison_outputs_keep_pair_slot(st)
    st.record_packed_row.fill_(-7)
    if receive == "ordered":
        st.dispatch_recv_ordered(routed)
    else:
        st.dispatch_recv()
    torch.cuda.synchronize()
    assert (st.packed_recv_count == 0).all() and (st.packed_recv_layout_range == 0).all()
    assert (st.tokens_per_expert == 0).all() and (st.record_packed_row == -7).all()
    y = torch.zeros((e // r, r * m, h), dtype=torch.bfloat16, device="cuda")
    st.send_flat.view(torch.int16).fill_(0x7FC0)
    st.combine_send(y)
    out = torch.empty((0, h), dtype=torch.bfloat16, device="cuda")
    st.combine_recv(topk.cuda(), torch.empty((0, k), dtype=torch.float32, device="cuda"), out)
    torch.cuda.synchronize()
    assert (st.send_flat.view(torch.int16) == 0x7FC0).all()


def test_send_by_dest_with_repeated_experts_and_full_pairs(rt):
    """Tokens naming an expert more than once: pairs beyond a pair's M slots are dropped from the counts,
    the prefixes and the buffer alike."""
    r, rank, t, m, h, k, e = 2, 1, 6, 6, 256, 4, 4
    g = torch.Generator().manual_seed(5)
    x = torch.randn((t, h), generator=g).to(torch.bfloat16)
    topk = torch.tensor([[2, 2, 0, -1], [2, 3, 3, 1], [3, 3, 3, 3], [2, 1, 2, 1], [-1, -1, 3, 3], [3, 3, 3, 3]])
    st = send_by_dest_on_gpu(rt, x, topk, rank, r, e, m, O.ROW_FP8)
    want = O.ll_send_by_dest(x, topk, rank, e, m, O.ROW_FP8, r)
    assert int(want["send_count"][3]) == m and int((want["pair_slot"] == -1).sum()) > 3
    check_send_by_dest(st, want, t)


def all_to_all_dispatch(states, fmt):
    """The dispatch all-to-all between ranks that share the GPU: the gathered counts, then one slice copy per
    (source, destination) pair -- no regrouping of rows on the way."""
    r = len(states)
    routed = torch.stack([st.send_count for st in states])
    cums = [st.send_cumsum.cpu().tolist() for st in states]
    for d, dst in enumerate(states):
        dst.recv_by_source.fill_(0xEE)
        dst.exchange_metadata(routed)
        for s, src in enumerate(states):
            lo, hi = cums[s][d], cums[s][d + 1]
            assert hi - lo <= dst.slot_rows
            dst.recv_by_source[s * dst.slot_rows:s * dst.slot_rows + hi - lo] = src.send_rows[lo:hi]
    return routed


@pytest.mark.parametrize("receive", ["from_tails", "ordered", "ordered_as_a_large_batch"])
@pytest.mark.parametrize("delivery", ["flat", "slotted", "direct"])
@pytest.mark.parametrize("fmt", [O.ROW_FP8, O.ROW_BF16])
@pytest.mark.parametrize("r,t,h,k,e", [(4, 40, 512, 3, 16), (8, 700, 512, 8, 64), (3, 5, 256, 2, 3)],
                         ids=["small", "chunked_receive", "one_expert_per_rank"])
def test_all_to_all_round_trip_on_one_gpu(rt, oracle_c, fmt, delivery, receive, r, t, h, k, e):
    """Every rank on the one GPU, the transport replaced by slice copies of contiguous ranges: send by
    destination, exchange metadata from the gathered counts, receive by source, experts, return by
    destination (into a flat buffer that is copied range by range, or -- `direct` -- straight into the
    peers' receive buffers), reduce from the flat (or slotted) buffer.  Dispatch outputs bit-exact against
    the oracle, per-record rows against its loops, the combine against the float32 chain.
    (deep_ep/buffer.py:2266-2301,2601-2608,2735; csrc/transport/ll_pipeline.cpp:1204-1361)"""
    run_all_to_all_round_trip(rt, oracle_c, fmt, delivery, receive, r, t, h, k, e)


@pytest.mark.parametrize("delivery,receive", [("flat", "ordered"), ("direct", "from_tails")])
def test_all_to_all_round_trip_at_the_headline_shape(rt, oracle_c, delivery, receive):
    """The same with all 32 ranks of the headline world (128 tokens x 7168, top-8 of 256 experts, FP8) on the one
    GPU; the dispatch outputs of three ranks and the combined rows of the same three against the oracle."""
    run_all_to_all_round_trip(rt, oracle_c, O.ROW_FP8, delivery, receive, 32, 128, 7168, 8, 256, check_ranks=(0, 5, 31))


@pytest.mark.parametrize("seed", range(16))
def test_all_to_all_round_trip_random_worlds(rt, oracle_c, seed):
    """Seeded random small worlds through the same flow: odd rank counts, one to five experts a rank, one token
    to a few hundred (both sides of the 2048 entries up to which the send builds its own tables), every format,
    receive and delivery."""
    rng = np.random.default_rng(1000 + seed)
    r = int(rng.choice([1, 2, 3, 4, 6, 8, 16]))
    epr = int(rng.choice([1, 2, 3, 5]))
    e = r * epr
    k = int(rng.integers(1, min(8, e) + 1))
    t = int(rng.choice([1, 2, 7, 33, 64, 129, 260, 300]))
    h = int(rng.choice([128, 256, 512, 1024, 1536, 2048]))
    fmt = [O.ROW_FP8, O.ROW_BF16, O.ROW_FP8_POW2, O.ROW_FP8_UE8M0][int(rng.integers(4))]
    if fmt == O.ROW_FP8_UE8M0 and (h // 128) % 4:
        h = 512  # packed UE8M0 scales come four to a word
    delivery = ["flat", "slotted", "direct"][int(rng.integers(3))]
    receive = ["from_tails", "ordered", "ordered_as_a_large_batch"][int(rng.integers(3))]
    run_all_to_all_round_trip(rt, oracle_c, fmt, delivery, receive, r, t, h, k, e)


@pytest.mark.parametrize("t", [48, 1100], ids=["decode_size", "large_batch"])
def test_all_to_all_step_replays_in_a_hip_graph(rt, t):
    """A rank's five calls over the all-to-all surface captured once and replayed: they must allocate nothing
    and record no memset, and every replay, with eager work and synchronisations in between, must leave what the
    eager calls left (the peers' messages and answers stay where the eager exchange put them)."""
    r, rank, h, k, e, fmt = 4, 1, 1024, 8, 32, O.ROW_FP8
    epr = e // r
    x_all, topk_all, w_all = make_world(r, t, h, k, e, seed=77, drop=5)
    states = []
    for s_ in range(r):
        st = rt.ll.AllToAllState(rt.ll.LLShape(r, s_, e, t, h, k, fmt))
        st.dispatch_send(x_all[s_].cuda(), topk_all[s_].cuda())
        states.append(st)
    torch.cuda.synchronize()
    routed = all_to_all_dispatch(states, fmt)  # also runs every rank's exchange_metadata
    me = states[rank]
    x, topk, w = x_all[rank].cuda(), topk_all[rank].cuda(), w_all[rank].cuda()
    y = torch.empty((epr, r * t, h), dtype=torch.bfloat16, device="cuda")
    rt.capi.check(rt.capi.load().deepep_synth_bf16_rows(rt.capi.ptr(y), epr * r * t, h, h * 2, None, 0, 31, 0,
                                                        torch.cuda.current_stream().cuda_stream))
    me.recv_flat.normal_()  # the peers' answers
    out = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
    meta = me.meta
    lib, capi = rt.capi.load(), rt.capi
    meta_args = [capi.ptr(routed), e, r, rank, me.slot_rows, me.row_capacity] + [capi.ptr(meta[n]) for n in (
        "send_counts", "recv_counts", "totals", "combine_remote_recv_offset", "source_rank", "source_offset",
        "padded_index", "combine_send_offset", "num_recv_tokens", "tokens_per_expert")]

    def step():
        me.dispatch_send(x, topk)
        capi.check(lib.deepep_ll_exchange_metadata(*meta_args, torch.cuda.current_stream().cuda_stream))
        me.dispatch_recv_ordered(routed)
        me.combine_send(y)
        me.combine_recv(topk, w, out)

    n_records = int(meta["num_recv_tokens"][1])  # the records past them are nobody's to write
    outputs = lambda: (me.send_rows, me.send_expert_prefix, me.send_cumsum, me.pair_slot, me.packed_recv_count,
                       me.packed_recv_layout_range, me.record_packed_row[:n_records], me.send_flat.view(torch.int16),
                       out.view(torch.int16))
    me.send_rows.fill_(0xEE)
    me.send_flat.view(torch.int16).fill_(0x7FC0)
    step()
    torch.cuda.synchronize()
    want = [v.clone() for v in outputs()]
    n_rows = int(me.packed_recv_count.sum())
    assert n_rows > (8192 if t > 1024 else 0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        step()
    for replay in range(4):
        me.send_rows.fill_(0xEE)  # eager work between the replays: scribble over what the step writes
        me.send_flat.view(torch.int16).fill_(0x7FC0)
        out.zero_()
        me.packed_recv_count.fill_(-1)
        me.record_packed_row.fill_(-7)
        me.pair_slot.fill_(-9)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for i, (got, exp) in enumerate(zip(outputs(), want)):
            assert torch.equal(got, exp), f"replay {replay}: output {i}"


def test_all_to_all_round_trip_with_large_batches(rt, oracle_c):
    """4096 tokens a rank, 8 ranks x 32 experts, hidden 2048 (every rank on the one GPU needs ~9 GB then): the
    send runs on chunk histograms with the prefix launch, the receive on the ordered index and the flat row copy,
    the return and the reduce on their streaming forms; one rank against the oracle."""
    import gc
    gc.collect()
    torch.cuda.empty_cache()
    free, _ = torch.cuda.mem_get_info()
    if free < 90 * 2 ** 30:
        pytest.skip(f"needs ~75 GB of free HBM, {free >> 30} GiB are free")
    run_all_to_all_round_trip(rt, oracle_c, O.ROW_FP8, "flat", "ordered", 8, 4096, 2048, 8, 256, check_ranks=(3,))


def run_all_to_all_round_trip(rt, oracle_c, fmt, delivery, receive, r, t, h, k, e, check_ranks=None):
    epr = e // r
    checked = range(r) if check_ranks is None else check_ranks
    x_all, topk_all, w_all = make_world(r, t, h, k, e, seed=555 + r, drop=min(6, t))
    states = []
    for rank in range(r):
        st = rt.ll.AllToAllState(rt.ll.LLShape(r, rank, e, t, h, k, fmt))
        st.dispatch_send(x_all[rank].cuda(), topk_all[rank].cuda())
        states.append(st)
    torch.cuda.synchronize()
    routed = all_to_all_dispatch(states, fmt)
    ys = []
    for rank, st in enumerate(states):
        poison_outputs_keep_pair_slot(st)
        st.record_packed_row.fill_(-7)
        st.tokens_per_expert.fill_(-7)
        if receive.startswith("ordered"):  # the messages are in this build's own order: placed from the counts alone
            if receive == "ordered_as_a_large_batch":  # the index launch + flat row copy instead of the single launch
                st.expected_rows = 9000
            st.dispatch_recv_ordered(routed)
        else:
            st.dispatch_recv()
        torch.cuda.synchronize()
        assert torch.equal(st.tokens_per_expert, st.packed_recv_count)
        if rank in checked:
            want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, t, fmt)
            check_dispatch(st, want, fmt)
            n = int(st.meta["num_recv_tokens"][1])
            rec = O.ll_record_packed_rows(list(topk_all), rank, e, t)
            assert n == rec.numel() and torch.equal(st.record_packed_row[:n].cpu().long(), rec)
            assert (st.record_packed_row[n:] == -7).all()
        # the experts: a seeded row per packed slot
        y = torch.empty((epr, r * t, h), dtype=torch.bfloat16, device="cuda")
        rt.capi.check(rt.capi.load().deepep_synth_bf16_rows(rt.capi.ptr(y), epr * r * t, h, h * 2, None, 0, 900 + rank,
                                                            0, torch.cuda.current_stream().cuda_stream))
        ys.append(y)
    peer_table = torch.tensor([st.recv_flat.data_ptr() for st in states], dtype=torch.int64, device="cuda")
    peer_rows = torch.tensor([st.recv_flat.shape[0] for st in states], dtype=torch.int64, device="cuda")
    for st in states:
        st.recv_flat.view(torch.int16).fill_(0x7FC0)
        st.send_flat.view(torch.int16).fill_(0x7FC0)
    for rank, st in enumerate(states):
        if delivery == "direct":
            st.combine_send(ys[rank], peer_table, peer_rows)
        else:
            st.combine_send(ys[rank])
    torch.cuda.synchronize()
    slot_rows = t * min(k, epr)
    slotted = [torch.full((r * slot_rows, h), float("nan"), dtype=torch.bfloat16, device="cuda") for _ in states]
    if delivery != "direct":  # the all-to-all back: one slice copy per (answering rank, asking rank) pair
        cums = [st.send_cumsum.cpu().tolist() for st in states]
        for d, ans in enumerate(states):
            recv_counts = ans.meta["recv_counts"].cpu().tolist()
            first = 0
            for s, ask in enumerate(states):
                n = recv_counts[s]
                assert n == cums[s][d + 1] - cums[s][d]
                assert int(ans.meta["combine_remote_recv_offset"][s]) == cums[s][d]
                ask.recv_flat[cums[s][d]:cums[s][d] + n] = ans.send_flat[first:first + n]
                slotted[s][d * slot_rows:d * slot_rows + n] = ans.send_flat[first:first + n]
                first += n
    else:
        assert all((st.send_flat.view(torch.int16) == 0x7FC0).all() for st in states)  # nothing went the long way
    for rank, st in enumerate(states):
        if rank not in checked:
            continue
        topk, w = topk_all[rank], w_all[rank]
        out = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
        out.view(torch.int16).fill_(0x7FC0)
        if delivery == "slotted":
            st.combine_recv(topk.cuda(), w.cuda(), out, recv=slotted[rank], slot_rows=slot_rows)
        else:
            st.combine_recv(topk.cuda(), w.cuda(), out)
        torch.cuda.synchronize()
        # which seeded row answers each pair: the packed row the owner of the expert gave it
        _, pair_slot = O.route(topk, e, t)
        live = pair_slot >= 0
        pair_rows = torch.zeros((t, k, h), dtype=torch.bfloat16)
        for d in range(r):
            lr = states[d].packed_recv_layout_range.cpu()
            sel = live & (topk // epr == d)
            ti, ki = torch.nonzero(sel, as_tuple=True)
            if ti.numel() == 0:
                continue
            le = (topk[ti, ki] % epr)
            begin = (lr[le, rank] >> 32)
            keys = (le * (r * t) + begin + pair_slot[ti, ki].long()).numpy().astype(np.uint32)
            pair_rows[ti, ki] = O.synth_bf16_rows(keys, h, 900 + d)
        chain = torch.empty((t, h), dtype=torch.int16)
        live8 = live.to(torch.uint8).contiguous()
        oracle_c.oracle_combine_chain(ctypes.c_void_p(pair_rows.view(torch.int16).data_ptr()),
                                      ctypes.c_void_p(w.contiguous().data_ptr()), ctypes.c_void_p(live8.data_ptr()),
                                      t, k, h, ctypes.c_void_p(chain.data_ptr()))
        assert torch.equal(out.cpu().view(torch.int16), chain), (rank, delivery)
        ref = O.ll_combine(pair_rows, topk, w, live)
        err = (out.cpu().double() - ref).abs()
        assert (err <= 1e-2 * ref.abs() + 1e-2 * ref.abs().mean()).all()  # the 1e-2 bar against the float64 sum


def test_all_to_all_hand_derived_world(rt):
    """The same flow on the two-rank world worked out on paper (tests/golden/ll_tiny_world.json): message order,
    tables, per-record packed rows, the flat buffers of both directions and the combined rows -- no oracle."""
    g, x_all, topk_all = load_tiny_world()
    e, m, h, t, k, r = g["num_experts"], g["max_tokens"], g["hidden"], g["num_tokens"], g["num_topk"], g["num_ranks"]
    states = []
    for rank in range(r):
        st = rt.ll.AllToAllState(rt.ll.LLShape(r, rank, e, m, h, k, O.ROW_BF16))
        st.dispatch_send(x_all[rank].cuda(), topk_all[rank].cuda())
        states.append(st)
    torch.cuda.synchronize()
    tail_at = O.row_payload(h, O.ROW_BF16) - 16
    for rank, st in enumerate(states):
        want = g["send_by_dest"][f"rank{rank}"]
        assert st.send_expert_prefix.cpu().tolist() == want["send_expert_prefix"]
        assert st.send_counts.cpu().tolist() == want["send_counts"]
        assert st.send_cumsum.cpu().tolist() == want["send_cumsum"]
        n = want["send_cumsum"][-1]
        tails = st.send_rows[:n, tail_at:tail_at + 16].cpu().contiguous().view(torch.int32)
        assert tails[:, 0].tolist() == want["row_token"] and tails[:, 1].tolist() == want["row_topk_slot"]
        assert tails[:, 3].tolist() == want["row_local_expert"]
        slot = st.pair_slot[:t].cpu()
        prefix = torch.tensor(want["send_expert_prefix"])
        row = torch.where(slot >= 0, prefix[topk_all[rank].clamp(min=0)] + slot, torch.full_like(slot, -1))
        assert row.tolist() == want["pair_send_row"]
    all_to_all_dispatch(states, O.ROW_BF16)
    for rank, st in enumerate(states):
        st.dispatch_recv()
        torch.cuda.synchronize()
        rec = g["record_packed_row"][f"rank{rank}"]
        assert st.record_packed_row[:len(rec)].cpu().tolist() == rec
        want, layout = tiny_world_expected(g, f"rank{rank}_ascending")
        assert st.packed_recv_count.cpu().tolist() == want["count"]
        assert torch.equal(st.packed_recv_layout_range.cpu(), layout)
        st.combine_send(st.packed_recv_x)  # identity experts
        torch.cuda.synchronize()
        flat = g["combine_send_flat_identity_experts"][f"rank{rank}"]
        assert st.send_flat[:len(flat)].cpu().float()[:, 0].tolist() == flat
    cums = [st.send_cumsum.cpu().tolist() for st in states]
    for d, ans in enumerate(states):
        recv_counts, first = ans.meta["recv_counts"].cpu().tolist(), 0
        for s, ask in enumerate(states):
            ask.recv_flat[cums[s][d]:cums[s][d] + recv_counts[s]] = ans.send_flat[first:first + recv_counts[s]]
            first += recv_counts[s]
    want_back = g["combine_recv_flat_rank0_identity_experts"]
    assert states[0].recv_flat[:len(want_back)].cpu().float()[:, 0].tolist() == want_back
    out = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
    w = torch.tensor(g["topk_weights_rank0"], dtype=torch.float32, device="cuda")
    states[0].combine_recv(topk_all[0].cuda(), w, out)
    torch.cuda.synchronize()
    expect = torch.tensor(g["combine_rank0_identity_experts"]).view(-1, 1).expand(-1, h)
    assert torch.equal(out.cpu().float(), expect)


@pytest.mark.parametrize("t,hint", [(24, 0), (1500, 0), (1500, 1500)],
                         ids=["one_workgroup_per_source", "chunked", "one_workgroup_per_source_past_its_hint"])
def test_dispatch_recv_by_source_clamps_a_pair_to_max_tokens(rt, t, hint):
    """Slots wider than M and senders that put more than M rows into one (expert, source) pair: the pair keeps
    its first M rows in arrival order, the counts and ranges count only those, and an expert's ranges stay
    inside its R * M packed slots -- what the staged receive does with an over-full count."""
    r, rank, h, k, e, fmt = 2, 0, 512, 4, 8, O.ROW_FP8
    m = t // 3  # what the receiver was built for; the senders route as if M were t
    x_all, topk_all, _ = make_world(r, t, h, k, e, seed=11, drop=0)
    topk_all[1, :, :] = torch.tensor([0, 1, 2, 3])  # source 1: t rows for each of rank 0's experts
    slot_rows = 4 * t
    buf = rows_by_source(x_all, topk_all, rank, e, t, fmt, slot_rows)
    routed = torch.stack([O.route(topk_all[s], e, t)[0] for s in range(r)]).to(torch.int32)
    capacity = 8 * t
    lib, capi = rt.capi.load(), rt.capi
    meta = rt.ll.exchange_metadata(routed.clamp(max=slot_rows).cuda(), rank, slot_rows, capacity)
    st = rt.ll.LowLatencyState(rt.ll.LLShape(r, rank, e, m, h, 1, fmt), keep_remote_rows=False)
    poison_outputs(st)
    ws = torch.empty(lib.deepep_ll_by_source_workspace_bytes(e, capacity), dtype=torch.uint8, device="cuda")
    rec = torch.full((capacity,), -7, dtype=torch.int32, device="cuda")
    capi.check(lib.deepep_ll_dispatch_recv_by_source(
        capi.ptr(buf.cuda()), slot_rows, capi.ptr(meta["recv_counts"]), capi.ptr(meta["source_offset"]),
        capi.ptr(meta["num_recv_tokens"]), capacity, h, e, r, m, fmt, capi.ptr(st.packed_recv_x),
        capi.ptr(st.packed_recv_scales), capi.ptr(st.packed_recv_src_info), capi.ptr(st.packed_recv_layout_range),
        capi.ptr(st.packed_recv_count), None, None, capi.ptr(rec), hint, capi.ptr(ws), ws.numel(),
        torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    epr, n_slots = e // r, r * m
    tail_at = O.row_payload(h, fmt) - 16
    tail = buf[:, tail_at:tail_at + 16].contiguous().view(torch.int32)
    recv_counts = meta["recv_counts"].cpu().tolist()
    kept = [[[] for _ in range(r)] for _ in range(epr)]
    want_rec, i = [], 0
    for s in range(r):
        for j in range(recv_counts[s]):
            row = s * slot_rows + j
            le = int(tail[row, 3])
            if len(kept[le][s]) < m:
                kept[le][s].append((row, i))
            i += 1
    want_rec = [-1] * i
    count = st.packed_recv_count.cpu().tolist()
    layout = st.packed_recv_layout_range.cpu()
    px = st.packed_recv_x.view(torch.uint8).cpu()
    for le in range(epr):
        begin = 0
        for s in range(r):
            rows = kept[le][s]
            assert int(layout[le, s]) == (((begin << 32) | len(rows)) if rows else 0), (le, s)
            if rows:
                idx = torch.tensor([row for row, _ in rows])
                assert torch.equal(px[le, begin:begin + len(rows)], buf[idx, :h])
                for pos, (_, rec_i) in enumerate(rows):
                    want_rec[rec_i] = le * n_slots + begin + pos
            begin += len(rows)
        assert count[le] == begin and begin <= n_slots
    assert max(count) == n_slots or t < 30  # source 1 alone fills its half of every expert
    assert rec[:i].cpu().tolist() == want_rec


def test_ordered_receive_with_slots_too_small_and_counts_too_large(rt):
    """The ordered receive on hostile inputs: a source whose message does not fit its slot loses the rows past
    it (their records read -1, the ranges count only what was kept), and a count above M is read as M."""
    r, rank, t, h, k, e, fmt = 2, 0, 30, 512, 4, 8, O.ROW_FP8
    epr = e // r
    x_all, topk_all, _ = make_world(r, t, h, k, e, seed=17, drop=0)
    topk_all[1, :, :] = torch.tensor([0, 1, 2, 3])  # source 1 sends t rows to each of rank 0's four experts
    slot_rows = 2 * t + 7  # ... but its slot holds two experts' worth and a bit
    states = []
    for s_ in range(r):
        st = rt.ll.AllToAllState(rt.ll.LLShape(r, s_, e, t, h, k, fmt), slot_rows=slot_rows)
        st.dispatch_send(x_all[s_].cuda(), topk_all[s_].cuda())
        states.append(st)
    torch.cuda.synchronize()
    routed = torch.stack([st.send_count for st in states])
    dst = states[rank]
    dst.recv_by_source.fill_(0xEE)
    for s_, src in enumerate(states):
        lo, hi = [int(v) for v in src.send_cumsum[rank:rank + 2].cpu()]
        n = min(hi - lo, slot_rows)
        dst.recv_by_source[s_ * slot_rows:s_ * slot_rows + n] = src.send_rows[lo:lo + n]
    routed_big = routed.clone()
    routed_big[0, 1] += 1000  # nonsense from source 0 for expert 1: read as M rows
    for mat, hint in ((routed, t * k), (routed_big, t * k), (routed, 9000), (routed_big, 9000)):
        poison_outputs_keep_pair_slot(dst)
        dst.record_packed_row.fill_(-7)
        dst.expected_rows = hint  # the single launch, then the index launch + flat row copy
        dst.dispatch_recv_ordered(mat)
        torch.cuda.synchronize()
        sent = mat[:, rank * epr:(rank + 1) * epr].cpu().clamp(max=t)  # [source, local expert]
        want_rec, begin = [], [0] * epr
        kept = torch.zeros((epr, r), dtype=torch.int64)
        for s_ in range(r):
            first = 0
            for le in range(epr):
                c = int(sent[s_, le])
                kept[le, s_] = max(0, min(c, slot_rows - first))
                first += c
        layout = dst.packed_recv_layout_range.cpu()
        for le in range(epr):
            b = 0
            for s_ in range(r):
                n = int(kept[le, s_])
                assert int(layout[le, s_]) == (((b << 32) | n) if n else 0)
                b += n
            assert int(dst.packed_recv_count[le]) == b
        for s_ in range(r):
            for le in range(epr):
                b = int(kept[le, :s_].sum())
                want_rec += [le * r * t + b + j if j < int(kept[le, s_]) else -1 for j in range(int(sent[s_, le]))]
        n_rec = min(len(want_rec), dst.row_capacity)
        assert dst.record_packed_row[:n_rec].cpu().tolist() == want_rec[:n_rec]
        if mat is routed:  # the rows kept are the oracle's rows, in place
            want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, t, fmt)
            px = dst.packed_recv_x.view(torch.uint8).cpu()
            for le in range(epr):
                n0 = int(kept[le, 0])
                assert torch.equal(px[le, :n0], want["packed_recv_x"][le, :n0])  # source 0 fits whole
                n1 = int(kept[le, 1])
                full0 = int(want["packed_recv_layout_range"][le, 0] & 0xFFFFFFFF)
                assert torch.equal(px[le, n0:n0 + n1], want["packed_recv_x"][le, full0:full0 + n1])
