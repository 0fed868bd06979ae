"""Property tests of the CPU oracle on tiny worlds: brute-force definitions written as literal loops,
drawn shapes with dropped (-1) selections.  A wrong index, sign or order in the oracle fails one of them."""
import torch
from hypothesis import given, settings, strategies as st

from oracle import deepep_oracle as O


@st.composite
def worlds(draw):
    r = draw(st.sampled_from([1, 2, 3, 4]))
    epr = draw(st.integers(1, 3))
    e = r * epr
    k = draw(st.integers(1, min(e, 4)))
    t = draw(st.integers(0, 6))
    m = t + draw(st.integers(0, 2)) if t else 1
    seed = draw(st.integers(0, 10 ** 6))
    g = torch.Generator().manual_seed(seed)
    topk_all = []
    for _ in range(r):
        rows = [torch.randperm(e, generator=g)[:k] for _ in range(t)]
        tk = torch.stack(rows) if t else torch.zeros((0, k), dtype=torch.int64)
        drop = torch.rand(tk.shape, generator=g) < draw(st.sampled_from([0.0, 0.2, 0.6]))
        topk_all.append(torch.where(drop, torch.full_like(tk, -1), tk))
    x_all = [(torch.arange(t, dtype=torch.float32).view(-1, 1) + 100 * s + 1).expand(-1, 128).to(torch.bfloat16).contiguous()
             for s in range(r)]
    return r, e, k, t, m, draw(st.integers(0, r - 1)), x_all, topk_all


@settings(max_examples=80, deadline=None)
@given(worlds())
def test_layout_is_the_brute_force_count(w):
    r, e, k, t, m, rank, _, topk_all = w
    topk = topk_all[rank]
    per_rank, per_rdma, per_expert, is_in = O.get_dispatch_layout(topk, e, r)
    epr = e // r
    for ex in range(e):
        assert per_expert[ex].item() == sum(1 for i in range(t) for j in range(k) if topk[i, j].item() == ex)
    for dst in range(r):
        members = [any(0 <= topk[i, j].item() and topk[i, j].item() // epr == dst for j in range(k)) for i in range(t)]
        assert per_rank[dst].item() == sum(members)
        assert [bool(v) for v in is_in[:, dst]] == members
    assert per_rdma is None


@settings(max_examples=80, deadline=None)
@given(worlds())
def test_route_slots_are_the_serial_scan(w):
    r, e, k, t, m, rank, _, topk_all = w
    topk = topk_all[rank]
    send_count, pair_slot = O.route(topk, e, m)
    seen = [0] * e
    for i in range(t):
        for j in range(k):
            ex = topk[i, j].item()
            if ex < 0:
                assert pair_slot[i, j].item() == -1
                continue
            want = seen[ex] if seen[ex] < m else -1
            assert pair_slot[i, j].item() == want
            seen[ex] += 1
    assert send_count.tolist() == [min(c, m) for c in seen]


@settings(max_examples=60, deadline=None)
@given(worlds())
def test_dispatch_is_the_brute_force_gather(w):
    r, e, k, t, m, rank, x_all, topk_all = w
    got = O.ll_dispatch(x_all, topk_all, rank, e, m, O.ROW_BF16)
    epr = e // r
    order = list(range(r))  # csrc/kernels/efa_kernels.cu:991-1010: ascending source rank
    for le in range(epr):
        ex = rank * epr + le
        rows, srcs, begin = [], [], {}
        for s in order:
            begin[s] = len(rows)
            for i in range(t):
                for j in range(k):
                    if topk_all[s][i, j].item() == ex:
                        rows.append(x_all[s][i])
                        srcs.append(i)
        n = len(rows)
        assert got["packed_recv_count"][le].item() == n
        assert got["packed_recv_src_info"][le, :n].tolist() == srcs
        if n:
            have = got["packed_recv_x"][le, :n].contiguous().view(torch.bfloat16)
            assert torch.equal(have, torch.stack(rows))
        for s in range(r):
            cnt = sum(1 for i in range(t) for j in range(k) if topk_all[s][i, j].item() == ex)
            lr = got["packed_recv_layout_range"][le, s].item()
            assert lr == (((begin[s] << 32) | cnt) if cnt else 0)


@settings(max_examples=60, deadline=None)
@given(worlds(), st.integers(0, 10 ** 6))
def test_combine_is_the_weighted_sum_and_is_linear(w, seed):
    r, e, k, t, m, rank, x_all, topk_all = w
    if t == 0:
        return
    g = torch.Generator().manual_seed(seed)
    topk = topk_all[rank]
    wts = torch.rand((t, k), generator=g)
    rows_a = torch.randn((t, k, 128), generator=g).to(torch.bfloat16)
    rows_b = torch.randn((t, k, 128), generator=g).to(torch.bfloat16)
    out_a = O.ll_combine(rows_a, topk, wts)
    for i in range(t):
        acc = torch.zeros(128, dtype=torch.float64)
        for j in range(k):
            if topk[i, j].item() >= 0:
                acc += wts[i, j].double() * rows_a[i, j].double()
        assert torch.allclose(out_a[i], acc, rtol=1e-12, atol=1e-12)
    both = O.ll_combine((rows_a.double() + rows_b.double()), topk, wts)
    assert torch.allclose(both, out_a + O.ll_combine(rows_b, topk, wts), rtol=1e-12, atol=1e-12)
    chain = O.ll_combine_f32_chain(rows_a, wts, topk >= 0).double()
    scale = out_a.abs().max().clamp(min=1.0)
    assert (chain - out_a).abs().max() <= scale * 2 ** -7  # one bf16 rounding of a float32 chain


@settings(max_examples=60, deadline=None)
@given(worlds())
def test_exchange_metadata_matches_the_dispatch(w):
    r, e, k, t, m, rank, x_all, topk_all = w
    routed = torch.stack([O.route(tk, e, m)[0] for tk in topk_all]).to(torch.int32)
    meta = O.ll_exchange_metadata(routed, rank, m)
    got = O.ll_dispatch(x_all, topk_all, rank, e, m, O.ROW_BF16)
    per_source = (got["packed_recv_layout_range"] & 0xFFFFFFFF).sum(0)
    assert meta["recv_counts"].tolist() == per_source.tolist()
    assert meta["total_recv"] == int(got["packed_recv_count"].sum())
    epr = e // r
    assert meta["send_counts"].tolist() == [int(routed[rank, d * epr:(d + 1) * epr].sum()) for d in range(r)]
    assert meta["source_rank"].tolist() == [s for s in range(r) for _ in range(int(per_source[s]))]


@settings(max_examples=60, deadline=None)
@given(worlds())
def test_all_to_all_round_trip_returns_every_pair_its_own_row(w):
    """Both directions over one contiguous message per peer, the messages moved by literal slice copies:
    the per-record packed rows must point at what the dispatch put there, and with identity experts every
    live pair must get back exactly the row its token sent."""
    r, e, k, t, m, _, x_all, topk_all = w
    epr, h = e // r, 128
    sent = [O.ll_send_by_dest(x_all[s], topk_all[s], s, e, m, O.ROW_BF16, r) for s in range(r)]
    routed = torch.stack([sd["send_count"] for sd in sent]).to(torch.int32)
    flats, metas = [], []
    for d in range(r):
        # the message of source s to rank d, and where its rows land in arrival order
        arrived = torch.cat([sent[s]["rows"][int(sent[s]["send_cumsum"][d]):int(sent[s]["send_cumsum"][d + 1])]
                             for s in range(r)]) if r else None
        meta = O.ll_exchange_metadata(routed, d, m)
        assert meta["total_recv"] == arrived.shape[0]
        packed = O.ll_dispatch(x_all, topk_all, d, e, m, O.ROW_BF16)
        rec = O.ll_record_packed_rows(topk_all, d, e, m)
        assert rec.numel() == arrived.shape[0]
        px = packed["packed_recv_x"].view(epr * r * m, -1)
        tail_at = O.row_payload(h, O.ROW_BF16) - 16
        for i in range(rec.numel()):
            assert torch.equal(px[int(rec[i])], arrived[i, :2 * h])  # the record's row is where the dispatch put it
            tail = arrived[i, tail_at:tail_at + 16].contiguous().view(torch.int32)
            assert int(rec[i]) // (r * m) == int(tail[3])  # ... inside the expert its tail names
            assert int(packed["packed_recv_src_info"].view(-1)[int(rec[i])]) == int(tail[0])
        y = packed["packed_recv_x"].view(epr, r * m, 2 * h).contiguous().view(torch.bfloat16)  # identity experts
        flats.append(O.ll_combine_send_by_dest(y, rec, meta["padded_index"], meta["combine_send_offset"]))
        metas.append(meta)
    for s in range(r):
        # the answers for rank s: peer d's rows for source s, landing behind what s sent to the ranks below d
        total = int(sent[s]["send_cumsum"][r])
        back = torch.zeros((total, h), dtype=torch.bfloat16)
        for d in range(r):
            first = int(metas[d]["recv_counts"][:s].sum())
            n = int(metas[d]["recv_counts"][s])
            at = int(metas[d]["combine_remote_recv_offset"][s])
            assert at == int(sent[s]["send_cumsum"][d]) and n == int(sent[s]["send_counts"][d])
            back[at:at + n] = flats[d][first:first + n]
        pair_rows, live = O.ll_combine_recv_flat_rows(back, 0, sent[s]["send_expert_prefix"], topk_all[s],
                                                      sent[s]["pair_slot"], epr)
        assert torch.equal(live, sent[s]["pair_slot"] >= 0)
        for i in range(t):
            for j in range(k):
                if live[i, j]:
                    assert torch.equal(pair_rows[i, j], x_all[s][i])
        # the slotted form of the same buffer: rank d's answers start at row d * slot_rows
        slot_rows = m * epr
        slotted = torch.zeros((r * slot_rows, h), dtype=torch.bfloat16)
        for d in range(r):
            lo, hi = int(sent[s]["send_cumsum"][d]), int(sent[s]["send_cumsum"][d + 1])
            slotted[d * slot_rows:d * slot_rows + hi - lo] = back[lo:hi]
        again, _ = O.ll_combine_recv_flat_rows(slotted, slot_rows, sent[s]["send_expert_prefix"], topk_all[s],
                                               sent[s]["pair_slot"], epr)
        assert torch.equal(again, pair_rows)
