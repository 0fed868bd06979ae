"""Pins the CPU oracle: library routines, closed forms, brute force and invariants.

No GPU.  A plausible mistake in the oracle (wrong rounding, dropped clamp, wrong
segment order, transposed index) must fail at least one test here.
"""
import ctypes

import numpy as np
import pytest
import torch

from oracle import deepep_oracle as O


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


# --------------------------------------------------------------------------
# FP8
# --------------------------------------------------------------------------
def test_e4m3_encoder_matches_torch_cast_on_every_bf16_input(oracle_c):
    # All 65536 bf16 bit patterns as float32, plus values that bf16 * float32
    # scale products reach: dense sweep around every e4m3 rounding boundary.
    bf = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    grid = []
    for b in range(256):
        v = oracle_c.oracle_e4m3_decode(b)
        if v == v:
            grid.append(v)
    grid = torch.tensor(sorted(set(grid)), dtype=torch.float32)
    mids = (grid[1:] + grid[:-1]) / 2
    near = torch.cat([torch.nextafter(mids, torch.tensor(float("inf"))), mids,
                      torch.nextafter(mids, torch.tensor(-float("inf")))])
    rnd = torch.empty(200000).uniform_(-448, 448, generator=torch.Generator().manual_seed(7))
    tiny = torch.empty(50000).uniform_(-0.05, 0.05, generator=torch.Generator().manual_seed(8))
    x = torch.cat([bf, grid, near, rnd, tiny])
    x = x[torch.isfinite(x)].clamp(-448, 448).contiguous()
    want = x.to(torch.float8_e4m3fn).view(torch.uint8)
    got = torch.empty_like(want)
    oracle_c.oracle_e4m3_encode_many(_ptr(x), _ptr(got), x.numel())
    assert torch.equal(got, want)


def test_e4m3_known_answers(oracle_c):
    # Hand-checked bytes of the OCP format: 1-4-3, bias 7.
    cases = [(0.0, 0x00), (-0.0, 0x80), (1.0, 0x38), (-1.0, 0xB8), (448.0, 0x7E), (-448.0, 0xFE), (2.0 ** -9, 0x01),
             (2.0 ** -6, 0x08), (0.3, 42), (447.9, 126), (17.0, 88), (1.0625, 0x38), (1.1875, 0x3A), (2.0 ** -10, 0x00),
             (3 * 2.0 ** -10, 0x02)]
    for v, b in cases:
        assert oracle_c.oracle_e4m3_encode(v) == b, (v, b)
        assert torch.tensor([v]).to(torch.float8_e4m3fn).view(torch.uint8).item() == b, (v, b)


def test_e4m3_decode_roundtrip(oracle_c):
    for b in range(256):
        v = oracle_c.oracle_e4m3_decode(b)
        if v != v:
            assert b & 0x7F == 0x7F
            continue
        assert oracle_c.oracle_e4m3_encode(v) == b
        assert torch.tensor([b], dtype=torch.uint8).view(torch.float8_e4m3fn).float().item() == v


@pytest.mark.parametrize("fmt", [O.ROW_FP8, O.ROW_FP8_POW2, O.ROW_FP8_UE8M0])
def test_torch_cast_matches_scalar_c_cast(oracle_c, fmt):
    g = torch.Generator().manual_seed(11)
    x = torch.randn((37, 512), generator=g)
    x[3] *= 100
    x[5] = 0
    x[7, :128] = 1e-6
    x[9, 5] = 448 * 3.0
    x[11] = -x[11].abs()
    x = x.to(torch.bfloat16)
    q, s = O.per_token_cast_to_fp8(x, round_scale=fmt != O.ROW_FP8, use_ue8m0=fmt == O.ROW_FP8_UE8M0)
    q2 = torch.empty((37, 512), dtype=torch.uint8)
    sb = 1 if fmt == O.ROW_FP8_UE8M0 else 4
    s2 = torch.empty((37, 4 * sb), dtype=torch.uint8)
    xb = x.view(torch.int16).contiguous()
    oracle_c.oracle_per_token_cast(_ptr(xb), 37, 512, fmt, _ptr(q2), _ptr(s2))
    assert torch.equal(q.view(torch.uint8), q2)
    assert torch.equal(s.contiguous().view(torch.uint8).view(37, -1), s2)


def test_cast_special_cases():
    x = torch.zeros((2, 256), dtype=torch.bfloat16)
    x[1, :128] = 2.0
    x[1, 128:] = -3.0
    x[1, 130] = 1.5
    q, s = O.per_token_cast_to_fp8(x)
    assert s[0, 0].item() == np.float32(1e-4) / np.float32(448.0)
    assert (q[0].view(torch.uint8) == 0).all()
    assert s[1, 0].item() == np.float32(2.0) / np.float32(448.0) and (q[1, :128].view(torch.uint8) == 0x7E).all()
    assert (q[1, 128:130].view(torch.uint8) == 0xFE).all() and q[1, 130].float().item() == 224.0
    # dequantised amax is exact
    back = O.per_token_cast_back(q, s)
    assert back[1, 0].item() == 2.0 and back[1, 128].item() == -3.0 and back[1, 130].item() == 1.5
    # round_scale: scale is the smallest power of two >= amax/448; ue8m0 carries its exponent byte
    q2, s2 = O.per_token_cast_to_fp8(x, round_scale=True)
    for v, raw in zip(s2[1].tolist(), (2.0 / 448, 3.0 / 448)):
        assert np.log2(v) == np.ceil(np.log2(raw)) and v >= raw > v / 2
    x512 = torch.randn((3, 512)).to(torch.bfloat16)
    _, sp = O.per_token_cast_to_fp8(x512, round_scale=True)
    _, su = O.per_token_cast_to_fp8(x512, round_scale=True, use_ue8m0=True)
    assert su.dtype == torch.int32 and su.shape == (3, 1)
    assert torch.equal(su.view(torch.uint8).view(3, 4).to(torch.int32), (sp.view(torch.int32) >> 23) & 0xFF)
    assert torch.equal(O.per_token_cast_back(_, su).float(), O.per_token_cast_back(_, sp).float())


def test_pow2_ceil_exact():
    s = torch.tensor([1.0, 1.0000001, 0.5, 0.75, 3.0, 2.0 ** -20, 2.0 ** -20 * 1.5, 2.2e-7])
    want = torch.tensor([1.0, 2.0, 0.5, 1.0, 4.0, 2.0 ** -20, 2.0 ** -19, 2.0 ** -22])
    assert torch.equal(O.pow2_ceil(s), want)


def test_cast_error_bound_and_reference_torch_helper():
    x = (torch.randn((64, 1024), generator=torch.Generator().manual_seed(5)) * 3).to(torch.bfloat16)
    q, s = O.per_token_cast_to_fp8(x)
    xv = x.view(64, -1, 128)
    amax = xv.abs().float().amax(dim=2).view(64, -1).clamp(1e-4)
    # IEEE division written with numpy, element by element, gives the same bytes
    inv = torch.from_numpy(np.float32(448.0) / amax.numpy())
    q_np = (xv.float() * inv.unsqueeze(2)).clamp(-448, 448).to(torch.float8_e4m3fn).view(64, 1024)
    assert torch.equal(q.view(torch.uint8), q_np.view(torch.uint8))
    assert torch.equal(s, torch.from_numpy(amax.numpy() / np.float32(448.0)))
    back = O.per_token_cast_back(q, s).float()
    err = (back - x.float()).abs().view(64, -1, 128)
    # half an e4m3 step at the top binade is 16 (scaled units); the bf16 round of the result adds 2^-9 relative
    assert (err <= amax.unsqueeze(2) * (16 / 448.0 + 2.0 ** -8)).all()
    # The reference's torch helper (reciprocal-multiply) has the same scales and differs from
    # the kernel's division in well under 1 % of bytes, each by one e4m3 code.
    qh, sh = O.per_token_cast_to_fp8_torch_helper(x)
    assert torch.equal(sh, s)
    a, b = q.view(torch.uint8).to(torch.int32), qh.view(torch.uint8).to(torch.int32)
    diff = a != b
    assert diff.float().mean().item() < 0.01
    assert ((a - b).abs()[diff] == 1).all()


# --------------------------------------------------------------------------
# Layout
# --------------------------------------------------------------------------
def _brute_layout(topk, num_experts, num_ranks):
    t, k = topk.shape
    epr = num_experts // num_ranks
    pe = [0] * num_experts
    pr = [0] * num_ranks
    pn = [0] * (num_ranks // 8)
    is_in = [[False] * num_ranks for _ in range(t)]
    for i in range(t):
        for j in range(k):
            e = int(topk[i, j])
            if e >= 0:
                pe[e] += 1
                is_in[i][e // epr] = True
        for r in range(num_ranks):
            pr[r] += is_in[i][r]
        for n in range(num_ranks // 8):
            pn[n] += any(is_in[i][8 * n:8 * n + 8])
    return pr, pn, pe, is_in


@pytest.mark.parametrize("t,k,e,r", [(1, 1, 2, 2), (13, 3, 16, 4), (40, 8, 64, 16), (0, 4, 8, 8), (9, 6, 48, 24)])
def test_layout_matches_brute_force(t, k, e, r):
    g = torch.Generator().manual_seed(t * 31 + e)
    topk = torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(t)]) if t else torch.zeros((0, k), dtype=torch.int64)
    if t > 2:
        topk[1, 0] = -1
        topk[2, :] = -1
    pr, pn, pe, is_in = O.get_dispatch_layout(topk, e, r)
    bpr, bpn, bpe, bis = _brute_layout(topk, e, r)
    assert pr.tolist() == bpr and pe.tolist() == bpe and is_in.tolist() == bis
    if r > 8 and r % 8 == 0:
        assert pn.tolist() == bpn
    else:
        assert pn is None
    # closed forms of tests/test_intranode.py:41-58
    for i in range(e):
        assert pe[i].item() == (topk == i).sum().item()


def test_routing_sort_and_channel_prefix():
    g = torch.Generator().manual_seed(3)
    is_in = torch.rand((53, 6), generator=g) < 0.4
    ids, counts, cumsum, total = O.moe_routing_sort(is_in)
    assert total == int(is_in.sum()) and counts.tolist() == is_in.sum(0).tolist()
    for r in range(6):
        seg = ids[cumsum[r]:cumsum[r + 1]].tolist()
        assert seg == [t for t in range(53) if is_in[t, r]]
    cpm = O.channel_prefix_matrix(is_in, 10)
    per = -(-53 // 10)
    for d in range(6):
        run = 0
        for c in range(10):
            b = min(per * c, 53)
            run += sum(bool(is_in[t, d]) for t in range(b, min(b + per, 53)))
            assert cpm[d, c].item() == run
    assert cpm[:, -1].tolist() == counts.tolist()


# --------------------------------------------------------------------------
# Dispatch / combine
# --------------------------------------------------------------------------
def _world(r, t, h, k, e, seed, drop=5):
    g = torch.Generator().manual_seed(seed)
    xs = [torch.randn((t, h), generator=g).to(torch.bfloat16) for _ in range(r)]
    tk = [torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(t)]) for _ in range(r)]
    for _ in range(drop):
        s, i, j = [int(torch.randint(0, n, (1,), generator=g)) for n in (r, t, k)]
        tk[s][i, j] = -1
    return xs, tk


@pytest.mark.parametrize("fmt", [O.ROW_FP8, O.ROW_BF16, O.ROW_FP8_UE8M0])
def test_vectorised_dispatch_equals_serial_restatement(fmt):
    xs, tk = _world(4, 8, 512, 3, 16, seed=2)
    for rank in range(4):
        a = O.ll_dispatch(xs, tk, rank, 16, 8, fmt)
        b = O._serial_dispatch(xs, tk, rank, 16, 8, fmt)
        for key in a:
            assert torch.equal(a[key], b[key]), (rank, key)


def test_ranges_are_the_serial_prefix_over_ascending_source_ranks():
    """csrc/kernels/efa_kernels.cu:991-1010: begin(e, s) is the running sum of cnt(e, s') over s' < s, a
    range is 0 where the count is 0, and the counts are the pairs naming the expert on each source."""
    xs, tk = _world(4, 8, 512, 3, 16, seed=5, drop=4)
    for rank in range(4):
        got = O.ll_dispatch(xs, tk, rank, 16, 8, O.ROW_FP8)
        for le in range(4):
            cursor = 0
            for s in range(4):
                cnt = sum(1 for row in tk[s].tolist() for e in row if e == rank * 4 + le)
                lr = int(got["packed_recv_layout_range"][le, s])
                assert lr == (((cursor << 32) | cnt) if cnt else 0), (rank, le, s)
                cursor += cnt
            assert cursor == int(got["packed_recv_count"][le])


def test_dispatch_invariants_of_reference_test():
    # tests/test_low_latency.py:59-60,119-147: x = rank-128 with the token index in the last 128 columns.
    r, t, h, k, e = 4, 16, 256, 4, 16
    g = torch.Generator().manual_seed(9)
    xs = []
    for rank in range(r):
        x = torch.ones((t, h), dtype=torch.bfloat16) * (rank - 128)
        x[:, -128:] = torch.arange(t).to(torch.bfloat16).view(-1, 1)
        xs.append(x)
    tk = [torch.topk(torch.randn((t, e), generator=g).abs() + 1, k, dim=-1)[1] for _ in range(r)]
    for s in range(r):
        tk[s][s, 0] = -1
    all_tk = torch.stack(tk)
    for rank in range(r):
        out = O.ll_dispatch(xs, tk, rank, e, t, O.ROW_FP8)
        epr = e // r
        for i in range(epr):
            expert = rank * epr + i
            n = out["packed_recv_count"][i].item()
            lr = out["packed_recv_layout_range"][i]
            assert n == (lr & 0xFFFFFFFF).sum().item() == (all_tk == expert).sum().item()
            q = out["packed_recv_x"][i, :n].view(torch.float8_e4m3fn)
            sc = out["packed_recv_scales"][i, :n].view(torch.float32)
            recv = O.per_token_cast_back(q, sc).float()
            assert torch.equal(recv[:, :-128].amin(-1), recv[:, :-128].amax(-1))
            src = out["packed_recv_src_info"][i, :n]
            assert (recv[:, -128:] - src.view(-1, 1) % t).sum().item() == 0
            for j in range(r):
                begin, cnt = (lr[j] >> 32).item(), (lr[j] & 0xFFFFFFFF).item()
                assert cnt == (all_tk[j] == expert).sum().item()
                assert (recv[begin:begin + cnt, :-128] - j + 128).sum().item() == 0
                assert src[begin:begin + cnt].tolist() == sorted(src[begin:begin + cnt].tolist())


def test_route_slots_and_staged_rows():
    xs, tk = _world(2, 10, 256, 3, 8, seed=4, drop=3)
    send_count, pair_slot = O.route(tk[0], 8, 10)
    seen = {}
    for t in range(10):
        for k in range(3):
            e = int(tk[0][t, k])
            if e < 0:
                assert pair_slot[t, k] == -1
                continue
            assert pair_slot[t, k] == seen.get(e, 0)
            seen[e] = seen.get(e, 0) + 1
    assert send_count.tolist() == [seen.get(e, 0) for e in range(8)]
    sc, ps, experts, slots, rows = O.staged_rows(xs[0], tk[0], 1, 8, 10, O.ROW_FP8, num_ranks=2)
    assert O.row_payload(256, O.ROW_FP8) == 256 + 16 + 16
    assert rows.shape[1] == O.row_stride(256, O.ROW_FP8) == 384  # whole 128-byte lines
    assert (rows[:, 288:] == 0).all()
    tail = rows[:, 272:288].contiguous().view(torch.int32)
    assert (tail[:, 2] == 1).all() and torch.equal(tail[:, 3].long(), experts % 4)  # 8 experts on 2 ranks
    q, s = O.per_token_cast_to_fp8(xs[0])
    assert torch.equal(rows[:, :256], q.view(torch.uint8)[tail[:, 0].long()])
    assert torch.equal(rows[:, 256:264].contiguous().view(torch.float32), s[tail[:, 0].long()])


def test_combine_closed_form_and_chain(oracle_c):
    t, k, h = 12, 5, 256
    g = torch.Generator().manual_seed(6)
    x = torch.randn((t, h), generator=g).to(torch.bfloat16)
    w = torch.randn((t, k), generator=g).abs()
    topk = torch.randint(0, 32, (t, k), generator=g)
    topk[0, 1] = -1
    topk[3, :] = -1
    live = topk >= 0
    rows = x.unsqueeze(1).expand(t, k, h).contiguous()
    ref = O.ll_combine(rows, topk, w)
    # tests/test_low_latency.py:181: combined == x * sum of live weights
    want = x.double() * (w.double() * live.double()).sum(1, keepdim=True)
    assert torch.allclose(ref, want, rtol=1e-12, atol=0)
    assert (ref[3] == 0).all()
    chain = O.ll_combine_f32_chain(rows, w, live)
    out = torch.empty((t, h), dtype=torch.int16)
    live8 = live.to(torch.uint8).contiguous()
    oracle_c.oracle_combine_chain(_ptr(rows.view(torch.int16)), _ptr(w.contiguous()), _ptr(live8), t, k, h, _ptr(out))
    assert torch.equal(out.view(torch.bfloat16), chain)
    rel = (chain.double() - ref).abs() / ref.abs().clamp(min=1e-2)
    assert rel.max().item() < 1e-2
    assert O.calc_diff(chain, ref) < 1e-5
    # a random-output case: the chain is within bf16 rounding of the float64 sum
    rows2 = torch.randn((t, k, h), generator=g).to(torch.bfloat16)
    ref2 = O.ll_combine(rows2, topk, w)
    chain2 = O.ll_combine_f32_chain(rows2, w, live)
    assert ((chain2.double() - ref2).abs() <= ref2.abs() * 2 ** -8 + 1e-6).all()


def test_size_hint_hand_values():
    # by hand for (128, 7168, 32, 256): dmsg = 16 + max(14336, 7168 + 224) = 14352, cmsg = 224 + 14336 = 14560;
    # send = recv = max(128 * 14352, 256 * 128 * 14560) = 477102080; sig = 1024;
    # total = 4 * 477102080 + 2048 = 1908410368 -> (total + 128) // 128 * 128
    assert O.get_low_latency_rdma_size_hint(128, 7168, 32, 256) == 1908410496
    # tiny case by hand: M=1,H=128,E=2: dmsg=16+256=272, cmsg=4+256=260; send=max(272,520)=520; recv=max(544,520)=544
    # sig=128 -> total = 1040+1088+256 = 2384 -> (2384+128)//128*128 = 2432
    assert O.get_low_latency_rdma_size_hint(1, 128, 2, 2) == 2432
    # the reference's cooperative send stride (csrc/kernels/coop_dispatch_send.cu:73-75) is this build's row payload
    assert O.row_payload(7168, O.ROW_FP8) == 7408 and O.row_payload(7168, O.ROW_BF16) == 14352
    assert O.row_payload(7168, O.ROW_FP8_UE8M0) == 7168 + 64 + 16
    assert O.row_stride(7168, O.ROW_FP8) == 7424 and O.row_stride(7168, O.ROW_BF16) == 14464
    assert O.row_stride(7168, O.ROW_FP8_UE8M0) == 7296 and O.row_stride(512, O.ROW_FP8) == 640


# --------------------------------------------------------------------------
# Seeded world: numpy restatement vs the C one, and distribution sanity
# --------------------------------------------------------------------------
def test_seeded_rows_numpy_equals_c(oracle_c):
    for x in (0, 1, 0xDEADBEEF, 0xFFFFFFFF, 12345):
        assert int(O.mix32(x)) == oracle_c.oracle_mix32(x)
    keys = np.array([0, 1, 2, 99, 2 ** 31, 2 ** 32 - 1, 777], dtype=np.uint32)
    for period in (0, 3):
        a = O.synth_bf16_rows(keys, 384, seed=42, outlier_period=period)
        b = torch.empty((len(keys), 384), dtype=torch.int16)
        oracle_c.oracle_synth_bf16_rows(keys.ctypes.data_as(ctypes.c_void_p), len(keys), 384, 42, period, _ptr(b))
        assert torch.equal(a.view(torch.int16), b)
    big = O.synth_bf16_rows(np.arange(64, dtype=np.uint32), 7168, seed=1).float()
    assert abs(big.mean().item()) < 0.01 and abs(big.std().item() - 1.0) < 0.02
    hot = O.synth_bf16_rows(np.arange(4000, dtype=np.uint32), 8, seed=1, outlier_period=100).float()
    frac = ((hot.abs().amax(1)) > 20).float().mean().item()
    assert 0.004 < frac < 0.02


@pytest.mark.parametrize("cdf_name", ["uniform", "zipf"])
def test_seeded_topk_numpy_equals_c(oracle_c, cdf_name):
    e, k, t = 64, 8, 50
    cdf = O.uniform_cdf(e) if cdf_name == "uniform" else O.zipf_cdf(e)
    assert cdf[-1] == 0xFFFFFFFF and (np.diff(cdf.astype(np.int64)) >= 0).all()
    ranks = np.array([0, 3, 5], dtype=np.int32)
    a = O.synth_topk_idx(cdf, ranks, t, k, seed=17)
    b = torch.empty((3, t, k), dtype=torch.int64)
    oracle_c.oracle_synth_topk_idx(cdf.ctypes.data_as(ctypes.c_void_p), ranks.ctypes.data_as(ctypes.c_void_p), 3, t, k,
                                   e, 17, _ptr(b))
    assert torch.equal(a, b)
    srt = torch.sort(a, dim=-1).values
    assert (srt[..., 1:] != srt[..., :-1]).all() and a.min() >= 0 and a.max() < e
    if cdf_name == "zipf":
        assert (a == 0).any(-1).float().mean() > 0.5  # the hottest expert is in most tokens


# ---- normal mode: top-k remap, source metadata, combine reduce -------------------------------------
def _normal_world(t, k, e, r, seed):
    g = torch.Generator().manual_seed(seed)
    topk = torch.argsort(torch.rand((t, e), generator=g), dim=1)[:, :k].contiguous()
    topk[t // 2, 0] = -1
    topk[0, :] = -1     # a token sent nowhere
    topk[1, 1:] = -1    # a token held by exactly one rank
    w = torch.rand((t, k), generator=g)
    _, _, _, is_in = O.get_dispatch_layout(topk, e, r)
    ids, counts, cumsum, _ = O.moe_routing_sort(is_in)
    return topk, w, is_in, ids, counts, cumsum


def test_topk_remap_against_the_kernels_per_element_rule():
    # csrc/kernels/efa_kernels.cu:352-386, one (row, k) at a time
    t, k, e, r = 37, 4, 24, 6
    topk, w, _, ids, _, cumsum = _normal_world(t, k, e, r, seed=3)
    got_e, got_w = O.topk_remap(topk, w, ids, cumsum, e // r)
    total = int(cumsum[r])
    assert got_e.shape == (total, k)
    for row in range(total):
        dst = max(d for d in range(r) if int(cumsum[d]) <= row and int(cumsum[d + 1]) > row)
        tok = int(ids[row])
        for kk in range(k):
            ex = int(topk[tok, kk])
            lo, hi = dst * (e // r), (dst + 1) * (e // r)
            if lo <= ex < hi and ex >= 0:
                assert int(got_e[row, kk]) == ex - lo and float(got_w[row, kk]) == float(w[tok, kk])
            else:
                assert int(got_e[row, kk]) == -1 and float(got_w[row, kk]) == 0.0
    # every send row keeps at least one selection: that is why the token was sent to that rank
    assert ((got_e >= 0).sum(1) >= 1).all()


def test_build_recv_src_meta_against_the_kernels_per_element_rule():
    # csrc/kernels/efa_kernels.cu:456-481
    cumsum = torch.tensor([0, 3, 3, 4, 9, 9, 11, 11, 12, 15, 15, 15, 16, 20, 20, 21, 30, 31], dtype=torch.int64)
    r, local = cumsum.numel() - 1, 8
    meta = O.build_recv_src_meta(cumsum, local).view(torch.int32).view(-1, 2)
    assert meta.shape[0] == int(cumsum[r])
    for i in range(meta.shape[0]):
        src = max(s for s in range(r) if int(cumsum[s]) <= i < int(cumsum[s + 1]))
        assert meta[i].tolist() == [src // local, 1 << (src % local)]


def test_combine_reduce_definitions_agree():
    t, k, e, r, h = 29, 3, 16, 4, 256
    topk, w, is_in, ids, counts, cumsum = _normal_world(t, k, e, r, seed=8)
    g = torch.Generator().manual_seed(1)
    total = int(cumsum[r])
    rows = torch.randn((total, h), generator=g).to(torch.bfloat16)
    rw = torch.rand((total, k), generator=g)
    b0 = torch.randn((t, h), generator=g).to(torch.bfloat16)
    ref_x, ref_w = O.combine_reduce(rows, rw, ids, t, b0, None)
    # the same sum written as a loop over (token, rank) pairs
    want = b0.double().clone()
    pos = 0
    for rank in range(r):
        for tok in range(t):
            if is_in[tok, rank]:
                want[tok] += rows[pos].double()
                pos += 1
    assert pos == total and torch.equal(ref_x, want)
    chain_x, chain_w = O.combine_reduce_f32_chain(rows, rw, ids, cumsum, t, b0, None)
    err = (chain_x.double() - ref_x).abs()
    assert (err <= 2.0 ** -8 * ref_x.abs() + 1e-6).all()  # one bf16 rounding of a float32 sum of <= 5 terms
    assert torch.allclose(chain_w.double(), ref_w, rtol=1e-6, atol=1e-7)
    # a token held by exactly one rank gets its row back bit for bit (no bias)
    chain_nb, _ = O.combine_reduce_f32_chain(rows, None, ids, cumsum, t)
    single = torch.nonzero(is_in.sum(1) == 1).flatten()
    assert single.numel() > 0
    for tok in single.tolist():
        j = int(torch.nonzero(ids == tok).flatten()[0])
        assert torch.equal(chain_nb[tok].view(torch.int16), rows[j].view(torch.int16))
    # a token sent nowhere gives zeros
    none = torch.nonzero(is_in.sum(1) == 0).flatten()
    for tok in none.tolist():
        assert (chain_nb[tok] == 0).all()


# ---------------------------------------------------------------------------
# the hand-derived two-rank world of tests/golden/ll_tiny_world.json
# ---------------------------------------------------------------------------
from tiny_world import load_tiny_world, tiny_world_expected  # noqa: E402


@pytest.mark.parametrize("key,rank", [("rank0_ascending", 0), ("rank1_ascending", 1)])
@pytest.mark.parametrize("fmt", [O.ROW_BF16, O.ROW_FP8])
def test_oracle_against_the_hand_derived_world(key, rank, fmt):
    g, x_all, topk_all = load_tiny_world()
    e, m, h = g["num_experts"], g["max_tokens"], g["hidden"]
    got = O.ll_dispatch(x_all, topk_all, rank, e, m, fmt)
    want, layout = tiny_world_expected(g, key)
    assert got["packed_recv_count"].tolist() == want["count"]
    assert torch.equal(got["packed_recv_layout_range"], layout)
    for le, n in enumerate(want["count"]):
        assert got["packed_recv_src_info"][le, :n].tolist() == want["src_info"][le]
        values = torch.tensor(want["row_value"][le], dtype=torch.float32)
        if fmt == O.ROW_BF16:
            rows = got["packed_recv_x"][le, :n].contiguous().view(torch.bfloat16).float()
            assert torch.equal(rows, values.view(-1, 1).expand(-1, h))
        else:
            assert (got["packed_recv_x"][le, :n] == g["fp8"]["payload_byte"]).all()
            scales = got["packed_recv_scales"][le, :n].contiguous().view(torch.float32).view(-1)
            assert torch.equal(scales, values / torch.tensor(448.0))  # one group per row
    if rank == 0:
        send_count, pair_slot = O.route(topk_all[0], e, m)
        assert send_count.tolist() == g["route_rank0"]["send_count"]
        assert pair_slot.tolist() == g["route_rank0"]["pair_slot"]
        pr, pn, pe, is_in = O.get_dispatch_layout(topk_all[0], e, g["num_ranks"])
        assert pe.tolist() == g["layout_rank0"]["num_tokens_per_expert"]
        assert pr.tolist() == g["layout_rank0"]["num_tokens_per_rank"] and pn is None
        assert is_in.tolist() == g["layout_rank0"]["is_token_in_rank"]


def test_oracle_combine_against_the_hand_derived_world():
    g, x_all, topk_all = load_tiny_world()
    w = torch.tensor(g["topk_weights_rank0"], dtype=torch.float32)
    pair_rows = x_all[0].unsqueeze(1).expand(-1, g["num_topk"], -1)  # identity experts
    want = torch.tensor(g["combine_rank0_identity_experts"]).view(-1, 1).expand(-1, g["hidden"])
    assert torch.equal(O.ll_combine(pair_rows, topk_all[0], w).float(), want)
    assert torch.equal(O.ll_combine_f32_chain(pair_rows, w, topk_all[0] >= 0).float(), want)


def test_oracle_normal_mode_against_the_hand_derived_world():
    g, _, _ = load_tiny_world()
    want = g["normal_mode_rank0"]
    is_in = torch.tensor(g["layout_rank0"]["is_token_in_rank"])
    ids, counts, cumsum, total = O.moe_routing_sort(is_in)
    assert ids.tolist() == want["sorted_token_ids"] and counts.tolist() == want["send_counts"]
    assert cumsum.tolist() == want["send_cumsum"] and total == 4
    assert O.channel_prefix_matrix(is_in, 2).tolist() == want["channel_prefix_matrix_2_channels"]
    assert O.channel_prefix_matrix(is_in, 3).tolist() == want["channel_prefix_matrix_3_channels"]


@pytest.mark.parametrize("rank", [0, 1])
def test_oracle_exchange_metadata_against_the_hand_derived_world(rank):
    g, _, topk_all = load_tiny_world()
    routed = torch.tensor(g["all_num_routed"], dtype=torch.int32)
    for s in range(g["num_ranks"]):  # the matrix itself: row s is rank s's per-expert pair count
        assert routed[s].tolist() == O.route(topk_all[s], g["num_experts"], g["max_tokens"])[0].tolist()
    got = O.ll_exchange_metadata(routed, rank, g["max_tokens"])
    want = g["exchange_metadata"][f"rank{rank}"]
    for key, value in want.items():
        assert (got[key].tolist() if torch.is_tensor(got[key]) else got[key]) == value, key
    assert not got["corrupt"]


def test_oracle_exchange_metadata_identities_and_corrupt_counts():
    r, e, m, rank = 6, 24, 40, 4
    g = torch.Generator().manual_seed(9)
    topk_all = [torch.stack([torch.randperm(e, generator=g)[:5] for _ in range(m)]) for _ in range(r)]
    routed = torch.stack([O.route(tk, e, m)[0] for tk in topk_all]).to(torch.int32)
    got = O.ll_exchange_metadata(routed, rank, m)
    epr = e // r
    # what the dispatch itself delivers: rows from source s = its pairs on this rank's experts
    want = O.ll_dispatch([torch.zeros((m, 128), dtype=torch.bfloat16)] * r, topk_all, rank, e, m, O.ROW_BF16)
    per_source = (want["packed_recv_layout_range"] & 0xFFFFFFFF).sum(0)
    assert got["recv_counts"].tolist() == per_source.tolist()
    assert got["total_recv"] == int(want["packed_recv_count"].sum())
    assert got["send_counts"].tolist() == routed[rank].view(r, epr).sum(1).tolist()
    assert got["padded_index"].tolist() == list(range(got["total_recv"])) == got["combine_send_offset"].tolist()
    assert got["combine_remote_recv_offset"].tolist() == routed[:, :rank * epr].sum(1).tolist()
    routed[2, 7] = m + 1  # one impossible count: nobody sends or receives this time
    bad = O.ll_exchange_metadata(routed, rank, m)
    assert bad["corrupt"] and bad["total_send"] == 0 and bad["total_recv"] == 0
    assert bad["send_counts"].sum() == 0 and bad["recv_counts"].sum() == 0 and bad["source_rank"].numel() == 0


def test_round_scale_has_one_answer_for_every_bf16_amax():
    """The reference rounds a scale up to a power of two as exp2(ceil(log2(s))) in float32
    (csrc/kernels/efa_kernels.cu:158, deep_ep/buffer.py:1601); oracle and kernel take the smallest power of
    two >= s from the bit pattern.  The two can only differ where log2f's rounding error carries ceil over an
    integer, i.e. for s a hair above a power of two.  On this path s = amax / 448 with amax a bf16 value (or the
    1e-4 clamp), and that never happens: over every positive finite bf16 amax, log2(s) is either an integer
    exactly (amax = 1.75 * 2^j) or at least 0.006 away from one — four hundred times the spacing of float32
    near the largest |log2(s)| — so any log2f good to a few ulps gives the same ceiling.  torch's own
    float32 log2 / ceil / exp2 on the CPU, the form the reference's Python writes, agrees on every one."""
    bits = torch.arange(1, 0x7F80, dtype=torch.int32)  # every positive finite bf16, subnormals included
    amax = (bits << 16).view(torch.float32).clamp(min=1e-4)
    amax = torch.cat([amax, torch.tensor([1e-4])])
    s = amax / 448.0
    exact = np.log2(s.numpy().astype(np.float64))
    off = np.abs(exact - np.round(exact))
    is_pow2 = (s.view(torch.int32) & 0x7FFFFF).numpy() == 0
    assert (off[is_pow2] == 0).all() and is_pow2.sum() > 100
    assert off[~is_pow2].min() > 0.006
    assert np.abs(exact).max() < 128 and np.spacing(np.float32(127.0)) < 0.006 / 400
    want = np.exp2(np.ceil(exact)).astype(np.float32)
    assert np.array_equal(O.pow2_ceil(s).numpy(), want)
    assert torch.equal(torch.exp2(torch.ceil(torch.log2(s))), O.pow2_ceil(s))


@pytest.mark.parametrize("rank", [0, 1])
def test_oracle_all_to_all_surface_against_the_hand_derived_world(rank):
    """Message order, per-record packed rows and the flat buffers of both directions, against values worked
    out on paper (tests/golden/ll_tiny_world.json)."""
    g, x_all, topk_all = load_tiny_world()
    e, m, h, r = g["num_experts"], g["max_tokens"], g["hidden"], g["num_ranks"]
    want = g["send_by_dest"][f"rank{rank}"]
    got = O.ll_send_by_dest(x_all[rank], topk_all[rank], rank, e, m, O.ROW_BF16, r)
    assert got["send_expert_prefix"].tolist() == want["send_expert_prefix"]
    assert got["send_counts"].tolist() == want["send_counts"]
    assert got["send_cumsum"].tolist() == want["send_cumsum"]
    assert got["pair_send_row"].tolist() == want["pair_send_row"]
    tail_at = O.row_payload(h, O.ROW_BF16) - 16
    tails = got["rows"][:, tail_at:tail_at + 16].contiguous().view(torch.int32)
    assert tails[:, 0].tolist() == want["row_token"] and tails[:, 1].tolist() == want["row_topk_slot"]
    assert tails[:, 2].tolist() == [rank] * len(want["row_token"]) and tails[:, 3].tolist() == want["row_local_expert"]
    values = got["rows"][:, :2 * h].contiguous().view(torch.bfloat16).float()
    assert torch.equal(values, torch.tensor([g["x_value"][rank][t] for t in want["row_token"]],
                                            dtype=torch.float32).view(-1, 1).expand(-1, h))
    rec = O.ll_record_packed_rows(topk_all, rank, e, m)
    assert rec.tolist() == g["record_packed_row"][f"rank{rank}"]
    meta = g["exchange_metadata"][f"rank{rank}"]
    packed = O.ll_dispatch(x_all, topk_all, rank, e, m, O.ROW_BF16)
    y = packed["packed_recv_x"].view(e // r, r * m, 2 * h).contiguous().view(torch.bfloat16)
    flat = O.ll_combine_send_by_dest(y, rec, torch.tensor(meta["padded_index"]), torch.tensor(meta["combine_send_offset"]))
    assert flat.float()[:, 0].tolist() == g["combine_send_flat_identity_experts"][f"rank{rank}"]
    assert (flat.float() == flat.float()[:, :1]).all()
    if rank == 0:
        back = torch.tensor(g["combine_recv_flat_rank0_identity_experts"], dtype=torch.float32).view(-1, 1).expand(-1, h)
        pair_rows, live = O.ll_combine_recv_flat_rows(back.to(torch.bfloat16), 0, got["send_expert_prefix"], topk_all[0],
                                                      got["pair_slot"], e // r)
        w = torch.tensor(g["topk_weights_rank0"], dtype=torch.float32)
        out = O.ll_combine_f32_chain(pair_rows, w, live)
        assert out.float()[:, 0].tolist() == g["combine_rank0_identity_experts"]
