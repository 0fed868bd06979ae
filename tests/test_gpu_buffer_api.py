"""GPU tests of the deep_ep.Buffer API, written after the reference's own drivers
(tests/test_low_latency.py:38-193, tests/test_intranode.py:35-66) with the other ranks
supplied by the loopback world instead of real processes."""
import random

import numpy as np
import pytest
import torch

from oracle import deepep_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def deep_ep():
    import deep_ep as mod
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return mod


def hash_tensor(t: torch.Tensor) -> int:
    """tests/utils.py:274."""
    return t.contiguous().view(torch.int8).to(torch.int64).sum().item() ^ t.numel()


def reference_world(num_ranks, num_tokens, hidden, num_experts, num_topk, seed):
    """Inputs of every rank as tests/test_low_latency.py:49-76 builds them (CPU generator)."""
    xs, tks, ws = [], [], []
    for rank in range(num_ranks):
        g = torch.Generator().manual_seed(seed + rank)
        rnd = random.Random(seed + rank)
        x = torch.ones((num_tokens, hidden), dtype=torch.bfloat16) * (rank - 128)
        x[:, -128:] = torch.arange(num_tokens).to(torch.bfloat16).view(-1, 1)
        scores = torch.randn((num_tokens, num_experts), generator=g).abs() + 1
        topk_idx = torch.topk(scores, num_topk, dim=-1, largest=True, sorted=True)[1]
        w = torch.randn((num_tokens, num_topk), generator=g).abs()
        for _ in range(10):
            topk_idx[rnd.randint(0, num_tokens - 1), rnd.randint(0, num_topk - 1)] = -1
        xs.append(x)
        tks.append(topk_idx)
        ws.append(w)
    return torch.stack(xs), torch.stack(tks), torch.stack(ws)


def reference_test_main(deep_ep, buffer, num_ranks, rank, num_tokens, hidden, num_topk, num_experts, seed, check=True,
                        cache=None):
    """The body of the reference's test_main (tests/test_low_latency.py:38-193) for one rank: every payload
    format, both completion styles, two inputs; returns the XOR of the hashes of every output (:118-193).
    check=False repeats the calls and the hashing only (the pressure loop, :316-329), taking the experts'
    outputs from `cache`, which a checking run filled."""
    num_local_experts = num_experts // num_ranks
    x_all, topk_all, w_all = reference_world(num_ranks, num_tokens, hidden, num_experts, num_topk, seed=seed)
    x_rand = (torch.randn((num_tokens, hidden), generator=torch.Generator().manual_seed(5)) * 0.1).to(torch.bfloat16)
    topk_idx = topk_all[rank].cuda().to(deep_ep.topk_idx_t)
    topk_weights = w_all[rank].cuda()
    all_topk_idx = topk_all
    cache = {} if cache is None else cache

    hash_value, num_times, hashes = 0, 0, {}
    for which, x_cpu in (("const", x_all[rank]), ("rand", x_rand)):
        world_x = x_all.clone()
        world_x[rank] = x_cpu
        buffer.loopback_set_world(world_x.cuda(), topk_all.cuda())
        current_x = x_cpu.cuda()
        for return_recv_hook in (False, True):
            for use_fp8 in (False, True):
                for round_scale in (False, True) if use_fp8 else (False,):
                    for use_ue8m0 in (False, True) if round_scale else (False,):
                        num_times += 1
                        for _ in range((num_times % 2) + 1):
                            stats = torch.zeros((num_local_experts,), dtype=torch.int, device="cuda")
                            packed_recv_x, packed_recv_count, handle, event, hook = buffer.low_latency_dispatch(
                                current_x, topk_idx, num_tokens, num_experts, use_fp8=use_fp8,
                                round_scale=round_scale, use_ue8m0=use_ue8m0,
                                cumulative_local_expert_recv_stats=stats, async_finish=not return_recv_hook,
                                return_recv_hook=return_recv_hook, topk_weights=topk_weights)
                            hook() if return_recv_hook else event.current_stream_wait()
                        torch.cuda.synchronize()
                        count_cpu = packed_recv_count.cpu()
                        key = (which, use_fp8, round_scale, use_ue8m0)
                        h = 0
                        for i in range(num_local_experts):  # the hash of what arrived, taken where it lies
                            n = int(count_cpu[i])
                            if n == 0:
                                continue
                            if use_fp8:
                                h ^= hash_tensor(packed_recv_x[0][i, :n]) ^ hash_tensor(packed_recv_x[1][i, :n])
                            else:
                                h ^= hash_tensor(packed_recv_x[i, :n])
                        if check:
                            if use_fp8:
                                assert packed_recv_x[0].dtype == torch.float8_e4m3fn
                                assert packed_recv_x[0].shape == (num_local_experts, num_ranks * num_tokens, hidden)
                                want_scale = (hidden // 512, torch.int32) if use_ue8m0 else (hidden // 128, torch.float32)
                                assert packed_recv_x[1].shape[-1] == want_scale[0] and packed_recv_x[1].dtype == want_scale[1]
                                fp8_cpu, scales_cpu = packed_recv_x[0].cpu(), packed_recv_x[1].cpu()
                            else:
                                assert packed_recv_x.dtype == torch.bfloat16
                                recv_cpu = packed_recv_x.cpu()
                            src_info_cpu, layout_cpu = handle[0].cpu(), handle[1].cpu()
                            assert handle[2:] == (num_tokens, hidden, num_experts)
                            assert src_info_cpu.dtype == torch.int32 and layout_cpu.shape == (num_local_experts, num_ranks)
                            simulated = torch.zeros((num_local_experts, num_ranks * num_tokens, hidden), dtype=torch.bfloat16)
                            for i in range(num_local_experts):
                                expert_id = rank * num_local_experts + i
                                n = int(count_cpu[i])
                                lr = layout_cpu[i]
                                int_mask = (2 ** 32) - 1
                                assert int(stats[i]) == n
                                assert n == int((lr & int_mask).sum())
                                assert n == int((all_topk_idx == expert_id).sum())
                                if n == 0:
                                    continue
                                if use_fp8:
                                    recv_x = O.per_token_cast_back(fp8_cpu[i, :n], scales_cpu[i, :n])
                                else:
                                    recv_x = recv_cpu[i, :n]
                                simulated[i, :n] = recv_x
                                src = src_info_cpu[i, :n]
                                if which == "const":
                                    rf = recv_x.float()
                                    amin = rf[:, :-128].amin(dim=-1)
                                    assert torch.equal(amin, rf[:, :-128].amax(dim=-1))
                                    if round_scale:
                                        assert O.calc_diff(rf[:, -1], src.float()) < 0.007
                                    else:
                                        # the recipe stores the token index as bf16 (exact up to 256 tokens)
                                        stored = (src % num_tokens).to(torch.bfloat16).float().view(-1, 1)
                                        assert (rf[:, -128:] - stored).sum().item() == 0
                                    for j in range(num_ranks):
                                        begin, cnt = int(lr[j] >> 32), int(lr[j] & int_mask)
                                        if not round_scale:
                                            assert int((amin == j - 128).sum()) == int((all_topk_idx[j] == expert_id).sum())
                                            assert (rf[begin:begin + cnt, :-128] - j + 128).sum().item() == 0
                            cache[key] = simulated.cuda()
                        # combine, with and without the zero-copy buffer
                        sim_dev = cache[key]
                        for zero_copy in (False, True):
                            if zero_copy:
                                buffer.get_next_low_latency_combine_buffer(handle)[:, :, :] = sim_dev
                            out = torch.empty((num_tokens, hidden), dtype=torch.bfloat16, device="cuda")
                            combined_x, event, hook = buffer.low_latency_combine(
                                sim_dev, topk_idx, topk_weights, handle, async_finish=not return_recv_hook,
                                zero_copy=zero_copy, return_recv_hook=return_recv_hook, out=out)
                            hook() if return_recv_hook else event.current_stream_wait()
                            torch.cuda.synchronize()
                            if check:
                                assert combined_x.data_ptr() == out.data_ptr()
                                want = x_cpu.float() * topk_weights.cpu().masked_fill(topk_idx.cpu() == -1, 0).sum(dim=1).view(-1, 1)
                                diff = O.calc_diff(want, combined_x.cpu())
                                assert torch.isnan(combined_x.float()).sum().item() == 0
                                if not round_scale:
                                    assert diff < (9e-4 if use_fp8 else 1e-5), f"{diff=} {use_fp8=} {zero_copy=}"
                            h ^= hash_tensor(combined_x)
                        # the same inputs give the same bytes on every call (tests/test_low_latency.py:319-329)
                        if key in hashes:
                            assert hashes[key] == h
                        hashes[key] = h
                        hash_value ^= h
    return hash_value


@pytest.mark.parametrize("num_ranks,rank,num_tokens,hidden,num_topk,num_experts",
                         [(8, 2, 128, 2048, 8, 288), (16, 15, 64, 7168, 8, 256),
                          (4, 1, 2100, 512, 8, 64)])  # a prefill-sized batch: histograms + send, index + flat copies
def test_low_latency_as_the_reference_tests_it(deep_ep, num_ranks, rank, num_tokens, hidden, num_topk, num_experts):
    assert num_experts % num_ranks == 0
    num_rdma_bytes = deep_ep.Buffer.get_low_latency_rdma_size_hint(num_tokens, hidden, num_ranks, num_experts)
    buffer = deep_ep.Buffer(None, num_rdma_bytes=num_rdma_bytes, low_latency_mode=True,
                            num_qps_per_rank=num_experts // num_ranks, explicitly_destroy=True,
                            sim_num_ranks=num_ranks, sim_rank=rank)
    reference_test_main(deep_ep, buffer, num_ranks, rank, num_tokens, hidden, num_topk, num_experts, seed=1)
    buffer.clean_low_latency_buffer(num_tokens, hidden, num_experts)
    buffer.destroy()


def test_pressure_every_rerun_hashes_the_same(deep_ep):
    """The reference's pressure check (tests/test_low_latency.py:316-329) at the headline shape, one rank of
    EP=32 with 128 tokens x 7168 and top-8 of 256 experts: test_main once for the reference hash, then twenty
    more times, and every rerun must hash every output to the same value; the loop stops at the first that
    does not.  No kernel on this path claims a slot or adds with an atomic in HBM, so nothing depends on
    scheduling."""
    num_ranks, rank, num_tokens, hidden, num_topk, num_experts = 32, 5, 128, 7168, 8, 256
    buffer = deep_ep.Buffer(None, low_latency_mode=True, num_qps_per_rank=num_experts // num_ranks,
                            explicitly_destroy=True, sim_num_ranks=num_ranks, sim_rank=rank)
    for seed in (0,):
        experts_outputs = {}
        ref_hash = reference_test_main(deep_ep, buffer, num_ranks, rank, num_tokens, hidden, num_topk, num_experts,
                                       seed=seed, check=True, cache=experts_outputs)
        for rerun in range(20):
            got = reference_test_main(deep_ep, buffer, num_ranks, rank, num_tokens, hidden, num_topk, num_experts,
                                      seed=seed, check=False, cache=experts_outputs)
            assert got == ref_hash, f"Error: seed={seed} rerun={rerun}"
    buffer.clean_low_latency_buffer(num_tokens, hidden, num_experts)
    buffer.destroy()


def test_dispatch_matches_oracle_through_the_api(deep_ep):
    num_ranks, rank, t, h, k, e = 32, 9, 128, 7168, 8, 256
    buffer = deep_ep.Buffer(None, low_latency_mode=True, explicitly_destroy=True, sim_num_ranks=num_ranks,
                            sim_rank=rank, sim_seed=77)
    x, topk_idx = buffer.loopback_synthesise(t, h, k, e)
    (recv_x, recv_scales), recv_count, handle, event, hook = buffer.low_latency_dispatch(x, topk_idx, t, e)
    event.current_stream_wait()
    torch.cuda.synchronize()
    assert hook is None
    topk_all = O.synth_topk_idx(O.uniform_cdf(e), np.arange(num_ranks), t, k, 77)
    x_all = O.synth_bf16_rows(np.arange(num_ranks * t, dtype=np.uint32), h, 77).view(num_ranks, t, h)
    # at this size the API's dispatch is one launch
    want = O.ll_dispatch(list(x_all), list(topk_all), rank, e, t, O.ROW_FP8)
    assert torch.equal(recv_count.cpu(), want["packed_recv_count"])
    assert torch.equal(handle[1].cpu(), want["packed_recv_layout_range"])
    px, ps, si = recv_x.view(torch.uint8).cpu(), recv_scales.view(torch.uint8).cpu(), handle[0].cpu()
    for le in range(e // num_ranks):
        n = int(recv_count[le])
        assert torch.equal(px[le, :n], want["packed_recv_x"][le, :n])
        assert torch.equal(ps[le, :n].reshape(n, -1), want["packed_recv_scales"][le, :n])
        assert torch.equal(si[le, :n], want["packed_recv_src_info"][le, :n])
    buffer.destroy()


def test_combine_accumulates_into_out_through_the_api(deep_ep):
    """accumulate=True starts the float32 sum from what `out` holds (csrc/kernels/coop_combine_recv.cuh:174-179):
    checked bit for bit against the float32 FMA chain started from the previous contents."""
    num_ranks, rank, t, h, k, e = 8, 5, 48, 1024, 4, 64
    buffer = deep_ep.Buffer(None, low_latency_mode=True, explicitly_destroy=True, sim_num_ranks=num_ranks,
                            sim_rank=rank, sim_seed=11)
    x, topk_idx = buffer.loopback_synthesise(t, h, k, e)
    topk_idx = topk_idx.clone()
    topk_idx[7, 2] = -1
    topk_idx[9, :] = -1  # a token sent nowhere keeps what `out` held
    w = torch.rand((t, k), generator=torch.Generator().manual_seed(2)).cuda()
    recv_x, recv_count, handle, _, _ = buffer.low_latency_dispatch(x, topk_idx, t, e, use_fp8=False)
    y = recv_x.clone()  # identity experts on the bf16 rows: every pair's answer is x[t] itself
    prev = torch.randn((t, h), generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    plain, _, _ = buffer.low_latency_combine(y, topk_idx, w, handle)
    plain = plain.clone()
    out = prev.cuda()
    got, _, _ = buffer.low_latency_combine(y, topk_idx, w, handle, out=out, accumulate=True)
    torch.cuda.synchronize()
    assert got.data_ptr() == out.data_ptr()
    pair_rows = x.cpu().unsqueeze(1).expand(t, k, h)
    live = topk_idx.cpu() >= 0
    want_plain = O.ll_combine_f32_chain(pair_rows, w.cpu(), live)
    want_acc = O.ll_combine_f32_chain(pair_rows, w.cpu(), live, initial=prev)
    assert torch.equal(plain.cpu().view(torch.int16), want_plain.view(torch.int16))
    assert torch.equal(got.cpu().view(torch.int16), want_acc.view(torch.int16))
    assert torch.equal(got[9].cpu().view(torch.int16), prev[9].view(torch.int16))
    with pytest.raises(AssertionError, match="accumulate adds to `out`"):
        buffer.low_latency_combine(y, topk_idx, w, handle, accumulate=True)
    buffer.destroy()


def test_layout_calls_on_two_streams_in_flight_together(deep_ep):
    """An asynchronous call (on the buffer's stream) followed by a synchronous one (on the caller's) before
    the first event is waited on: each stream has its own scratch, so both give the right counts."""
    num_ranks, num_experts, num_tokens, num_topk = 8, 256, 4096, 8
    buffer = deep_ep.Buffer(None, explicitly_destroy=True, sim_num_ranks=num_ranks, sim_rank=1)
    g = torch.Generator().manual_seed(99)
    topk_a = torch.topk(torch.rand((num_tokens, num_experts), generator=g), num_topk, dim=-1)[1]
    topk_b = torch.topk(torch.rand((num_tokens, num_experts), generator=g), num_topk, dim=-1)[1]
    dev_a, dev_b = topk_a.cuda(), topk_b.cuda()
    want_a = O.get_dispatch_layout(topk_a, num_experts, num_ranks)
    want_b = O.get_dispatch_layout(topk_b, num_experts, num_ranks)
    for _ in range(20):
        ra = buffer.get_dispatch_layout(dev_a, num_experts, async_finish=True)
        rb = buffer.get_dispatch_layout(dev_b, num_experts)
        ra[4].current_stream_wait()
        torch.cuda.synchronize()
        for got, want in ((ra, want_a), (rb, want_b)):
            assert torch.equal(got[0].cpu(), want[0]) and torch.equal(got[2].cpu(), want[2])
            assert torch.equal(got[3].cpu(), want[3])
    buffer.destroy()


def test_profile_report_line(deep_ep, monkeypatch, capsys):
    """DEEPEP_PROFILE=1 prints the reference's report line (deep_ep/buffer.py:67-76) every
    DEEPEP_PROFILE_INTERVAL calls, after DEEPEP_PROFILE_WARMUP uncounted ones."""
    import re
    from deepep_efa_amd import buffer as buffer_module
    monkeypatch.setattr(buffer_module, "_PROFILE_ENABLED", True)
    monkeypatch.setattr(buffer_module, "_PROFILE_PRINT_EVERY", 2)
    monkeypatch.setattr(buffer_module, "_PROFILE_WARMUP", 1)
    buffer = deep_ep.Buffer(None, low_latency_mode=True, explicitly_destroy=True, sim_num_ranks=4, sim_rank=2)
    x, topk_idx = buffer.loopback_synthesise(16, 512, 2, 16)
    w = torch.ones((16, 2), dtype=torch.float32, device="cuda")
    for call in range(5):  # 1 warm-up + 2 reports of 2 calls each
        recv, _, handle, _, _ = buffer.low_latency_dispatch(x, topk_idx, 16, 16, use_fp8=False)
        buffer.low_latency_combine(recv, topk_idx, w, handle)
    torch.cuda.synchronize()
    lines = [l for l in capsys.readouterr().err.splitlines() if l.startswith("[LL_PROFILE")]
    assert len(lines) == 4
    pattern = r"\[LL_PROFILE rank=2\] (DISPATCH|COMBINE) \(avg of 2\): start->end=\d+\.\d+us \| TOTAL=\d+\.\d+us"
    assert all(re.fullmatch(pattern, l) for l in lines), lines
    assert [l.split()[2] for l in lines] == ["DISPATCH", "COMBINE", "DISPATCH", "COMBINE"]
    buffer.destroy()


def test_get_dispatch_layout_api(deep_ep):
    """tests/test_intranode.py:35-66 recipe, plus the event plumbing of csrc/deep_ep.cpp:526-574."""
    for num_ranks, num_experts, num_tokens, num_topk in ((8, 256, 4096, 8), (16, 256, 128, 8), (64, 256, 333, 6)):
        buffer = deep_ep.Buffer(None, explicitly_destroy=True, sim_num_ranks=num_ranks, sim_rank=1)
        g = torch.Generator().manual_seed(num_ranks)
        scores = torch.randn((num_tokens, num_experts), generator=g).abs() + 1
        topk_idx = torch.topk(scores, num_topk, dim=-1)[1]
        topk_idx[3, 1] = -1
        dev = topk_idx.cuda()
        want = O.get_dispatch_layout(topk_idx, num_experts, num_ranks)
        for async_finish in (False, True):
            prev = buffer.capture() if async_finish else None
            per_rank, per_rdma, per_expert, is_in, event = buffer.get_dispatch_layout(
                dev, num_experts, previous_event=prev, async_finish=async_finish,
                allocate_on_comm_stream=async_finish)
            if async_finish:
                event.current_stream_wait()
            else:
                assert event.event is None
            torch.cuda.synchronize()
            assert per_rank.dtype == torch.int32 and is_in.dtype == torch.bool
            assert torch.equal(per_rank.cpu(), want[0]) and torch.equal(per_expert.cpu(), want[2])
            assert torch.equal(is_in.cpu(), want[3])
            assert (per_rdma is None) == (want[1] is None)
            if want[1] is not None:
                assert torch.equal(per_rdma.cpu(), want[1])
        with pytest.raises(RuntimeError, match=r"Failed: Assertion error deep_ep_cpp.cpp:\d+ 'topk_idx.dim\(\) == 2'"):
            buffer.get_dispatch_layout(dev.view(-1), num_experts)
        buffer.destroy()


def test_api_argument_errors_and_masks(deep_ep):
    buffer = deep_ep.Buffer(None, low_latency_mode=True, explicitly_destroy=True, enable_shrink=True,
                            sim_num_ranks=4, sim_rank=0)
    x = torch.zeros((8, 512), dtype=torch.bfloat16, device="cuda")
    topk = torch.zeros((8, 2), dtype=torch.int64, device="cuda")
    with pytest.raises(RuntimeError, match="x.size\\(0\\) <= num_max_dispatch_tokens_per_rank"):
        buffer.low_latency_dispatch(x, topk, 4, 16)
    with pytest.raises(RuntimeError, match="num_experts % num_ranks == 0"):
        buffer.low_latency_dispatch(x, topk, 8, 18)
    with pytest.raises(RuntimeError, match="scalar_type\\(\\) == torch::kBFloat16"):
        buffer.low_latency_dispatch(x.float(), topk, 8, 16)
    with pytest.raises(RuntimeError, match="not use_ue8m0 or round_scale"):
        buffer.low_latency_dispatch(x, topk, 8, 16, use_ue8m0=True)
    # combine before any dispatch of that shape
    handle = (torch.zeros((4, 32), dtype=torch.int32, device="cuda"),
              torch.zeros((4, 4), dtype=torch.int64, device="cuda"), 8, 512, 16)
    y = torch.zeros((4, 32, 512), dtype=torch.bfloat16, device="cuda")
    w = torch.ones((8, 2), dtype=torch.float32, device="cuda")
    with pytest.raises(RuntimeError, match="ll.dispatched"):
        buffer.low_latency_combine(y, topk, w, handle)
    # masks: a local tensor in the reference fork (deep_ep/buffer.py:2805-2829)
    status = torch.zeros(4, dtype=torch.int, device="cuda")
    buffer.low_latency_update_mask_buffer(2, True)
    buffer.low_latency_query_mask_buffer(status)
    assert status.tolist() == [0, 0, 1, 0]
    buffer.low_latency_update_mask_buffer(2, False)
    buffer.low_latency_update_mask_buffer(1, True)
    buffer.low_latency_query_mask_buffer(status)
    assert status.tolist() == [0, 1, 0, 0]
    buffer.low_latency_clean_mask_buffer()
    buffer.low_latency_query_mask_buffer(status)
    assert status.tolist() == [0, 0, 0, 0]
    for moves_tokens_between_gpus in (buffer.dispatch, buffer.combine, buffer.internode_dispatch,
                                      buffer.internode_combine):
        with pytest.raises(NotImplementedError):
            moves_tokens_between_gpus(x)
    t = buffer.get_local_buffer_tensor(torch.int32, use_rdma_buffer=True)
    assert t.dtype == torch.int32 and t.is_cuda
    assert isinstance(buffer.get_comm_stream(), torch.cuda.Stream)
    buffer.destroy()
    with pytest.raises(NotImplementedError):
        class FakeGroup:
            def rank(self): return 0
            def size(self): return 2
        deep_ep.Buffer(FakeGroup())


def test_normal_mode_layout_and_pack(deep_ep):
    """4096 tokens x 7168, top-8 of 256 experts, 8 ranks: layout -> per-rank sort -> channel prefix -> pack."""
    from deepep_efa_amd import deep_ep_cpp, normal
    t, h, k, e, r = 4096, 7168, 8, 256, 8
    buffer = deep_ep.Buffer(None, explicitly_destroy=True, sim_num_ranks=r, sim_rank=0, sim_seed=3)
    x, topk_idx = buffer.loopback_synthesise(t, h, k, e)
    per_rank, _, per_expert, is_in, _ = buffer.get_dispatch_layout(topk_idx, e)
    ids, counts, cumsum, total = normal.moe_routing_sort(is_in)
    torch.cuda.synchronize()
    topk_cpu = O.synth_topk_idx(O.uniform_cdf(e), np.arange(r), t, k, 3)[0]
    assert torch.equal(topk_idx.cpu(), topk_cpu)
    w_rank, _, w_expert, w_is_in = O.get_dispatch_layout(topk_cpu, e, r)
    assert torch.equal(per_rank.cpu(), w_rank) and torch.equal(per_expert.cpu(), w_expert)
    w_ids, w_counts, w_cumsum, w_total = O.moe_routing_sort(w_is_in)
    assert total == w_total and torch.equal(ids.cpu(), w_ids) and torch.equal(counts.cpu(), w_counts)
    assert torch.equal(cumsum.cpu(), w_cumsum)
    for c in (10, 12):
        assert torch.equal(normal.channel_prefix_matrix(is_in, c).cpu(), O.channel_prefix_matrix(w_is_in, c))
    # bf16 pack
    packed, none = normal.pack_rows(x, None, ids, cumsum)
    assert none is None and packed.shape == (total, h)
    x_cpu = x.cpu()
    assert torch.equal(packed.cpu().view(torch.int16), x_cpu[w_ids].view(torch.int16))
    # fp8 + scales pack (inputs quantised by the caller, as the reference's normal mode does)
    q, s = deep_ep_cpp.per_token_cast_to_fp8(x, False, False)
    pq, psc = normal.pack_rows(q, s, ids, cumsum)
    wq, ws = O.per_token_cast_to_fp8(x_cpu)
    assert torch.equal(pq.cpu().view(torch.uint8), wq.view(torch.uint8)[w_ids])
    assert torch.equal(psc.cpu(), ws[w_ids])
    buffer.destroy()


@pytest.mark.parametrize("num_ranks,rank,t,h,k,e", [
    (16, 4, 64, 2048, 6, 64),   # one launch per direction
    (8, 3, 2200, 512, 8, 64),   # the large-batch kernels: histograms + send + index + copy, index + copy + reduce
], ids=["decode_size", "large_batch"])
def test_dispatch_and_combine_replay_in_a_hip_graph(deep_ep, num_ranks, rank, t, h, k, e):
    """Decode loops capture the dispatch + combine pair once and replay it.  The captured calls must
    allocate nothing and record no memset; every replay, with eager work and synchronisations in
    between, must give the eager result."""
    buffer = deep_ep.Buffer(None, low_latency_mode=True, explicitly_destroy=True, sim_num_ranks=num_ranks,
                            sim_rank=rank, sim_seed=21)
    x, topk_idx = buffer.loopback_synthesise(t, h, k, e)
    w = torch.softmax(torch.randn((t, k), generator=torch.Generator().manual_seed(4)), dim=-1).cuda()

    def step():
        (rx, rs), cnt, handle, _, _ = buffer.low_latency_dispatch(x, topk_idx, t, e)
        y = (rx.float().view(rx.shape[0], rx.shape[1], h // 128, 128) * rs.unsqueeze(-1)).view(rx.shape).to(torch.bfloat16)
        out, _, _ = buffer.low_latency_combine(y, topk_idx, w, handle)
        return rx, rs, cnt, handle, out

    rx, rs, cnt, handle, out = step()  # eager: also fills the per-shape caches
    torch.cuda.synchronize()
    want = [v.clone() for v in (rx.view(torch.uint8), rs, cnt, handle[0], handle[1], out)]
    live = torch.arange(rx.shape[1], device="cuda").view(1, -1) < cnt.view(-1, 1)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        grx, grs, gcnt, ghandle, gout = step()
    for replay in range(4):
        for v in (grx.view(torch.uint8), grs, gout):  # eager work between replays: scribble over the outputs
            v.fill_(0)
        gcnt.fill_(-1)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = (grx.view(torch.uint8), grs, gcnt, ghandle[0], ghandle[1], gout)
        assert torch.equal(got[2], want[2]) and torch.equal(got[4], want[4]), f"replay {replay}: counts / layout"
        assert torch.equal(got[0][live], want[0][live]), f"replay {replay}: payload"
        assert torch.equal(got[1][live], want[1][live]), f"replay {replay}: scales"
        assert torch.equal(got[3][live], want[3][live]), f"replay {replay}: src_info"
        assert torch.equal(got[5].view(torch.int16), want[5].view(torch.int16)), f"replay {replay}: combined"
    buffer.destroy()
