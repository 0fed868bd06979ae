"""Bench of the low-latency dispatch + combine hot path on one MI355X.

A step is one pass of the hot path for one rank of an EP=32 world: dispatch
(route + quantise + pack into per-expert slots, then compaction of the rows
received) and combine (return of the expert outputs, then the top-k weighted
reduce), for 128 tokens x 7168 hidden, top-8 of 256 experts, FP8 dispatch and
BF16 combine.  At this size each of the two is one kernel launch.  The 31 peer
ranks' rows are synthesised in HBM from a seed before the timed region and
stay resident.

Prints ONE JSON line.  `value` is microseconds of stream time per step over K
steps: the steps are enqueued by HIP-graph replays so the GPU never waits for
the host (launching call by call from Python costs more than the kernels take;
that figure is reported beside it).  Per-entry durations are measured the same
way; the roofline of the slower of the two step kernels is in the same line,
quoted with every launch after a flush of the caches (replayed back to back the
step's 66 MB never leave the 256 MB memory-side cache).  The sections at 4096
tokens take two or more sets of buffers in turn for the same reason: a call
must not find its bytes where the call before left them.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def algorithmic_bytes(t, h, k, p, rv, stride, e, r, own=0, packed=None):
    """Bytes each entry point must move (reads + writes), from the generated routing.
    p = live (token,k) pairs of this rank, rv = rows this rank receives, own = rows it sends to itself.
    The one-call entries handle the own rows once: quantised straight into the packed tensors on dispatch,
    read straight from the expert outputs on combine."""
    g = h // 128
    if packed is None:  # FP8 payload + float32 scales + source index
        packed = h + 4 * g + 4
    small = e * 4 + (e // r) * r * 8 + (e // r) * 4
    return {
        "dispatch_send": t * 2 * h + t * k * 8 + p * stride + t * k * 4 + e * 4,
        "dispatch_recv": rv * stride + rv * packed + small,
        "combine_send": rv * 2 * h * 2 + (e // r) * r * 8,
        "combine_recv": p * 2 * h + t * k * 16 + t * 2 * h,
        "dispatch": (t * 2 * h + t * k * 8 + (p - own) * stride + own * packed + t * k * 4 + e * 4
                     + (rv - own) * (stride + packed) + small),
        "combine": (rv - own) * 2 * h * 2 + (e // r) * r * 8 + p * 2 * h + t * k * 16 + t * 2 * h,
        # zero copy: no row is returned, the transport sends the ranges of layout_range from the expert outputs
        "combine_zero_copy": (e // r) * r * 8 + p * 2 * h + t * k * 16 + t * 2 * h,
        "exchange_metadata": r * e * 4 + rv * 16 + r * 24,
        # the staged receive's bytes plus, per row, the record, the tail read and the descriptor
        "dispatch_recv_by_source": rv * stride + rv * packed + small + rv * 12,
        "dispatch_recv_by_source_ordered": rv * stride + rv * packed + small + r * e * 4 + rv * 8,
        # the all-to-all shaped transport: one buffer per direction, contiguous per peer
        "dispatch_send_by_dest": t * 2 * h + t * k * 8 * 2 + p * stride + t * k * 4 + e * 8,
        "combine_send_by_dest": rv * 2 * h * 2 + rv * 16,
        "combine_recv_flat": p * 2 * h + t * k * 16 + e * 4 + t * 2 * h,
        # the five launches (or launch pairs) of a step over that transport: send by destination, exchange
        # metadata, ordered receive, return by destination, reduce from the flat buffer
        "all_to_all_step": (t * 2 * h + t * k * 8 * 2 + p * stride + t * k * 4 + e * 8) + (r * e * 4 + rv * 16 + r * 24)
                           + (rv * stride + rv * packed + small + r * e * 4 + rv * 8) + (rv * 2 * h * 2 + rv * 16)
                           + (p * 2 * h + t * k * 16 + e * 4 + t * 2 * h),
        "all_to_all_step_without_metadata_launch": (t * 2 * h + t * k * 8 * 2 + p * stride + t * k * 4 + e * 8)
                           + (rv * stride + rv * packed + small + r * e * 4 + rv * 8) + (rv * 2 * h * 2 + rv * 16)
                           + (p * 2 * h + t * k * 16 + e * 4 + t * 2 * h),
    }


def load_bench_probe():
    """The measuring-stick kernels (bench_probe.hip beside this file, a library of its own: nothing of it is in
    libdeepep_hip.so).  Built by __graft_entry__.build(); built here only if that has not happened."""
    import ctypes
    path = os.path.join(ROOT, "bench_probe.so")
    if not os.path.exists(path):
        import importlib.util
        spec = importlib.util.spec_from_file_location("deepep_build", os.path.join(ROOT, "deepep_efa_amd", "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build_bench_probe()
    lib = ctypes.CDLL(path)
    c = ctypes
    lib.bench_probe_row_scatter.restype = c.c_int
    lib.bench_probe_row_scatter.argtypes = [c.c_void_p, c.c_int, c.c_int, c.c_void_p, c.c_int, c.c_void_p, c.c_int64,
                                            c.c_void_p]
    lib.bench_probe_stream_copy.restype = c.c_int
    lib.bench_probe_stream_copy.argtypes = [c.c_void_p, c.c_void_p, c.c_int64, c.c_void_p]
    return lib


def time_calls(torch, fn, n):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(n):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / n


def time_calls_median(torch, fn, n=10, samples=5):
    """The large entries (tens to hundreds of microseconds a call): `samples` runs of `n` eager calls, each run
    between its own pair of events; the median run with the fastest and slowest beside it.  Independent of
    --steps."""
    runs = sorted(time_calls(torch, fn, n) for _ in range(samples))
    return runs[len(runs) // 2], [round(runs[0], 2), round(runs[-1], 2)]


def time_graph_samples(torch, fn, warmup, steps, samples=10):
    """`fn` enqueued by HIP-graph replays so that the GPU never waits for the host: the time is the stream's,
    kernels plus the gaps between them.  The graph holds a whole multiple of `steps` calls, at least 100 (what
    a replay costs by itself, a few microseconds, is then under a tenth of a microsecond per call whatever
    `steps` is: with graphs of 20 steps the 128-token step read 16.2 us, with graphs of 200 steps 15.8) and at
    most 1000; a sample is one replay between its own pair of events, and `samples` of them are taken whatever
    `steps` is.  Returns the median per call with the fastest and slowest sample beside it, so the figure does
    not depend on how many steps were asked for."""
    per_graph = min(1000, steps * max(1, -(-100 // steps)))
    replays = 1
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    with torch.cuda.graph(g):
        for _ in range(per_graph):
            fn()
    for _ in range(max(1, -(-warmup // per_graph))):
        g.replay()
    torch.cuda.synchronize()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(samples)]
    for e0, e1 in events:
        e0.record()
        for _ in range(replays):
            g.replay()
        e1.record()
    torch.cuda.synchronize()
    per_call = sorted(e0.elapsed_time(e1) * 1e3 / (replays * per_graph) for e0, e1 in events)
    del g
    return {"us": per_call[len(per_call) // 2], "min_us": per_call[0], "max_us": per_call[-1],
            "calls_per_graph": per_graph, "replays_per_sample": replays, "samples": samples}


def rotating(fns):
    """One callable that runs the given callables in turn.  Each works on its own set of buffers, so that a call
    finds none of its bytes in the 256 MB memory-side cache where the call before left them: calls on one set
    of buffers, back to back, measure that cache and not HBM unless a single call moves far more than it holds."""
    turn = [0]

    def call():
        turn[0] = (turn[0] + 1) % len(fns)
        fns[turn[0]]()
    return call


def phase_marks(torch, args):
    """Where the microseconds go inside the two step kernels: the timing build (bench_phase.hip: the library's
    sources with the DEEPEP_PHASE hook writing the 100 MHz wall clock) runs the headline step, replayed and after
    read flushes, and prints for each kind of workgroup the mean / latest time since the launch's first mark at
    which its first and its last wave pass every mark."""
    import ctypes

    import numpy as np
    from deepep_efa_amd import _capi
    path = os.path.join(ROOT, "bench_phase.so")
    if not os.path.exists(path):
        raise ImportError(f"{path} is missing: build it with `python deepep_efa_amd/build.py`")
    _capi._lib, _capi.LIB_PATH = None, path  # every C-ABI call below goes to the timing build
    lib = _capi.load()
    from deepep_efa_amd import ll_runtime, loopback
    t, h, k, e, r, rank = args.tokens, args.hidden, args.topk, args.experts, args.ranks, args.rank
    st = ll_runtime.LowLatencyState(ll_runtime.LLShape(r, rank, e, t, h, k, ll_runtime.ROW_FP8))
    world = loopback.LoopbackWorld(r, rank, seed=args.seed)
    world.synthesise(t, h, k, e)
    x, topk = world.own_inputs()
    w = torch.softmax(torch.randn((t, k), generator=torch.Generator().manual_seed(args.seed)), dim=-1).cuda()
    out = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
    y = torch.randn((e // r, r * t, h), device="cuda").to(torch.bfloat16)
    st.dispatch_send(x, topk)
    world.dispatch_from_peers(st)
    st.dispatch_recv()
    world.combine_from_peers(st, mode=1, seed=args.seed + 2)
    torch.cuda.synchronize()
    assert lib.deepep_ll_dispatch_is_single_launch(t, k, e, r, t * k) == 1, "the marks are read per workgroup of one launch"
    log = torch.zeros((16384, 16), dtype=torch.int64, device="cuda")
    lib.bench_phase_set_log.argtypes = [ctypes.c_void_p]
    assert lib.bench_phase_set_log(ctypes.c_void_p(log.data_ptr())) == 0
    flush = torch.zeros(128 << 20, dtype=torch.int32, device="cuda")

    def collect(fn, cold, reps=40):
        acc, n = None, 0
        for i in range(reps + 5):
            if cold:
                flush.max()
            else:
                fn()
            log.zero_()
            torch.cuda.synchronize()
            fn()
            torch.cuda.synchronize()
            if i < 5:
                continue
            ticks = log.cpu().numpy().astype("float64")
            us = (ticks - ticks[ticks > 0].min()) * 0.01
            us[ticks == 0] = float("nan")
            acc = us if acc is None else acc + us
            n += 1
        return acc / n

    def report(title, us, groups, names):
        print(title)
        for gname, rows in groups:
            blk = us[rows]
            if blk.size == 0 or np.isnan(blk).all():
                continue
            with np.errstate(all="ignore"):
                mean, latest = np.nanmean(blk, axis=0), np.nanmax(blk, axis=0)
            print(f"  {gname} ({blk.shape[0]} workgroups)")
            for half, label in ((0, "first wave"), (8, "last wave ")):
                cells = [f"{names[gname][i]} {mean[half + i]:.2f}/{latest[half + i]:.2f}" for i in range(8)
                         if i in names[gname] and not np.isnan(mean[half + i])]
                print(f"    {label}: " + "   ".join(cells))

    send_marks = {0: "start", 1: "indices back", 3: "ranked+quantised", 4: "addresses known", 5: "stores begin",
                  6: "stores issued"}
    recv_marks = {0: "start", 1: "segment table", 2: "row loads begin", 3: "first row stored"}
    names = {"send": send_marks, "receive": recv_marks, "metadata": {0: "start", 1: "segment table"},
             "reduce": {0: "start", 1: "rows back", 2: "summed", 3: "stored"},
             "row return": {0: "start", 1: "segment table", 2: "copies issued"}}
    stamp = build_stamp(lib)
    print(f"per-phase marks, {t} tokens x {h}, top-{k} of {e} experts, rank {rank} of {r}: mean/latest microseconds since "
          "the launch's first mark, averaged over 40 launches")
    print(f"build: abi={stamp['abi']} source={stamp['source_sha']}")
    for cold in (False, True):
        state = "every launch after 512 MiB of reads" if cold else "replayed"
        us = collect(lambda: st.dispatch(x, topk), cold)
        live = np.where(~np.isnan(us).all(axis=1))[0]
        blocks = int(live.max()) + 1
        report(f"ll_dispatch_fused_kernel, {state} ({blocks} workgroups)", us,
               [("send", slice(0, t)), ("receive", slice(t + 1, blocks - 1)), ("metadata", slice(blocks - 1, blocks))],
               names)
        us = collect(lambda: st.combine(y, topk, w, out), cold)
        live = np.where(~np.isnan(us).all(axis=1))[0]
        blocks = int(live.max()) + 1
        reduce_blocks = (t * ((2 * h + 1023) // 1024) + 3) // 4
        report(f"ll_combine_fused_kernel, {state} ({blocks} workgroups)", us,
               [("reduce", slice(0, reduce_blocks)), ("row return", slice(reduce_blocks, blocks))], names)
    lib.bench_phase_set_log(None)


def calibrate_copy(torch, _capi, lib):
    """A plain copy through the pack kernel with identity row ids: 32768 rows x 14336 B read and written once.
    Under `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` the counters of pack_rows_kernel divided into the
    known 469762048 bytes give the scale of each counter on this GPU."""
    rows, row_bytes = 32768, 14336
    src = torch.empty((rows, row_bytes), dtype=torch.uint8, device="cuda").random_(0, 255)
    dst = torch.empty_like(src)
    ids = torch.arange(rows, dtype=torch.int64, device="cuda")
    n_dev = torch.tensor([rows], dtype=torch.int64, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream

    def fn():
        _capi.check(lib.deepep_pack_rows(_capi.ptr(src), None, _capi.ptr(ids), _capi.ptr(n_dev), rows, rows, row_bytes,
                                         0, _capi.ptr(dst), None, stream))
    us = time_calls(torch, fn, 10)
    assert torch.equal(src, dst)
    print(json.dumps({"calibrate_copy": {"kernel": "pack_rows_kernel", "bytes_read": rows * row_bytes,
                                         "bytes_written": rows * row_bytes, "us": round(us, 2),
                                         "GBps": round(2 * rows * row_bytes / us / 1e3, 1)}}))


def build_stamp(lib):
    """What identifies the kernels being timed: the ABI revision the loaded library reports and a hash of the
    kernel sources in the tree.  Profile summaries under profiles/ carry the same pair."""
    import hashlib
    digest = hashlib.sha256()
    csrc = os.path.join(ROOT, "deepep_efa_amd", "csrc")
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".hpp", ".cpp")):
            with open(os.path.join(csrc, name), "rb") as f:
                digest.update(name.encode() + b"\0" + f.read())
    return {"abi": int(lib.deepep_abi_version()), "source_sha": digest.hexdigest()[:12]}


def read_traffic_summary(kernel, stamp):
    """L2 <-> fabric bytes per launch of `kernel` from the committed rocprofv3 counter summary, or None when
    there is none or it was taken on other kernel sources than the ones being timed (its `build:` line)."""
    path = os.path.join(ROOT, "profiles", "ll_dispatch_combine_ep32_128tok_fabric_traffic.txt")
    if not os.path.exists(path):
        return None
    want = f"build: abi={stamp['abi']} source={stamp['source_sha']}"
    lines = open(path).read().splitlines()
    if not any(line.strip() == want for line in lines):
        return None
    for line in lines:
        parts = line.split()
        if len(parts) >= 4 and parts[0] == kernel and parts[1].isdigit() and parts[2].isdigit():
            return int(parts[1]) + int(parts[2])
    return None


def all_to_all_entries(torch, _capi, lib, ll_runtime, st, world, x, topk, weights, y, out):
    """The same rank's step over a transport that ships one contiguous message per peer (an all-to-all):
    send by destination; receive from the per-source buffer (placing the rows from their tails through the
    exchange-metadata records, or, for messages in this build's own order, from the gathered counts alone);
    return by destination; reduce from the flat buffer.  The peers' messages are the staged rows regrouped by
    source rank (expert by expert, the order the send side emits), set up once.  Returns the callables."""
    sh = st.shape
    r, e, m, el = sh.num_ranks, sh.num_experts, sh.max_tokens, sh.num_local_experts
    a2a = ll_runtime.AllToAllState(sh)
    a2a.dispatch_send(x, topk)
    staging = st.recv_staging.view(el, r, m, st.stride)
    count = st.recv_count.view(el, r).cpu()
    for src in range(r):
        off = src * a2a.slot_rows
        for le in range(el):
            c = int(count[le, src])
            a2a.recv_by_source[off:off + c] = staging[le, src, :c]
            off += c
    tk = world.topk_idx_all.view(r, -1)
    routed = torch.stack([torch.bincount(tk[s][tk[s] >= 0], minlength=e) for s in range(r)]).to(torch.int32)
    a2a.exchange_metadata(routed)
    a2a.dispatch_recv()
    a2a.recv_flat.normal_()  # the peers' answers, one row per row sent
    torch.cuda.synchronize()
    meta = a2a.meta
    meta_args = [_capi.ptr(routed), e, r, sh.rank, a2a.slot_rows, a2a.row_capacity] + [_capi.ptr(meta[n]) for n in (
        "send_counts", "recv_counts", "totals", "combine_remote_recv_offset", "source_rank", "source_offset",
        "padded_index", "combine_send_offset", "num_recv_tokens", "tokens_per_expert")]

    def whole_step():  # everything one rank launches for a step over such a transport, in stream order
        a2a.dispatch_send(x, topk)
        _capi.check(lib.deepep_ll_exchange_metadata(*meta_args, torch.cuda.current_stream().cuda_stream))
        a2a.dispatch_recv_ordered(routed)
        a2a.combine_send(y)
        a2a.combine_recv(topk, weights, out)

    def critical_path():
        # The ordered receive does not read the exchange metadata (the return by destination does): on a
        # real transport that launch goes to a side stream while the rows are on the wire, and what is
        # left in stream order between the inputs and the combined rows are these four.
        a2a.dispatch_send(x, topk)
        a2a.dispatch_recv_ordered(routed)
        a2a.combine_send(y)
        a2a.combine_recv(topk, weights, out)

    return {
        "all_to_all_step": whole_step,
        "all_to_all_step_without_metadata_launch": critical_path,
        "dispatch_send_by_dest": lambda: a2a.dispatch_send(x, topk),
        "dispatch_recv_by_source": lambda: a2a.dispatch_recv(),
        "dispatch_recv_by_source_ordered": lambda: a2a.dispatch_recv_ordered(routed),
        "combine_send_by_dest": lambda: a2a.combine_send(y),
        "combine_recv_flat": lambda: a2a.combine_recv(topk, weights, out),
    }


def bench_pack(torch, _capi, lib, loopback, args):
    """Normal-mode layout + pack at 4096 tokens x 7168, top-8 of 256 experts, 8 ranks x 32 experts."""
    t, h, k, e, r = 4096, 7168, 8, 256, 8
    world = loopback.LoopbackWorld(r, 0, seed=args.seed)
    world.synthesise(t, h, k, e)
    x, topk = world.own_inputs()
    stream = torch.cuda.current_stream().cuda_stream
    i32 = dict(dtype=torch.int32, device="cuda")
    per_rank, per_expert = torch.empty(r, **i32), torch.empty(e, **i32)
    is_in = torch.empty((t, r), dtype=torch.bool, device="cuda")
    ws = torch.empty(max(256, lib.deepep_layout_workspace_bytes(t, r, e)), dtype=torch.uint8, device="cuda")
    ids = torch.empty(t * r, dtype=torch.int64, device="cuda")
    counts, cumsum = torch.empty(r, **i32), torch.empty(r + 1, dtype=torch.int64, device="cuda")
    ws2 = torch.empty(max(256, lib.deepep_routing_sort_workspace_bytes(t, r)), dtype=torch.uint8, device="cuda")
    cpm = torch.empty((r, 10), **i32)
    row_of_pair = torch.empty((t, r), **i32)  # the sort's inverse table: with it the combine reduce is one launch

    def layout():
        _capi.check(lib.deepep_get_dispatch_layout(_capi.ptr(topk), t, k, r, e, _capi.ptr(per_rank), None,
                                                   _capi.ptr(per_expert), _capi.ptr(is_in), _capi.ptr(ws), ws.numel(),
                                                   stream))

    def sort():
        _capi.check(lib.deepep_moe_routing_sort(_capi.ptr(is_in), t, r, _capi.ptr(ids), _capi.ptr(counts),
                                                _capi.ptr(cumsum), _capi.ptr(row_of_pair), _capi.ptr(ws2), ws2.numel(),
                                                stream))

    def prefix():
        _capi.check(lib.deepep_channel_prefix_matrix(_capi.ptr(is_in), t, r, 10, _capi.ptr(cpm), stream))

    layout(), sort(), prefix()
    torch.cuda.synchronize()
    s = int(cumsum[r])
    total_dev = cumsum[r:]
    # The HBM-bound entries rotate over several sets of buffers (see `rotating`): seven for the cast (89 MB a
    # call), two for the packs and the reduce (321 to 622 MB a call).
    sets = 7
    xs = [x] + [x.clone() for _ in range(sets - 1)]
    qs = [torch.empty((t, h), dtype=torch.uint8, device="cuda") for _ in range(sets)]
    scs = [torch.empty((t, h // 128), dtype=torch.float32, device="cuda") for _ in range(sets)]
    q, sc = qs[0], scs[0]
    for i in range(sets):
        _capi.check(lib.deepep_per_token_cast_to_fp8(_capi.ptr(xs[i]), t, h, 1, _capi.ptr(qs[i]), _capi.ptr(scs[i]),
                                                     stream))
    out16s = [torch.empty((s, h), dtype=torch.bfloat16, device="cuda") for _ in range(2)]
    out8s = [torch.empty((s, h), dtype=torch.uint8, device="cuda") for _ in range(2)]
    outss = [torch.empty((s, h // 128), dtype=torch.float32, device="cuda") for _ in range(2)]
    out16 = out16s[0]

    def pack_bf16_on(i):
        return lambda: _capi.check(lib.deepep_pack_rows(_capi.ptr(xs[i]), None, _capi.ptr(ids), _capi.ptr(total_dev), s,
                                                        t, 2 * h, 0, _capi.ptr(out16s[i]), None, stream))

    def pack_fp8_on(i):
        return lambda: _capi.check(lib.deepep_pack_rows(_capi.ptr(qs[i]), _capi.ptr(scs[i]), _capi.ptr(ids),
                                                        _capi.ptr(total_dev), s, t, h, h // 32, _capi.ptr(out8s[i]),
                                                        _capi.ptr(outss[i]), stream))

    def cast_on(i):
        return lambda: _capi.check(lib.deepep_per_token_cast_to_fp8(_capi.ptr(xs[i]), t, h, 1, _capi.ptr(qs[i]),
                                                                    _capi.ptr(scs[i]), stream))

    pack_bf16 = rotating([pack_bf16_on(i) for i in range(2)])
    pack_fp8 = rotating([pack_fp8_on(i) for i in range(2)])
    cast = rotating([cast_on(i) for i in range(sets)])

    # the steps either side of the pack: top-k remap of the send rows, source metadata of the rows
    # received (here: as many as were sent), and the per-token reduce of the rows that come back
    # (here: the packed rows themselves, i.e. every rank returns what it was sent)
    weights = torch.rand((t, k), device="cuda")
    remap_e = torch.empty((s, k), dtype=torch.int64, device="cuda")
    remap_w = torch.empty((s, k), dtype=torch.float32, device="cuda")
    meta = torch.empty((s, 8), dtype=torch.uint8, device="cuda")
    comb_xs = [torch.empty((t, h), dtype=torch.bfloat16, device="cuda") for _ in range(2)]
    comb_w = torch.empty((t, k), dtype=torch.float32, device="cuda")
    ws3 = torch.empty(max(256, lib.deepep_combine_reduce_workspace_bytes(t, r)), dtype=torch.uint8, device="cuda")
    pack_bf16(), pack_bf16()

    def remap():
        _capi.check(lib.deepep_topk_remap(_capi.ptr(topk), _capi.ptr(weights), _capi.ptr(ids), _capi.ptr(cumsum), t, k, r,
                                          e // r, s, _capi.ptr(remap_e), _capi.ptr(remap_w), stream))

    def src_meta():
        _capi.check(lib.deepep_build_recv_src_meta(_capi.ptr(cumsum), r, 8, s, _capi.ptr(meta), stream))

    remap()

    def reduce_on(i):
        return lambda: _capi.check(lib.deepep_combine_reduce(
            _capi.ptr(out16s[i]), _capi.ptr(remap_w), _capi.ptr(ids), _capi.ptr(cumsum), _capi.ptr(is_in), None, None,
            t, h, k, r, s, _capi.ptr(row_of_pair), _capi.ptr(comb_xs[i]), _capi.ptr(comb_w), None, 0, stream))

    def reduce_from_list_on(i):  # without the sort's table: the positions are rebuilt from the list first
        return lambda: _capi.check(lib.deepep_combine_reduce(
            _capi.ptr(out16s[i]), _capi.ptr(remap_w), _capi.ptr(ids), _capi.ptr(cumsum), _capi.ptr(is_in), None, None,
            t, h, k, r, s, None, _capi.ptr(comb_xs[i]), _capi.ptr(comb_w), _capi.ptr(ws3), ws3.numel(), stream))

    reduce = rotating([reduce_on(i) for i in range(2)])
    reduce_from_list = rotating([reduce_from_list_on(i) for i in range(2)])

    res = {"workload": "4096 tokens x 7168 bf16, top-8 of 256 experts, 8 ranks x 32 experts", "rows_packed": s,
           "buffers": "cast, packs and reduce rotate over 7 / 2 / 2 sets of buffers, so no call finds its bytes in "
                      "the memory-side cache"}
    for name, fn, nbytes in (("layout", layout, t * k * 8 + t * r + 4 * (r + e)),
                             ("routing_sort", sort, 2 * t * r + s * 8),
                             ("channel_prefix", prefix, t * r + r * 10 * 4),
                             ("cast_fp8", cast, t * 2 * h + t * h + t * (h // 32)),
                             ("pack_bf16", pack_bf16, s * 2 * h * 2 + s * 8),
                             ("pack_fp8", pack_fp8, s * (h + h // 32) * 2 + s * 8),
                             ("topk_remap", remap, s * 8 + s * k * 12 * 2),
                             ("recv_src_meta", src_meta, s * 8),
                             ("combine_reduce", reduce, s * 2 * h + s * k * 4 + t * r * 5 + t * 2 * h + t * k * 4),
                             ("combine_reduce_from_the_list", reduce_from_list,
                              s * 2 * h + s * k * 4 + s * 12 + t * r + t * 2 * h + t * k * 4)):
        us, spread = time_calls_median(torch, fn)
        res[name] = {"us": round(us, 2), "bytes": nbytes, "GBps": round(nbytes / us / 1e3, 1),
                     "frac_of_8TBps": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4), "us_min_max": spread}
    # The packs read every source row once per destination rank that wants it (s / t times on average).  The
    # figure above counts each of those reads; if the caches served all but the first, HBM would see only the
    # unique bytes: every source row once, every packed row once.  The counters say the L2 does not serve them
    # (it fetches the full read bytes from the fabric); whether the memory-side cache does they cannot tell.
    for name, row in (("pack_bf16", 2 * h), ("pack_fp8", h + h // 32)):
        unique = t * row + s * row + s * 8
        res[name]["unique_bytes"] = unique
        res[name]["frac_of_8TBps_on_unique_bytes"] = round(unique / res[name]["us"] / 1e3 / HBM_PEAK_GBS, 4)
    return res


def bench_ll_large(torch, _capi, lib, ll_runtime, loopback, args, skewed=False):
    """The same four LL entry points at 4096 tokens (8 ranks x 32 experts), where they are HBM-bound;
    skewed: at 8192 tokens, 64 ranks x 4 experts, Zipf(1.2) expert popularity with rank 0 holding the hottest
    experts and 1 % of the rows scaled by 100 (needs ~150 GB of HBM)."""
    t, h, k, e, r, rank = (8192, 7168, 8, 256, 64, 0) if skewed else (4096, 7168, 8, 256, 8, 3)
    shape = ll_runtime.LLShape(r, rank, e, t, h, k, ll_runtime.ROW_FP8)
    st = ll_runtime.LowLatencyState(shape)
    world = loopback.LoopbackWorld(r, rank, seed=args.seed + 7)
    if skewed:
        world.synthesise(t, h, k, e, popularity="zipf", outlier_period=100)
    else:
        world.synthesise(t, h, k, e)
    x, topk = world.own_inputs()
    weights = torch.softmax(torch.randn((t, k), generator=torch.Generator().manual_seed(1)), dim=-1).cuda()
    out = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
    epr, n_slots = e // r, r * t
    y = torch.empty((epr, n_slots, h), dtype=torch.bfloat16, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    _capi.check(lib.deepep_synth_bf16_rows(_capi.ptr(y), epr * n_slots, h, h * 2, None, 0, 5, 0, stream))
    # 4096 tokens: two sets of buffers taken in turn (see `rotating`; a send moves 302 MB, little more than the
    # memory-side cache holds).  The skewed size moves gigabytes per call and keeps one set.
    states = [st] if skewed else [st, ll_runtime.LowLatencyState(shape)]
    xs = [x] + [x.clone() for _ in states[1:]]
    for s_, x_ in zip(states, xs):
        s_.dispatch_send(x_, topk)
        world.dispatch_from_peers(s_)
        s_.dispatch_recv()
        world.combine_from_peers(s_, mode=1, seed=9)
    torch.cuda.synchronize()
    p = int((st.pair_slot[:t] >= 0).sum())
    rv = int(st.packed_recv_count.sum())
    own = int((st.packed_recv_layout_range[:, rank] & 0xFFFFFFFF).sum())
    nbytes = algorithmic_bytes(t, h, k, p, rv, st.payload_bytes, e, r, own)
    balanced_hint = st.expected_rows
    if skewed:
        # The hint a caller has: the rows the step before received (packed_recv_count is an output of every
        # dispatch; deep_ep.Buffer reads it back without blocking and sizes the next large call by it).  The
        # row copies take their grid from it; with the balanced guess T * K, twenty times too low here, they
        # walk the batch in a loop, which the *_with_balanced_hint lines show.
        for s_ in states:
            s_.expected_rows = rv

    def with_hint(fn, s_, hint):
        def call():
            keep, s_.expected_rows = s_.expected_rows, hint
            try:
                fn()
            finally:
                s_.expected_rows = keep
        return call

    def on_every_state(make):
        return rotating([make(s_, x_) for s_, x_ in zip(states, xs)])

    calls = {
        "dispatch_send": on_every_state(lambda s_, x_: lambda: s_.dispatch_send(x_, topk)),
        "dispatch_recv": on_every_state(lambda s_, x_: lambda: s_.dispatch_recv()),
        "combine_send": on_every_state(lambda s_, x_: lambda: s_.combine_send(y)),
        "combine_recv": on_every_state(lambda s_, x_: lambda: s_.combine_recv(topk, weights, out)),
        # the one-call entries (what deep_ep.Buffer launches): the rank's own rows are written / read in place
        "dispatch": on_every_state(lambda s_, x_: lambda: s_.dispatch(x_, topk)),
        "combine": on_every_state(lambda s_, x_: lambda: s_.combine(y, topk, weights, out)),
    }
    if skewed:
        calls["dispatch_recv_with_balanced_hint"] = with_hint(lambda: st.dispatch_recv(), st, balanced_hint)
        calls["combine_send_with_balanced_hint"] = with_hint(lambda: st.combine_send(y), st, balanced_hint)
        nbytes["dispatch_recv_with_balanced_hint"] = nbytes["dispatch_recv"]
        nbytes["combine_send_with_balanced_hint"] = nbytes["combine_send"]
    if not skewed:  # the same step over an all-to-all shaped transport (two sets of buffers like the others)
        per_state = [all_to_all_entries(torch, _capi, lib, ll_runtime, s_, world, x_, topk, weights, y, out)
                     for s_, x_ in zip(states, xs)]
        for name in per_state[0]:
            calls[name] = rotating([entries[name] for entries in per_state])
    res = {"workload": f"LL dispatch+combine at {t} tokens x {h}, top-{k} of {e} experts, {r} ranks x {epr} experts"
                       + (", Zipf(1.2) expert popularity, 1 % outlier rows" if skewed else ""),
           "pairs_sent": p, "rows_received": rv, "rows_to_own_experts": own, "expected_rows_hint": st.expected_rows,
           "buffers": "one set" if skewed else "two sets taken in turn, so no call finds its bytes in the memory-side cache"}
    for name, fn in calls.items():
        if skewed:  # millisecond kernels: every call between its own events, so the spread shows
            samples = sorted(time_calls(torch, fn, 1) for _ in range(6))
            us = samples[len(samples) // 2]
            spread = [round(samples[0], 2), round(samples[-1], 2)]
        else:
            us, spread = time_calls_median(torch, fn)
        res[name] = {"us": round(us, 2), "bytes": nbytes[name], "GBps": round(nbytes[name] / us / 1e3, 1),
                     "frac_of_8TBps": round(nbytes[name] / us / 1e3 / HBM_PEAK_GBS, 4), "us_min_max": spread}
    if not skewed:  # what the same send measures when every call goes to the same buffers
        us, _ = time_calls_median(torch, lambda: st.dispatch_send(x, topk))
        res["dispatch_send"]["us_on_one_set_of_buffers"] = round(us, 2)
    # The send's memory traffic without the send: a bare kernel that reads every token row and stores one
    # byte per element to the rows the send writes (remote experts' slots; the rows for this rank's own
    # experts go to the same buffer at the expert's slots too).  What it reaches is what this access
    # pattern gets from HBM on this GPU.
    slot = st.pair_slot[:t].long()
    dst_rows = torch.where(slot >= 0, topk.clamp(min=0) * st.shape.max_tokens + slot, torch.full_like(slot, -1))
    dst_rows = dst_rows.to(torch.int32).contiguous()
    probe_lib = load_bench_probe()

    def probe_on(s_, x_):
        def call():
            rc = probe_lib.bench_probe_row_scatter(_capi.ptr(x_), t, h, _capi.ptr(dst_rows), k, _capi.ptr(s_.send_slots),
                                                   s_.stride, stream)
            assert rc == 0, rc
        return call

    probe = on_every_state(probe_on)
    if skewed:
        samples = sorted(time_calls(torch, probe, 1) for _ in range(6))
        us = samples[len(samples) // 2]
    else:
        us, _ = time_calls_median(torch, probe)
    probe_bytes = t * 2 * h + p * h
    res["bare_row_scatter"] = {"us": round(us, 2), "bytes": probe_bytes, "GBps": round(probe_bytes / us / 1e3, 1),
                               "frac_of_8TBps": round(probe_bytes / us / 1e3 / HBM_PEAK_GBS, 4),
                               "what": "reads the token rows and stores hidden bytes to each row the send writes: "
                                       "the send's traffic pattern without routing, quantisation or scales"}
    res["dispatch_send"]["us_per_byte_against_bare_row_scatter"] = round(
        (res["dispatch_send"]["us"] / nbytes["dispatch_send"]) / (us / probe_bytes), 3)
    # For scale beside the row copies: one contiguous streaming copy of as many bytes as the receive copy reads
    # (and writes), 16 bytes per thread, nothing to look up.
    half = (nbytes["dispatch_recv"] // 2) // 4096 * 4096
    pairs = [(torch.empty(half, dtype=torch.uint8, device="cuda"), torch.empty(half, dtype=torch.uint8, device="cuda"))
             for _ in range(1 if skewed else 2)]

    def copy_on(a, b):
        def call():
            assert probe_lib.bench_probe_stream_copy(_capi.ptr(a), _capi.ptr(b), half, stream) == 0
        return call

    plain = rotating([copy_on(a, b) for a, b in pairs])
    if skewed:
        samples = sorted(time_calls(torch, plain, 1) for _ in range(6))
        us = samples[len(samples) // 2]
    else:
        us, _ = time_calls_median(torch, plain)
    res["plain_stream_copy"] = {"us": round(us, 2), "bytes": 2 * half, "GBps": round(2 * half / us / 1e3, 1),
                                "frac_of_8TBps": round(2 * half / us / 1e3 / HBM_PEAK_GBS, 4),
                                "what": "one contiguous copy of the bytes the receive copy moves"}
    del pairs
    return res


def bench_api_step(torch, args):
    """The same step through deep_ep.Buffer (what a MoE layer calls): low_latency_dispatch + low_latency_combine
    for rank 5 of the EP=32 world, launched call by call from Python and as a captured HIP graph.  The peers'
    rows and their answers are staged once and stay resident, as in the C-ABI step above."""
    import deep_ep
    t, h, k, e, r, rank = args.tokens, args.hidden, args.topk, args.experts, args.ranks, args.rank
    buffer = deep_ep.Buffer(None, low_latency_mode=True, explicitly_destroy=True, sim_num_ranks=r, sim_rank=rank,
                            sim_seed=args.seed)
    x, topk_idx = buffer.loopback_synthesise(t, h, k, e)
    x, topk_idx = x.clone(), topk_idx.clone()
    weights = torch.softmax(torch.randn((t, k), generator=torch.Generator().manual_seed(args.seed)), dim=-1).cuda()
    buffer.loopback_set_combine_mode(1, args.seed + 2)
    (rx, rs), count, handle, _, _ = buffer.low_latency_dispatch(x, topk_idx, t, e)
    y = torch.zeros((e // r, r * t, h), dtype=torch.bfloat16, device="cuda")
    buffer.low_latency_combine(y, topk_idx, weights, handle)
    torch.cuda.synchronize()
    buffer.loopback_clear_world()  # the exchange is done: later calls run this rank's own kernels only

    def step(zero_copy=False):
        _, _, hd, _, _ = buffer.low_latency_dispatch(x, topk_idx, t, e)
        buffer.low_latency_combine(y, topk_idx, weights, hd, zero_copy=zero_copy)

    # zero_copy: the expert outputs are written into the buffer of get_next_low_latency_combine_buffer
    # and sent from there, so the combine returns no rows (deep_ep/buffer.py:2831-2852)
    buffer.get_next_low_latency_combine_buffer(handle)
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    wall0 = time.perf_counter()
    ev0.record()
    for _ in range(args.steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    res = {"eager_us": round(ev0.elapsed_time(ev1) * 1e3 / args.steps, 2),
           "eager_host_wall_us": round((time.perf_counter() - wall0) * 1e6 / args.steps, 2), "graph_us": None}
    if not args.no_graph:
        try:
            res["graph_us"] = round(time_graph_samples(torch, step, args.warmup, args.steps)["us"], 2)
            res["graph_zero_copy_us"] = round(
                time_graph_samples(torch, lambda: step(zero_copy=True), args.warmup, args.steps)["us"], 2)
        except Exception as exc:
            res["graph_us"] = None
            res["graph_error"] = type(exc).__name__
    buffer.destroy()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--tokens", type=int, default=128)
    ap.add_argument("--hidden", type=int, default=7168)
    ap.add_argument("--topk", type=int, default=8)
    ap.add_argument("--experts", type=int, default=256)
    ap.add_argument("--ranks", type=int, default=32)
    ap.add_argument("--rank", type=int, default=5)
    ap.add_argument("--seed", type=int, default=2024)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-pack", action="store_true", help="skip the normal-mode layout + pack section")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a plain row copy of known size (for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-profiler", action="store_true",
                    help="skip the per-launch GPU timestamps taken with torch.profiler (for runs under rocprofv3)")
    ap.add_argument("--row-format", choices=["fp8", "bf16", "fp8_pow2", "fp8_ue8m0"], default="fp8",
                    help="dispatch payload (the headline workload is fp8); other formats skip the CPU baseline")
    ap.add_argument("--cold-trace", type=int, default=0, metavar="N",
                    help="only run N eager dispatch / combine pairs, each call after a 512 MiB flush of the caches "
                         "(writes, or reads with --cold-by-reads), for a rocprofv3 kernel trace")
    ap.add_argument("--cold-by-reads", action="store_true")
    ap.add_argument("--no-skew-stress", action="store_true", help="skip the skewed 8192-token stress section")
    ap.add_argument("--only-ll-4096", action="store_true",
                    help="only time the LL entry points at 4096 tokens (8 ranks x 32 experts) and print that section")
    ap.add_argument("--phase-marks", action="store_true",
                    help="only print the in-kernel phase timestamps of the two step kernels (timing build "
                         "bench_phase.so)")
    ap.add_argument("--skew-stress", action="store_true",
                    help="only time the LL entry points at the skewed 8192-token, 64-rank stress size and print that")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU's share of the expert-parallel world; --gpus must be 1 "
              "(the peers are synthesised in HBM, nothing runs on a second GPU)", file=sys.stderr)
        sys.exit(2)

    import torch
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    torch.cuda.set_device(0)
    if args.phase_marks:
        phase_marks(torch, args)
        return
    from deepep_efa_amd import _capi, ll_runtime, loopback

    lib = _capi.load()
    if args.calibrate_copy:
        calibrate_copy(torch, _capi, lib)
        return
    if args.skew_stress:
        print(json.dumps(bench_ll_large(torch, _capi, lib, ll_runtime, loopback, args, skewed=True)))
        return
    if args.only_ll_4096:
        print(json.dumps(bench_ll_large(torch, _capi, lib, ll_runtime, loopback, args)))
        return
    t, h, k, e, r, rank = args.tokens, args.hidden, args.topk, args.experts, args.ranks, args.rank
    fmt = {"fp8": ll_runtime.ROW_FP8, "bf16": ll_runtime.ROW_BF16, "fp8_pow2": ll_runtime.ROW_FP8_POW2,
           "fp8_ue8m0": ll_runtime.ROW_FP8_UE8M0}[args.row_format]
    if fmt != ll_runtime.ROW_FP8:
        args.no_cpu_baseline = True
    shape = ll_runtime.LLShape(r, rank, e, t, h, k, fmt)
    st = ll_runtime.LowLatencyState(shape)
    world = loopback.LoopbackWorld(r, rank, seed=args.seed)
    world.synthesise(t, h, k, e)
    x, topk = world.own_inputs()
    weights = torch.softmax(torch.randn((t, k), generator=torch.Generator().manual_seed(args.seed)), dim=-1).cuda()
    out = torch.empty((t, h), dtype=torch.bfloat16, device="cuda")
    epr, n_slots = e // r, r * t
    y = torch.empty((epr, n_slots, h), dtype=torch.bfloat16, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    _capi.check(lib.deepep_synth_bf16_rows(_capi.ptr(y), epr * n_slots, h, h * 2, None, 0, args.seed + 1, 0, stream))

    # the exchange, done once: peers' dispatch rows and their combine answers stay resident
    st.dispatch_send(x, topk)
    world.dispatch_from_peers(st)
    st.dispatch_recv()
    world.combine_from_peers(st, mode=1, seed=args.seed + 2)
    torch.cuda.synchronize()
    p = int((st.pair_slot[:t] >= 0).sum())
    rv = int(st.packed_recv_count.sum())
    own = int((st.packed_recv_layout_range[:, rank] & 0xFFFFFFFF).sum())

    # the gathered route counts of the whole world, as a count all-gather would leave them
    tk = world.topk_idx_all.view(r, -1)
    routed = torch.stack([torch.bincount(tk[s][tk[s] >= 0], minlength=e) for s in range(r)]).to(torch.int32)
    meta_out = ll_runtime.exchange_metadata(routed, rank, t, r * t)  # buffers made once, reused below
    meta_args = [_capi.ptr(routed), e, r, rank, t, r * t] + [_capi.ptr(meta_out[n]) for n in (
        "send_counts", "recv_counts", "totals", "combine_remote_recv_offset", "source_rank", "source_offset",
        "padded_index", "combine_send_offset", "num_recv_tokens", "tokens_per_expert")]

    if args.cold_trace > 0:
        flush = torch.zeros(128 << 20, dtype=torch.int32, device="cuda")
        for i in range(args.cold_trace):
            for call in (lambda: st.dispatch(x, topk), lambda: st.combine(y, topk, weights, out)):
                if args.cold_by_reads:
                    flush.max()
                else:
                    flush.fill_(i)
                call()
            torch.cuda.synchronize()
        print(json.dumps({"cold_trace": args.cold_trace, "flush": "reads" if args.cold_by_reads else "writes"}))
        return

    calls = {
        "exchange_metadata": lambda: _capi.check(lib.deepep_ll_exchange_metadata(
            *meta_args, torch.cuda.current_stream().cuda_stream)),
        "dispatch": lambda: st.dispatch(x, topk),  # send + receive phase, one launch at this size
        "combine": lambda: st.combine(y, topk, weights, out),  # row return + reduce, one launch at this size
        "combine_zero_copy": lambda: st.combine(y, topk, weights, out, zero_copy=True),  # the reduce alone
        "dispatch_send": lambda: st.dispatch_send(x, topk),
        "dispatch_recv": lambda: st.dispatch_recv(),
        "combine_send": lambda: st.combine_send(y),
        "combine_recv": lambda: st.combine_recv(topk, weights, out),
    }
    # the same step over an all-to-all shaped transport: one contiguous message per peer in each direction
    calls.update(all_to_all_entries(torch, _capi, lib, ll_runtime, st, world, x, topk, weights, y, out))
    step_calls = ("dispatch", "combine")  # what deep_ep.Buffer.low_latency_dispatch / _combine launch
    phase_calls = ("dispatch_send", "dispatch_recv", "combine_send", "combine_recv")

    def step():
        for name in step_calls:
            calls[name]()

    def step_by_phase():
        for name in phase_calls:
            calls[name]()

    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def time_eager(fn, warmup, reps):
        """`reps` calls launched one by one from Python: includes the host's launch cost when that
        is longer than the kernels (it is, at this size: ~9 us per call through ctypes)."""
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        wall0 = time.perf_counter()
        ev0.record()
        for _ in range(reps):
            fn()
        ev1.record()
        torch.cuda.synchronize()
        return ev0.elapsed_time(ev1) * 1e3 / reps, (time.perf_counter() - wall0) * 1e6 / reps

    flush = torch.zeros(128 << 20, dtype=torch.int32, device="cuda")

    def time_cold(fn, reps=40, by_reads=False):
        """One call at a time, each after 512 MiB of other traffic has pushed the step's data out of
        the 256 MB last-level cache; the call is a one-step HIP graph (so that its launches are queued
        while the flush still runs) between its own pair of events.  Median over `reps`.
        The flush writes the 512 MiB (what the reference's bench does before each timed call: the
        caches are then full of lines that must be written back first) or, `by_reads`, reads them
        (the caches are left full of clean lines, as after a GEMM over expert weights)."""
        launch = fn
        if not args.no_graph:
            try:
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    fn()
                launch = g.replay
            except Exception:
                launch = fn
        samples = []
        for i in range(reps + 3):
            if by_reads:
                flush.max()
            else:
                flush.fill_(i)
            ev0.record()
            launch()
            ev1.record()
            torch.cuda.synchronize()
            if i >= 3:
                samples.append(ev0.elapsed_time(ev1) * 1e3)
        samples.sort()
        return samples[len(samples) // 2]

    def kernel_time_after_flush(fn, by_reads, reps=30):
        """Average duration of the library's kernels in one call of `fn`, every call after a 512 MiB flush
        (reads or writes), from the GPU's own start/end timestamps of each launch as torch.profiler collects them
        — the clock rocprofv3's kernel trace reads.  HIP events cannot isolate a 10 us kernel that has to follow
        a flush: a pair of them around one launch costs ~7 us by itself (the *_two_trivial_launches_us lines).
        None when the profiler is unavailable."""
        if args.no_profiler:
            return None
        try:
            from torch.profiler import ProfilerActivity, profile
            for i in range(3):
                flush.max() if by_reads else flush.fill_(i)
                fn()
            torch.cuda.synchronize()
            with profile(activities=[ProfilerActivity.CUDA]) as prof:
                for i in range(reps):
                    flush.max() if by_reads else flush.fill_(i)
                    fn()
                    torch.cuda.synchronize()
            total = 0.0
            for ev in prof.events():
                if ev.device_type == torch.autograd.DeviceType.CUDA and "deepep" in ev.name:
                    total += ev.device_time if hasattr(ev, "device_time") else ev.cuda_time
            return total / reps if total > 0 else None
        except Exception:
            return None

    eager_us, host_wall_us = time_eager(step, args.warmup, args.steps)
    eager_phase_us, _ = time_eager(step_by_phase, 10, args.steps)
    graph_us = graph_phase_us = step_samples = None
    per_call, per_call_spread = {}, {}
    timing = "eager launches"
    if not args.no_graph:
        try:
            step_samples = time_graph_samples(torch, step, args.warmup, args.steps)
            graph_us = step_samples["us"]
            graph_phase_us = time_graph_samples(torch, step_by_phase, 10, args.steps)["us"]
            for name, fn in calls.items():
                got = time_graph_samples(torch, fn, 10, args.steps)
                per_call[name] = got["us"]
                per_call_spread[name] = [round(got["min_us"], 2), round(got["max_us"], 2)]
            timing = (f"HIP graphs of {step_samples['calls_per_graph']} steps each; median of "
                      f"{step_samples['samples']} samples of {step_samples['replays_per_sample']} back-to-back "
                      "replays, whatever --steps is")
        except Exception as exc:  # fall back to eager timing, and say so
            graph_us = None
            timing = f"eager launches (graph capture unavailable: {type(exc).__name__})"
    if graph_us is None:
        # the same call `steps` times back to back between two events
        for name, fn in calls.items():
            per_call[name], _ = time_eager(fn, 10, args.steps)
    cold_us = time_cold(step)
    tiny = torch.zeros(64, dtype=torch.int32, device="cuda")
    cold_floor_us = time_cold(lambda: (tiny.add_(1), tiny.add_(1)))  # two trivial launches, timed the same way
    cold_reads_us = time_cold(step, by_reads=True)
    cold_reads_floor_us = time_cold(lambda: (tiny.add_(1), tiny.add_(1)), by_reads=True)
    # the two step kernels alone, each launch after a flush: where their bytes really come from HBM
    cold_kernel_us = {name: {"read_flush": kernel_time_after_flush(calls[name], True),
                             "write_flush": kernel_time_after_flush(calls[name], False)} for name in step_calls}
    us_per_step = graph_us if graph_us is not None else eager_us
    us_per_phase_step = graph_phase_us if graph_phase_us is not None else eager_phase_us

    nbytes = algorithmic_bytes(t, h, k, p, rv, st.payload_bytes, e, r, own, packed=st.data_bytes + st.scale_bytes + 4)
    kernels = {n: {"us": round(per_call[n], 2), "bytes": nbytes[n],
                   "GBps": round(nbytes[n] / per_call[n] / 1e3, 1)} for n in calls}
    for n, spread in per_call_spread.items():
        kernels[n]["us_min_max"] = spread
    dom = max(step_calls, key=per_call.get)
    stamp = build_stamp(lib)
    warm = nbytes[dom] / per_call[dom] / 1e3
    # Back-to-back replays leave the step's ~66 MB in the 256 MB memory-side cache, so that rate is not an HBM
    # rate.  The headline roofline is therefore the same kernel with every launch after 512 MiB of reads (the
    # state a GEMM over expert weights leaves): its bytes then come from HBM.
    cold_dom = cold_kernel_us[dom]["read_flush"]
    if cold_dom is not None:
        roofline = {"bound": "hbm", "kernel": dom, "achieved": round(nbytes[dom] / cold_dom / 1e3, 1),
                    "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(nbytes[dom] / cold_dom / 1e3 / HBM_PEAK_GBS, 4),
                    "traffic": None, "duration_us": round(cold_dom, 2),
                    "state": "every launch after 512 MiB of reads have flushed the caches: the bytes come from HBM",
                    "timer": "GPU start/end timestamps of each launch (torch.profiler), 30 launches"}
    else:  # no profiler: the cache-resident figure, named for what it is
        roofline = {"bound": "hbm", "kernel": dom, "achieved": round(warm, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(warm / HBM_PEAK_GBS, 4), "traffic": None, "duration_us": round(per_call[dom], 2),
                    "state": "back-to-back replays, data resident in the 256 MB memory-side cache: not an HBM rate",
                    "timer": "HIP events over graph replays"}
    roofline_cache_resident = {
        "bound": "memory-side cache (256 MB), not HBM", "kernel": dom, "achieved": round(warm, 1),
        "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(warm / HBM_PEAK_GBS, 4),
        "duration_us": round(per_call[dom], 2), "timer": "HIP events over graph replays, launches back to back"}
    result = {
        "metric": "us per LL dispatch+combine (128 tok,7168,top-8); pack/combine HBM GB/s",
        "value": round(us_per_step, 2),
        "value_min_max": ([round(step_samples["min_us"], 2), round(step_samples["max_us"], 2)]
                          if step_samples is not None else None),
        "unit": "us",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(us_per_step / 1e3, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ("fp8_e4m3 dispatch (f32 scale math)" if fmt != ll_runtime.ROW_BF16 else "bf16 dispatch") +
                 ", bf16 combine (f32 accumulate)",
        "data": "synthetic",
        "config": {"workload": "LL dispatch+combine, one GPU's share of EP=32: 128 tokens x 7168, top-8 of 256 "
                               "experts, 8 local experts; 31 peers synthesised in HBM from a seed",
                   "tokens": t, "hidden": h, "topk": k, "experts": e, "ranks": r, "rank": rank,
                   "pairs_sent": p, "rows_received": rv, "rows_to_own_experts": own,
                   "launches_per_step": 2},
        "kernel_time_us": round(sum(per_call[n] for n in step_calls), 2),
        "step_by_phase_us": round(us_per_phase_step, 2),  # the same step as four launches
        "timing": timing,
        "eager_us_per_step": round(eager_us, 2),  # launched call by call from Python: host-bound
        "eager_host_wall_us_per_step": round(host_wall_us, 2),
        "cold_cache_us_per_step": round(cold_us, 2),  # every step after a 512 MiB flush of the last-level cache
        "cold_cache_two_trivial_launches_us": round(cold_floor_us, 2),  # what that way of timing costs by itself
        "cold_cache_read_flush_us_per_step": round(cold_reads_us, 2),  # the same after 512 MiB of reads
        "cold_cache_read_flush_two_trivial_launches_us": round(cold_reads_floor_us, 2),
        "kernels": kernels,
        # the reference's own bandwidth accounting (tests/test_low_latency.py:236-242): bytes per valid
        # selection H + H/128*4 + 16 for the FP8 dispatch and 2H for the combine, over the call's time
        "reference_formula_GBps": {
            "dispatch": round(p * (h + h // 128 * 4 + 16) / per_call["dispatch"] / 1e3, 1),
            "combine": round(p * 2 * h / per_call["combine"] / 1e3, 1)},
        "roofline": roofline,
        "roofline_cache_resident": roofline_cache_resident,
        "cold_kernel_us": {n: {k: (round(v, 2) if v is not None else None) for k, v in d.items()}
                           for n, d in cold_kernel_us.items()},
        "build": stamp,
    }

    traffic = read_traffic_summary(dom, stamp)
    if traffic is not None and (t, h, k, e, r) == (128, 7168, 8, 256, 32):
        result["roofline"]["traffic"] = traffic
    cpu_inputs = None
    if not args.no_cpu_baseline:  # host copies for the CPU leg, taken before the device buffers are released
        cpu_inputs = (x.cpu(), topk.cpu(), weights.cpu(), st.recv_staging.view(epr, r, t, st.stride).cpu(),
                      st.recv_count.view(epr, r).cpu())
    del st, y
    torch.cuda.empty_cache()
    if fmt == ll_runtime.ROW_FP8:
        result["api_step_us"] = bench_api_step(torch, args)
        torch.cuda.empty_cache()
    if not args.no_pack:
        result["normal_mode_pack"] = bench_pack(torch, _capi, lib, loopback, args)
        result["ll_4096_tokens"] = bench_ll_large(torch, _capi, lib, ll_runtime, loopback, args)
        torch.cuda.empty_cache()
        free, _ = torch.cuda.mem_get_info()
        if args.no_skew_stress:
            pass
        elif free >= 170 * 2 ** 30:
            result["skew_stress"] = bench_ll_large(torch, _capi, lib, ll_runtime, loopback, args, skewed=True)
            torch.cuda.empty_cache()
        else:
            result["skew_stress"] = {"skipped": f"needs ~150 GB of free HBM, {free >> 30} GiB are free"}

    if not args.no_cpu_baseline:
        from oracle import cpu_baseline
        torch.cuda.synchronize()
        cpu = cpu_baseline.CpuRankStep(*cpu_inputs, e, r, rank, t)
        med, threads, runs = cpu_baseline.time_cpu_step(cpu, budget_s=12.0)
        result["cpu_baseline"] = {"value": round(med * 1e6, 1), "unit": "us", "cores": threads, "kind": "port",
                                  "host_cpu_count": os.cpu_count(),
                                  "sample": f"the same rank-{rank} dispatch+combine step in torch on the host, "
                                            f"median of {runs} runs on {threads} threads"}
        # the reference's own CPU-runnable case: layout counts + FP8 cast + weighted combine sum at EP=16
        med, threads, runs = cpu_baseline.time_reference_case(budget_s=5.0)
        result["cpu_baseline_ep16_case"] = {
            "value": round(med * 1e6, 1), "unit": "us", "cores": threads, "kind": "port",
            "host_cpu_count": os.cpu_count(),
            "sample": "128 tokens x 7168, top-8 of 256 experts, simulated EP=16: get_dispatch_layout counts + "
                      f"per-128-channel FP8 cast + weighted top-k combine sum in torch, median of {runs} runs on "
                      f"{threads} threads"}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
