"""Bench of the low-latency dispatch + combine hot path on one MI355X.

A step is one pass of the hot path for one rank of an EP=32 world:
dispatch_send (route + quantise + pack) -> dispatch_recv -> combine_send ->
combine_recv, for 128 tokens x 7168 hidden, top-8 of 256 experts, FP8
dispatch and BF16 combine.  The 31 peer ranks' rows are synthesised in HBM
from a seed before the timed region and stay resident.

Prints ONE JSON line.  `value` is microseconds per dispatch+combine measured
over K back-to-back steps on one stream (launch gaps included); the
per-kernel durations, measured with events around each entry point, and the
roofline of the slowest kernel are in the same line.
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


def algorithmic_bytes(t, h, k, p, rv, stride, e, r):
    """Bytes each kernel must move (reads + writes), from the generated routing.
    p = live (token,k) pairs of this rank, rv = rows this rank receives."""
    g = h // 128
    return {
        "dispatch_send": t * 2 * h + t * k * 8 + p * stride + t * k * 4 + e * 4,
        "dispatch_recv": rv * stride + rv * (h + 4 * g + 4) + e * 4 + (e // r) * r * 8 + (e // r) * 4,
        "combine_send": rv * 2 * h * 2 + (e // r) * r * 8,
        "combine_recv": p * 2 * h + t * k * 16 + t * 2 * h,
    }


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
    ap.add_argument("--no-graph", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU's share of the expert-parallel world; --gpus must be 1 "
              "(the peers are synthesised in HBM, nothing runs on a second GPU)", file=sys.stderr)
        sys.exit(2)

    import torch
    from deepep_efa_amd import _capi, ll_runtime, loopback

    lib = _capi.load()
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    torch.cuda.set_device(0)
    t, h, k, e, r, rank = args.tokens, args.hidden, args.topk, args.experts, args.ranks, args.rank
    shape = ll_runtime.LLShape(r, rank, e, t, h, k, ll_runtime.ROW_FP8)
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

    calls = {
        "dispatch_send": lambda: st.dispatch_send(x, topk),
        "dispatch_recv": lambda: st.dispatch_recv(),
        "combine_send": lambda: st.combine_send(y),
        "combine_recv": lambda: st.combine_recv(topk, weights, out),
    }

    def step():
        for fn in calls.values():
            fn()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    wall0 = time.perf_counter()
    ev0.record()
    for _ in range(args.steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - wall0
    us_per_step = ev0.elapsed_time(ev1) * 1e3 / args.steps

    # per entry point: the same call `steps` times back to back between two events.  Consecutive
    # launches on one stream leave well under a microsecond between kernels on this GPU, so the
    # mean is the kernel's duration (the rocprofv3 summary under profiles/ is the cross-check).
    per_call = {}
    for name, fn in calls.items():
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        ev0.record()
        for _ in range(args.steps):
            fn()
        ev1.record()
        torch.cuda.synchronize()
        per_call[name] = ev0.elapsed_time(ev1) * 1e3 / args.steps

    graph_us = None
    if not args.no_graph:
        try:
            g = torch.cuda.CUDAGraph()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                step()
            torch.cuda.current_stream().wait_stream(side)
            with torch.cuda.graph(g):
                step()
            for _ in range(10):
                g.replay()
            torch.cuda.synchronize()
            ev0.record()
            for _ in range(args.steps):
                g.replay()
            ev1.record()
            torch.cuda.synchronize()
            graph_us = ev0.elapsed_time(ev1) * 1e3 / args.steps
        except Exception as exc:  # graph capture is an extra, never the headline
            graph_us = f"unavailable: {type(exc).__name__}"

    nbytes = algorithmic_bytes(t, h, k, p, rv, st.stride, e, r)
    kernels = {n: {"us": round(per_call[n], 2), "bytes": nbytes[n],
                   "GBps": round(nbytes[n] / per_call[n] / 1e3, 1)} for n in calls}
    dom = max(per_call, key=per_call.get)
    achieved = nbytes[dom] / per_call[dom] / 1e3
    result = {
        "metric": "us per LL dispatch+combine (128 tok,7168,top-8); pack/combine HBM GB/s",
        "value": round(us_per_step, 2),
        "unit": "us",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(us_per_step / 1e3, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3 dispatch (f32 scale math), bf16 combine (f32 accumulate)",
        "data": "synthetic",
        "config": {"workload": "LL dispatch+combine, one GPU's share of EP=32: 128 tokens x 7168, top-8 of 256 "
                               "experts, 8 local experts; 31 peers synthesised in HBM from a seed",
                   "tokens": t, "hidden": h, "topk": k, "experts": e, "ranks": r, "rank": rank,
                   "pairs_sent": p, "rows_received": rv},
        "kernel_time_us": round(sum(per_call.values()), 2),
        "graph_replay_us": graph_us if not isinstance(graph_us, float) else round(graph_us, 2),
        "host_wall_us_per_step": round(wall * 1e6 / args.steps, 2),
        "kernels": kernels,
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None},
    }

    if not args.no_cpu_baseline:
        from oracle import cpu_baseline
        torch.cuda.synchronize()
        staged = st.recv_staging.view(epr, r, t, st.stride).cpu()
        cpu = cpu_baseline.CpuRankStep(x.cpu(), topk.cpu(), weights.cpu(), staged, st.recv_count.view(epr, r).cpu(),
                                       e, r, rank, t)
        med, threads, runs = cpu_baseline.time_cpu_step(cpu, budget_s=15.0)
        result["cpu_baseline"] = {"value": round(med * 1e6, 1), "unit": "us", "cores": threads, "kind": "port",
                                  "sample": f"the same rank-{rank} dispatch+combine step in torch on the host, "
                                            f"median of {runs} runs"}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
