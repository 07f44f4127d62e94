#!/usr/bin/env python3
"""Benchmark of the MoE token-routing hot path on one MI355X.

One step = one pass of the hot path over one batch of synthetic tokens: dispatch (layout + fused
BF16->FP8 e4m3 cast + scatter into the rank-major receive buffer) followed by combine (gather +
fp32 reduce + BF16 store) at T=8192, H=7168, top-8 of 256 experts, 8 logical ranks, uniform-random
routing.  Inputs are resident in HBM before the timed region; outputs are pre-sized for the worst
case so no host synchronisation sits inside a step.  Calls go straight through the C ABI.

Prints one JSON line: whole-step achieved HBM GB/s (algorithmic bytes / time), per-op us/call,
a roofline object for the dominant kernel (combine), one for the dispatch call, and a CPU baseline (the
torch-CPU oracle timed on the same workload, all tokens, a few passes).  The default run adds two blocks that take a
few seconds more: `other_workloads` (C4, the expanded layout and the BF16 payload at the headline shape, C2 and the
low-latency C5: us per dispatch / combine, algorithmic bytes, fraction of peak) and `us_per_api_call` (what a caller of
`deep_ep.ElasticBuffer.dispatch` / `.combine` and of `deep_ep.Buffer.low_latency_dispatch` / `low_latency_combine` pays
per call through the Python wrapper and the compiled extension, outputs allocated inside the call, by the host clock;
the low-latency step also as a replayed HIP graph).  --brief leaves them out; --workload C5 prints the headline objects
for the low-latency pair of kernels; --overlap times dispatch and combine under a GPU-filling compute stream.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "deepep-ascend_amd"))
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0

# HBM bytes per launch measured with rocprofv3 (--pmc FETCH_SIZE and --pmc WRITE_SIZE in separate runs, KiB per
# dispatch, each scaled by what the same counter reads for a plain copy kernel of known size: x2.000 for
# FETCH_SIZE, x1.000 for WRITE_SIZE on this machine).  Keyed by (workload, layout, payload, operation); "dispatch" is
# the whole call (one kernel where the single launch applies, layout kernel + move kernel otherwise).
MEASURED_TRAFFIC_BYTES = {
    # profiles/bench_C3_hbm_counters.md
    ("C3", "compact", "fp8", "dispatch"): 459281822,
    ("C3", "compact", "fp8", "combine"): 751991366,
    ("C3", "expanded", "fp8", "dispatch"): 1862368 + 613156339,
    ("C3", "expanded", "fp8", "combine"): 1074426190,
    ("C3", "compact", "bf16", "dispatch"): 1844575 + 755717968,
    ("C3", "compact", "bf16", "combine"): 751994813,
    # profiles/bench_C4_C2_hbm_counters.md
    ("C4", "compact", "fp8", "dispatch"): 425752286,
    ("C4", "compact", "fp8", "combine"): 690500110,
    ("C2", "compact", "bf16", "dispatch"): 97414801,
    ("C2", "compact", "bf16", "combine"): 96362205,
    # profiles/bench_C5_low_latency_hbm_counters.md
    ("C5", "packed", "fp8", "ll_dispatch"): 23993245,
    ("C5", "packed", "fp8", "ll_combine"): 30425179,
}


def algorithmic_bytes(T, H, K, E, R, N_r, N_e, fp8=True, expanded=False):
    """Bytes a perfect implementation must move (each payload byte read once, written once)."""
    s_in = T * H * 2
    b_row = H * (1 if fp8 else 2) + ((H // 128) * 4 if fp8 else 0)
    meta = K * 8 + K * 4 + (K + 2) * 4
    layout = T * K * 8 + T * R + (R + E) * 4
    if expanded:
        dispatch = s_in + T * K * 12 + N_e * (b_row + 4) + N_r * (K + 2) * 4
    else:
        dispatch = s_in + T * K * 12 + N_r * (b_row + meta)
    n_in = N_e if expanded else N_r
    combine = n_in * H * 2 + T * K * 8 + T * H * 2
    return {"layout": layout, "dispatch": dispatch, "combine": combine}


class RoutingCalls:
    """Buffers (worst-case sized, allocated once) and argument blocks of a dispatch + combine pair on one workload,
    launched straight through the C ABI."""

    def __init__(self, torch, _abi, dev, case, fp8, expanded, launches=0):
        self.torch, self._abi = torch, _abi
        T, H, K, E, R, M = case.T, case.H, case.K, case.E, case.R, case.M
        self.T, self.H, self.K, self.E, self.R, self.M = T, H, K, E, R, M
        self.x, idx, w = case.x.to(dev), case.topk_idx.to(dev), case.topk_weights.to(dev)
        x = self.x
        # realised routing statistics (for the algorithmic bytes)
        valid = case.topk_idx >= 0
        self.N_e = N_e = int(valid.sum())
        dst = torch.where(valid, case.topk_idx // (E // R), torch.full_like(case.topk_idx, -1))
        self.N_r = N_r = int(sum(int((dst == r).any(dim=1).sum()) for r in range(R)))
        self.ab = algorithmic_bytes(T, H, K, E, R, N_r, N_e, fp8=fp8, expanded=expanded)

        i32 = dict(dtype=torch.int32, device=dev)
        cap = M * R
        ecap = M * min(K, E)
        rows = ecap if expanded else cap
        ws_bytes = _abi.lib.deep_ep_hip_workspace_bytes(T, K, E, R)
        self.workspace = workspace = torch.zeros(ws_bytes, dtype=torch.uint8, device=dev)
        psum_rank, psum_expert, unaligned = torch.empty(R, **i32), torch.empty(E, **i32), torch.empty(E, **i32)
        slot = torch.empty((T, K), **i32)
        meta = torch.empty((cap, K + 2), **i32)
        recv_x = torch.empty((rows, H), dtype=torch.float8_e4m3fn if fp8 else torch.bfloat16, device=dev)
        recv_sf = torch.empty((rows, H // 128), dtype=torch.float32, device=dev) if fp8 else None
        recv_idx = torch.empty((cap, K), dtype=torch.int64, device=dev) if not expanded else None
        recv_w = torch.empty((rows,) if expanded else (cap, K), dtype=torch.float32, device=dev)
        y = torch.randn((rows, H), dtype=torch.float32, device=dev).to(torch.bfloat16)   # "expert outputs"
        out = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
        out_w = torch.empty((T, K), dtype=torch.float32, device=dev)
        self.keep = (idx, w, psum_rank, psum_expert, unaligned, slot, meta, recv_x, recv_sf, recv_idx, recv_w, y, out, out_w)

        d = self.d = _abi.DispatchArgs()
        d.payload = _abi.PAYLOAD_CAST_FP8 if fp8 else _abi.PAYLOAD_BF16
        d.do_expand = int(expanded)
        d.num_tokens, d.hidden, d.num_topk, d.num_experts, d.num_ranks = T, H, K, E, R
        d.rank_idx, d.num_max_tokens_per_rank, d.expert_alignment = 0, M, 1
        d.x, d.topk_idx, d.topk_weights = x.data_ptr(), idx.data_ptr(), w.data_ptr()
        d.num_sf_packs = H // 128 if fp8 else 0
        d.psum_num_recv_tokens_per_rank = psum_rank.data_ptr()
        d.psum_num_recv_tokens_per_expert = psum_expert.data_ptr()
        d.num_unaligned_recv_tokens_per_expert = unaligned.data_ptr()
        d.dst_buffer_slot_idx, d.recv_src_metadata = slot.data_ptr(), meta.data_ptr()
        d.recv_x = recv_x.data_ptr()
        d.recv_sf = recv_sf.data_ptr() if fp8 else 0
        d.recv_sf_token_stride, d.recv_sf_hidden_stride = (H // 128, 1) if fp8 else (0, 0)
        d.recv_topk_idx = recv_idx.data_ptr() if recv_idx is not None else 0
        d.recv_topk_weights = recv_w.data_ptr()
        d.recv_capacity, d.expanded_capacity = cap, (ecap if expanded else 0)
        d.workspace, d.workspace_bytes = workspace.data_ptr(), ws_bytes
        d.tuning = _abi.Tuning.from_env()
        d.tuning.dispatch_launches = launches

        c = self.c = _abi.CombineArgs()
        c.tuning = _abi.Tuning.from_env()
        c.do_expand, c.allow_multiple_reduction = int(expanded), 1
        c.num_tokens, c.hidden, c.num_topk, c.num_experts, c.num_ranks = T, H, K, E, R
        c.rank_idx, c.num_max_tokens_per_rank = 0, M
        c.x, c.num_x_rows = y.data_ptr(), rows
        c.topk_weights = recv_w.data_ptr()
        c.topk_idx, c.dst_buffer_slot_idx = idx.data_ptr(), slot.data_ptr()
        c.recv_src_metadata, c.num_recv_rows = meta.data_ptr(), cap
        c.psum_num_recv_tokens_per_rank = psum_rank.data_ptr()
        c.combined_x, c.combined_topk_weights = out.data_ptr(), out_w.data_ptr()
        c.workspace, c.workspace_bytes = workspace.data_ptr(), ws_bytes

        self.stream = torch.cuda.current_stream()
        self.sp = self.stream.cuda_stream

    def on_stream(self, stream):
        """Launch on `stream` from now on (it must be ordered behind everything launched so far)."""
        self.stream, self.sp = stream, stream.cuda_stream

    def dispatch(self, phases=None):
        self.d.phases = (self._abi.PHASE_LAYOUT | self._abi.PHASE_MOVE) if phases is None else phases
        self._abi.check(self._abi.lib.deep_ep_hip_launch_dispatch(ctypes.byref(self.d), self.sp), "dispatch")

    def combine(self):
        self._abi.check(self._abi.lib.deep_ep_hip_launch_combine(ctypes.byref(self.c), self.sp), "combine")

    def step(self):
        self.dispatch()
        self.combine()

    def launches(self):
        self.d.phases = self._abi.PHASE_LAYOUT | self._abi.PHASE_MOVE
        return self._abi.lib.deep_ep_hip_dispatch_kernel_launches(ctypes.byref(self.d))

    def status(self):
        return int(self.workspace[:4].view(self.torch.int32).item())

    def loop_us(self, fn, iters):
        """Average duration in us of fn over iters back-to-back launches, by HIP events on the launch stream."""
        torch = self.torch
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(self.stream)
        for _ in range(iters):
            fn()
        e1.record(self.stream)
        e1.synchronize()
        return e0.elapsed_time(e1) * 1e3 / iters


def _quantiles(samples):
    samples = sorted(samples)
    pick = lambda q: samples[min(len(samples) - 1, int(q * len(samples)))]
    return {"min": round(samples[0], 2), "p50": round(pick(0.5), 2), "p95": round(pick(0.95), 2)}


def host_timed(torch, fn, calls=60, warm=5):
    """What a caller pays per call, by the host clock.  `waited`: each call between two device synchronisations (host
    work of the call + launch + kernels + the wait for the result); `issue`: the same calls back to back, the time until
    the call returns to the caller (device work only shows if the queue fills up)."""
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    waited, issue = [], []
    for _ in range(calls):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        t1 = time.perf_counter()
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        waited.append((t2 - t0) * 1e6)
        issue.append((t1 - t0) * 1e6)
    return {"waited_us": _quantiles(waited), "issue_us": _quantiles(issue)}


def routing_api_figures(torch, dev, case, kernel_us):
    """us per call of `deep_ep.ElasticBuffer.dispatch` / `.combine` (Python wrapper -> compiled extension -> C ABI, outputs
    allocated inside the call) at the headline shape, against the kernel time of the same operation."""
    import deep_ep
    T, H, K, E, R, M = case.T, case.H, case.K, case.E, case.R, case.M
    x, idx, w = case.x.to(dev), case.topk_idx.to(dev), case.topk_weights.to(dev)
    buf = deep_ep.ElasticBuffer(deep_ep.LogicalGroup(0, R), num_max_tokens_per_rank=M, hidden=H, num_topk=K)
    out = {"binding": deep_ep._binding.name, "calls": 60}
    no_sync = lambda: buf.dispatch(x, idx, w, num_experts=E, do_cpu_sync=False, cast_to_fp8=True)
    out["dispatch_no_cpu_sync"] = host_timed(torch, no_sync)
    out["dispatch_cpu_sync"] = host_timed(torch, lambda: buf.dispatch(x, idx, w, num_experts=E, cast_to_fp8=True))
    (recv_x, recv_sf), recv_idx, recv_w, handle, _ = no_sync()
    y = torch.randn((recv_x.shape[0], H), dtype=torch.float32, device=dev).to(torch.bfloat16)
    out["combine"] = host_timed(torch, lambda: buf.combine(y, handle, topk_weights=recv_w))
    buf.check_device_status()
    d_us, c_us = kernel_us
    out["kernel_us"] = {"dispatch": round(d_us, 2), "combine": round(c_us, 2)}
    out["host_overhead_us"] = {"dispatch_no_cpu_sync": round(out["dispatch_no_cpu_sync"]["waited_us"]["p50"] - d_us, 2),
                               "dispatch_cpu_sync": round(out["dispatch_cpu_sync"]["waited_us"]["p50"] - d_us, 2),
                               "combine": round(out["combine"]["waited_us"]["p50"] - c_us, 2)}
    return out


def low_latency_api_figures(torch, ll, kernel_us):
    """us per call of `deep_ep.Buffer.low_latency_dispatch` / `low_latency_combine` at the C5 shape, eager and as a
    replayed HIP graph of one dispatch + combine step, against the kernel time."""
    import deep_ep
    x, idx, w = ll.inputs
    buf = deep_ep.Buffer(deep_ep.LogicalGroup(0, ll.R), low_latency_mode=True)
    out = {"binding": deep_ep._binding.name, "calls": 60}
    dispatch = lambda: buf.low_latency_dispatch(x, idx, ll.M, ll.E, use_fp8=True)
    out["low_latency_dispatch"] = host_timed(torch, dispatch)
    recv, count, handle, _, _ = dispatch()
    combine = lambda: buf.low_latency_combine(ll.y, idx, w, handle)
    out["low_latency_combine"] = host_timed(torch, combine)

    def step():
        recv, count, handle, _, _ = dispatch()
        return buf.low_latency_combine(ll.y, idx, w, handle)

    out["step_eager"] = host_timed(torch, step)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        for _ in range(3):
            step()                                   # the buffer's workspaces exist and were last used on this stream
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            captured = step()
    torch.cuda.current_stream().wait_stream(side)
    out["step_graph_replay"] = host_timed(torch, graph.replay)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    stream = torch.cuda.current_stream()
    e0.record(stream)
    for _ in range(30):
        graph.replay()
    e1.record(stream)
    e1.synchronize()
    out["step_graph_replay"]["device_us_back_to_back"] = round(e0.elapsed_time(e1) * 1e3 / 30, 2)
    d_us, c_us = kernel_us
    out["kernel_us"] = {"low_latency_dispatch": round(d_us, 2), "low_latency_combine": round(c_us, 2), "step": round(d_us + c_us, 2)}
    out["host_overhead_us"] = {"low_latency_dispatch": round(out["low_latency_dispatch"]["waited_us"]["p50"] - d_us, 2),
                               "low_latency_combine": round(out["low_latency_combine"]["waited_us"]["p50"] - c_us, 2),
                               "step_eager": round(out["step_eager"]["waited_us"]["p50"] - d_us - c_us, 2),
                               "step_graph_replay": round(out["step_graph_replay"]["waited_us"]["p50"] - d_us - c_us, 2)}
    del captured
    return out


def other_workloads(torch, rc, _abi, dev, c3_case, iters=12):
    """The other benchmark configurations in brief: us per dispatch / combine in a hot loop (HIP events on the launch
    stream, straight through the C ABI), their algorithmic bytes and the fraction of the 8 TB/s peak."""
    out = {}
    specs = (("C4", rc.c4, True, False), ("C3_expanded", lambda: c3_case, True, True), ("C3_bf16", lambda: c3_case, False, False),
             ("C2", rc.c2, False, False))
    for name, make, fp8, expanded in specs:
        case = make()
        rt = RoutingCalls(torch, _abi, dev, case, fp8, expanded)
        for _ in range(3):
            rt.step()
        torch.cuda.synchronize()
        d_us, c_us = rt.loop_us(rt.dispatch, iters), rt.loop_us(rt.combine, iters)
        d_bytes, c_bytes = rt.ab["layout"] + rt.ab["dispatch"], rt.ab["combine"]
        out[name] = {"workload": f"{case.name}: T={rt.T} H={rt.H} E={rt.E} R={rt.R} K={rt.K}, "
                                 f"{'FP8 (fused cast)' if fp8 else 'BF16'} dispatch, {'expanded' if expanded else 'compact'} layout, "
                                 f"N_r={rt.N_r}, N_e={rt.N_e}",
                     "dispatch_us": round(d_us, 2), "combine_us": round(c_us, 2), "dispatch_kernel_launches": rt.launches(),
                     "dispatch_bytes": d_bytes, "combine_bytes": c_bytes,
                     "dispatch_frac": round(d_bytes / d_us * 1e-3 / HBM_PEAK_GBS, 4),
                     "combine_frac": round(c_bytes / c_us * 1e-3 / HBM_PEAK_GBS, 4), "device_status": rt.status()}
        del rt
        torch.cuda.empty_cache()
    ll = LowLatencyCalls(torch, rc, _abi, dev)
    for _ in range(5):
        ll.step()
    torch.cuda.synchronize()
    d_us, c_us = ll.loop_us(ll.dispatch, 30), ll.loop_us(ll.combine, 30)
    out["C5"] = {"workload": f"C5 low latency: R={ll.R} T={ll.T} H={ll.H} E={ll.E} K={ll.K} M={ll.M}, rows on rank 0: {ll.n_e}",
                 "dispatch_us": round(d_us, 2), "combine_us": round(c_us, 2), "dispatch_bytes": ll.dispatch_bytes,
                 "combine_bytes": ll.combine_bytes, "dispatch_frac": round(ll.dispatch_bytes / d_us * 1e-3 / HBM_PEAK_GBS, 4),
                 "combine_frac": round(ll.combine_bytes / c_us * 1e-3 / HBM_PEAK_GBS, 4)}
    api = low_latency_api_figures(torch, ll, kernel_us=(d_us, c_us))
    del ll
    torch.cuda.empty_cache()
    return out, api


def under_compute_load(torch, dev, rt, iters=20):
    """us per dispatch / combine on a communication stream of their own while a chain of 8192^3 BF16 matrix products
    keeps the GPU busy on another stream (what overlapping the routing with a neighbouring micro-batch's GEMMs looks
    like), and the same without the load."""
    comm, load = torch.cuda.Stream(), torch.cuda.Stream()
    a = torch.randn((8192, 8192), device=dev, dtype=torch.bfloat16)
    c = torch.empty_like(a)
    torch.cuda.synchronize()
    rt.on_stream(comm)
    out = {}
    for name, fn in (("dispatch", rt.dispatch), ("combine", rt.combine)):
        fn()
        torch.cuda.synchronize()
        quiet = rt.loop_us(fn, iters)
        done = torch.cuda.Event()
        with torch.cuda.stream(load):
            for _ in range(40):
                torch.mm(a, a, out=c)
            done.record(load)
        time.sleep(0.002)                                  # the products are running
        busy = rt.loop_us(fn, iters)
        out[name] = {"alone_us": round(quiet, 2), "under_load_us": round(busy, 2), "load_outlasted_the_measurement": not done.query()}
        torch.cuda.synchronize()
    out["device_status"] = rt.status()
    rt.on_stream(torch.cuda.current_stream())
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="C3", choices=["C2", "C3", "C4", "C5"])
    ap.add_argument("--ll-batch-sweep", action="store_true",
                    help="with --workload C5: also time the low-latency kernels at 64 to 512 tokens per rank")
    ap.add_argument("--expanded", action="store_true", help="expert-major (expanded) receive layout")
    ap.add_argument("--bf16", action="store_true", help="BF16 dispatch instead of the fused FP8 cast")
    ap.add_argument("--launches", type=int, default=0, choices=[0, 1, 2],
                    help="dispatch: 0 library's choice (single launch), 1 single launch even where it does not pay, 2 layout kernel + move kernel")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample-tokens", type=int, default=0, help="tokens the CPU baseline runs over (0: all of the workload)")
    ap.add_argument("--routing", default="case", choices=["case", "sequential"],
                    help="sequential: every token goes to ranks 0..4 (dest rows of consecutive tokens are adjacent)")
    ap.add_argument("--stream-yardsticks", action="store_true",
                    help="also time plain torch kernels with the same read/write mixes (context for the roofline fractions)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run a plain 1 GiB read + 1 GiB write elementwise kernel (scale for rocprof byte counters)")
    ap.add_argument("--fresh-input", action="store_true",
                    help="per-kernel timings: rewrite x with a copy kernel right before every (untimed) call, as a producer would")
    ap.add_argument("--l2-flush", action="store_true", help="zero a 256 MB buffer between per-kernel timings")
    ap.add_argument("--overlap", action="store_true",
                    help="also time dispatch and combine on a stream of their own while matrix products fill the GPU on another")
    ap.add_argument("--persistent-movers", type=int, default=0,
                    help="dispatch move phase as a persistent kernel with a work queue and this many mover wavefronts per compute unit: 4, 8 or 15 (implies two launches)")
    ap.add_argument("--wave-spans", action="store_true",
                    help="fused-cast compact dispatch only: load the measurement build of the library (mover wavefronts record "
                         "their start and end) and report the span of a launch's wavefronts beside its launch-to-launch time")
    ap.add_argument("--brief", action="store_true", help="only the headline workload: no other workloads, no API-level figures")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (logical ranks share its HBM); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    if args.wave_spans:
        stamps_lib = os.path.join(ROOT, "deepep-ascend_amd", "deep_ep", "libdeep_ep_hip_stamps.so")
        if not os.path.exists(stamps_lib) or args.bf16 or args.expanded or args.workload == "C5" or args.persistent_movers:
            print("bench.py: --wave-spans needs libdeep_ep_hip_stamps.so (python deepep-ascend_amd/build.py) and the fused-cast "
                  "compact dispatch", file=sys.stderr)
            sys.exit(2)
        os.environ["DEEP_EP_HIP_LIBRARY"] = stamps_lib
        args.brief = True                 # the API-level figures go through the compiled extension, which holds the product library

    import torch
    import routing_cases as rc
    from deep_ep import _abi

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.workload == "C5":
        print(json.dumps(bench_low_latency(args, torch, rc, _abi, dev)))
        return
    case = {"C2": rc.c2, "C3": rc.c3, "C4": rc.c4}[args.workload]()
    if args.routing == "sequential":
        E_l = case.E // case.R
        base = torch.tensor([0, E_l, 2 * E_l, 3 * E_l, 4 * E_l, 1, E_l + 1, 2 * E_l + 1][:case.K], dtype=torch.int64)
        case.topk_idx = base.unsqueeze(0).repeat(case.T, 1).contiguous()
    fp8 = not args.bf16
    expanded = args.expanded
    rt = RoutingCalls(torch, _abi, dev, case, fp8, expanded, args.launches)
    rt.d.tuning.persistent_movers = args.persistent_movers
    T, H, K, E, R, M = rt.T, rt.H, rt.K, rt.E, rt.R, rt.M
    N_r, N_e, ab, x, workspace, stream = rt.N_r, rt.N_e, rt.ab, rt.x, rt.workspace, rt.stream
    dispatch, combine, step = rt.dispatch, rt.combine, rt.step

    flush_buf = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev) if args.l2_flush else None
    x_master = x.clone() if args.fresh_input else None

    def timed(fn, iters, flush=False):
        """Average duration in us of fn over iters launches, by HIP events on the launch stream."""
        if flush or args.fresh_input:
            total = 0.0
            for _ in range(iters):
                if flush:
                    flush_buf.zero_()
                if args.fresh_input:
                    x.copy_(x_master)          # a producer kernel has just written the input (untimed)
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream); fn(); e1.record(stream)
                e1.synchronize()
                total += e0.elapsed_time(e1)
            return total * 1e3 / iters
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(iters):
            fn()
        e1.record(stream)
        e1.synchronize()
        return e0.elapsed_time(e1) * 1e3 / iters

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    status = int(workspace[:4].view(torch.int32).item())
    if status != 0:
        print(f"bench.py: device status {status} after warm-up (bad routing input or overflow)", file=sys.stderr)
        sys.exit(1)

    # ---- the timed region: exactly `steps` steps ----
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    step_us = timed(step, args.steps)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3

    # ---- per-kernel durations (same launches, one kind at a time) ----
    k = max(args.steps, 10)
    for phases in (_abi.PHASE_LAYOUT, _abi.PHASE_MOVE):     # kernels the steps above may not have launched yet
        dispatch(phases)
    torch.cuda.synchronize()
    layout_us = timed(lambda: dispatch(_abi.PHASE_LAYOUT), k, args.l2_flush)
    move_us = timed(lambda: dispatch(_abi.PHASE_MOVE), k, args.l2_flush)
    dispatch_us = timed(lambda: dispatch(_abi.PHASE_LAYOUT | _abi.PHASE_MOVE), k, args.l2_flush)
    combine_us = timed(combine, k, args.l2_flush)

    def distribution(fn, iters, flush, before=None):
        """min / p50 / p95 / mean in us over single launches, each bracketed by its own pair of HIP events (the
        events add a few us to every sample).  flush: a 256 MB buffer is zeroed before each launch.  before: run
        (untimed) ahead of every launch."""
        buf = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev) if flush else None
        samples = []
        for _ in range(iters):
            if flush:
                buf.zero_()
            if before is not None:
                before()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream); fn(); e1.record(stream)
            e1.synchronize()
            samples.append(e0.elapsed_time(e1) * 1e3)
        samples.sort()
        pick = lambda q: samples[min(len(samples) - 1, int(q * len(samples)))]
        return {"min": round(samples[0], 2), "p50": round(pick(0.5), 2), "p95": round(pick(0.95), 2),
                "mean": round(sum(samples) / len(samples), 2)}

    full_dispatch = lambda: dispatch(_abi.PHASE_LAYOUT | _abi.PHASE_MOVE)
    dist = {"dispatch": distribution(full_dispatch, k, False), "combine": distribution(combine, k, False),
            "dispatch_after_cache_flush": distribution(full_dispatch, k, True),
            "combine_after_cache_flush": distribution(combine, k, True)}
    # The input as a producing layer leaves it: just written by another kernel, hence in the memory-side cache.
    x_source = x.clone()
    dist["dispatch_after_input_written"] = distribution(full_dispatch, k, False, before=lambda: x.copy_(x_source))
    del x_source
    # ... and written in place (what a normalisation leaves behind: no second tensor competes for the cache)
    dist["dispatch_after_input_rewritten_in_place"] = distribution(full_dispatch, k, False, before=lambda: x.mul_(1.0))

    def gbs(nbytes, us):
        return nbytes / us * 1e-3

    step_bytes = ab["layout"] + ab["dispatch"] + ab["combine"]
    traffic_key = (case.name, "expanded" if expanded else "compact", "fp8" if fp8 else "bf16")
    if args.routing != "case":
        traffic_key = ("other",) * 3
    result = {
        "metric": "dispatch+combine achieved HBM GB/s (algorithmic bytes / step time), 8192x7168 top-8 of 256, 8 logical ranks",
        "value": round(gbs(step_bytes, step_us), 1),
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_us * 1e-3, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3 dispatch (bf16 in) / bf16 combine (fp32 accumulate)" if fp8 else "bf16",
        "data": "synthetic",
        "config": {"workload": f"{case.name}: T={T} H={H} E={E} R={R} K={K} "
                               f"{'expanded' if expanded else 'compact'} layout, N_r={N_r}, N_e={N_e}",
                   "l2_flush": bool(args.l2_flush), "fresh_input": bool(args.fresh_input),
                   "dispatch_launches": args.launches, "persistent_movers": args.persistent_movers},
        "us_per_single_launch": dist,
        "us_per_call": {"dispatch": round(dispatch_us, 2), "dispatch_layout": round(layout_us, 2),
                        "dispatch_move": round(move_us, 2), "combine": round(combine_us, 2)},
        "achieved_gbs": {"dispatch": round(gbs(ab["layout"] + ab["dispatch"], dispatch_us), 1),
                         "dispatch_move": round(gbs(ab["dispatch"], move_us), 1),
                         "combine": round(gbs(ab["combine"], combine_us), 1)},
        "frac_of_peak": {"dispatch": round(gbs(ab["layout"] + ab["dispatch"], dispatch_us) / HBM_PEAK_GBS, 4),
                         "combine": round(gbs(ab["combine"], combine_us) / HBM_PEAK_GBS, 4)},
        "algorithmic_bytes": ab,
        "roofline": {"kernel": "combine_kernel", "bound": "hbm",
                     "achieved": round(gbs(ab["combine"], combine_us), 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs(ab["combine"], combine_us) / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES.get(traffic_key + ("combine",))},
        "roofline_dispatch": {"kernel": ("dispatch_cast" if fp8 else "dispatch_copy") + "_single_launch_kernel (whole call; where the "
                                        "single launch does not apply: layout_kernel + " + ("dispatch_cast_kernel)" if fp8 else "dispatch_copy_kernel)"),
                              "bound": "hbm", "achieved": round(gbs(ab["layout"] + ab["dispatch"], dispatch_us), 1),
                              "peak": HBM_PEAK_GBS, "unit": "GB/s",
                              "frac": round(gbs(ab["layout"] + ab["dispatch"], dispatch_us) / HBM_PEAK_GBS, 4),
                              "traffic": MEASURED_TRAFFIC_BYTES.get(traffic_key + ("dispatch",))},
        "wall_ms_timed_region": round(wall_ms, 3),
    }

    if args.calibration_copy:
        calibration_copy(torch, dev)

    if args.stream_yardsticks:
        result["stream_yardsticks_gbs"] = stream_yardsticks(torch, dev)

    if args.overlap:
        result["under_compute_load"] = under_compute_load(torch, dev, rt)

    if args.wave_spans:
        result["wave_spans_us"] = wave_spans(torch, _abi, rt, timed, k)

    headline = (args.workload == "C3" and fp8 and not expanded and args.routing == "case" and not args.l2_flush and
                not args.fresh_input and args.persistent_movers == 0)
    if headline and not args.brief:
        result["us_per_api_call"] = {"C3": routing_api_figures(torch, dev, case, kernel_us=(dispatch_us, combine_us))}
        torch.cuda.empty_cache()
        result["other_workloads"], result["us_per_api_call"]["C5"] = other_workloads(torch, rc, _abi, dev, case)

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(case, args.cpu_sample_tokens, fp8, expanded)
    print(json.dumps(result))


def wave_spans(torch, _abi, rt, timed, iters):
    """With the measurement build of the library: for the whole dispatch (one launch) and for its move phase on a finished
    layout, the launch-to-launch time of a hot loop, and for the loop's last launch the time from the start of its first
    mover wavefront to the moment the last one had issued its stores / had them acknowledged (100 MHz wall clock).  The
    stamps cost every wavefront a wait for its own stores, so the launches are a little longer than the library's."""
    import numpy as np
    pairs = rt.d.tuning.cast_pairs if rt.d.tuning.cast_pairs in (1, 2) else (1 if rt.H <= 1024 else 2)
    waves = rt.T * ((rt.H + pairs * 1024 - 1) // (pairs * 1024))
    out = {"wavefronts": waves}
    for name, phases in (("dispatch", _abi.PHASE_LAYOUT | _abi.PHASE_MOVE), ("dispatch_move", _abi.PHASE_MOVE)):
        for _ in range(10):                              # the loop below starts from the state its own launches leave behind
            rt.dispatch(phases)
        period = timed(lambda: rt.dispatch(phases), iters)
        torch.cuda.synchronize()
        raw = (ctypes.c_longlong * (3 * waves))()
        if _abi.lib.deep_ep_hip_debug_wave_stamps(raw, waves) != 0:
            raise RuntimeError("reading the wavefront stamps failed")
        a = np.frombuffer(raw, dtype=np.int64).reshape(waves, 3)
        first = a[:, 0].min()
        out[name] = {"launch_to_launch": round(period, 2),
                     "first_start_to_last_store_issued": round(float(a[:, 1].max() - first) / 100.0, 2),
                     "first_start_to_last_store_acknowledged": round(float(a[:, 2].max() - first) / 100.0, 2),
                     "first_wavefront_done": round(float(a[:, 2].min() - first) / 100.0, 2),
                     "wavefronts_done_after_10_us": int((a[:, 2] - first <= 1000).sum()),
                     "last_wavefront_start": round(float(a[:, 0].max() - first) / 100.0, 2),
                     "median_wavefront_lifetime": round(float(np.median(a[:, 2] - a[:, 0])) / 100.0, 2)}
    return out


def calibration_copy(torch, dev):
    """A plain elementwise kernel of known size (reads 2^30 bytes, writes 2^30 bytes): what a byte counter reads for
    it fixes the counter's scale."""
    a = torch.ones(256 * 1024 * 1024, dtype=torch.float32, device=dev)
    b = torch.empty_like(a)
    for _ in range(3):
        torch.mul(a, 1.0, out=b)
    torch.cuda.synchronize()


def stream_yardsticks(torch, dev, iters=10):
    """What plain library kernels reach on this GPU for the traffic mixes of the routing kernels (GB/s of HBM
    bytes moved): a fill (write only), an elementwise kernel (1 read : 1 write), a 1 : 3 broadcast (the dispatch
    mix: every source row written to several destinations) and a 3 : 1 elementwise kernel (towards the combine mix)."""
    n = 256 * 1024 * 1024                                  # fp32 elements: 1 GiB per tensor, beyond the 256 MB last-level cache
    a = torch.ones(n, dtype=torch.float32, device=dev)
    a2 = torch.ones(n, dtype=torch.float32, device=dev)
    a3 = torch.ones(n, dtype=torch.float32, device=dev)
    b = torch.empty(n, dtype=torch.float32, device=dev)
    b3 = torch.empty((3, n), dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream()

    def timed(fn):
        for _ in range(2):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(iters):
            fn()
        e1.record(stream)
        e1.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / iters

    nbytes = n * 4
    out = {
        "write_only_fill": round(nbytes / timed(lambda: b.fill_(1.0)) * 1e-9, 1),
        "elementwise_1r_1w": round(2 * nbytes / timed(lambda: torch.mul(a, 1.0, out=b)) * 1e-9, 1),
        "broadcast_1r_3w": round(4 * nbytes / timed(lambda: torch.mul(a.unsqueeze(0).expand(3, n), 1.0, out=b3)) * 1e-9, 1),
        "elementwise_3r_1w": round(4 * nbytes / timed(lambda: torch.addcmul(a, a2, a3, out=b)) * 1e-9, 1),
    }
    return out


class LowLatencyCalls:
    """C5: low-latency decode.  Destination rank 0 of 8 receives from all 8 logical source ranks (128 tokens each,
    hidden 7168, top-8 of 256): FP8 dispatch into [32, 1024, 7168] packed buffers, weighted BF16 combine back.
    Buffers allocated once, launches straight through the C ABI."""
    R, T, H, E, K, M = 8, 128, 7168, 256, 8, 128

    def __init__(self, torch, rc, _abi, dev, tokens_per_rank=None, two_kernels=False):
        self.torch, self._abi = torch, _abi
        if tokens_per_rank is not None:
            self.T = self.M = tokens_per_rank
        R, T, H, E, K, M = self.R, self.T, self.H, self.E, self.K, self.M
        E_l, rows = E // R, R * M
        self.cpu_inputs = x_cpu, idx_cpu, w_cpu = rc.c5_sources(seed=0, R=R, T=T, H=H, E=E, K=K)
        x, idx, w = x_cpu.to(dev), idx_cpu.to(dev), w_cpu.to(dev)
        self.inputs = (x, idx, w)
        self.n_e = n_e = int(((idx_cpu >= 0) & (idx_cpu < E_l)).sum())            # (token, lane) pairs that land on rank 0
        px = torch.empty((E_l, rows, H), dtype=torch.float8_e4m3fn, device=dev)
        ps = torch.empty((E_l, H // 128, rows), dtype=torch.float32, device=dev)
        cnt = torch.empty(E_l, dtype=torch.int32, device=dev)
        info = torch.empty((E_l, rows), dtype=torch.int32, device=dev)
        rng = torch.zeros((E_l, R), dtype=torch.int64, device=dev)
        lane_rows = torch.empty((R * T, K), dtype=torch.int32, device=dev)    # what Buffer keeps beside the handle
        self.y = y = torch.randn((E_l, rows, H), dtype=torch.float32, device=dev).to(torch.bfloat16)
        out = torch.empty((R, T, H), dtype=torch.bfloat16, device=dev)
        ws = torch.zeros(max(_abi.lib.deep_ep_hip_ll_workspace_bytes(R, T, K, E_l), 4096), dtype=torch.uint8, device=dev)
        self.keep = (px, ps, cnt, info, rng, lane_rows, out, ws)
        d = self.d = _abi.LLDispatchArgs()
        d.use_fp8, d.num_src_ranks, d.src_rank_begin, d.src_token_stride = 1, R, 0, T
        d.hidden, d.num_topk, d.num_experts, d.expert_begin, d.num_local_experts = H, K, E, 0, E_l
        d.num_ranks, d.num_max_dispatch_tokens_per_rank = R, M
        d.x, d.topk_idx = x.data_ptr(), idx.data_ptr()
        d.packed_recv_x, d.packed_recv_x_scales, d.packed_recv_count = px.data_ptr(), ps.data_ptr(), cnt.data_ptr()
        d.packed_recv_src_info, d.packed_recv_layout_range = info.data_ptr(), rng.data_ptr()
        d.lane_rows = lane_rows.data_ptr()
        d.workspace, d.workspace_bytes = ws.data_ptr(), ws.numel()
        d.tuning = _abi.Tuning.from_env()
        if two_kernels:
            d.tuning.ll_two_kernels = 1
        c = self.c = _abi.LLCombineArgs()
        c.num_src_ranks, c.src_rank_begin, c.src_token_stride = R, 0, T
        c.hidden, c.num_topk, c.num_experts, c.expert_begin, c.num_local_experts, c.num_ranks = H, K, E, 0, E_l, R
        c.num_max_dispatch_tokens_per_rank = M
        c.x, c.topk_idx, c.topk_weights = y.data_ptr(), idx.data_ptr(), w.data_ptr()
        c.packed_recv_src_info, c.packed_recv_layout_range, c.combined_x = info.data_ptr(), rng.data_ptr(), out.data_ptr()
        c.lane_rows = 0 if os.environ.get("BENCH_LL_SEARCH") else lane_rows.data_ptr()
        c.workspace, c.workspace_bytes = ws.data_ptr(), ws.numel()
        c.tuning = _abi.Tuning.from_env()
        self.stream = torch.cuda.current_stream()
        self.sp = self.stream.cuda_stream
        self.dispatch_bytes = R * T * H * 2 + R * T * K * 8 + n_e * (H + (H // 128) * 4 + 4) + E_l * (4 + R * 8)
        self.combine_bytes = n_e * H * 2 + R * T * K * 12 + R * T * H * 2

    def dispatch(self):
        self._abi.check(self._abi.lib.deep_ep_hip_launch_ll_dispatch(ctypes.byref(self.d), self.sp), "ll dispatch")

    def combine(self):
        self._abi.check(self._abi.lib.deep_ep_hip_launch_ll_combine(ctypes.byref(self.c), self.sp), "ll combine")

    def step(self):
        self.dispatch()
        self.combine()

    def loop_us(self, fn, iters):
        torch = self.torch
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(self.stream)
        for _ in range(iters):
            fn()
        e1.record(self.stream)
        e1.synchronize()
        return e0.elapsed_time(e1) * 1e3 / iters


def bench_low_latency(args, torch, rc, _abi, dev):
    ll = LowLatencyCalls(torch, rc, _abi, dev)
    R, T, H, E, K, M, n_e = ll.R, ll.T, ll.H, ll.E, ll.K, ll.M, ll.n_e
    for _ in range(args.warmup):
        ll.step()
    torch.cuda.synchronize()
    step_us = ll.loop_us(ll.step, args.steps)
    d_us, c_us = ll.loop_us(ll.dispatch, max(args.steps, 20)), ll.loop_us(ll.combine, max(args.steps, 20))
    d_bytes, c_bytes = ll.dispatch_bytes, ll.combine_bytes
    sweep = None
    if args.ll_batch_sweep:
        # other batch sizes of the same shape: the single-kernel dispatch (one item per wavefront up to 128 tokens per
        # rank here, several beyond) against the counting + move kernels, and the combine
        sweep = {}
        for t in (64, 128, 192, 256, 384, 512):
            one, two = LowLatencyCalls(torch, rc, _abi, dev, t), LowLatencyCalls(torch, rc, _abi, dev, t, two_kernels=True)
            for calls in (one, two):
                for _ in range(5):
                    calls.step()
            torch.cuda.synchronize()
            sweep[f"{R}x{t}"] = {"dispatch_us": round(one.loop_us(one.dispatch, 50), 2),
                                 "dispatch_two_kernels_us": round(two.loop_us(two.dispatch, 50), 2),
                                 "combine_us": round(one.loop_us(one.combine, 50), 2)}
            del one, two
    if args.calibration_copy:
        calibration_copy(torch, dev)
    result = {"metric": "low-latency dispatch+combine us/call, 8 sources x 128 tokens x 7168, top-8 of 256, destination rank 0",
            "value": round(step_us, 2), "unit": "us", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(step_us * 1e-3, 5), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
            "dtype": "fp8_e4m3 dispatch / bf16 weighted combine", "data": "synthetic",
            "config": {"workload": f"C5: R={R} T={T} H={H} E={E} K={K} M={M}, rows on rank 0: {n_e}"},
            "us_per_call": {"ll_dispatch": round(d_us, 2), "ll_combine": round(c_us, 2)},
            "achieved_gbs": {"ll_dispatch": round(d_bytes / d_us * 1e-3, 1), "ll_combine": round(c_bytes / c_us * 1e-3, 1)},
            "algorithmic_bytes": {"ll_dispatch": d_bytes, "ll_combine": c_bytes},
            "roofline": {"kernel": "ll_fused_kernel", "bound": "hbm", "achieved": round(d_bytes / d_us * 1e-3, 1),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(d_bytes / d_us * 1e-3 / HBM_PEAK_GBS, 4),
                         "traffic": MEASURED_TRAFFIC_BYTES.get(("C5", "packed", "fp8", "ll_dispatch"))},
            "roofline_combine": {"kernel": "ll_combine_kernel", "bound": "hbm", "achieved": round(c_bytes / c_us * 1e-3, 1),
                                 "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(c_bytes / c_us * 1e-3 / HBM_PEAK_GBS, 4),
                                 "traffic": MEASURED_TRAFFIC_BYTES.get(("C5", "packed", "fp8", "ll_combine"))}}
    if sweep is not None:
        result["low_latency_batch_sweep"] = sweep
    result["us_per_api_call"] = low_latency_api_figures(torch, ll, kernel_us=(d_us, c_us))
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline_low_latency(*ll.cpu_inputs, R, M, E)
    return result


def cpu_baseline_low_latency(x, idx, w, R, M, E):
    """The CPU oracle on the whole low-latency workload: what destination rank 0 receives from the R source ranks
    (FP8 cast + packed scatter), then the weighted combine back to every source rank."""
    import torch
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import routing_oracle as oracle

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    E_l, H = E // R, x.shape[2]
    y = torch.zeros((E_l, R * M, H), dtype=torch.bfloat16)

    def one_pass():
        _, _, _, info, ranges = oracle.ll_dispatch(list(x), list(idx), M, E, R, 0)
        for s in range(R):
            oracle.ll_combine(y, idx[s], w[s], info, ranges, s, E, R, 0)

    one_pass()   # warm-up
    iters, t0 = 0, time.perf_counter()
    while True:
        one_pass()
        iters += 1
        elapsed = time.perf_counter() - t0
        if elapsed > 10.0 or iters >= 10:
            break
    per_pass = elapsed / iters
    return {"value": round(per_pass * 1e6, 1), "unit": "us", "cores": cores, "kind": "port",
            "sample": f"the whole workload ({R} sources x {x.shape[1]} tokens), 1 warm-up + {iters} timed passes of "
                      f"ll_dispatch + ll_combine for every source (torch CPU, eager)"}


def cpu_baseline(case, sample_tokens, fp8, expanded):
    """The torch-CPU oracle (the reference path restated) timed on the first `sample_tokens` tokens of
    the same workload: layout + (FP8 cast +) dispatch + combine, all host cores."""
    import torch
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import routing_oracle as oracle

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    n = case.T if sample_tokens <= 0 else min(sample_tokens, case.T)
    x, idx, w = case.x[:n].contiguous(), case.topk_idx[:n].contiguous(), case.topk_weights[:n].contiguous()
    T, H, K, E, R = n, case.H, case.K, case.E, case.R

    def one_pass():
        oracle.layout(idx, E, R)
        payload = oracle.per_token_cast_to_fp8(x) if fp8 else x
        r = oracle.dispatch(payload, idx, w, E, R, 0, n, do_expand=expanded)
        rows = r.recv_x[0].shape[0] if isinstance(r.recv_x, tuple) else r.recv_x.shape[0]
        y = torch.zeros((rows, H), dtype=torch.bfloat16)
        oracle.combine(y, idx, r.recv_src_metadata, r.dst_buffer_slot_idx, r.psum_num_recv_tokens_per_scaleup_rank,
                       E, R, 0, n, topk_weights=r.recv_topk_weights, do_expand=expanded)
        return r

    r = one_pass()   # warm-up
    iters, t0 = 0, time.perf_counter()
    while True:
        one_pass()
        iters += 1
        elapsed = time.perf_counter() - t0
        if elapsed > 10.0 or iters >= 2:
            break
    per_pass = elapsed / iters
    valid = idx >= 0
    N_e = int(valid.sum())
    N_r = r.num_recv_tokens
    ab = algorithmic_bytes(T, H, K, E, R, N_r, N_e, fp8=fp8, expanded=expanded)
    total = ab["layout"] + ab["dispatch"] + ab["combine"]
    return {"value": round(total / per_pass * 1e-9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"{'all' if n == case.T else 'first ' + str(n) + ' of'} {case.T} tokens of the same workload, 1 warm-up + {iters} timed passes of "
                      f"layout+dispatch+combine (torch CPU, eager), {per_pass * 1e3:.1f} ms/pass",
            "ms_per_pass": round(per_pass * 1e3, 2)}


if __name__ == "__main__":
    main()
