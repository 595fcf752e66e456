"""Benchmark of the quantized-matmul / MoE hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--skip-secondary]

Headline (`value`): prefill tok/s of BASELINE configs[3], the Q4_K MoE expert GEMM at T = 2048 — one step
is router top-10 -> expert permutation -> ragged grouped gate/up GEMM + SwiGLU -> grouped down GEMM ->
shared expert -> weighted combine, on synthetic inputs already resident in HBM. The same JSON line carries
the decode-side numbers (configs 0, 2, 4 as HBM GB/s), config 1 (dense dequant-GEMM), the roofline of the
dominant kernel measured live with events around each launch, and a CPU baseline timed on this host.
"""
import argparse
import copy
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0     # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0  # dense f16 / bf16 matrix peak


def timed(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def timed_batches(torch, fn, batches=50, warmup=3):
    """`batches` launches of `fn`, each bracketed by its own pair of events (the engine's BatchResult.gpu_ms, src/graph.mm:3979-3984):
    mean, median and min in ms. The event pairs add a few microseconds of idle time per batch that the back-to-back loop of
    `timed` does not see."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(batches)]
    for start, stop in pairs:
        start.record()
        fn()
        stop.record()
    torch.cuda.synchronize()
    ms = sorted(start.elapsed_time(stop) for start, stop in pairs)
    return {"batches": batches, "mean_ms": sum(ms) / len(ms), "median_ms": ms[len(ms) // 2] if len(ms) % 2 else 0.5 * (ms[len(ms) // 2 - 1] + ms[len(ms) // 2]),
            "min_ms": ms[0]}


def graph_of(torch, fn, result, times=1):
    """`fn` recorded `times` times into one HIP graph (the launches of a step replayed by the driver instead of being
    issued one by one from Python), or None when capture fails or a replay does not reproduce the eager result bit for
    bit. The check replays three times with eager work and synchronisations in between."""
    fn()
    torch.cuda.synchronize()
    want = result.clone()
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(times):
                fn()
        for _ in range(3):
            result.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            if not torch.equal(result, want):
                return None
        return graph
    except Exception as error:  # capture not possible here: time the eager launches instead
        print(f"graph capture failed: {error}", file=sys.stderr)
        torch.cuda.synchronize()
        return None


def profiled(capi, torch, fn, steps):
    torch.cuda.synchronize()
    capi.profile_begin()
    for _ in range(steps):
        fn()
    rows = capi.profile_end()
    return {k: {"launches": v[0], "avg_us": 1e3 * v[1] / max(v[0], 1), "min_us": 1e3 * v[2]} for k, v in rows.items()}


def measured_traffic(kernel):
    """HBM bytes per launch of `kernel` as measured with hardware counters and recorded under profiles/
    (a line `traffic_bytes_per_launch[<kernel>] = N`), or None when no such measurement is on file."""
    folder = os.path.join(ROOT, "profiles")
    if os.path.isdir(folder):
        for name in sorted(os.listdir(folder)):
            if name.endswith((".md", ".txt")):
                for text in open(os.path.join(folder, name)):
                    if text.startswith(f"traffic_bytes_per_launch[{kernel}] ="):
                        return float(text.split("=")[1])
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--skip-secondary", action="store_true")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches only (no HIP graph replay)")
    ap.add_argument("--skip-comparison", action="store_true",
                    help="leave out the untimed comparison runs (shared expert on a second stream): a kernel trace then holds "
                         "the timed step's launches and the roofline launches only")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path is built and measured on a single MI355X (--gpus 1); "
              "across GPUs the experts would be sharded and the routed rows exchanged all-to-all, which is not built here",
              file=sys.stderr)
        sys.exit(2)

    import torch
    capi = importlib.import_module("tokspur-public_amd.capi")
    synth = importlib.import_module("tokspur-public_amd.synth")
    capi.dll()  # fails loudly when the HIP library has not been built
    torch.cuda.set_device(0)
    gpu = capi.Device()
    t_setup = time.time()

    # ------------------------------------------------------------------ config 3 (headline)
    T, C, H, E, S = 2048, 2048, 512, 512, 10
    logits = synth.zipf_router_logits(synth.tensor_seed(3, 1), T, E, scale=synth.ZIPF_BIAS_SCALE)
    x = synth.round_bf16(synth.activations_f32(synth.tensor_seed(3, 2), (T, C)))
    gate = synth.matrix(12, synth.tensor_seed(3, 10), H * E, C)
    up = synth.matrix(12, synth.tensor_seed(3, 11), H * E, C)
    down = synth.matrix(14, synth.tensor_seed(3, 12), C * E, H)
    w = capi.PlanarMoeWeights(gpu, 12, 14, C, H, E, gate, up, down)
    sg = synth.matrix(12, synth.tensor_seed(3, 20), H, C)
    su = synth.matrix(12, synth.tensor_seed(3, 21), H, C)
    sd = synth.matrix(14, synth.tensor_seed(3, 22), C, H)
    ws = capi.PlanarMoeWeights(gpu, 12, 14, C, H, 2, np.concatenate([sg, sg]), np.concatenate([su, su]), np.concatenate([sd, sd]))
    shared = capi.PlanarSharedExpert(gpu, C, H, sg, su, sd)
    d_logits, d_x = gpu.upload(logits), gpu.upload(x)
    ids, wts = gpu.zeros((T, S), "int32"), gpu.zeros((T, S))
    scratch, scratch_s = capi.GroupedScratch(gpu, T, S, E, C, H, with_shared=True), capi.GroupedScratch(gpu, T, 1, 2, C, H)
    y, ys, out = gpu.empty((T * S, C)), gpu.empty((T, C)), gpu.empty((T, C))
    ids_shared, shared_logit = gpu.zeros(T, "int32"), gpu.full(T, 20.0)

    def routed_only():
        capi.planar_nax_grouped_moe(gpu, w, ids, d_x, T, S, scratch, y=y)

    side = torch.cuda.Stream()  # default priority: the shared expert only needs x, so it runs beside the routed experts

    def step_two_streams():  # the shared expert as a grouped product of its own beside the routed experts
        main = torch.cuda.current_stream()
        side.wait_stream(main)
        with torch.cuda.stream(side):
            capi.planar_nax_grouped_moe(gpu, ws, ids_shared, d_x, T, 1, scratch_s, y=ys)
        gpu.route(d_logits, S, 0, True, tokens=T, out=(ids, wts))
        routed_only()
        main.wait_stream(side)
        gpu.mixture(y, wts, ys, shared_logit, C, S, tokens=T, out=out)

    def step_c3():  # the shared expert's rows ride in the routed experts' two GEMM launches
        gpu.route(d_logits, S, 0, True, tokens=T, out=(ids, wts))
        capi.planar_nax_grouped_moe(gpu, w, ids, d_x, T, S, scratch, y=y, shared=shared, shared_y=ys)
        gpu.mixture(y, wts, ys, shared_logit, C, S, tokens=T, out=out)

    # Part of set-up, before any warm-up or timed step: 30 untimed steps (~15 ms) bring the GPU from idle to its working
    # clocks. Without them the W = 3 warm-up steps end before the clocks have risen and the timed steps start ~12 % slow.
    for _ in range(30):
        step_c3()
    torch.cuda.synchronize()
    two_streams_ms_step = None
    if not args.skip_comparison:
        two_streams_ms_step = timed(torch, step_two_streams, args.steps, args.warmup)
        torch.cuda.synchronize()
        reference_out = out.clone()
    eager_ms_step = timed(torch, step_c3, args.steps, args.warmup)
    torch.cuda.synchronize()
    assert args.skip_comparison or torch.equal(out, reference_out), "the two ways of running the shared expert disagree"
    graph = None if args.no_graph else graph_of(torch, step_c3, out)
    graph_ms_step = timed(torch, graph.replay, args.steps, args.warmup) if graph is not None else None
    # the step is reported the way it ran fastest; both ways are in the line
    ms_step = eager_ms_step if graph_ms_step is None or graph_ms_step >= eager_ms_step else graph_ms_step
    # the same step under the engine's protocol: 3 warm-up batches, then 50 batches with an event pair around each
    batches = max(50, args.steps)
    protocol = {"eager": timed_batches(torch, step_c3, batches, 3),
                "graph": timed_batches(torch, graph.replay, batches, 3) if graph is not None else None}
    assert gpu.error() == 0, "device error word set during the timed region"
    counts = scratch.counts.cpu().numpy().view(np.uint32)
    nonempty = int((counts > 0).sum())
    flops_step = (T * S + T) * 6291456.0
    bytes_step = (nonempty + 1) * 2039808 + 8388608 + 16777216 + 4194304
    prof = profiled(capi, torch, routed_only, 5)
    gu = prof["gemm_gate_up_swiglu"]
    # dominant kernel: the routed gate/up GEMM. 142 FLOP per weight byte is below the MI355X ridge (2.5e15 / 8e12 = 312),
    # so HBM bounds it. Algorithmic bytes per launch: every non-empty expert's Q4_K gate+up rows once (2 x 512 rows x 8
    # blocks x 144 B = 1 179 648 B per expert), the f16 activations once, the f16 h rows once.
    gu_flops = T * S * 2.0 * (2 * H) * C
    gu_bytes = nonempty * 2 * H * (C // 256) * 144 + T * C * 2 + T * S * H * 2
    gu_s = gu["avg_us"] * 1e-6
    roofline = {"kernel": "gemm_gate_up_swiglu (routed experts of configs[3]: persistent workgroups, a task's activation rows resident in registers, Q4_K planar weight tiles streamed global->LDS once per task -> integer f16 MFMA 32x32x16 + SwiGLU)",
                "bound": "hbm", "achieved": gu_bytes / gu_s / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": gu_bytes / gu_s / 1e9 / HBM_PEAK_GBPS, "traffic": measured_traffic("gemm_gate_up_swiglu"),
                "avg_launch_us": gu["avg_us"], "bytes_per_launch": gu_bytes, "flops_per_launch": gu_flops,
                "mfma_tflops": gu_flops / gu_s / 1e12, "mfma_frac": gu_flops / gu_s / 1e12 / MFMA_F16_PEAK_TFLOPS}
    # a plain copy of known size, once, outside every timed region: the yardstick for a profiler's HBM byte counters
    cal_src = gpu.zeros(64 << 20, "int32")
    cal_dst = gpu.empty(64 << 20, "int32")
    capi.calibration_copy(gpu, cal_dst, cal_src)
    torch.cuda.synchronize()
    del cal_src, cal_dst
    configs = {"c3_moe_prefill": {
        "tok_per_s": T / (ms_step * 1e-3), "ms_per_step": ms_step, "tflops": flops_step / (ms_step * 1e-3) / 1e12,
        "mfma_frac": flops_step / (ms_step * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS,
        "hbm_gbps": bytes_step / (ms_step * 1e-3) / 1e9, "hbm_frac": bytes_step / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "expert_loads": {"nonempty": nonempty, "min": int(counts.min()), "median": int(np.median(counts)), "max": int(counts.max())},
        "kernels_us": {k: round(v["avg_us"], 2) for k, v in prof.items()},
        "launch": "HIP graph replay of the step's kernels" if ms_step is graph_ms_step else "eager launches from Python",
        "eager_ms_per_step": eager_ms_step, "graph_ms_per_step": graph_ms_step,
        "per_batch_events": protocol,
        "shared_expert": "rides in the routed experts' gate/up and down launches" + (
            "" if two_streams_ms_step is None else
            f" (same bits as run beside them on a second stream: {two_streams_ms_step:.3f} ms per step that way, eager)")}}

    # ------------------------------------------------------------------ the whole sublayer, router projection included
    # What encode_moe_mm_many enqueues for a chunk (src/moe_mm_many.cpp:126-283): router projection as ONE f32 GEMM
    # (kernels/moe_router_f32_batch.metal:13) -> batch top-k -> routed experts -> shared expert as three dense Q8_0 products
    # with SwiGLU between -> shared router -> batch mixture. The router weights are random here, so the expert loads are
    # near uniform (the headline step draws Zipf-biased logits instead of projecting them).
    rw = gpu.upload(synth.activations_f32(synth.tensor_seed(3, 30), (E, C)) / np.float32(np.sqrt(C)))
    srw = gpu.upload(synth.activations_f32(synth.tensor_seed(3, 31), (1, C)) / np.float32(np.sqrt(C)))
    q8g, q8u = gpu.upload(synth.matrix(8, synth.tensor_seed(3, 32), H, C)), gpu.upload(synth.matrix(8, synth.tensor_seed(3, 33), H, C))
    q8d = gpu.upload(synth.matrix(8, synth.tensor_seed(3, 34), C, H))
    lg_l, sl_l = gpu.empty((T, E)), gpu.empty(T)
    sg_l, su_l, sd_l = gpu.empty((T, H)), gpu.empty((T, H)), gpu.empty((T, C))
    q8ws = gpu.empty(max(capi.dense_mm_q8_workspace_bytes(T, C, H), capi.dense_mm_q8_workspace_bytes(T, H, C)), "uint8")
    scratch_l = capi.GroupedScratch(gpu, T, S, E, C, H)

    def step_sublayer():
        gpu.router_f32_batch(rw, d_x, T, C, E, out=lg_l)
        gpu.route(lg_l, S, 0, True, tokens=T, out=(ids, wts))
        capi.planar_nax_grouped_moe(gpu, w, ids, d_x, T, S, scratch_l, y=y)
        capi.dense_mm_q8_staged(gpu, capi.LAYOUT_GGUF, q8g, d_x, T, C, H, out=sg_l, workspace=q8ws)
        capi.dense_mm_q8_staged(gpu, capi.LAYOUT_GGUF, q8u, d_x, T, C, H, out=su_l, workspace=q8ws)
        gpu.swiglu(sg_l, su_l, out=sg_l)
        capi.dense_mm_q8_staged(gpu, capi.LAYOUT_GGUF, q8d, sg_l, T, H, C, out=sd_l, workspace=q8ws)
        gpu.gemv_rows(0, srw, d_x, sl_l, T, C, 1, C * 4, 4)
        gpu.mixture(y, wts, sd_l, sl_l, C, S, tokens=T, out=out)

    sub_eager = timed(torch, step_sublayer, args.steps, args.warmup)
    sub_graph = None if args.no_graph else graph_of(torch, step_sublayer, out)
    sub_graph_ms = timed(torch, sub_graph.replay, args.steps, args.warmup) if sub_graph is not None else None
    sub_ms = sub_eager if sub_graph_ms is None or sub_graph_ms >= sub_eager else sub_graph_ms
    sub_counts = scratch_l.counts.cpu().numpy().view(np.uint32)
    configs["c3_sublayer_with_router"] = {
        "tok_per_s": T / (sub_ms * 1e-3), "ms_per_step": sub_ms, "eager_ms_per_step": sub_eager, "graph_ms_per_step": sub_graph_ms,
        "per_batch_events": {"eager": timed_batches(torch, step_sublayer, batches, 3),
                             "graph": timed_batches(torch, sub_graph.replay, batches, 3) if sub_graph is not None else None},
        "expert_loads": {"nonempty": int((sub_counts > 0).sum()), "min": int(sub_counts.min()), "median": int(np.median(sub_counts)), "max": int(sub_counts.max())},
        "kernels_us": {k: round(v["avg_us"], 2) for k, v in profiled(capi, torch, step_sublayer, 5).items()},
        "composition": "router f32 GEMM -> top-10 -> grouped gate/up + SwiGLU -> grouped down -> shared expert as 3 dense Q8_0 GEMMs + SwiGLU -> shared router -> mixture"}
    assert gpu.error() == 0, "device error word set during the sublayer steps"
    del sub_graph

    # ------------------------------------------------------------------ CPU baseline (rank 0, bounded sample)
    cpu = None
    if not args.skip_cpu:
        from oracle import oracle
        ref, orc = oracle.ref(), oracle.lib()
        lib, kind = (ref, "reference") if ref is not None else (orc, "port")
        id_host = ids.cpu().numpy().view(np.uint32).reshape(-1)
        gsz, dsz = (C // 256) * 144 * H, (H // 256) * 210 * C
        t0, done = time.perf_counter(), 0
        while done < 512 and time.perf_counter() - t0 < 12.0:
            rid = (done * 397) % (T * S)
            e, xv = int(id_host[rid]), x[rid // S]
            g = lib.reference_gemv(12, gate[e * gsz:(e + 1) * gsz], C, H, xv)
            u = lib.reference_gemv(12, up[e * gsz:(e + 1) * gsz], C, H, xv)
            gf = g.astype(np.float32)
            h = (gf / (np.float32(1) + np.exp(-gf))) * u.astype(np.float32)
            lib.reference_gemv(14, down[e * dsz:(e + 1) * dsz], H, C, h)
            done += 1
        per_route = (time.perf_counter() - t0) / done
        cpu = {"value": T / (per_route * (T * S + T)), "unit": "tok/s", "cores": 1, "kind": kind,
               "sample": f"{done} of {T * S + T} expert routes of configs[3] (dequantize + double-accumulate GEMV for gate, up, down), "
                         f"{per_route * 1e3:.1f} ms per route, extrapolated linearly"}
        # the same arithmetic, weight rows split over the host cores this process may use (the restated code: the
        # reference ships its GEMV single-threaded)
        cores = max(1, min(16, len(os.sched_getaffinity(0))))
        t0, done = time.perf_counter(), 0
        while done < 2048 and time.perf_counter() - t0 < 6.0:
            rid = (done * 397) % (T * S)
            e, xv = int(id_host[rid]), x[rid // S]
            g = orc.reference_gemv_mt(12, gate[e * gsz:(e + 1) * gsz], C, H, xv, cores)
            u = orc.reference_gemv_mt(12, up[e * gsz:(e + 1) * gsz], C, H, xv, cores)
            gf = g.astype(np.float32)
            h = (gf / (np.float32(1) + np.exp(-gf))) * u.astype(np.float32)
            orc.reference_gemv_mt(14, down[e * dsz:(e + 1) * dsz], H, C, h, cores)
            done += 1
        per_route_mt = (time.perf_counter() - t0) / done
        cpu["all_cores"] = {"value": T / (per_route_mt * (T * S + T)), "unit": "tok/s", "cores": cores, "kind": "port",
                            "sample": f"{done} routes, {per_route_mt * 1e3:.2f} ms per route"}

    # ------------------------------------------------------------------ secondary configs
    if not args.skip_secondary:
        k2 = max(5, args.steps // 2)
        # config 1: dense Q4_K dequant-GEMM, raw GGUF rows, bf16 in / bf16 out
        w1 = gpu.upload(synth.matrix(12, synth.tensor_seed(1, 1), 8192, C))
        for m in (128, 512, 2048):
            xb = gpu.upload(synth.bf16_bits(synth.activations_f32(synth.tensor_seed(1, 2 + m), (m, C))))
            o1, ws1 = gpu.empty((m, 8192), "int16"), gpu.empty(capi.dense_mm_workspace_bytes(m, C), "uint8")
            ms = timed(torch, lambda: capi.dense_mm(gpu, 12, capi.LAYOUT_GGUF, w1, xb, m, C, 8192, out=o1, out_bf16=True, workspace=ws1), k2, 2)
            fl = 2.0 * m * C * 8192
            configs[f"c1_dense_gemm_m{m}"] = {"tok_per_s": m / (ms * 1e-3), "ms": ms, "tflops": fl / (ms * 1e-3) / 1e12,
                                              "mfma_frac": fl / (ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS}
        # config 3 with the engine's own down kind: Q4_K co-located gate/up (the same tensors) and Q8_0 planes down (kind 9), whose
        # weights the down kernel decodes to halves on the fly
        down8 = synth.matrix(8, synth.tensor_seed(3, 13), C * E, H)
        w8 = capi.PlanarMoeWeights(gpu, 12, 8, C, H, E, gate, up, down8)
        del down8

        def routed_q8_down():
            capi.planar_nax_grouped_moe(gpu, w8, ids, d_x, T, S, scratch, y=y)

        gpu.route(d_logits, S, 0, True, tokens=T, out=(ids, wts))  # the headline's routes again (the sublayer drew its own)
        ms = timed(torch, routed_q8_down, k2, 2)
        configs["c3_routed_q4k_gate_up_q8_down"] = {"ms": ms, "tok_per_s": T / (ms * 1e-3),
                                                    "kernels_us": {k: round(v["avg_us"], 2) for k, v in profiled(capi, torch, routed_q8_down, 5).items()}}
        del w8
        # NOT a BASELINE configuration: the engine's own expert shape (2560 channels, 640 hidden units: src/moe_mm_many_plan.cpp:7,31)
        # with its kinds, Q4_K co-located gate/up and Q8_0 planes down, 2048 tokens, 512 experts, top-10, uniform router. Neither
        # resident kernel takes this shape (they want 2048 columns resp. 512 hidden units): gate/up runs on the general
        # integer-factor kernel, down on the staged kernel. 64 synthetic experts repeated eight times.
        Ce, He = 2560, 640
        rep = E // 64
        ge = np.tile(synth.matrix(12, synth.tensor_seed(3, 30), He * 64, Ce), rep)
        ue = np.tile(synth.matrix(12, synth.tensor_seed(3, 31), He * 64, Ce), rep)
        de = np.tile(synth.matrix(8, synth.tensor_seed(3, 32), Ce * 64, He), rep)
        we = capi.PlanarMoeWeights(gpu, 12, 8, Ce, He, E, ge, ue, de)
        del ge, ue, de
        xe = gpu.upload(synth.round_bf16(synth.activations_f32(synth.tensor_seed(3, 33), (T, Ce))))
        ids_e, wts_e = gpu.zeros((T, S), "int32"), gpu.zeros((T, S))
        gpu.route(gpu.upload(synth.activations_f32(synth.tensor_seed(3, 34), (T, E))), S, 0, True, tokens=T, out=(ids_e, wts_e))
        scratch_e, ye = capi.GroupedScratch(gpu, T, S, E, Ce, He), gpu.empty((T * S, Ce))

        def routed_engine_shape():
            capi.planar_nax_grouped_moe(gpu, we, ids_e, xe, T, S, scratch_e, y=ye)

        ms = timed(torch, routed_engine_shape, k2, 2)
        fl_e = T * S * 3 * 2.0 * Ce * He
        configs["engine_shape_2560x640_q4k_gate_up_q8_down_not_a_baseline_config"] = {
            "ms": ms, "tok_per_s": T / (ms * 1e-3), "tflops": fl_e / (ms * 1e-3) / 1e12,
            "kernels_us": {k: round(v["avg_us"], 2) for k, v in profiled(capi, torch, routed_engine_shape, 5).items()}}
        assert gpu.error() == 0
        del we, xe, scratch_e, ye
        # config 0: dense Q4_K GEMV over a rotation of distinct weight copies (> 512 MB) so every read comes from HBM
        w0 = synth.matrix(12, synth.tensor_seed(0, 1), 4096, C)
        x0, y0 = gpu.upload(synth.activations_f32(synth.tensor_seed(0, 2), C)), gpu.empty(4096)
        copies = [gpu.upload(w0) for _ in range(120)]
        state = {"i": 0}

        def gemv_rot():
            gpu.gemv(12, copies[state["i"] % len(copies)], x0, C, 4096, y=y0)
            state["i"] += 1

        eager_ms = timed(torch, gemv_rot, 240, 120)
        state["i"] = 0
        graph0 = None if args.no_graph else graph_of(torch, gemv_rot, y0, times=len(copies))  # one rotation: 120 launches, 120 matrices
        graph_ms = timed(torch, graph0.replay, 6, 2) / len(copies) if graph0 is not None else None
        ms = eager_ms if graph_ms is None or graph_ms >= eager_ms else graph_ms
        b0 = 4096 * 8 * 144 + 8192 + 16384
        configs["c0_gemv_q4k"] = {"us": ms * 1e3, "eager_us": eager_ms * 1e3, "graph_us": None if graph_ms is None else graph_ms * 1e3,
                                  "hbm_gbps": b0 / (ms * 1e-3) / 1e9, "hbm_frac": b0 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                                  "launch": "HIP graph replay of 120 launches" if ms is graph_ms else "eager launches from Python",
                                  "note": "per-launch time over a 566 MB rotation of weight copies; a 4.7 MB launch is latency bound"}
        del graph0
        ms = timed(torch, lambda: gpu.gemv(12, copies[0], x0, C, 4096, y=y0), 240, 20)
        configs["c0_gemv_q4k"]["cache_resident_us"] = ms * 1e3
        state["i"] = 0
        k0 = profiled(capi, torch, gemv_rot, 120)
        configs["c0_gemv_q4k"]["kernel_us"] = round(min(v["avg_us"] for v in k0.values()), 2)
        del copies
        # NOT a BASELINE configuration: the same Q4_K GEMV kernel at sizes where HBM, not launch latency, bounds it (the 4.7 MB of
        # config 0 cannot show the kernel's bandwidth). Weights: config 0's rows repeated; two copies alternate.
        for big_rows in (65536, 262144):
            wb = np.tile(w0, big_rows // 4096)
            pair = [gpu.upload(wb), gpu.upload(wb)]
            yb = gpu.empty(big_rows)
            state["i"] = 0

            def gemv_big():
                gpu.gemv(12, pair[state["i"] % 2], x0, C, big_rows, y=yb)
                state["i"] += 1

            ms = timed(torch, gemv_big, 40, 10)
            bb = big_rows * 8 * 144 + 8192 + big_rows * 4
            configs[f"gemv_q4k_{big_rows}x2048_not_a_baseline_config"] = {"us": ms * 1e3, "hbm_gbps": bb / (ms * 1e-3) / 1e9,
                                                                           "hbm_frac": bb / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, "bytes": bb}
            del pair, wb, yb
        # config 2: MoE verify T = 8 on the config-3 experts. Eight router inputs in rotation select different experts from step
        # to step, and four copies of the whole 1.06 GB expert set take turns as well: any one copy is read every fourth step,
        # with ~450 MB of other copies' experts in between, so no expert's planes are still in the 256 MB last-level cache
        # when a step asks for them (with one copy, a quarter of a step's experts had been read one or two steps before)
        T2 = 8
        expert_sets = [w]
        for _ in range(3):
            twin = copy.copy(w)
            twin.pair_lo, twin.pair_hi, twin.down, twin.union_meta = w.pair_lo.clone(), w.pair_hi.clone(), w.down.clone(), w.union_meta.clone()
            expert_sets.append(twin)
        sets = []
        for i in range(8):
            lg = gpu.upload(synth.activations_f32(synth.tensor_seed(2, 100 + i), (T2, E)))
            sets.append((lg, gpu.upload(synth.activations_f32(synth.tensor_seed(2, 200 + i), (T2, C)))))
        ids2, wts2 = gpu.zeros((T2, S), "int32"), gpu.zeros((T2, S))
        h2, y2, hs2, ys2, out2 = gpu.empty((T2 * S, H)), gpu.empty((T2 * S, C)), gpu.empty((T2, H)), gpu.empty((T2, C)), gpu.empty((T2, C))
        ids_s2, sl2 = gpu.zeros(T2, "int32"), gpu.full(T2, 20.0)
        used = []
        for lg, _ in sets:
            gpu.route(lg, S, 0, True, tokens=T2, out=(ids2, wts2))
            used.append(len(set(ids2.cpu().numpy().reshape(-1).tolist())))

        def step_c2_two_streams():  # the shared expert as a routed call of its own beside the routed experts
            lg, xx = sets[state["i"] % len(sets)]
            w2 = expert_sets[state["i"] % len(expert_sets)]
            state["i"] += 1
            main = torch.cuda.current_stream()
            side.wait_stream(main)
            with torch.cuda.stream(side):
                capi.planar_moe_routed_m8(gpu, ws, ids_s2, xx, T2, 1, h=hs2, y=ys2)
            gpu.route(lg, S, 0, True, tokens=T2, out=(ids2, wts2))
            capi.planar_moe_routed_m8(gpu, w2, ids2, xx, T2, S, h=h2, y=y2)
            main.wait_stream(side)
            gpu.mixture(y2, wts2, ys2, sl2, C, S, tokens=T2, out=out2)

        def step_c2():  # the shared expert as one more record of the routed experts' two launches
            lg, xx = sets[state["i"] % len(sets)]
            w2 = expert_sets[state["i"] % len(expert_sets)]
            state["i"] += 1
            gpu.route(lg, S, 0, True, tokens=T2, out=(ids2, wts2))
            capi.planar_moe_routed_m8(gpu, w2, ids2, xx, T2, S, h=h2, y=y2, shared=shared, shared_h=hs2, shared_y=ys2)
            gpu.mixture(y2, wts2, ys2, sl2, C, S, tokens=T2, out=out2)

        two_streams_ms = None
        if not args.skip_comparison:
            two_streams_ms = timed(torch, step_c2_two_streams, 48, 16)
            state["i"] = 0
            step_c2_two_streams()
            torch.cuda.synchronize()
            reference_out2 = out2.clone()
            state["i"] = 0
            step_c2()
            torch.cuda.synchronize()
            assert torch.equal(out2, reference_out2), "the two ways of running the shared expert disagree (config 2)"
        eager_ms = timed(torch, step_c2, 48, 16)
        state["i"] = len(sets) - 1  # the check inside graph_of runs the last set once more, then the capture starts at set 0
        graph2 = None if args.no_graph else graph_of(torch, step_c2, out2, times=len(sets))
        graph_ms = timed(torch, graph2.replay, 6, 2) / len(sets) if graph2 is not None else None
        if graph_ms is None or graph_ms >= eager_ms:
            graph2, ms = None, eager_ms
        else:
            ms = graph_ms
        b2 = (float(np.mean(used)) + 1) * 2039808 + 147456
        configs["c2_moe_verify_t8"] = {"us": ms * 1e3, "eager_us": eager_ms * 1e3, "graph_us": None if graph_ms is None else graph_ms * 1e3,
                                       "distinct_experts_mean": float(np.mean(used)),
                                       "hbm_gbps": b2 / (ms * 1e-3) / 1e9, "hbm_frac": b2 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                                       "launch": "HIP graph replay of eight steps" if graph2 is not None else "eager launches from Python",
                                       "two_streams_us": None if two_streams_ms is None else two_streams_ms * 1e3}
        state["i"] = 0
        configs["c2_moe_verify_t8"]["kernels_us"] = {k: round(v["avg_us"], 2) for k, v in profiled(capi, torch, step_c2, 8).items()}
        configs["c2_moe_verify_t8"]["note"] = "eight router inputs x four copies of the expert set in rotation: every expert plane comes from HBM"
        del expert_sets, graph2
        # config 4: Q8_0 LM head, vocab 151936 x 2048, both arms: raw GGUF rows and the same matrix as q8_lanes_v1 rows. M = 16 goes
        # through the dense Q8_0 GEMM entry point (either layout: one pass, K halves summed)
        V = 151936
        w4_host = synth.matrix(8, synth.tensor_seed(4, 1), V, C)
        w4 = gpu.upload(w4_host)
        w4_lanes = gpu.upload(capi.q8_lanes_pack_rows(C, w4_host))
        del w4_host
        for m in (1, 4, 8, 16):
            x4 = gpu.upload(synth.activations_f32(synth.tensor_seed(4, 2 + m), (m, C)))
            y4 = gpu.empty((m, V))

            def lm_head():
                if m > 8:  # one pass over the matrix for up to sixteen rows
                    capi.dense_mm_q8(gpu, capi.LAYOUT_GGUF, w4, x4, m, C, V, out=y4)
                else:
                    gpu.q8_matvec_many(w4, x4, C, V, m, y=y4)

            ms = timed(torch, lm_head, k2, 2)
            b4 = 330612736 + 615936 * m
            configs[f"c4_lm_head_q8_m{m}"] = {"us": ms * 1e3, "hbm_gbps": b4 / (ms * 1e-3) / 1e9, "hbm_frac": b4 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}
            tk_scratch, tk_rows = gpu.empty(capi.logit_topk_scratch_bytes(m, V), "uint8"), gpu.empty(capi.logit_topk_output_bytes(m), "uint8")

            def lm_head_argmax():
                lm_head()
                capi.logit_topk(gpu, y4, m, V, scratch=tk_scratch, out=tk_rows)

            configs[f"c4_lm_head_q8_m{m}"]["us_with_top64"] = timed(torch, lm_head_argmax, k2, 2) * 1e3
            y4_lanes = gpu.empty((m, V))

            def lm_head_lanes():
                capi.dense_mm_q8(gpu, capi.LAYOUT_Q8_LANES_V1, w4_lanes, x4, m, C, V, out=y4_lanes)

            lanes_ms = timed(torch, lm_head_lanes, k2, 2)
            lm_head()
            both = (y4.cpu().numpy(), y4_lanes.cpu().numpy())
            assert float(np.max(np.abs(both[0] - both[1]) / np.maximum(1.0, np.abs(both[0])))) <= 5e-5, "the two row layouts disagree (config 4)"
            configs[f"c4_lm_head_q8_m{m}"].update({"lanes_us": lanes_ms * 1e3, "lanes_hbm_frac": b4 / (lanes_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS})
        assert gpu.error() == 0, "device error word set during the secondary configurations"

    line = {
        "metric": "prefill tok/s + decode HBM GB/s, Q4_K MoE expert GEMM, 1 MI355X",
        "value": T / (ms_step * 1e-3), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",  # f16 MFMA, f32 accumulate
        "data": "synthetic",
        "config": {"workload": "configs[3] MoE grouped-GEMM prefill: T=2048 tokens, hidden 2048, 512 experts, top-10 renormalised softmax "
                               "router with Zipf(1.1)-biased logits (bias scale 0.25), gate+up Q4_K [2x512,2048] + SwiGLU, down Q6_K [2048,512], "
                               "1 shared expert, weighted combine; integer weight factors and bf16 activations on the f16 matrix cores, f32 scales and accumulate",
                   "tokens": T, "experts": E, "selected": S, "routes": T * S},
        "roofline": roofline, "cpu_baseline": cpu, "configs": configs,
        "setup_s": round(time.time() - t_setup, 1),
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
