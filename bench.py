#!/usr/bin/env python3
"""Benchmark of the frozen quantized-linear hot path on one MI355X.

Workload (BASELINE.json configs[1], "decode dequant-GEMV"): K=4096, N=14336 (Llama-3-8B FFN
up-projection), weights ~ N(0, 0.02) quantised once to int8 (per-channel scales) and once to
int4 (group 128), activations bf16 ~ N(0,1), forward only.  One "step" = one int4 M=1 GEMV
plus one int8 M=1 GEMV.  Inputs are resident in HBM before the timed region; successive steps
rotate through >= 512 MB of distinct weight copies so the 256 MB Infinity Cache cannot serve
the reads.  `value` is algorithmic bytes moved per second (weights + scales + X + Y).

The launches of the timed region are captured once into a HIP graph and replayed, so the GPU,
not the Python launch path, sets the pace; per-kernel durations for the roofline object come
from HIP events around single-kernel graphs on the same stream.

Also reported in `extra`: M in {4,16} decode rates, the cache-resident M=1 rate, the
compute-bound rows (configs[2..3]) in TFLOP/s, the fp32 compute type (configs[0]'s layer) and the MoE
frozen-expert layer (configs[4]) in tokens/s.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
MFMA_FP32_PEAK_TFLOPS = 157.3
K_DEC, N_DEC = 4096, 14336
# HBM bytes per launch of the dominant kernel from rocprofv3 counters (profiles/decode_gemv_hbm_traffic.md).  A counter run
# cannot happen inside this script, so the figure is carried here with the state of the tree it was collected on.
MEASURED_TRAFFIC_INT8_M1 = 59406822
MEASURED_TRAFFIC_COLLECTED = "commit a3f0718 (after the last change to rowlin_int8_digits_kernel); read again at commit fdff18f: the same counts"


def algorithmic_bytes(kind, M, N=N_DEC, K=K_DEC, group=128):
    """Bytes one launch has to move: packed weights + scales + X (bf16) + Y (fp32)."""
    if kind == "int4":
        w = N * K // 2 + (N * K // group) * 2
    else:
        w = N * K + N * 4
    return w + M * K * 2 + M * N * 4


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--replays", type=int, default=5,
                    help="the K-step timed region is run this many times; the median run is reported")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary rows (M=4/16, GEMM TFLOP/s)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy three times (reference point for rocprofv3 --pmc "
                         "FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from caif_amd import capi, torch_ops as T

    capi.lib()                                    # fail loudly when the HIP library is missing
    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)

    # ---------------------------------------------------------------- synthetic weights, quantised on the GPU
    w = torch.empty(N_DEC, K_DEC, device=dev).normal_(0, 0.02, generator=gen)
    p4, s4 = T.quantize_int4_per_group(w, 128)
    q8, s8 = T.quantize_int8(w.reshape(K_DEC, N_DEC), per_channel=True)     # the reference's [in,out] labelling
    q8 = q8.reshape(-1)
    del w
    copies4 = max(2, -(-512 * 2**20 // algorithmic_bytes("int4", 1)))       # >= 512 MB of distinct weights
    copies8 = max(2, -(-512 * 2**20 // algorithmic_bytes("int8", 1)))
    W4 = [T.FrozenWeight(p4.clone(), T.W_INT4_GROUP, s4.clone(), N_DEC, K_DEC, 1, 128) for _ in range(copies4)]
    W8 = [T.FrozenWeight(q8.clone(), T.W_INT8, s8.clone(), N_DEC, K_DEC, N_DEC) for _ in range(copies8)]
    # M = 1, 4, 16 are the configuration's rows; 32 rows (two 16-row tiles in one pass over the weight) is an extra row
    X = {m: torch.empty(m, K_DEC, device=dev).normal_(0, 1, generator=gen).to(torch.bfloat16) for m in (1, 4, 16, 32)}
    Y = {m: torch.empty(m, N_DEC, device=dev) for m in (1, 4, 16, 32)}
    ws = torch.empty(4 << 20, dtype=torch.uint8, device=dev)      # partial sums of the 32-row kernel's two reduction slices

    def gemv(fw, m):
        T.qlinear_forward(X[m], fw, T.BF16, T.F32, out=Y[m], workspace=ws)

    def step(i):
        gemv(W4[i % copies4], 1)
        gemv(W8[i % copies8], 1)

    def capture(fn, count):
        """Record fn(0..count-1) into one HIP graph on a side stream (no memsets are recorded)."""
        g = torch.cuda.CUDAGraph()
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            fn(0)
            torch.cuda.synchronize()
            with torch.cuda.graph(g, stream=s):
                for i in range(count):
                    fn(i)
        torch.cuda.synchronize()
        return g

    def time_graph(g, launches, reps=5):
        """Average milliseconds per launch, HIP events around graph replays (median of reps)."""
        g.replay()
        torch.cuda.synchronize()
        times = []
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            g.replay()
            e1.record()
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1) / launches)
        return sorted(times)[len(times) // 2]

    # ---------------------------------------------------------------- the timed region: K steps
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    graph = capture(step, args.steps)
    graph.replay()
    torch.cuda.synchronize()
    # exactly K steps per timed run, each run bracketed by a device synchronisation on both sides; one run of a
    # 20-step graph lasts well under a millisecond, so the median of several runs is what is reported
    runs_ms = []
    for _ in range(max(1, args.replays)):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        runs_ms.append((t1 - t0) * 1e3 / args.steps)
    ms_per_step = sorted(runs_ms)[len(runs_ms) // 2]
    step_bytes = algorithmic_bytes("int4", 1) + algorithmic_bytes("int8", 1)
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    if args.calibrate_copy:
        src = torch.empty(256 * 2**20, dtype=torch.uint8, device=dev).fill_(3)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---------------------------------------------------------------- per-kernel durations (HIP events)
    L = 128
    per = {}
    for kind, Ws, nc in (("int4", W4, copies4), ("int8", W8, copies8)):
        for m in (1, 4, 16, 32):
            if m != 1 and args.no_extra:
                continue
            g = capture(lambda i, Ws=Ws, nc=nc, m=m: gemv(Ws[i % nc], m), L)
            ms = time_graph(g, L)
            per[(kind, m)] = {"us": ms * 1e3, "GBps": algorithmic_bytes(kind, m) / (ms * 1e-3) / 1e9}
            del g
    resident = {}
    for kind, Ws in (("int4", W4), ("int8", W8)):
        g = capture(lambda i, Ws=Ws: gemv(Ws[0], 1), L)
        ms = time_graph(g, L)
        resident[kind] = algorithmic_bytes(kind, 1) / (ms * 1e-3) / 1e9
        del g

    dom = ("int8", 1)           # the kernel that takes most of a step
    roofline = {
        "bound": "hbm",
        "kernel": "rowlin_int8_digits_kernel<bf16 X, per-channel scales, 4 chunks/row> M=1 K=4096 N=14336",
        "achieved": round(per[dom]["GBps"], 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(per[dom]["GBps"] / HBM_PEAK_GBS, 4),
        "avg_launch_us": round(per[dom]["us"], 3),
        "algorithmic_bytes_per_launch": algorithmic_bytes("int8", 1),
        # HBM bytes per launch of this kernel from two rocprofv3 --pmc runs (FETCH_SIZE x 1.9997 and
        # WRITE_SIZE x 1.0000, factors from a plain 256 MiB copy in the same runs): 59.35 MB read +
        # 0.06 MB written; the summary is profiles/decode_gemv_hbm_traffic.md
        "traffic": MEASURED_TRAFFIC_INT8_M1,
        "traffic_collected_at": MEASURED_TRAFFIC_COLLECTED,
    }

    extra = {
        "decode_GBps": {f"{k}_M{m}": round(v["GBps"], 1) for (k, m), v in per.items()},
        "decode_us": {f"{k}_M{m}": round(v["us"], 3) for (k, m), v in per.items()},
        "decode_cache_resident_GBps_M1": {k: round(v, 1) for k, v in resident.items()},
        "decode_frac_of_hbm_peak_M1": {k: round(per[(k, 1)]["GBps"] / HBM_PEAK_GBS, 4) for k in ("int4", "int8")},
        "weight_copies_rotated": {"int4": copies4, "int8": copies8},
        "timed_runs_ms_per_step": [round(v, 6) for v in runs_ms],
    }
    if not args.no_extra:
        del W4[1:], W8[1:]                        # the rotated copies are not needed below
        for name, fn in (("decode_other_shapes", lambda: decode_other_rows(torch, T, dev, gen, capture, time_graph)),
                         ("quantise_ops", lambda: quantise_rows(torch, T, dev, gen)),
                         ("compute_bound", lambda: compute_bound_rows(torch, T, dev, gen, capture, time_graph))):
            try:
                extra.update(fn())
            except Exception as e:   # secondary rows must not take the headline down
                extra[name + "_error"] = repr(e)

    out = {
        "metric": "dequant-GEMM HBM GB/s (M=1 int4/int8) + MFMA TFLOP/s (M=2048 fwd+dX)",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "decode dequant-GEMV K=4096 N=14336 M=1: one int4(g128) + one int8(per-channel) "
                               "launch per step, weights rotated over >=512 MB (BASELINE configs[1])",
                   "bytes_per_step": step_bytes},
        "roofline": roofline,
        "extra": extra,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(np, q8.cpu().numpy(), s8.cpu().numpy(), p4.cpu().numpy(),
                                           s4.cpu().view(torch.int16).numpy().view(np.uint16),
                                           X[1].float().cpu().numpy())
        if not args.no_extra:
            extra["cpu_host_path_configs0"] = cpu_configs0(np)
    print(json.dumps(out))


def decode_other_rows(torch, T, dev, gen, capture, time_graph):
    """Decode launches beside the headline shape.
    `decode_tall_M1`: the same M = 1 kernels on a weight eight times as tall (N = 114688, K = 4096; 235 MB int4,
    470 MB int8, and successive launches read different copies): one launch streams long enough that its start
    and end no longer weigh, so the rate it reaches is the kernels' streaming rate and the distance of the N = 14336 launches
    from it is what a launch's ramp and tail cost.
    `decode_down_proj`: the FFN down projection of the same model (N = 4096, K = 14336), M = 1 and 16."""
    out = {"decode_tall_M1": {}, "decode_down_proj": {}}
    x1 = torch.empty(1, K_DEC, device=dev).normal_(0, 1, generator=gen).to(torch.bfloat16)
    ws = torch.empty(4 << 20, dtype=torch.uint8, device=dev)      # the 16-row kernel's reduction slices at K = 14336: 1.8 MB
    N_TALL = 8 * N_DEC
    w = torch.empty(N_TALL, K_DEC, device=dev).normal_(0, 0.02, generator=gen)
    p4, s4 = T.quantize_int4_per_group(w, 128)
    q8, s8 = T.quantize_int8(w.reshape(K_DEC, N_TALL), per_channel=True)
    del w
    y = torch.empty(1, N_TALL, device=dev)
    # each launch reads a different copy, and the copies together exceed 512 MB, so none of it comes from cache
    tall = (("int4", [T.FrozenWeight(p4.clone() if i else p4, T.W_INT4_GROUP, s4, N_TALL, K_DEC, 1, 128)
                      for i in range(3)]),
            ("int8", [T.FrozenWeight(q8.reshape(-1).clone() if i else q8.reshape(-1), T.W_INT8, s8, N_TALL, K_DEC,
                                     N_TALL) for i in range(2)]))
    for kind, fws in tall:
        g = capture(lambda i, fws=fws: T.qlinear_forward(x1, fws[i % len(fws)], T.BF16, T.F32, out=y, workspace=ws),
                    12)
        ms = time_graph(g, 12)
        del g
        nbytes = algorithmic_bytes(kind, 1, N=N_TALL)
        out["decode_tall_M1"][kind] = {"N": N_TALL, "copies_rotated": len(fws), "us": round(ms * 1e3, 2),
                                       "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                                       "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    # yardstick, not part of the path: what kernels that are not this library's read per second from the same
    # rotated buffers (each launch a different 470 MB copy, so nothing comes from cache): the runtime's device-to-device
    # copy, half reads, half writes (torch's reductions run far below the memory rate and say nothing here)
    try:
        bufs = [fw.wq for fw in tall[1][1]]
        nb = bufs[0].numel()
        sink = torch.empty(nb, dtype=torch.int8, device=dev)

        def timed(fn, n=6):
            fn(0)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(n):
                fn(i)
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / n

        ms_cpy = timed(lambda i: sink.copy_(bufs[i % len(bufs)]))
        out["hbm_stream_yardstick_GBps"] = {"bytes": nb, "device_copy_read_plus_write": round(2 * nb / (ms_cpy * 1e-3) / 1e9, 1)}
        del bufs, sink
    except Exception as e:   # a yardstick must not take the rows down
        out["hbm_stream_yardstick_GBps"] = None
        print(f"bench: HBM stream yardstick skipped: {type(e).__name__}: {e}", file=sys.stderr)
    del tall, fws
    del p4, s4, q8, s8, y
    N, K = 4096, 14336
    copies = 10                                  # 10 x 59 MB (int8) / 20 x 30 MB (int4) > 512 MB: HBM, not cache
    w = torch.empty(N, K, device=dev).normal_(0, 0.02, generator=gen)
    p4, s4 = T.quantize_int4_per_group(w, 128)
    q8, s8 = T.quantize_int8(w.reshape(K, N), per_channel=True)
    del w
    W4 = [T.FrozenWeight(p4.clone(), T.W_INT4_GROUP, s4, N, K, 1, 128) for _ in range(2 * copies)]
    W8 = [T.FrozenWeight(q8.reshape(-1).clone(), T.W_INT8, s8, N, K, N) for _ in range(copies)]
    for m in (1, 16):
        x = torch.empty(m, K, device=dev).normal_(0, 1, generator=gen).to(torch.bfloat16)
        y = torch.empty(m, N, device=dev)
        for kind, Ws in (("int4", W4), ("int8", W8)):
            g = capture(lambda i, Ws=Ws: T.qlinear_forward(x, Ws[i % len(Ws)], T.BF16, T.F32, out=y, workspace=ws), 40)
            ms = time_graph(g, 40)
            del g
            nbytes = algorithmic_bytes(kind, m, N=N, K=K)
            out["decode_down_proj"][f"{kind}_M{m}_N{N}_K{K}"] = {
                "us": round(ms * 1e3, 2), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    # the input gradient with 16 rows through the same down-projection weights (dY [16, 4096] -> dX [16, 14336]):
    # one pass over the weight on the fp32 matrix core, its row ranges meeting in the workspace
    from caif_amd import capi
    out["few_row_input_gradient"] = {}
    dy = torch.empty(16, N, device=dev).normal_(0, 1e-3, generator=gen).to(torch.bfloat16)
    dx = torch.empty(16, K, device=dev)
    for kind, Ws, wk in (("int4", W4, T.W_INT4_GROUP), ("int8", W8, T.W_INT8)):
        nb = capi.lib().caifx_qlinear_workspace_bytes(16, N, K, T.BF16, T.BF16, wk, 1)
        wsb = torch.empty(max(nb, 1), dtype=torch.uint8, device=dev)
        g = capture(lambda i, Ws=Ws: T.qlinear_backward_input(dy, Ws[i % len(Ws)], T.BF16, T.F32, out=dx, workspace=wsb), 40)
        ms = time_graph(g, 40)
        del g
        nbytes = algorithmic_bytes(kind, 16, N=N, K=K)      # the same weight, 16 rows in, 16 rows out
        out["few_row_input_gradient"][f"{kind}_M16_N{N}_K{K}"] = {
            "us": round(ms * 1e3, 2), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    return out


def quantise_rows(torch, T, dev, gen):
    """The quantise / pack ops on the decode weight (fp32 [4096, 14336], 235 MB): eager calls timed with HIP
    events, the input rotating over three copies.  Bytes counted: one read of the input plus the codes and scales
    written; the int8 schemes need the maxima before the first code, so a second read of the input is part of
    their cost and shows as a lower fraction (their second pass walks the rows backwards, so the part of the
    input the first pass read last is still in the Infinity Cache)."""
    rows, cols = K_DEC, N_DEC
    # three copies taken in turn (705 MB): a call does not find its input in the 256 MB Infinity Cache
    ws = [torch.empty(rows, cols, device=dev).normal_(0, 0.02, generator=gen) for _ in range(3)]
    turn = [0]

    def w():
        turn[0] = (turn[0] + 1) % len(ws)
        return ws[turn[0]]

    n = rows * cols
    out = {}

    def timed(fn, iters=10):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        ts = []
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                fn()
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1) / iters)
        return sorted(ts)[1]

    for name, fn, nbytes in (
            ("int8_per_channel_4096x14336", lambda: T.quantize_int8(w(), per_channel=True), n * 4 + n + cols * 4),
            ("int8_per_tensor_4096x14336", lambda: T.quantize_int8(w(), per_channel=False), n * 4 + n + 4),
            ("int4_group128_4096x14336", lambda: T.quantize_int4_per_group(w(), 128), n * 4 + n // 2 + n // 128 * 2)):
        ms = timed(fn)
        out[name] = {"us": round(ms * 1e3, 1), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                     "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    # the dequantisers (checkpoint export path): codes + scales in, fp32 out
    q8, s8 = T.quantize_int8(ws[0], per_channel=True)
    p4, s4 = T.quantize_int4_per_group(ws[0], 128)
    for name, fn, nbytes in (
            ("dequant_int8_per_channel_4096x14336", lambda: T.dequantize_int8(q8, s8, per_channel=True), n + cols * 4 + n * 4),
            ("dequant_int4_group128_4096x14336", lambda: T.dequantize_int4_per_group(p4, s4, n, 128),
             n // 2 + n // 128 * 2 + n * 4)):
        ms = timed(fn)
        out[name] = {"us": round(ms * 1e3, 1), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                     "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    return {"quantise_ops": out}


def compute_bound_rows(torch, T, dev, gen, capture, time_graph):
    """configs[2] and configs[3]: int4 g128 dequant-GEMM forward (+ dX) in TFLOP/s."""
    rows = {}
    L = 8
    for (M, N, K, with_dx) in ((2048, 4096, 4096, True), (2048, 11008, 4096, True), (4096, 11008, 4096, True)):
        w = torch.empty(N, K, device=dev).normal_(0, 0.02, generator=gen)
        p, s = T.quantize_int4_per_group(w, 128)
        del w
        fw = T.FrozenWeight(p, T.W_INT4_GROUP, s, N, K, 1, 128)
        x = torch.empty(M, K, device=dev).normal_(0, 1, generator=gen).to(torch.bfloat16)
        dy = torch.empty(M, N, device=dev).normal_(0, 1e-3, generator=gen).to(torch.bfloat16)
        y = torch.empty(M, N, device=dev)
        dx = torch.empty(M, K, device=dev)
        from caif_amd import capi
        nb = max(capi.lib().caifx_qlinear_workspace_bytes(M, N, K, T.BF16, T.BF16, T.W_INT4_GROUP, b) for b in (0, 1))
        ws = torch.empty(max(nb, 1), dtype=torch.uint8, device=dev)
        flops = 2.0 * M * N * K
        g = capture(lambda i: T.qlinear_forward(x, fw, T.BF16, T.F32, out=y, workspace=ws), L)
        ms_f = time_graph(g, L, reps=3)
        del g
        key = f"int4_M{M}_N{N}_K{K}"
        rows[key] = {"fwd_us": round(ms_f * 1e3, 2), "fwd_TFLOPs": round(flops / (ms_f * 1e-3) / 1e12, 1)}
        if with_dx:
            g = capture(lambda i: T.qlinear_backward_input(dy, fw, T.BF16, T.F32, out=dx, workspace=ws), L)
            ms_b = time_graph(g, L, reps=3)
            del g
            rows[key].update({"dx_us": round(ms_b * 1e3, 2), "dx_TFLOPs": round(flops / (ms_b * 1e-3) / 1e12, 1),
                              "fwd_dx_frac_of_mfma_peak":
                                  round(2 * flops / ((ms_f + ms_b) * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)})
        # yardstick, not part of the path: the vendor library's dense bf16 GEMM (torch.matmul) on the same shape with
        # the weight already dequantised, i.e. what the platform's own kernel reaches without any unpacking
        try:
            wd = torch.empty(N, K, device=dev).normal_(0, 0.02, generator=gen).to(torch.bfloat16)
            yd = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
            g = capture(lambda i: torch.matmul(x, wd.t(), out=yd), L)
            ms_v = time_graph(g, L, reps=3)
            del g, wd, yd
            rows[key]["vendor_dense_bf16_fwd_TFLOPs"] = round(flops / (ms_v * 1e-3) / 1e12, 1)
        except Exception as e:   # the yardstick must not take the row down
            rows[key]["vendor_dense_bf16_fwd_TFLOPs"] = None
            print(f"bench: vendor GEMM yardstick skipped: {type(e).__name__}: {e}", file=sys.stderr)
        # second yardstick: the matrix pipes alone (no loads, stores or unpacking) on this row's own values.  Their
        # clock follows the power the operand bit patterns draw, so this, not the published peak, is what a kernel
        # that did everything else for free would reach on N(0,1) activations and N(0,0.02) weights
        try:
            wvals = torch.empty(16384, device=dev).normal_(0, 0.02, generator=gen)
            iters = 600
            fl, keep = T.probe_mfma_bf16(x, wvals, iters)         # untimed: clocks settle
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(3):
                fl, keep = T.probe_mfma_bf16(x, wvals, iters)
            e1.record()
            torch.cuda.synchronize()
            pipes = 3 * fl / (e0.elapsed_time(e1) * 1e-3) / 1e12
            rows[key]["mfma_pipes_alone_on_these_values_TFLOPs"] = round(pipes, 1)
            rows[key]["fwd_frac_of_pipes_alone"] = round(rows[key]["fwd_TFLOPs"] / pipes, 4)
            del keep, wvals
        except Exception as e:
            rows[key]["mfma_pipes_alone_on_these_values_TFLOPs"] = None
            print(f"bench: matrix-pipe yardstick skipped: {type(e).__name__}: {e}", file=sys.stderr)
        if (M, N) == (4096, 11008):
            # configs[3]: what the LoRA adapter does with the frozen base around its own small GEMMs: the base
            # output cast to bf16 and added to the low-rank branch, forward and backward.  "chain" is the
            # reference's sequence (fp32 result, cast, Add); "fused" folds cast and Add into the GEMM's store.
            lora_y = torch.empty(M, N, device=dev).normal_(0, 1e-2, generator=gen).to(torch.bfloat16)
            lora_x = torch.empty(M, K, device=dev).normal_(0, 1e-4, generator=gen).to(torch.bfloat16)
            yb = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
            xb = torch.empty(M, K, device=dev, dtype=torch.bfloat16)

            def chain(i):
                T.qlinear_forward(x, fw, T.BF16, T.F32, out=y, workspace=ws)
                T.add(y.to(torch.bfloat16), lora_y)
                T.qlinear_backward_input(dy, fw, T.BF16, T.F32, out=dx, workspace=ws)
                T.add(dx.to(torch.bfloat16), lora_x)

            def fused(i):
                T.qlinear_forward(x, fw, T.BF16, T.BF16, out=yb, workspace=ws, addend=lora_y)
                T.qlinear_backward_input(dy, fw, T.BF16, T.BF16, out=xb, workspace=ws, addend=lora_x)

            g = capture(chain, 4)
            ms_c = time_graph(g, 4, reps=3)
            del g
            g = capture(fused, 4)
            ms_u = time_graph(g, 4, reps=3)
            del g
            rows["lora_base_fwd_bwd_M4096_N11008_K4096"] = {
                "gemm_cast_add_chain_us": round(ms_c * 1e3, 1), "fused_store_us": round(ms_u * 1e3, 1)}
    # float-storage cell on the 16-bit matrix cores: weight stored in bf16, bf16 compute (what the reference's bf16
    # add-MoE runs, CHANGES.md:132-135), forward and input gradient, beside the vendor GEMM on the same operands
    try:
        M, N, K = 2048, 4096, 4096
        wd = torch.empty(N, K, device=dev).normal_(0, 0.02, generator=gen).to(torch.bfloat16)
        fw = T.FrozenWeight(wd.reshape(-1), T.W_BF16, None, N, K)
        x = torch.empty(M, K, device=dev).normal_(0, 1, generator=gen).to(torch.bfloat16)
        dy = torch.empty(M, N, device=dev).normal_(0, 1e-3, generator=gen).to(torch.bfloat16)
        y, dx = torch.empty(M, N, device=dev), torch.empty(M, K, device=dev)
        yv = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
        ws = torch.empty(1 << 20, dtype=torch.uint8, device=dev)
        flops = 2.0 * M * N * K
        g = capture(lambda i: T.qlinear_forward(x, fw, T.BF16, T.F32, out=y, workspace=ws), L)
        ms_f = time_graph(g, L, reps=3)
        del g
        g = capture(lambda i: T.qlinear_backward_input(dy, fw, T.BF16, T.F32, out=dx, workspace=ws), L)
        ms_b = time_graph(g, L, reps=3)
        del g
        g = capture(lambda i: torch.matmul(x, wd.t(), out=yv), L)
        ms_v = time_graph(g, L, reps=3)
        del g
        rows[f"bf16_storage_M{M}_N{N}_K{K}"] = {
            "fwd_us": round(ms_f * 1e3, 2), "fwd_TFLOPs": round(flops / (ms_f * 1e-3) / 1e12, 1),
            "dx_us": round(ms_b * 1e3, 2), "dx_TFLOPs": round(flops / (ms_b * 1e-3) / 1e12, 1),
            "vendor_dense_bf16_fwd_TFLOPs": round(flops / (ms_v * 1e-3) / 1e12, 1),
            "fwd_frac_of_vendor": round(ms_v / ms_f, 4)}
        del wd, fw, x, dy, y, dx, yv
    except Exception as e:
        rows["bf16_storage_error"] = repr(e)
    return {"prefill_gemm": rows, "few_tile_gemm": few_tile_rows(torch, T, dev, gen, capture, time_graph),
            "fp32_compute": fp32_rows(torch, T, dev, gen, capture, time_graph),
            "moe_frozen_experts": moe_rows(torch, T, dev, gen)}


def few_tile_rows(torch, T, dev, gen, capture, time_graph):
    """Between the decode regime and a full round of tiles (int4 g128, K = N = 4096, bf16): forward at M = 64 and
    128 and the input gradient at M = 64, with the workspace the library asks for (workgroups share each tile's
    reduction) and without one (plain launch)."""
    from caif_amd import capi
    N = K = 4096
    w = torch.empty(N, K, device=dev).normal_(0, 0.02, generator=gen)
    p, s = T.quantize_int4_per_group(w, 128)
    del w
    fw = T.FrozenWeight(p, T.W_INT4_GROUP, s, N, K, 1, 128)
    none = torch.empty(1, dtype=torch.uint8, device=dev)
    rows, L = {}, 16
    for M, backward in ((64, False), (128, False), (64, True)):
        src = torch.empty(M, N if backward else K, device=dev).normal_(0, 1, generator=gen).to(torch.bfloat16)
        dst = torch.empty(M, K if backward else N, device=dev)
        nb = capi.lib().caifx_qlinear_workspace_bytes(M, N, K, T.BF16, T.BF16, T.W_INT4_GROUP, int(backward))
        ws = torch.empty(max(nb, 1), dtype=torch.uint8, device=dev)
        fn = T.qlinear_backward_input if backward else T.qlinear_forward
        us = {}
        for name, buf in (("shared_reduction_us", ws), ("plain_us", none)):
            g = capture(lambda i, buf=buf: fn(src, fw, T.BF16, T.F32, out=dst, workspace=buf), L)
            us[name] = round(time_graph(g, L, reps=3) * 1e3, 2)
            del g
        rows[f"int4_{'dx' if backward else 'fwd'}_M{M}_N{N}_K{K}"] = us
    return rows


def fp32_rows(torch, T, dev, gen, capture, time_graph):
    """configs[0] on the GPU (int8 per-channel, K = N = 4096, fp32 X[16, 4096], fp32 compute: forward + dX) and
    the same layer at M = 2048, against the fp32 matrix-core peak."""
    N = K = 4096
    w = torch.empty(K, N, device=dev).normal_(0, 0.02, generator=gen)       # the reference's [in,out] labelling
    q, s = T.quantize_int8(w, per_channel=True)
    del w
    fw = T.FrozenWeight(q.reshape(-1), T.W_INT8, s, N, K, N)
    from caif_amd import capi
    rows = {}
    for M, L in ((16, 32), (2048, 8)):
        # the workspace the library asks for (few rows: partial sums of reduction slices / row ranges)
        nb = max(capi.lib().caifx_qlinear_workspace_bytes(M, N, K, T.F32, T.F32, T.W_INT8, b) for b in (0, 1))
        ws = torch.empty(max(nb, 1), dtype=torch.uint8, device=dev)
        x = torch.empty(M, K, device=dev).normal_(0, 1, generator=gen)
        dy = torch.empty(M, N, device=dev).normal_(0, 1e-3, generator=gen)
        y, dx = torch.empty(M, N, device=dev), torch.empty(M, K, device=dev)
        g = capture(lambda i: T.qlinear_forward(x, fw, T.F32, T.F32, out=y, workspace=ws), L)
        ms_f = time_graph(g, L, reps=3)
        del g
        g = capture(lambda i: T.qlinear_backward_input(dy, fw, T.F32, T.F32, out=dx, workspace=ws), L)
        ms_b = time_graph(g, L, reps=3)
        del g
        flops = 2.0 * M * N * K
        rows[f"int8_M{M}_N{N}_K{K}"] = {
            "fwd_us": round(ms_f * 1e3, 2), "dx_us": round(ms_b * 1e3, 2),
            "fwd_TFLOPs": round(flops / (ms_f * 1e-3) / 1e12, 2), "dx_TFLOPs": round(flops / (ms_b * 1e-3) / 1e12, 2),
            "fwd_dx_frac_of_fp32_mfma_peak": round(2 * flops / ((ms_f + ms_b) * 1e-3) / 1e12 / MFMA_FP32_PEAK_TFLOPS, 4)}
        if M == 16:
            # sixteen rows against a 16.8 MB weight: the weight stream bounds it, not the matrix pipes
            nbytes = N * K + N * 4 + M * K * 4 + M * N * 4
            rows[f"int8_M{M}_N{N}_K{K}"].update({
                "bound": "hbm", "algorithmic_bytes": nbytes,
                "fwd_frac_of_hbm_peak": round(nbytes / (ms_f * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                "dx_frac_of_hbm_peak": round(nbytes / (ms_b * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)})
    return rows


def moe_rows(torch, T, dev, gen):
    """configs[4]: 64 frozen SwiGLU experts (int8 per-channel, gate/up 2048->1408, down 1408->2048), 4096
    bf16 tokens, top-6 routing with uniform random expert ids: forward + backward dX as grouped
    dequant-GEMMs over the token-sorted buffer.  Eager launches timed with HIP events."""
    E, D, H, tokens, top_k = 64, 2048, 1408, 4096, 6

    def bank(n, k):
        ws = []
        for _ in range(E):
            w = torch.empty(k, n, device=dev).normal_(0, 0.02, generator=gen)     # the reference's [in,out] labelling
            q, s = T.quantize_int8(w, per_channel=True)
            ws.append(T.FrozenWeight(q.reshape(-1), T.W_INT8, s, n, k, n))
        return T.GroupedFrozenWeights(ws)

    gate, up, down = bank(H, D), bank(H, D), bank(D, H)
    ids = torch.randint(0, E, (tokens * top_k,), device=dev, generator=gen)
    counts = torch.bincount(ids, minlength=E)
    offsets = torch.zeros(E + 1, dtype=torch.int32, device=dev)
    offsets[1:] = torch.cumsum(counts, 0).to(torch.int32)
    rows = tokens * top_k
    x = torch.empty(rows, D, device=dev).normal_(0, 1, generator=gen).to(torch.bfloat16)
    gout = torch.empty(rows, D, device=dev).normal_(0, 1e-2, generator=gen).to(torch.bfloat16)
    bf = lambda r, c: torch.empty(r, c, dtype=torch.bfloat16, device=dev)
    up_o, gate_o, out, gh, gi_up, gi_gate = bf(rows, H), bf(rows, H), bf(rows, D), bf(rows, H), bf(rows, D), bf(rows, D)
    ws = torch.empty(1 << 20, dtype=torch.uint8, device=dev)
    state = {}

    hidden, grad_gate, grad_up = bf(rows, H), bf(rows, H), bf(rows, H)

    def fwd():
        T.qlinear_grouped_forward(x, offsets, up, T.BF16, T.BF16, out=up_o, workspace=ws)
        T.qlinear_grouped_forward(x, offsets, gate, T.BF16, T.BF16, out=gate_o, workspace=ws)
        T.silu_multiply(gate_o, up_o, out=hidden)
        T.qlinear_grouped_forward(hidden, offsets, down, T.BF16, T.BF16, out=out, workspace=ws)

    def bwd():
        T.qlinear_grouped_backward_input(gout, offsets, down, T.BF16, T.BF16, out=gh, workspace=ws)
        T.swiglu_backward(gate_o, up_o, gh, grad_gate, grad_up)
        T.qlinear_grouped_backward_input(grad_up, offsets, up, T.BF16, T.BF16, out=gi_up, workspace=ws)
        # gi_up + gi_gate folded into the second GEMM's store (same bits as the reference's Add)
        state["dx"] = T.qlinear_grouped_backward_input(grad_gate, offsets, gate, T.BF16, T.BF16, out=gi_gate,
                                                       workspace=ws, addend=gi_up)

    # the same two passes with the gating inside a GEMM's store (same bits, fewer launches and no grad_hidden
    # buffer; reported beside the separate launches, which are the faster form here)
    def fwd_gating_in_store():
        T.qlinear_grouped_forward(x, offsets, gate, T.BF16, T.BF16, out=gate_o, workspace=ws)
        T.qlinear_grouped_forward_swiglu(x, offsets, up, gate_o, T.BF16, out=(up_o, hidden))
        T.qlinear_grouped_forward(hidden, offsets, down, T.BF16, T.BF16, out=out, workspace=ws)

    def bwd_gating_in_store():
        T.qlinear_grouped_backward_input_swiglu(gout, offsets, down, gate_o, up_o, T.BF16, out=(grad_gate, grad_up))
        T.qlinear_grouped_backward_input(grad_up, offsets, up, T.BF16, T.BF16, out=gi_up, workspace=ws)
        T.qlinear_grouped_backward_input(grad_gate, offsets, gate, T.BF16, T.BF16, out=gi_gate, workspace=ws, addend=gi_up)

    def timed(fn, iters=10, reps=3):
        """Milliseconds per call: median of reps event-timed runs of iters eager calls, after iters untimed
        ones (the first few calls after the one-off quantisation above run at a lower clock)."""
        for _ in range(iters):
            fn()
        torch.cuda.synchronize()
        times = []
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                fn()
            e1.record()
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1) / iters)
        return sorted(times)[len(times) // 2]

    ms_f, ms_b = timed(fwd), timed(bwd)
    ms_f_fused, ms_b_fused = timed(fwd_gating_in_store), timed(bwd_gating_in_store)

    # Per-expert-segment GEMM efficiency (outside the timed runs): the grouped kernel stamps every 128 x 128 tile
    # with its expert, row count, start and end (100 MHz wall clock).  An expert's efficiency is the flops of its
    # segment over what the matrix pipes offer during its tiles' lifetimes, 2 cnt K N / (sum of tile durations x
    # peak / (256 compute units x the workgroups that share one)); partial last tiles and everything a tile waits
    # for count against it.
    def segment_efficiency(launch, n_cols, k_red):
        from caif_amd import capi
        tiles = ((rows + 127) // 128 + E) * ((n_cols + 127) // 128)
        stamps = torch.zeros(tiles * 4, dtype=torch.int64, device=dev)
        capi.call("caifx_qlinear_grouped_tile_stamps", stamps.data_ptr(), tiles)
        try:
            launch()
            torch.cuda.synchronize()
        finally:
            capi.call("caifx_qlinear_grouped_tile_stamps", None, 0)
        st = stamps.view(-1, 4).cpu()
        st = st[st[:, 3] > 0]
        cnt = counts.cpu()
        # word 1 of a stamp: rows of the tile, and from bit 32 up how many workgroups of the kernel that ran it
        # share a compute unit when that is not two (the int8 forward kernel runs one)
        resident = int(st[0, 1] >> 32) or 2
        share = MFMA_BF16_PEAK_TFLOPS * 1e12 / (256 * resident)
        effs = []
        for e in range(E):
            mine = st[st[:, 0] == e]
            if len(mine) == 0 or int(cnt[e]) == 0:
                continue
            busy_s = float((mine[:, 3] - mine[:, 2]).sum()) / 1e8
            effs.append(2.0 * int(cnt[e]) * n_cols * k_red / (busy_s * share))
        effs.sort()
        span_s = float(st[:, 3].max() - st[:, 2].min()) / 1e8
        return {"experts": len(effs), "tiles": int(len(st)), "workgroups_per_cu": resident, "min": round(effs[0], 4), "median": round(effs[len(effs) // 2], 4),
                "max": round(effs[-1], 4), "first_start_to_last_end_us": round(span_s * 1e6, 1)}

    try:
        seg = {"definition": "2*rows_e*K*N / (sum of the expert's tile durations * 2.5 PFLOP/s / (256 * workgroups_per_cu))",
               "gate_forward_2048_to_1408": segment_efficiency(
                   lambda: T.qlinear_grouped_forward(x, offsets, gate, T.BF16, T.BF16, out=gate_o, workspace=ws), H, D),
               "down_forward_1408_to_2048": segment_efficiency(
                   lambda: T.qlinear_grouped_forward(hidden, offsets, down, T.BF16, T.BF16, out=out, workspace=ws), D, H),
               "down_input_gradient": segment_efficiency(
                   lambda: T.qlinear_grouped_backward_input(gout, offsets, down, T.BF16, T.BF16, out=gh, workspace=ws), H, D),
               "gate_input_gradient": segment_efficiency(
                   lambda: T.qlinear_grouped_backward_input(grad_gate, offsets, gate, T.BF16, T.BF16, out=gi_gate,
                                                            workspace=ws), D, H)}
    except Exception as e:   # a diagnostic must not take the row down
        seg = {"error": repr(e)}
    # token routing around the experts (dispatch map, gather, weighted combine, and their backward passes),
    # on the same routing; HBM-bound row moves: algorithmic bytes = rows read + rows written
    idx2 = ids.reshape(tokens, top_k).to(torch.int32).contiguous()
    wts = torch.softmax(torch.empty(tokens, top_k, device=dev).normal_(0, 1, generator=gen), dim=1).to(torch.bfloat16)
    xt = torch.empty(tokens, D, device=dev).normal_(0, 1, generator=gen).to(torch.bfloat16)
    dmap, offs = T.moe_build_dispatch_map(idx2, E)
    packed, comb, gbuf, gin = bf(rows, D), bf(tokens, D), bf(rows, D), bf(tokens, D)
    row_b, tok_b = rows * D * 2, tokens * D * 2
    routing = {}
    for name, fn, nbytes in (
            ("build_dispatch_map", lambda: T.moe_build_dispatch_map(idx2, E), None),
            ("dispatch", lambda: T.moe_dispatch(xt, idx2, dmap, offs, rows, out=packed), tok_b + row_b),
            ("combine", lambda: T.moe_combine(out, idx2, wts, dmap, offs, out=comb), row_b + tok_b),
            ("combine_backward_grad_expert",
             lambda: T.moe_combine_backward_grad_expert(comb, idx2, wts, dmap, offs, rows, out=gbuf), tok_b + row_b),
            ("dispatch_backward", lambda: T.moe_dispatch_backward(gbuf, idx2, dmap, offs, out=gin), row_b + tok_b)):
        ms = timed(fn, iters=20)
        routing[name] = {"us": round(ms * 1e3, 2)}
        if nbytes:
            routing[name].update({"GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                                  "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)})
    routing_ms = sum(v["us"] for v in routing.values()) * 1e-3
    # decode: 16 tokens x top-6 = 96 rows over the same 64 experts (one to four rows each, some none): the gate
    # projection as one launch, memory bound on the touched experts' weights.  Two expert banks take turns so
    # that the 370 MB of both do not stay in the Infinity Cache.
    ids_d = torch.randint(0, E, (16 * top_k,), device=dev, generator=gen)
    counts_d = torch.bincount(ids_d, minlength=E)
    offs_d = torch.zeros(E + 1, dtype=torch.int32, device=dev)
    offs_d[1:] = torch.cumsum(counts_d, 0).to(torch.int32)
    xd = torch.empty(16 * top_k, D, device=dev).normal_(0, 1, generator=gen).to(torch.bfloat16)
    yd = torch.empty(16 * top_k, H, device=dev)
    banks = (gate, up)
    turn = [0]

    def decode_gate():
        turn[0] ^= 1
        T.qlinear_grouped_forward(xd, offs_d, banks[turn[0]], T.BF16, T.F32, out=yd, workspace=ws)

    ms_d = timed(decode_gate, iters=20)
    touched = int((counts_d > 0).sum())
    dec_bytes = touched * (D * H + H * 4) + 16 * top_k * (D * 2 + H * 4)
    decode = {"rows": 16 * top_k, "experts_touched": touched, "us": round(ms_d * 1e3, 2),
              "GBps": round(dec_bytes / (ms_d * 1e-3) / 1e9, 1),
              "frac_of_hbm_peak": round(dec_bytes / (ms_d * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    gemm_flops = 3 * 2.0 * rows * D * H
    return {"experts": E, "tokens": tokens, "top_k": top_k, "packed_rows": rows,
            "rows_per_expert_min_max": [int(counts.min()), int(counts.max())],
            "fwd_ms": round(ms_f, 4), "bwd_ms": round(ms_b, 4), "gating_in_gemm_store": {"fwd_ms": round(ms_f_fused, 4), "bwd_ms": round(ms_b_fused, 4)},
            "tokens_per_s_fwd_bwd": round(tokens / ((ms_f + ms_b) * 1e-3), 1),
            "routing": routing,
            "decode_gate_projection_16_tokens": decode,
            "tokens_per_s_fwd_bwd_with_routing": round(tokens / ((ms_f + ms_b + routing_ms) * 1e-3), 1),
            "grouped_gemm_TFLOPs_fwd": round(gemm_flops / (ms_f * 1e-3) / 1e12, 1),
            "grouped_gemm_TFLOPs_bwd": round(gemm_flops / (ms_b * 1e-3) / 1e12, 1),
            "per_expert_segment_gemm_efficiency": seg,
            "grouped_frac_of_mfma_peak": round(2 * gemm_flops / ((ms_f + ms_b) * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
            # the other bound of a pass: every expert weight (int8 codes + fp32 per-channel scales) streamed once
            "weight_bytes_per_pass": int(3 * E * D * H + E * (2 * H + D) * 4),
            "weight_stream_us_at_hbm_peak": round((3 * E * D * H + E * (2 * H + D) * 4) / (HBM_PEAK_GBS * 1e9) * 1e6, 1),
            "mfma_us_at_peak_per_pass": round(gemm_flops / (MFMA_BF16_PEAK_TFLOPS * 1e12) * 1e6, 1)}


def cpu_baseline(np, q8, s8, p4, s4_bits, x_values):
    """The reference's Host_e path for this layer is cblas_sgemm on an fp32 weight
    (src/caif_ops_host.cpp:112-139); it has no host dequantiser, so the timed CPU job is the
    oracle's OpenMP dequantise-to-fp32 followed by that sgemm (numpy's bundled OpenBLAS), on the
    same M=1 workload.  Bounded: at most ~20 s of CPU work."""
    from oracle import oracle as orc
    orc.build()
    omp_threads, blas_threads = cpu_threads(orc)
    cores = max(omp_threads, blas_threads)
    x = np.ascontiguousarray(x_values, np.float32)
    reps, t_deq, t_gemm = 0, 0.0, 0.0
    t_start = time.perf_counter()
    while reps < 20 and time.perf_counter() - t_start < 15.0:
        t0 = time.perf_counter()
        w4 = orc.frozen_weight_compute(p4, orc.W_INT4_GROUP, s4_bits, N_DEC, K_DEC, 1, 128, orc.F32)
        w8 = orc.frozen_weight_compute(q8, orc.W_INT8, s8, N_DEC, K_DEC, N_DEC, 128, orc.F32)
        t1 = time.perf_counter()
        y4 = x @ w4.T                              # cblas_sgemm(NoTrans, Trans, M, N, K)
        y8 = x @ w8.T
        t2 = time.perf_counter()
        t_deq += t1 - t0
        t_gemm += t2 - t1
        reps += 1
    del y4, y8
    step_bytes = algorithmic_bytes("int4", 1) + algorithmic_bytes("int8", 1)
    per_step = (t_deq + t_gemm) / reps
    return {
        "value": round(step_bytes / per_step / 1e9, 3),
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{reps} full steps of the same M=1 workload (int4 + int8, K=4096, N=14336): oracle OpenMP "
                  f"dequantise-to-fp32 ({t_deq / reps * 1e3:.1f} ms/step, {omp_threads} OpenMP threads) + "
                  f"numpy/OpenBLAS sgemm ({t_gemm / reps * 1e3:.1f} ms/step, {blas_threads} OpenBLAS threads)",
        "ms_per_step": round(per_step * 1e3, 3),
    }


def cpu_threads(orc):
    """(OpenMP threads of the oracle's loops, threads of numpy's BLAS) as the libraries themselves report them."""
    blas = 1
    try:
        from threadpoolctl import threadpool_info
        blas = max([p.get("num_threads", 1) for p in threadpool_info() if p.get("user_api") == "blas"] or [1])
    except Exception:
        pass
    return orc.max_threads(), blas


def cpu_configs0(np):
    """BASELINE configs[0] on the host cores: the reference's Host_e path is cblas_sgemm on an fp32 weight
    (src/caif_ops_host.cpp:54-139), forward (NoTrans, Trans) and input gradient (NoTrans, NoTrans); the weight is
    the oracle's dequantised int8 per-channel weight (dequantisation timed separately, the reference has no host
    dequantiser).  K = N = 4096, fp32 X[16, 4096] ~ N(0,1), dY ~ N(0, 1e-3)."""
    from oracle import oracle as orc
    orc.build()
    rng = np.random.default_rng(7)
    N = K = 4096
    w = rng.normal(0, 0.02, (K, N)).astype(np.float32)
    q, s = orc.quantize_int8_per_channel(w)
    x = rng.normal(0, 1, (16, K)).astype(np.float32)
    dy = rng.normal(0, 1e-3, (16, N)).astype(np.float32)
    t0 = time.perf_counter()
    wf = orc.frozen_weight_compute(q.reshape(-1), orc.W_INT8, s, N, K, N, 128, orc.F32)
    t_deq = time.perf_counter() - t0
    fwd, bwd = [], []
    for _ in range(7):
        t0 = time.perf_counter()
        y = x @ wf.T
        t1 = time.perf_counter()
        dx = dy @ wf
        t2 = time.perf_counter()
        fwd.append(t1 - t0)
        bwd.append(t2 - t1)
    del y, dx
    omp_threads, blas_threads = cpu_threads(orc)
    return {"workload": "int8 per-channel K=N=4096, fp32 X[16,4096]: sgemm forward + input gradient on the dequantised weight",
            "dequantise_ms": round(t_deq * 1e3, 2), "sgemm_fwd_ms": round(sorted(fwd)[3] * 1e3, 3),
            "sgemm_dx_ms": round(sorted(bwd)[3] * 1e3, 3), "openmp_threads": omp_threads, "openblas_threads": blas_threads}


if __name__ == "__main__":
    main()
