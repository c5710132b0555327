#!/usr/bin/env python3
"""Benchmark of the ternary-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

The workload is the benchmark's config 2, the decode GEMV: x fp16 [1,4096] times packed ternary
W [4096,4096] (per-tensor fp32 scale, fp16 bias).  One such GEMV moves 4 MiB, which the memory system
delivers in less time than a kernel takes to start and drain, so the library serves decode work through
`bt_ternary_gemv_grouped`: G independent GEMV units (own activations, weights, scale, bias, output) per
launch, every unit bit-identical to the single call.  One "step" is one such launch over G = 128 config-2
units; two sets of 128 weight matrices (2 x 512 MiB, four times the 256 MB Infinity Cache) alternate, so
every step streams its packed weights from HBM.  W warm-up steps, then exactly K steps (captured in one HIP
graph so that host launch overhead is not what is measured) are timed between two device synchronisations;
the graph is replayed several times and the median replay is reported.  Prints ONE JSON line.

The same line carries the roofline of the dominant kernel (HIP-event timed over the timed region), the same
GEMV one matrix per launch (`single_launch`), the CPU oracle timed on the host cores beside it, and the
secondary figures of the metric (int8 TOPS at M=2048, small-batch decode, large matrices, quantize+pack).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E
INT8_PEAK_TOPS = 5000.0     # MI355X dense int8 MFMA
BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16 / fp16 MFMA
METRIC = "packed ternary GEMM GB/s (M=1) & int8 TOPS (M=2048), % of roofline, 1 GPU"


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--units", type=int, default=128, help="config-2 GEMV units per launch (G)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary shapes")
    ap.add_argument("--no-block-stack", action="store_true", help="skip the 30-layer block stack (config 5)")
    ap.add_argument("--block-stack-only", type=int, default=0, metavar="LAYERS",
                    help="no GEMV timing: run the config-5 block stack with this many layers and print its "
                         "timings (the workload of profiles/block_stack_kernel_trace.txt)")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="CPU baseline sample length")
    ap.add_argument("--pmc-pass", action="store_true",
                    help="no timing: a few eager launches of each kernel plus a plain copy of known size, "
                         "for one `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` run")
    return ap.parse_args()


def graph_time(fn, steps, warmup, torch, min_replays=None):
    """(wall ms, event ms) for `steps` calls of fn(i) replayed as one HIP graph: the median over
    the timed replays, each between two synchronisations.  A graph of fewer than 200 steps is timed
    in runs of back-to-back replays that hold at least 200 steps together (the time of a run divided
    by its replays: the fixed cost of starting a replay, some 0.1 ms, then hides behind the replay
    before it as it does inside a long graph), and in 20 such runs instead of 5, so that neither
    that cost nor a clock ramp decides the figure."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(warmup):
            fn(i)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(steps):
            fn(i)
    graph.replay()  # untimed: first replay uploads the graph
    torch.cuda.synchronize()
    replays = min_replays or (5 if steps >= 200 else 20)
    in_a_row = 1 if steps >= 200 else -(-200 // steps)
    walls, events = [], []
    for _ in range(replays):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        for _ in range(in_a_row):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        walls.append((time.perf_counter() - t0) * 1e3 / in_a_row)
        events.append(e0.elapsed_time(e1) / in_a_row)
    walls.sort()
    events.sort()
    return walls[len(walls) // 2], events[len(events) // 2]


_probe_lib = None


def probe_grid_handover(torch, device):
    """Microseconds per grid-wide hand-over of an n-entry vector between persistent workgroups (bench_mfma_probe.so):
    what ONE stage boundary of a chain of dependent GEMVs inside one launch would cost, against the launch it would
    replace.  Per variant the time of 220 rounds minus that of 20, over 200 (best of 5), with the number of entries
    that arrived wrong and whether a bounded wait gave up (both must be 0)."""
    import ctypes
    global _probe_lib
    if _probe_lib is None:
        _probe_lib = ctypes.CDLL(os.path.join(ROOT, "bench_mfma_probe.so"))
    fn = _probe_lib.bench_probe_grid_handover
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_int] * 4 + [ctypes.c_void_p] * 5 + [ctypes.c_int, ctypes.c_void_p]
    st = torch.cuda.current_stream(device).cuda_stream
    res = {}
    for name, mode, n in (("barrier_only", 2, 2560), ("barrier_then_read_2560", 0, 2560), ("barrier_then_read_6912", 0, 6912),
                          ("poll_tagged_data_2560", 1, 2560), ("poll_tagged_data_6912", 1, 6912)):
        for wgs in (256, 512):
            ctr = torch.zeros(1, dtype=torch.int32, device=device)
            xcd = torch.zeros(256, dtype=torch.int32, device=device)
            data = torch.zeros(222 * n, dtype=torch.int32, device=device)
            status = torch.zeros(1, dtype=torch.int32, device=device)
            check = torch.zeros(1, dtype=torch.int32, device=device)
            times, wrong, gave_up = {}, 0, 0
            for rounds in (20, 220):
                best = None
                for _ in range(5):
                    for t in (ctr, xcd, data, status, check):
                        t.zero_()
                    torch.cuda.synchronize()
                    e0 = torch.cuda.Event(enable_timing=True)
                    e1 = torch.cuda.Event(enable_timing=True)
                    e0.record()
                    assert fn(mode, wgs, rounds, n, ctr.data_ptr(), xcd.data_ptr(), data.data_ptr(), status.data_ptr(),
                              check.data_ptr(), 1 << 20, st) == 0
                    e1.record()
                    torch.cuda.synchronize()
                    t_ms = e0.elapsed_time(e1)
                    best = t_ms if best is None else min(best, t_ms)
                    wrong += int(check[0])
                    gave_up |= int(status[0])
                times[rounds] = best
            res[f"{name}_{wgs}_workgroups"] = {"us": round((times[220] - times[20]) * 1e3 / 200, 2), "wrong_entries": wrong,
                                              "gave_up_in_round": gave_up}
    return res


def probe_mfma_int8(torch, device, blocks=2048, iters=4096, random_operands=0, return_clock=False):
    """Launches the int8 matrix-core rate probe (bench_mfma_probe.so, this benchmark's own aid) on the
    current stream; returns the number of integer operations the launch performs."""
    import ctypes
    global _probe_lib
    if _probe_lib is None:
        _probe_lib = ctypes.CDLL(os.path.join(ROOT, "bench_mfma_probe.so"))
        _probe_lib.bench_probe_mfma_i8.restype = ctypes.c_int
        _probe_lib.bench_probe_mfma_i8.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                                   ctypes.c_void_p, ctypes.c_void_p]
    out = torch.zeros(8, dtype=torch.int32, device=device)
    ops = ctypes.c_double(0.0)
    rc = _probe_lib.bench_probe_mfma_i8(blocks, iters, int(random_operands), out.data_ptr(), ctypes.addressof(ops),
                                        torch.cuda.current_stream(device).cuda_stream)
    assert rc == 0
    if return_clock:  # (synchronizes) shader-clock cycles per 100 MHz tick of workgroup 0's loop, in MHz
        cyc, ticks = int(out[2]), int(out[3])
        return ops.value, (100.0 * cyc / ticks if ticks > 0 else None)
    return ops.value


def probe_hbm_read(torch, device, nbytes=512 << 20):
    """GB/s of the benchmark's read-only probe kernel (bench_mfma_probe.so) over `nbytes` of device memory, for its
    three address patterns; each figure the median of 5 timed runs of 4 launches."""
    import ctypes
    global _probe_lib
    if _probe_lib is None:
        _probe_lib = ctypes.CDLL(os.path.join(ROOT, "bench_mfma_probe.so"))
    fn = _probe_lib.bench_probe_hbm_read
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    buf = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=device)
    out = torch.zeros(8, dtype=torch.int32, device=device)
    st = torch.cuda.current_stream(device).cuda_stream
    res = {}
    for name, pattern in (("grid_stride", 0), ("contiguous_per_workgroup", 1), ("contiguous_per_workgroup_nontemporal", 2)):
        assert fn(buf.data_ptr(), nbytes, pattern, out.data_ptr(), st) == 0  # warm
        torch.cuda.synchronize()
        ts = []
        for _ in range(5):
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(4):
                fn(buf.data_ptr(), nbytes, pattern, out.data_ptr(), st)
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1) / 4)
        ts.sort()
        res[name] = round(nbytes / (ts[2] * 1e-3) / 1e9, 1)
    del buf
    return res


def block_stack(torch, dev, layers=30, d_model=2560, heads=20, ffn=6912, batch=8, seq=512, vocab=32000):
    """Config 5 timed end to end in every variant (outputs are compared by tests/test_gpu_configs.py)."""
    from bittorch_amd.utils.block_stack import BlockStack
    c5 = BlockStack(dev, layers, d_model, heads, ffn, batch, seq, vocab)

    def timed(fn, reps, before=None):
        fn()
        torch.cuda.synchronize()
        best = 1e30
        for _ in range(reps):
            if before:
                before()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            best = min(best, (time.perf_counter() - t0) * 1e3)
        return best

    res = {"layers": layers, "d_model": d_model, "heads": heads, "ffn": ffn, "tokens": batch * seq,
           "ternary_weights": c5.n_tern,
           "ops_per_forward_ternary_layers": 2.0 * batch * seq * c5.n_tern}
    res["ms_requantize_every_forward"] = round(timed(c5.forward, 3, c5.drop_packed_caches), 3)   # what the reference does
    res["ms_packed_weights_cached"] = round(timed(c5.forward, 5), 3)
    infer = c5.convert()
    res["ms_inference_modules"] = round(timed(lambda: c5.forward(infer), 5), 3)
    c5.fuse()
    res["ms_inference_fused_glue"] = round(timed(lambda: c5.forward_fused(False), 5), 3)
    res["ms_inference_int8_path"] = round(timed(lambda: c5.forward_fused(True), 5), 3)
    c5.prepare_prefill(True)   # the opt-in second weight copy (field layout) under every int8 GEMM
    res["ms_inference_int8_path_prefill_copies"] = round(timed(lambda: c5.forward_fused(True), 5), 3)
    c5.prepare_prefill(False)
    res["ternary_TOPS_int8_path"] = round(res["ops_per_forward_ternary_layers"] / (res["ms_inference_int8_path"] * 1e-3) / 1e12, 1)
    res["ternary_TFLOPS_cached"] = round(res["ops_per_forward_ternary_layers"] / (res["ms_packed_weights_cached"] * 1e-3) / 1e12, 1)
    res["packed_weight_bytes"] = c5.n_tern // 4
    del c5, infer
    torch.cuda.empty_cache()
    return res


def measured_traffic(tag):
    """HBM bytes per launch from the committed hardware-counter summary (rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE runs of `--pmc-pass`, scaled by a copy kernel of known size);
    None if the summary is not there."""
    path = os.path.join(ROOT, "profiles", "pmc_hbm_traffic.txt")
    try:
        with open(path) as fh:
            for line in fh:
                if line.startswith("traffic_bytes_per_launch " + tag + ":"):
                    return int(line.split(":")[1])
    except OSError:
        pass
    return None


def pmc_pass(torch, _C, dev, gemv_steps, grouped_step):
    """Eager launches for hardware-counter collection (every dispatch gets its own counter row).
    The copy kernel moves a known number of bytes, which calibrates the counter's unit."""
    n_copy = 64 * 1024 * 1024 // 4
    src = torch.randn(n_copy, device=dev)
    dst = torch.empty_like(src)
    for _ in range(5):
        torch.mul(src, 1.0, out=dst)  # elementwise kernel: reads 64 MiB, writes 64 MiB
    for i in range(6):  # the headline: G config-2 units per launch
        grouped_step(i)
    for gemv_step in gemv_steps:  # one matrix per launch: the decode-tiled path, then the same GEMV on the row-major W_T
        for i in range(40):
            gemv_step(i)
    m, n, k = 2048, 4096, 4096
    c = torch.randint(0, 3, (4, k // 4, n), device=dev, dtype=torch.uint8)
    w = (c[0] | (c[1] << 2) | (c[2] << 4) | (c[3] << 6)).contiguous()
    xa = torch.randn(m, k, device=dev).bfloat16()
    sc = torch.rand(n, device=dev) * 0.05 + 0.01
    for _ in range(5):
        q, s = _C.act_quant_int8(xa)
        _C.ternary_gemm_int8(q, s, w, sc, None, k, out_dtype=torch.bfloat16)
    wt = _C.retile_weights(w, k)  # the benchmarked variant: tiled weights, operand-order activations
    for _ in range(5):
        q, s = _C.act_quant_int8(xa, True)
        _C.ternary_gemm_int8_tiled(q, s, wt, sc, None, k, n, torch.bfloat16, False, None, True)
    master = torch.randn(n, k, device=dev) * 0.02
    for _ in range(5):
        _C.ternary_quantize_pack(master, 0.05, True)
    # config 3 as 32 units of 16 int8 rows per launch (bt_ternary_gemm_i8_grouped), 16 x 4096 -> 11008
    g8, n3, k3 = 32, 11008, 4096
    tl = []
    for _ in range(g8):
        c = torch.randint(0, 3, (4, k3 // 4, n3), device=dev, dtype=torch.uint8)
        tl.append(_C.retile_weights((c[0] | (c[1] << 2) | (c[2] << 4) | (c[3] << 6)).contiguous(), k3))
    sc3 = torch.rand(n3, device=dev) * 0.05 + 0.01
    qs = [_C.act_quant_int8(torch.randn(16, k3, device=dev).bfloat16(), True) for _ in range(g8)]
    ys = [torch.empty(16, n3, dtype=torch.bfloat16, device=dev) for _ in range(g8)]
    tabs = (_C.pointer_table([q_ for q_, _ in qs]), _C.pointer_table([s_ for _, s_ in qs]), _C.pointer_table(tl),
            _C.pointer_table([sc3] * g8), None, _C.pointer_table(ys))
    for _ in range(5):
        _C.ternary_gemm_int8_grouped(*tabs, 16, k3, n3, out_dtype=torch.bfloat16, q_operand_order=True)
    torch.cuda.synchronize()
    print(json.dumps({"pmc_pass": "done", "copy_bytes_read": n_copy * 4, "copy_bytes_written": n_copy * 4,
                      "copy_kernel": "at::native vectorized elementwise (mul by scalar)"}))


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU's throughput; --gpus {args.gpus} is not supported "
              "(this path has no multi-GPU part: it shards by output columns without collectives)",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from bittorch_amd import _C  # ImportError if the HIP library is not built
    from bittorch_amd._lib import set_option

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    torch.manual_seed(0)

    if args.block_stack_only:
        print(json.dumps({"block_stack": block_stack(torch, dev, layers=args.block_stack_only)}))
        return

    # ---- config 2: decode GEMV units -------------------------------------------------------
    N = K = 4096
    weight_bytes = N * (K // 4)
    G = args.units
    nsets = 2 * G  # two alternating sets of G units: 2 x 512 MiB of packed weights at G = 128 (Infinity Cache: 256 MB)
    g = torch.Generator().manual_seed(0)
    w0 = (torch.randn(N, K, generator=g) * 0.02).to(dev)
    x = torch.randn(1, K, generator=g).half().to(dev)
    bias = (torch.randn(N, generator=g) * 0.01).half().to(dev)
    packed0, scale0, _ = _C.ternary_quantize_pack(w0, 0.05, per_channel=False)
    scale = scale0.reshape(1).float()
    zero_frac = float((_C.unpack_dequant(packed0, K, out_dtype=torch.int8) == 0).float().mean())
    packs = [packed0]
    for _ in range(nsets - 1):
        wi = torch.randn(N, K, device=dev) * 0.02
        packs.append(_C.ternary_quantize_pack(wi, 0.05, per_channel=False)[0])
    del wi
    torch.cuda.synchronize()

    # The product's decode path: TernaryLinearInference layers over the packed weights, each reading the
    # decode-tiled copy of its W_T.  Every unit has its own activations, bias and output.
    from bittorch_amd.nn import TernaryLinearInference
    import bittorch_amd as bt
    x_all = torch.cat([x] + [torch.randn(1, K, device=dev).half() for _ in range(nsets - 1)])  # [nsets, K], row u for unit u
    y_all = torch.empty(nsets, N, dtype=torch.float16, device=dev)
    xs = [x_all[u:u + 1] for u in range(nsets)]
    ys = [y_all[u:u + 1] for u in range(nsets)]
    biases = [bias] + [(torch.randn(N, device=dev) * 0.01).half() for _ in range(nsets - 1)]
    layers = [TernaryLinearInference(K, N, p, scale, b).prepare_decode() for p, b in zip(packs, biases)]
    tables = []
    for s0 in (0, G):
        sl = slice(s0, s0 + G)
        tables.append((_C.pointer_table(xs[sl]), _C.pointer_table([l.tiled_weights() for l in layers[sl]]),
                       _C.pointer_table([scale] * G), _C.pointer_table(biases[sl]), _C.pointer_table(ys[sl])))
    torch.cuda.synchronize()

    def step(i):  # one launch over G units, through the caller the kept API offers for it
        s0 = (i % 2) * G
        bt.ops.ternary_linear_grouped(layers[s0:s0 + G], x_all[s0:s0 + G], out=y_all[s0:s0 + G])

    def step_single(i):  # the same GEMV, one matrix per launch
        return layers[i % nsets](xs[i % nsets])

    def step_row_major(i):
        return _C.ternary_linear_packed_forward(xs[i % nsets], packs[i % nsets], scale, biases[i % nsets], K)

    # every unit of the grouped launch equals the single call bit for bit (checked here on the benchmark's own
    # operands; the parity tests proper are tests/test_gpu_gemv_exact.py)
    step(0)
    step(1)
    for u in (0, G - 1, G, nsets - 1):
        assert torch.equal(ys[u], step_single(u)), f"grouped unit {u} differs from the single call"

    if args.pmc_pass:
        pmc_pass(torch, _C, dev, (step_single, step_row_major), step)
        return
    wall_ms, ev_ms = graph_time(step, args.steps, args.warmup, torch)
    ms_per_step = wall_ms / args.steps
    kernel_us = ev_ms / args.steps * 1e3
    value = G * weight_bytes / (ms_per_step * 1e-3) / 1e9
    achieved = G * weight_bytes / (kernel_us * 1e-6) / 1e9
    single_steps = max(args.steps, 50) * 10
    _, ev_single = graph_time(step_single, single_steps, args.warmup * 10, torch)
    us_single = ev_single / single_steps * 1e3

    out = {
        "metric": METRIC,
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 x 2-bit ternary -> exact integer accumulate (int8 matrix cores), fp32 epilogue",
        "data": "synthetic (seed 0; N(0,0.02) master weights quantized with threshold 0.05, "
                f"{zero_frac * 100:.1f}% zeros; N(0,1) activations)",
        "config": {
            "workload": f"config 2 decode GEMV units: x fp16 [1,4096] x packed ternary W [4096,4096], per-tensor fp32 "
                        f"scale, fp16 bias; one step = one launch over {G} independent units (GROUPED STEADY STATE: the "
                        "70 % target is reached only here; the same GEMV one matrix per launch, which is what one "
                        "TernaryLinearInference.forward call gets, is the single_launch block of this line)",
            "path": "bittorch_amd.ops.ternary_linear_grouped over TernaryLinearInference layers' decode-tiled weight "
                    "copies (bt_ternary_gemv_grouped); every unit bit-identical to the single call (checked in this "
                    "run and by the GPU tests)",
            "M": 1, "N": N, "K": K,
            "units_per_step": G,
            "weight_sets": nsets,
            "weight_bytes_per_step": G * weight_bytes,
            "timing": "one HIP graph of all steps, median of the replays, each between two synchronisations",
        },
        "value_is": "grouped_steady_state_GBps",
        "headline": {
            "grouped_steady_state_GBps": round(value, 2),
            "grouped_steady_state_frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
            "single_launch_GBps": round(weight_bytes / (us_single * 1e-6) / 1e9, 1),
            "single_launch_frac_of_hbm_peak": round(weight_bytes / (us_single * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
            "note": f"value = {G} independent config-2 GEMVs per launch; a decode step of one sequence has 3-4 DEPENDENT "
                    "GEMVs per block, each a launch of its own at the single_launch rate (secondary."
                    "decode_token_per_block_bf16: microseconds per block)",
        },
        "roofline": {
            "kernel": "bt::gemv_planes_chunk_kernel (fp16 activations as six int8 digit rows, decode-tiled weights read front to back)",
            "bound": "hbm",
            "achieved": round(achieved, 2),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": measured_traffic("gemv_planes_chunk_kernel_G128_config2"),
            "launch_us": round(kernel_us, 3),
            "algorithmic_bytes_per_launch": G * weight_bytes,
        },
        "single_launch": {
            "note": "the same config-2 GEMV one matrix per launch (TernaryLinearInference.forward), a chain of launches "
                    "over the rotating weight sets: bounded by the launch, set-up and drain of a kernel, not by bytes",
            "kernel": "bt::gemv_planes_kernel",
            "launch_us": round(us_single, 3),
            "GBps": round(weight_bytes / (us_single * 1e-6) / 1e9, 1),
            "frac_of_hbm_peak": round(weight_bytes / (us_single * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
            "traffic": measured_traffic("gemv_planes_kernel_config2_tiled"),
            "algorithmic_bytes_per_launch": weight_bytes,
        },
    }

    # ---- secondary figures of the metric ------------------------------------------------
    if not args.no_extra:
        extra = {}

        _, ev_rm = graph_time(step_row_major, single_steps, args.warmup * 10, torch)
        us_rm = ev_rm / single_steps * 1e3
        extra["decode_gemv_row_major_W_T"] = {
            "us": round(us_rm, 3), "GBps": round(weight_bytes / (us_rm * 1e-6) / 1e9, 1),
            "frac_of_hbm_peak": round(weight_bytes / (us_rm * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
            "traffic": measured_traffic("gemv_planes_kernel_config2_row_major"),
            "note": "one matrix per launch through bittorch._C.ternary_linear_packed_forward on the reference-layout W_T [Kb, N]",
        }
        # units per launch: where the grouped launch leaves the launch-bound regime
        by_g = {}
        for gg in (1, 2, 4, 8, 16, 32, 64, 128):
            if gg > G:
                break
            tb = [tuple(t[:gg].contiguous() for t in tab) for tab in tables]
            reps = max(10, 2560 // gg // 4)
            _, ev_g = graph_time(lambda i: _C.ternary_gemv_grouped(*tb[i % 2], K, N, scale_len=1), reps, 5, torch)
            us_g = ev_g / reps * 1e3
            by_g[f"G{gg}"] = {"us_per_launch": round(us_g, 2), "GBps": round(gg * weight_bytes / (us_g * 1e-6) / 1e9, 1),
                              "frac_of_hbm_peak": round(gg * weight_bytes / (us_g * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)}
        if nsets >= 2 * G and G >= 64:
            # twice the headline's units in one launch (every weight set: 2 G x 4 MiB, four times the Infinity Cache at G = 128)
            g2 = 2 * G
            tb2 = (_C.pointer_table(xs[:g2]), _C.pointer_table([l.tiled_weights() for l in layers[:g2]]),
                   _C.pointer_table([scale] * g2), _C.pointer_table(biases[:g2]), _C.pointer_table(ys[:g2]))
            _, ev_g = graph_time(lambda i: _C.ternary_gemv_grouped(*tb2, K, N, scale_len=1), 20, 3, torch)
            us_g = ev_g / 20 * 1e3
            by_g[f"G{g2}"] = {"us_per_launch": round(us_g, 2), "GBps": round(g2 * weight_bytes / (us_g * 1e-6) / 1e9, 1),
                              "frac_of_hbm_peak": round(g2 * weight_bytes / (us_g * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)}
        extra["grouped_gemv_by_units_per_launch"] = by_g

        # the same launch on bf16 rows (each row scaled by its own largest exponent, summed as integers)
        xs_bf = [t.bfloat16() for t in xs[:2 * G]]
        bs_bf = [t.bfloat16() for t in biases[:2 * G]]
        ys_bf = [torch.empty(1, N, dtype=torch.bfloat16, device=dev) for _ in range(2 * G)]
        tb_bf = []
        for s0 in (0, G):
            sl = slice(s0, s0 + G)
            tb_bf.append((_C.pointer_table(xs_bf[sl]), tables[s0 // G][1], tables[s0 // G][2],
                          _C.pointer_table(bs_bf[sl]), _C.pointer_table(ys_bf[sl])))
        _, ev_bf = graph_time(lambda i: _C.ternary_gemv_grouped(*tb_bf[i % 2], K, N, scale_len=1,
                                                                bias_dtype=torch.bfloat16, x_dtype=torch.bfloat16),
                              args.steps, args.warmup, torch)
        us_bf = ev_bf / args.steps * 1e3
        extra["grouped_gemv_bf16_rows"] = {
            "us_per_launch": round(us_bf, 2), "GBps": round(G * weight_bytes / (us_bf * 1e-6) / 1e9, 1),
            "frac_of_hbm_peak": round(G * weight_bytes / (us_bf * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
            "note": f"G = {G} units per launch, bf16 rows, biases and outputs",
        }

        def rand_packed(n, k, count):
            outp = []
            for _ in range(count):
                c = torch.randint(0, 3, (4, (k + 3) // 4, n), device=dev, dtype=torch.uint8)
                outp.append((c[0] | (c[1] << 2) | (c[2] << 4) | (c[3] << 6)).contiguous())
            return outp

        def acts(m, k, outliers):
            a = torch.randn(m, k, device=dev)
            if outliers:
                a = torch.where(torch.rand(m, k, device=dev) < 0.001, a * 20, a)
            return a.bfloat16()

        # config 4: prefill, int8 activations on the matrix cores
        for (m, n, k) in ((2048, 4096, 4096), (2048, 11008, 4096)):
            ws = rand_packed(n, k, 2)
            xa = acts(m, k, True)
            sc = torch.rand(n, device=dev) * 0.05 + 0.01
            # the quantized activations in the layout the fused entry point uses (16-byte groups in
            # matrix-core operand order); the row-major variant is reported beside it
            q, s = _C.act_quant_int8(xa, operand_order=True)
            q_rm, _ = _C.act_quant_int8(xa)
            steps = 50
            # (the host leg before this leaves the GPU idle: bring the clocks back up before timing)
            for i in range(200):
                _C.ternary_gemm_int8(q_rm, s, ws[i % 2], sc, None, k, out_dtype=torch.bfloat16)
            torch.cuda.synchronize()
            _, ev = graph_time(lambda i: _C.ternary_gemm_int8(q, s, ws[i % 2], sc, None, k, out_dtype=torch.bfloat16,
                                                              q_operand_order=True), steps, 5, torch)
            _, ev_rm = graph_time(lambda i: _C.ternary_gemm_int8(q_rm, s, ws[i % 2], sc, None, k,
                                                                 out_dtype=torch.bfloat16), steps, 5, torch)
            ts = [_C.retile_weights(w, k) for w in ws]
            _, ev_tw = graph_time(lambda i: _C.ternary_gemm_int8_tiled(q, s, ts[i % 2], sc, None, k, n, torch.bfloat16,
                                                                       False, None, True), steps, 5, torch)
            # "quantizes activations to int8 on the fly": the quantizer's launch in the timed region, on the tiled copy
            # (what TernaryLinearInference pays from float activations) and through the reference's entry point
            def quant_then_gemm(i):
                q_, s_ = _C.act_quant_int8(xa, operand_order=True)
                return _C.ternary_gemm_int8_tiled(q_, s_, ts[i % 2], sc, None, k, n, torch.bfloat16, False, None, True)
            _, ev_qg = graph_time(quant_then_gemm, steps, 5, torch)
            _, ev_q = graph_time(lambda i: _C.act_quant_int8(xa, operand_order=True), steps, 5, torch)
            # the opt-in prefill copy in the field layout (TernaryLinearInference.prepare_prefill), row sums from the quantizer
            fs = [_C.retile_fields(t, k, n) for t in ts]
            _, _, rs = _C.act_quant_int8(xa, operand_order=True, return_rowsum=True)
            _, ev_fl = graph_time(lambda i: _C.ternary_gemm_int8_fields(q, s, rs, fs[i % 2], sc, None, k, n, torch.bfloat16,
                                                                        False, None, True), steps, 5, torch)
            del ts, fs
            _, ev_full = graph_time(lambda i: _C.ternary_linear_tensor_core_forward(xa, ws[i % 2], sc, None, k, 2),
                                    steps, 5, torch)
            ops = 2.0 * m * n * k
            tops = ops / (ev_tw / steps * 1e-3) / 1e12
            extra[f"prefill_int8_M{m}_N{n}_K{k}"] = {
                "gemm_us": round(ev_tw / steps * 1e3, 2),
                "tops": round(tops, 1),
                "frac_of_int8_peak": round(tops / INT8_PEAK_TOPS, 4),
                "note": "the layer's tiled weight copy and operand-order activations (TernaryLinearInference.forward_int8); "
                        "the functional API on the row-major W_T beside it",
                "gemm_us_row_major_W_T": round(ev / steps * 1e3, 2),
                "gemm_us_row_major_W_T_and_activations": round(ev_rm / steps * 1e3, 2),
                "with_act_quant_us": round(ev_full / steps * 1e3, 2),
                "tops_with_act_quant": round(ops / (ev_full / steps * 1e-3) / 1e12, 1),
                "act_quant_us": round(ev_q / steps * 1e3, 2),
                "act_quant_GBps": round(3.0 * m * k / (ev_q / steps * 1e-3) / 1e9, 1),
                "with_act_quant_us_tiled_weights": round(ev_qg / steps * 1e3, 2),
                "frac_of_int8_peak_with_act_quant_tiled_weights": round(ops / (ev_qg / steps * 1e-3) / 1e12 / INT8_PEAK_TOPS, 4),
                "gemm_us_prefill_copy_field_layout": round(ev_fl / steps * 1e3, 2),
            }
            # float path of the same shape (bf16 activations, fp32 accumulation on the 16-bit
            # matrix cores) and the vendor library on dense operands, for scale
            _, ev_f = graph_time(lambda i: _C.ternary_linear_packed_forward(xa, ws[i % 2], sc, None, k),
                                 steps, 5, torch)
            extra[f"prefill_bf16_M{m}_N{n}_K{k}"] = {
                "gemm_us": round(ev_f / steps * 1e3, 2),
                "tflops": round(ops / (ev_f / steps * 1e-3) / 1e12, 1),
                "frac_of_bf16_peak": round(ops / (ev_f / steps * 1e-3) / 1e12 / BF16_PEAK_TFLOPS, 4),
            }
            if hasattr(torch, "_int_mm"):
                wd = torch.randint(-1, 2, (k, n), device=dev, dtype=torch.int8)
                _, ev_v = graph_time(lambda i: torch._int_mm(q_rm, wd), steps, 5, torch)
                extra[f"prefill_int8_M{m}_N{n}_K{k}"]["vendor_int8_gemm_dense_tops"] = round(
                    ops / (ev_v / steps * 1e-3) / 1e12, 1)
                del wd
            wdf = torch.randn(n, k, device=dev).bfloat16()
            _, ev_v = graph_time(lambda i: torch.nn.functional.linear(xa, wdf), steps, 5, torch)
            extra[f"prefill_bf16_M{m}_N{n}_K{k}"]["vendor_bf16_gemm_dense_tflops"] = round(
                ops / (ev_v / steps * 1e-3) / 1e12, 1)
            del ws, xa, q, q_rm, s, wdf
        # what the matrix cores sustain on register operands only (no memory in the loop):
        # constant operands, pseudo-random int8 x ternary operands, and the GEMM's own register
        # footprint (32 accumulators, 8 A and 4 B fragments per wave)
        def probe(mode):
            probe_mfma_int8(torch, dev, 2048, 4096, mode)  # warm
            torch.cuda.synchronize()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(5):
                ops = probe_mfma_int8(torch, dev, 2048, 4096, mode)
            e1.record()
            torch.cuda.synchronize()
            return ops * 5 / (e0.elapsed_time(e1) * 1e-3) / 1e12

        probe_tops = {"constant_operands": probe(0), "random_operands": probe(1), "gemm_register_footprint": probe(2)}
        _, probe_mhz = probe_mfma_int8(torch, dev, 2048, 4096, 2, return_clock=True)
        extra["mfma_i8_register_only_probe"] = {
            "tops": {k: round(v, 1) for k, v in probe_tops.items()},
            "frac_of_int8_peak": round(probe_tops["gemm_register_footprint"] / INT8_PEAK_TOPS, 4),
            "shader_clock_MHz_under_this_load": None if probe_mhz is None else round(probe_mhz),
            "note": "2048 workgroups x 8 waves of back-to-back v_mfma_i32_16x16x64_i8, no memory traffic in the loop; "
                    "the clock is what workgroup 0 measures in its loop (cycle counter against the 100 MHz real-time "
                    "counter): the 5 POPS peak assumes 2.4 GHz",
        }
        # what a pure reader gets from the memory system on this box, next to the headline
        read_probe = probe_hbm_read(torch, dev)
        extra["hbm_read_only_probe"] = {
            "GBps": read_probe,
            "headline_frac_of_best_pattern": round(out["value"] / max(read_probe.values()), 4),
            "note": "512 MiB read by 512 workgroups of 512 threads (grid-stride: 4096 of 256), xor-reduced; the grouped "
                    "GEMV walks its weights in the third pattern",
        }
        # what one stage boundary of a chain of dependent GEMVs inside ONE launch would cost (persistent workgroups
        # handing a vector over through memory), against the kernel launch it would replace
        extra["grid_handover_probe"] = {
            "us_per_handover": probe_grid_handover(torch, dev),
            "note": "persistent workgroups of 512 threads on all 8 XCDs: every workgroup writes its slice of an n-entry "
                    "vector with agent-scope stores, then a barrier (one counter per XCD in its own L2, one agent-scope "
                    "counter of 8) and a plain read of the whole vector, or no barrier and consumers polling data whose "
                    "entries carry the round number; every wait bounded.  A dependent launch in a HIP graph costs "
                    "about 3.5 us (launch, one round trip to memory, drain) beyond its bytes: a hand-over costs as much, "
                    "so a chain of GEMVs in one launch would gain only what it can prefetch behind the wait",
        }
        for key in list(extra):
            if key.startswith("prefill_int8"):
                extra[key]["frac_of_probe"] = round(extra[key]["tops"] / probe_tops["gemm_register_footprint"], 4)
        # config 2 again with independent launches in flight: the same kernel on 1, 2, 4 and 8 branches
        # of one HIP graph (each branch its own chain of launches over its own weight sets).  A single
        # chain pays a launch gap and a full memory round trip per 4 MiB; with branches the chip's
        # bandwidth, not the latency of one launch, sets the rate.  Not the headline figure: a decode
        # step of one sequence is a single chain.
        def branches_time(nb, per_branch=250):
            streams = [torch.cuda.Stream() for _ in range(nb)]
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                main = torch.cuda.current_stream()
                for bi, st in enumerate(streams):
                    st.wait_stream(main)
                    with torch.cuda.stream(st):
                        for i in range(per_branch):
                            layers[(bi * per_branch + i) % nsets](xs[(bi * per_branch + i) % nsets])
                for st in streams:
                    main.wait_stream(st)
            graph.replay()
            torch.cuda.synchronize()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e-3 / (nb * per_branch)

        conc = {}
        for nb in (1, 2, 4, 8):
            t = branches_time(nb)
            conc[f"{nb}_branches"] = {"us_per_launch": round(t * 1e6, 3), "GBps": round(weight_bytes / t / 1e9, 1),
                                      "frac_of_hbm_peak": round(weight_bytes / t / 1e9 / HBM_PEAK_GBPS, 4)}
        extra["decode_gemv_independent_launches_in_flight"] = conc
        # config 3: small-batch decode, int8 activations
        for (m, n, k) in ((16, 11008, 4096), (16, 4096, 11008)):
            cnt = max(2, int(400e6 // (n * k // 4)))
            ws = rand_packed(n, k, cnt)
            xa = acts(m, k, False)
            sc = torch.rand(n, device=dev) * 0.05 + 0.01
            steps = 200
            _, ev = graph_time(lambda i: _C.ternary_linear_tensor_core_forward(xa, ws[i % cnt], sc, None, k, 2),
                               steps, 10, torch)
            us = ev / steps * 1e3
            gbps = n * ((k + 3) // 4) / (us * 1e-6) / 1e9
            ts = [_C.retile_weights(w, k) for w in ws]

            def tiled_step(i):
                q, s = _C.act_quant_int8(xa, True)
                return _C.ternary_gemm_int8_tiled(q, s, ts[i % cnt], sc, None, k, n, torch.bfloat16, False, None, True)

            _, ev_t = graph_time(tiled_step, steps, 10, torch)
            us_t = ev_t / steps * 1e3
            gbps_t = n * ((k + 3) // 4) / (us_t * 1e-6) / 1e9
            extra[f"decode_int8_M{m}_N{n}_K{k}"] = {
                "us": round(us_t, 2), "weight_GBps": round(gbps_t, 1),
                "frac_of_hbm_peak": round(gbps_t / HBM_PEAK_GBPS, 4),
                "us_row_major_W_T": round(us, 2), "weight_GBps_row_major_W_T": round(gbps, 1),
                "note": "activation quantization + GEMM per step; decode-tiled weights, and the tensor-core "
                        "forward on the reference-layout W_T beside it",
            }
            del ws, ts
        # large matrices at M = 1, where one launch is no longer bounded by its start and drain: a vocabulary
        # projection and a 64 MiB square layer, fp16 (exact GEMV where K allows), bf16 and int8 activations
        big = {}
        for (n, k) in ((128256, 4096), (16384, 16384)):
            cnt = max(2, int(600e6 // (n * k // 4)))
            ts = []
            for w in rand_packed(n, k, cnt):
                ts.append(_C.retile_weights(w, k))
                del w
            sc = torch.rand(n, device=dev) * 0.05 + 0.01
            x16 = torch.randn(1, k, device=dev).half()
            xb = x16.bfloat16()
            qb, sb = _C.act_quant_int8(xb, True)
            row = {"packed_weight_bytes": n * k // 4}
            for name, fn in (("fp16", lambda i: _C.ternary_linear_tiled_forward(x16, ts[i % cnt], sc, None, k, n)),
                             ("bf16", lambda i: _C.ternary_linear_tiled_forward(xb, ts[i % cnt], sc, None, k, n)),
                             ("int8", lambda i: _C.ternary_gemm_int8_tiled(qb, sb, ts[i % cnt], sc, None, k, n, torch.bfloat16,
                                                                           False, None, True))):
                _, ev_b = graph_time(fn, 40, 8, torch)
                us_b = ev_b / 40 * 1e3
                row[name] = {"us": round(us_b, 2), "GBps": round(n * k // 4 / (us_b * 1e-6) / 1e9, 1),
                             "frac_of_hbm_peak": round(n * k // 4 / (us_b * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)}
            big[f"N{n}_K{k}"] = row
            del ts
        extra["large_matrices_M1"] = big
        # config 3 as G units per launch (bt_ternary_gemm_i8_grouped): batched decode steps through several
        # same-shaped layers, int8 activations already quantized; two alternating sets of units beyond the
        # Infinity Cache; the single tiled call per unit beside it
        gi8 = {}
        for (n, k) in ((11008, 4096), (4096, 11008)):
            row = {}
            for G in (8, 32, 128):
                nsets_ = 2
                tl_ = [[_C.retile_weights(w, k) for w in rand_packed(n, k, G)] for _ in range(nsets_)]
                sc_ = torch.rand(n, device=dev) * 0.05 + 0.01
                qs_ = [_C.act_quant_int8(acts(16, k, False), True) for _ in range(G)]
                ys_ = [torch.empty(16, n, dtype=torch.bfloat16, device=dev) for _ in range(G)]
                tabs_ = [(_C.pointer_table([q for q, _ in qs_]), _C.pointer_table([s for _, s in qs_]),
                          _C.pointer_table(tl_[i]), _C.pointer_table([sc_] * G), None, _C.pointer_table(ys_))
                         for i in range(nsets_)]
                _, ev = graph_time(lambda i: _C.ternary_gemm_int8_grouped(*tabs_[i % nsets_], 16, k, n, out_dtype=torch.bfloat16,
                                                                         q_operand_order=True), 20, 4, torch)
                us = ev / 20 * 1e3
                row[f"G{G}"] = {"us": round(us, 2), "weight_GBps": round(G * n * k // 4 / (us * 1e-6) / 1e9, 1),
                                "frac_of_hbm_peak": round(G * n * k // 4 / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)}
                if G == 8:
                    _, ev1 = graph_time(lambda i: [_C.ternary_gemm_int8_tiled(qs_[u][0], qs_[u][1], tl_[i % nsets_][u], sc_, None,
                                                                             k, n, torch.bfloat16, False, None, True)
                                                   for u in range(8)], 20, 4, torch)
                    row["single_call_us_per_unit"] = round(ev1 / 20 * 1e3 / 8, 2)
                del tl_, tabs_, qs_, ys_
            gi8[f"M16_N{n}_K{k}"] = row
        extra["grouped_int8_units_config3"] = gi8
        # batched decode / short prefill on the config-2 layer (tiled weights): the streaming kernel runs the 16-row
        # blocks of a call concurrently in one launch; the tiled GEMM (forced with the library option STREAM_MAX_ROWS) beside it
        bd = {}
        n_, k_ = 4096, 4096
        ws = rand_packed(n_, k_, 8)
        ts = [_C.retile_weights(w, k_) for w in ws]
        sc = torch.rand(n_, device=dev) * 0.05 + 0.01
        for m in (32, 64, 128, 256):
            xa = acts(m, k_, False)
            q, s_ = _C.act_quant_int8(xa, True)
            row = {}
            for route, env in (("streaming", None), ("tiled_gemm", "16")):
                if env:
                    set_option("STREAM_MAX_ROWS", env)
                _, ev_f = graph_time(lambda i: _C.ternary_linear_tiled_forward(xa, ts[i % 8], sc, None, k_, n_), 40, 5, torch)
                _, ev_i = graph_time(lambda i: _C.ternary_gemm_int8_tiled(q, s_, ts[i % 8], sc, None, k_, n_, torch.bfloat16,
                                                                         False, None, True), 40, 5, torch)
                set_option("STREAM_MAX_ROWS", None)
                row[f"bf16_us_{route}"] = round(ev_f / 40 * 1e3, 2)
                row[f"int8_us_{route}"] = round(ev_i / 40 * 1e3, 2)
            row["int8_tops"] = round(2.0 * m * n_ * k_ / (row["int8_us_streaming"] * 1e-6) / 1e12, 1)
            bd[f"M{m}"] = row
        extra["batched_decode_N4096_K4096"] = bd
        del ws, ts
        # prefill chunks shorter than config 4's (chunked prefill): the tiled copy against the opt-in field-layout copy
        sp = {}
        n_ = k_ = 4096
        wt_ = rand_packed(n_, k_, 1)[0]
        tl_ = _C.retile_weights(wt_, k_)
        fl_ = _C.retile_fields(tl_, k_, n_)
        sc_ = torch.rand(n_, device=dev) * 0.05 + 0.01
        for m in (512, 1024):
            q_, s_, rs_ = _C.act_quant_int8(acts(m, k_, True), operand_order=True, return_rowsum=True)
            _, ev_t = graph_time(lambda i: _C.ternary_gemm_int8_tiled(q_, s_, tl_, sc_, None, k_, n_, torch.bfloat16, False, None, True), 40, 5, torch)
            _, ev_f = graph_time(lambda i: _C.ternary_gemm_int8_fields(q_, s_, rs_, fl_, sc_, None, k_, n_, torch.bfloat16, False, None, True), 40, 5, torch)
            sp[f"M{m}"] = {"gemm_us_tiled_copy": round(ev_t / 40 * 1e3, 2), "gemm_us_prefill_copy_field_layout": round(ev_f / 40 * 1e3, 2)}
        extra["short_prefill_int8_N4096_K4096"] = sp
        del wt_, tl_, fl_
        # quantize + pack of fp32 master weights
        for (n, k) in ((4096, 4096), (11008, 4096), (4096, 11008)):
            cnt = max(2, int(600e6 // (n * k * 4)))
            masters = [torch.randn(n, k, device=dev) * 0.02 for _ in range(cnt)]
            steps = 40
            _, ev = graph_time(lambda i: _C.ternary_quantize_pack(masters[i % cnt], 0.05, True), steps, 4, torch)
            us = ev / steps * 1e3
            nbytes = 4 * n * k + n * ((k + 3) // 4) + 4 * n
            extra[f"quantize_pack_N{n}_K{k}"] = {
                "us": round(us, 2), "GBps": round(nbytes / (us * 1e-6) / 1e9, 1),
                "frac_of_hbm_peak": round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
            }
            del masters
        # block glue (config-5 shapes, bf16): fused kernels against the torch sequences they replace
        import torch.nn.functional as F
        glue = {}
        for (m, k) in ((4096, 6912), (4096, 2560)):
            gs = [torch.randn(m, k, device=dev).bfloat16() for _ in range(4)]
            us_ = [torch.randn(m, k, device=dev).bfloat16() for _ in range(4)]
            nw = torch.ones(k, device=dev).bfloat16()
            nb = m * k * 2
            cases = {
                "swiglu": (lambda i: _C.swiglu(gs[i % 4], us_[i % 4]), 3 * nb),
                "swiglu_torch_2_kernels": (lambda i: F.silu(gs[i % 4]) * us_[i % 4], 3 * nb),
                "swiglu_quantized": (lambda i: _C.swiglu(gs[i % 4], us_[i % 4], False, True), 2 * nb + nb // 2),
                "swiglu_quantized_torch_plus_act_quant": (lambda i: _C.act_quant_int8(F.silu(gs[i % 4]) * us_[i % 4]), 2 * nb + nb // 2),
                "rmsnorm": (lambda i: _C.rmsnorm(gs[i % 4], nw, 1e-5), 2 * nb),
                "rmsnorm_torch": (lambda i: F.rms_norm(gs[i % 4], (k,), nw, 1e-5), 2 * nb),
                "rmsnorm_quantized": (lambda i: _C.rmsnorm(gs[i % 4], nw, 1e-5, False, True), nb + nb // 2),
                "rmsnorm_quantized_torch_plus_act_quant": (lambda i: _C.act_quant_int8(F.rms_norm(gs[i % 4], (k,), nw, 1e-5)), nb + nb // 2),
            }
            for name, (fn, nbytes) in cases.items():
                _, ev = graph_time(fn, 40, 4, torch)
                us = ev / 40 * 1e3
                glue[f"{name}_{m}x{k}"] = {"us": round(us, 2), "algorithmic_GBps": round(nbytes / (us * 1e-6) / 1e9, 1)}
            del gs, us_
        extra["block_glue_bf16"] = glue
        # one decode token through the ternary layers of a config-5 block (M = 1, bf16, HIP graph over 16 distinct
        # layers' weights): seven separate GEMVs + torch glue against q|k|v and gate|up as single launches with the
        # glue fused (RMSNorm and SwiGLU inside the GEMV kernels that consume them, residuals in their epilogues);
        # attention itself (KV cache) is left out of both
        import bittorch_amd as bt
        d_model, ffn, nl = 2560, 6912, 16  # 16 x 19.8 MB of packed weights: beyond the Infinity Cache
        def mk(i, o):
            pk = rand_packed(o, i, 1)[0]
            return bt.nn.TernaryLinearInference(i, o, pk, torch.rand(o, device=dev) * 0.05 + 0.01)
        layers_ = [{nm: mk(*sh) for nm, sh in (("q", (d_model, d_model)), ("k", (d_model, d_model)), ("v", (d_model, d_model)),
                                              ("o", (d_model, d_model)), ("gate", (d_model, ffn)), ("up", (d_model, ffn)),
                                              ("down", (ffn, d_model)))} for _ in range(nl)]
        for L in layers_:
            L["qkv"] = bt.utils.fuse_ternary_linear_inference(L["q"], L["k"], L["v"])
            L["mlp"] = bt.nn.TernarySwiGLU(L["gate"], L["up"], L["down"], compute="float", fuse_gate_up=True)
        xt = torch.randn(1, d_model, device=dev).bfloat16()
        nw = torch.ones(d_model, device=dev).bfloat16()
        eps = 1e-5

        def decode_plain(i):
            L = layers_[i % nl]
            h = F.rms_norm(xt, (d_model,), nw, eps)
            a, _k, _v = L["q"](h), L["k"](h), L["v"](h)    # q stands in for the attention output (k, v go to the cache)
            x1 = xt + L["o"](a)
            h2 = F.rms_norm(x1, (d_model,), nw, eps)
            return x1 + L["down"](F.silu(L["gate"](h2)) * L["up"](h2))

        def decode_fused(i):
            L = layers_[i % nl]
            qkv = L["qkv"](xt, None, (nw, eps))            # RMSNorm inside the GEMV kernel
            a = qkv[:, :d_model]                           # (a view: no launch between the projections)
            x1 = L["o"](a, xt)
            return L["mlp"](x1, nw, eps, residual=x1)

        def all_layers(flag):
            for L in layers_:
                for m in L.values():
                    for sub in m.modules():
                        if isinstance(sub, TernaryLinearInference):
                            sub.decode_tiled = flag
                            if flag:
                                sub.prepare_decode()

        all_layers(False)
        _, ev_p = graph_time(decode_plain, 64, 8, torch)
        _, ev_f = graph_time(decode_fused, 64, 8, torch)
        all_layers(True)
        torch.cuda.synchronize()
        _, ev_pt = graph_time(decode_plain, 64, 8, torch)
        _, ev_ft = graph_time(decode_fused, 64, 8, torch)
        extra["decode_token_per_block_bf16"] = {
            "us_seven_gemvs_torch_glue_row_major_W_T": round(ev_p / 64 * 1e3, 2),
            "us_fused_layers_and_glue_row_major_W_T": round(ev_f / 64 * 1e3, 2),
            "us_seven_gemvs_torch_glue": round(ev_pt / 64 * 1e3, 2),
            "us_fused_layers_and_glue": round(ev_ft / 64 * 1e3, 2),
            "packed_weight_bytes_per_block": (4 * d_model * d_model + 3 * d_model * ffn) // 4,
        }
        # the same fused sequence on fp16 rows (config 2's dtype): every GEMV is the exact kernel, RMSNorm and SwiGLU
        # prologues inside it
        xt = xt.half()
        nw = nw.half()
        _, ev_h = graph_time(decode_fused, 64, 8, torch)
        extra["decode_token_per_block_bf16"]["us_fused_layers_and_glue_fp16_rows"] = round(ev_h / 64 * 1e3, 2)
        del layers_
        # config 5: the 30-layer block stack, end to end
        if not args.no_block_stack:
            try:
                extra["block_stack_2B_forward"] = block_stack(torch, dev)
            except RuntimeError as err:  # e.g. not enough free HBM on a shared card
                extra["block_stack_2B_forward"] = {"skipped": str(err)[:200]}
        out["secondary"] = extra

    # ---- CPU baseline: the oracle (a scalar C port of the reference arithmetic) -------------
    if not args.no_cpu:
        from oracle import oracle as o
        o.build()
        x_np = x.float().cpu().numpy()
        p_np = packed0.cpu().numpy()
        s_np = scale.cpu().numpy()
        b_np = bias.float().cpu().numpy()
        threads = o.num_threads()
        o.linear_packed(x_np, p_np, s_np, K, b_np)  # warm
        t0 = time.perf_counter()
        iters = 0
        while time.perf_counter() - t0 < args.cpu_seconds:
            o.linear_packed(x_np, p_np, s_np, K, b_np)
            iters += 1
        dt = (time.perf_counter() - t0) / iters
        out["cpu_baseline"] = {
            "value": round(weight_bytes / dt / 1e9, 4),
            "unit": "GB/s",
            "cores": threads,
            "kind": "port",
            "sample": f"{iters} passes of the same M=1 4096x4096 GEMV through oracle/bt_oracle.c "
                      f"(OpenMP over output columns, {threads} threads), {args.cpu_seconds:.0f} s",
            "ms_per_step": round(dt * 1e3, 3),
        }
        # the reference's own CPU route (unpack + dense product) in plain torch, for scale
        torch.set_num_threads(max(1, min(threads, os.cpu_count() or 1)))
        from bittorch_amd.nn import TernaryLinearInference
        layer = TernaryLinearInference(K, N, packed0.cpu(), scale.cpu().expand(N).contiguous(), bias.float().cpu())
        xc = x.float().cpu()
        layer(xc)
        t0 = time.perf_counter()
        it2 = 0
        while time.perf_counter() - t0 < 3.0:
            layer(xc)
            it2 += 1
        dt2 = (time.perf_counter() - t0) / it2
        out["cpu_baseline"]["torch_unpack_linear_ms_per_step"] = round(dt2 * 1e3, 3)
        out["cpu_baseline"]["torch_unpack_linear_GBps"] = round(weight_bytes / dt2 / 1e9, 4)
        # the training module's plain-torch backend on the CPU (quantize the fp32 masters every call,
        # then a dense product), and the dense product alone on pre-quantized effective weights
        from bittorch_amd.nn import TernaryLinear

        def cpu_time(fn, seconds=3.0):
            fn()
            t0 = time.perf_counter()
            n = 0
            while time.perf_counter() - t0 < seconds:
                fn()
                n += 1
            return (time.perf_counter() - t0) / n

        tl = TernaryLinear(K, N, bias=True, per_channel=False, backend="python")
        with torch.no_grad():
            tl.weight.copy_(w0.cpu())
            tl.bias.copy_(bias.float().cpu())
            dt3 = cpu_time(lambda: tl(xc))
            w_tern, s_cpu = tl.get_quantized_weight()
            w_eff = (w_tern * s_cpu).contiguous()
            dt4 = cpu_time(lambda: torch.nn.functional.linear(xc, w_eff, tl.bias))
        out["cpu_baseline"]["torch_python_backend_requantize_ms_per_step"] = round(dt3 * 1e3, 3)
        out["cpu_baseline"]["torch_prequantized_dense_fp32_ms_per_step"] = round(dt4 * 1e3, 3)
        out["cpu_baseline"]["torch_threads"] = torch.get_num_threads()

    print(json.dumps(out))


if __name__ == "__main__":
    main()
