#!/usr/bin/env python3
"""Benchmark of the quantized-weight matmul hot path on one MI355X.

A step is one pass of the hot path over one batch: hipq_matmul on device-resident
inputs = activation quantizer (fp32 -> Q8_K) + Q4_K x Q8_K block-dot GEMM, at the
prefill shape BASELINE.json quotes its metric on (configs[1]: M=512, K=4096,
N=12288). Prints ONE JSON line. Also measured and attached to the same line: the
decode GEMV (M=1) over the same matrix at HBM-resident size and over a sweep of widths,
the kernels' own durations (start and stop events attached to every launch), the FC stack
of the whole 28-layer decoder of configs[4], host-memory calls, and the reference CPU path
timed on this box's host cores with both of its thread front-ends.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

M, K, N = 512, 4096, 12288
INT8_PEAK_TOPS = 5000.0  # MI355X dense int8 matrix peak, TOP/s
HBM_PEAK_GBS = 8000.0    # MI355X HBM3E peak, GB/s
# HBM bytes per launch from rocprofv3 FETCH_SIZE / WRITE_SIZE counter runs of this script, scaled by
# what the same counters read for kernels of known size in the same run (a 1 GiB read-only kernel, a 1 GiB
# fill, its 256 MiB device copies) (profiles/gemm_q4k_prefill_m512_k4096_n12288.txt,
# profiles/gemv_q4k_decode_m1_k4096.txt, profiles/moe_block_q4k_64tok_128experts.txt). Measured once, not live: counters need the profiler attached.
TRAFFIC_GEMM_C2 = 49.04e6 + 25.17e6
TRAFFIC_GEMV_C2 = 28.57e6 + 0.05e6
TRAFFIC_GEMV_LM_HEAD = 350.25e6 + 0.62e6
METRIC = "Q4 GEMV effective GB/s (%HBM peak); prefill GEMM int8 TOPS (%MFMA peak)"


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline_thread_pool(blocks_host, a_host, budget_s=8.0):
    """The same product through the reference's default x86 front-end (ggml_interface_mixed.cpp:532-638):
    a pool of hardware_concurrency() threads (bs_thread_pool_manager.hpp:41), whatever share of the
    machine this process has. Its thread count is what the pool reports."""
    import numpy as np
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    so = os.path.join(ROOT, "oracle", "_ref", "libnntr_ref_mixed.so")
    if not os.path.exists(so):
        return None
    lib = ctypes.CDLL(so)
    lib.ref_init()
    b = np.zeros_like(blocks_host)
    lib.ref_repack_q4_K_x8(ctypes.c_void_p(b.ctypes.data), ctypes.c_void_p(blocks_host.ctypes.data),
                           ctypes.c_size_t(blocks_host.size), ctypes.c_uint(N), ctypes.c_uint(K))
    c = np.zeros((M, N), np.float32)
    run = lambda: lib.ref_gemm_q4_K(ctypes.c_uint(M), ctypes.c_uint(N), ctypes.c_uint(K),
                                    ctypes.c_void_p(a_host.ctypes.data), ctypes.c_void_p(b.ctypes.data),
                                    ctypes.c_void_p(c.ctypes.data))
    run()
    t0, reps = time.perf_counter(), 0
    while True:
        run()
        reps += 1
        el = time.perf_counter() - t0
        if el > budget_s or reps >= 400:
            break
    sec = el / reps
    return {"value": round(2.0 * M * N * K / sec / 1e12, 4), "unit": "TOPS", "threads": int(lib.ref_max_threads()),
            "kind": "reference", "front_end": "thread pool of hardware_concurrency() threads (the x86 default)",
            "sample": "%d full passes (%.2f s each), same inputs" % (reps, sec)}


def cpu_baseline(blocks_host, a_host, gpu_out, budget_s=12.0):
    """The reference ggml-interface CPU path (oracle/_ref, built from the reference's
    own sources) on the same inputs; falls back to this repo's C port of it."""
    import numpy as np
    os.environ.setdefault("OMP_THREAD_LIMIT", "16")  # this box's CPU share
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import cpuref as cr
    lib, kind = cr.ref(), "reference"
    if lib is None:
        lib, kind = cr.oracle(), "port"
    hw = os.cpu_count() or 1
    limit = int(os.environ.get("OMP_THREAD_LIMIT", "16"))
    # the reference wrapper asks for hardware_concurrency()/2 threads (GEMM)
    cores = max(1, min(hw // 2, limit)) if kind == "reference" else min(hw, limit)
    if kind == "port":
        cr.oracle().orc_set_threads(cores)
    if kind == "reference":
        b = cr.repack_x8(lib, "q4_K", blocks_host, N, K)
        c = np.zeros((M, N), np.float32)
        run = lambda: lib.ref_gemm_q4_K(ctypes.c_uint(M), ctypes.c_uint(N), ctypes.c_uint(K),
                                        ctypes.c_void_p(a_host.ctypes.data), ctypes.c_void_p(b.ctypes.data),
                                        ctypes.c_void_p(c.ctypes.data))
    else:
        c = None

        def run():
            nonlocal c
            c = cr.gemm(lib, "q4_K", a_host, blocks_host, N)
    run()
    t0 = time.perf_counter()
    reps = 0
    while True:
        run()
        reps += 1
        el = time.perf_counter() - t0
        if el > budget_s or reps >= 400:
            break
    sec = el / reps
    err = float(np.abs(gpu_out - c).max() / np.abs(c).max())
    return {"value": round(2.0 * M * N * K / sec / 1e12, 4), "unit": "TOPS", "cores": cores, "kind": kind,
            "front_end": "OpenMP, hardware_concurrency() / 2 threads for a GEMM (ggml_interface_omp.cpp:331, 434)",
            "cpu_model": cpu_model(), "cpus_visible": os.cpu_count(),
            "sample": "%d full passes of the same M=%d K=%d N=%d Q4_K matmul (%.2f s each), same inputs"
                      % (reps, M, K, N, sec),
            "gpu_vs_cpu_max_rel_err": err}


def cpu_gemv_baseline(kind, n, k, host, nbytes, budget_s=4.0):
    """One-row matmul of the reference library (its OpenMP wrapper asks for 4 threads on this
    path, ggml_interface_omp.cpp:309, 410) on the GPU leg's weights and row: effective GB/s
    over the same algorithmic bytes, and whether the GPU's output carries the same bits."""
    import numpy as np
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import cpuref as cr
    lib = cr.ref()
    if lib is None:
        return None
    blocks, a, gpu_out = host
    b = blocks if kind == "q6_K" else cr.repack_x8(lib, kind, blocks, n, k)
    c = np.zeros((1, n), np.float32)
    fn = getattr(lib, "ref_gemm_" + kind)
    run = lambda: fn(ctypes.c_uint(1), ctypes.c_uint(n), ctypes.c_uint(k), ctypes.c_void_p(a.ctypes.data),
                     ctypes.c_void_p(b.ctypes.data), ctypes.c_void_p(c.ctypes.data))
    run()
    t0, reps = time.perf_counter(), 0
    while True:
        run()
        reps += 1
        el = time.perf_counter() - t0
        if el > budget_s or reps >= 2000:
            break
    return {"value": round(nbytes / (el / reps) / 1e9, 2), "unit": "GB/s", "threads": 4, "kind": "reference",
            "ms_per_call": round(el / reps * 1e3, 4), "sample": "%d calls" % reps,
            "gpu_output_bit_identical": bool(np.array_equal(gpu_out.view(np.uint32), c.view(np.uint32)))}


def plugin_moe_layer():
    """One qwen_moe layer of the C3 shape through libnntrainer_hip_context.so: router, routing and the three
    expert products in one incremental_forwarding call on host tensors; microseconds per call."""
    import subprocess
    lib = os.path.join(ROOT, "nntrainer_amd", "lib")
    exe, plugin = os.path.join(lib, "hipq_host_selftest"), os.path.join(lib, "libnntrainer_hip_context.so")
    if not (os.path.exists(exe) and os.path.exists(plugin)):
        return {"skipped": "the plug-in is not built (python -c 'import __graft_entry__ as g; g.build()')"}
    try:
        r = subprocess.run([exe, plugin, "moelayer", "200"], capture_output=True, text=True, timeout=180)
        if r.returncode != 0:
            return {"failed": (r.stdout + r.stderr)[-300:]}
        res = json.loads(r.stdout.strip().splitlines()[-1])
    except Exception as e:  # the bench line must still be printed
        return {"failed": repr(e)[:300]}
    res["workload"] = ("one qwen_moe layer, hidden 2048, 128 experts of 768, top 8, Q4_K (BASELINE configs[2]'s "
                       "block), created by the context's factory; incremental_forwarding on host tensors, the router's "
                       "weight given; one decode token and a chunk of 64 tokens; wall clock per call")
    return res


def plugin_c5_layer():
    """The quantized FCs of one C5 decoder layer through libnntrainer_hip_context.so (layers created by the
    context's factories, run with incremental_forwarding on host tensors): microseconds per layer."""
    import subprocess
    lib = os.path.join(ROOT, "nntrainer_amd", "lib")
    exe, plugin = os.path.join(lib, "hipq_host_selftest"), os.path.join(lib, "libnntrainer_hip_context.so")
    if not (os.path.exists(exe) and os.path.exists(plugin)):
        return {"skipped": "the plug-in is not built (python -c 'import __graft_entry__ as g; g.build()')"}
    try:
        r = subprocess.run([exe, plugin, "c5layer", "200"], capture_output=True, text=True, timeout=180)
        if r.returncode != 0:
            return {"failed": (r.stdout + r.stderr)[-300:]}
        res = json.loads(r.stdout.strip().splitlines()[-1])
    except Exception as e:  # the bench line must still be printed
        return {"failed": repr(e)[:300]}
    res["workload"] = ("one Qwen3-0.6B-shaped decoder layer (BASELINE configs[4]), Q4_0 weights, through the context "
                       "plug-in: layers from its factories, incremental_forwarding on host tensors, every call "
                       "synchronous; as the seven fully_connected layers of an unchanged graph, as qkv_layer + "
                       "fully_connected + mlp_swiglu + fully_connected, and as qkv_layer + fully_connected + mlp_swiglu "
                       "with down_unit (the whole MLP one call, hidden rows kept on the device); tensors in ordinary memory and in memory of the "
                       "context's allocator (page-locked); one decode row, and a prefill of 512 rows; wall clock per layer")
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path has no multi-GPU part (run with --gpus 1)")

    # ---- a C5 decoder layer's FCs through the framework plug-in (the layer API, host tensors, every
    # call synchronous): the plug-in's own driver as a child process, before this process touches the GPU
    plugin_layer = plugin_c5_layer()
    plugin_moe = plugin_moe_layer()

    import numpy as np
    import torch
    from nntrainer_amd import capi

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.init()
    capi.init(0)
    stream = torch.cuda.current_stream().cuda_stream
    gen = torch.Generator(device="cuda").manual_seed(1)

    # The headline's inputs are configs[1] as the parity test of the same configuration draws them
    # (tests/test_gpu_configs.py::test_c2_q4_K_prefill_gemm): the repository's bit-reproducible generator,
    # stream 1, weights N(0, 0.02) from sample 0 and activations N(0, 1) behind them; quantized on the
    # device by the byte-exact weight quantizer. The other sections below draw theirs from torch's
    # generator on the device (not the tests' data; shapes and distributions as stated there).
    from nntrainer_amd import synth
    w32_host = synth.normal(1, (N, K), 0.02)
    a_host_in = synth.normal(1, (M, K), 1.0, first=N * K)
    input_digest = {"weights_fp32": synth.digest(w32_host), "activations_fp32": synth.digest(a_host_in)}
    w32 = torch.from_numpy(w32_host).cuda()
    a = torch.from_numpy(a_host_in).cuda()
    del w32_host
    blocks = torch.empty(capi.weight_nbytes("q4_K", N, K), dtype=torch.uint8, device="cuda")
    capi.quantize_weights("q4_K", w32, N, K, blocks, stream=stream)
    torch.cuda.synchronize()
    n_copies = 20  # 20 x 28.3 MB = 566 MB of distinct weights, twice the 256 MB last-level cache
    weights = [capi.Weight("q4_K", N, K, blocks, mem=capi.MEM_DEVICE) for _ in range(n_copies)]
    del w32
    c = torch.empty((M, N), device="cuda", dtype=torch.float32)

    def timed(ws_, a_, m_, c_, iters):
        """(ms per call, {kernel: (launches, mean ms)}, ms of the kernels that are not the activation
        quantizer per call, name of the longest of them): `iters` hipq_matmul calls between two events,
        then the same calls again with a start and a stop event attached to every launch."""
        call_ms = capi.matmul_loop(ws_, a_, m_, c_, iters, stream=stream)
        with capi.LaunchTiming(4 * (iters + len(ws_)) + 16) as lt:
            capi.matmul_loop(ws_, a_, m_, c_, iters, stream=stream)
        kern = lt.by_kernel()
        calls = iters + len(ws_)
        prod = {k_: v_ for k_, v_ in kern.items() if "quantize" not in k_}
        prod_ms = sum(cnt * mean for cnt, mean in prod.values()) / calls
        main_k = max(prod, key=lambda k_: prod[k_][0] * prod[k_][1]) if prod else ""
        return call_ms, kern, prod_ms, main_k

    # ---- the timed region: K steps of the whole hot path -------------------
    # A block = `steps` calls of hipq_matmul from a C loop (hipq_bench_matmul_loop of libhipq_bench.so,
    # which links the product library and calls its public entry point), bracketed by synchronize() on
    # both sides (wall clock) and by two HIP events on the launch stream, nothing else in the stream:
    # ms_per_step. Each block is followed by the same loop with the library's kernel timing switched on
    # (hipq_launch_timing_begin / _end: every launch carries its own start and stop event, the kernel's
    # own duration as a kernel trace reports it): roofline.kernel_ms and quantizer_ms. Attaching events
    # to a launch delays the next launch by several microseconds, so the timed loop's own total is not
    # the step time. Blocks are repeated and medians reported: 20 steps are 1.5 ms, short enough for
    # the clock state of the moment to move one block by percents.
    for i in range(args.warmup):
        capi.matmul(weights[i % n_copies], a, M, c, stream=stream)
    torch.cuda.synchronize()
    blocks_timed, blocks_instr = [], []
    gemm_kernel_name = ""
    for rep in range(5):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev_step = capi.matmul_loop(weights, a, M, c, args.steps, stream=stream)
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) / (args.steps + n_copies)  # the loop makes one untimed call per weight first
        blocks_timed.append((ev_step, wall))
        with capi.LaunchTiming(4 * (args.steps + n_copies)) as lt:
            capi.matmul_loop(weights, a, M, c, args.steps, stream=stream)
        kern = lt.by_kernel()
        q_ms = sum(mean for k_, (cnt, mean) in kern.items() if "quantize" in k_)
        g_name = max((k_ for k_ in kern if "quantize" not in k_), key=lambda k_: kern[k_][1])
        blocks_instr.append((q_ms + kern[g_name][1], q_ms, kern[g_name][1]))
        gemm_kernel_name = g_name
    blocks_timed.sort()
    step_ms = blocks_timed[len(blocks_timed) // 2][0]
    blocks_instr.sort(key=lambda b: b[2])
    instr_ms, quant_ms, gemm_ms = blocks_instr[len(blocks_instr) // 2]
    sec = step_ms * 1e-3
    ops = 2.0 * M * N * K
    value = ops / sec / 1e12
    gemm_tops = ops / (gemm_ms * 1e-3) / 1e12

    # ---- the same step with operands in host memory (what the Layer API hands over) --------
    # Not `value`: the PCIe-inclusive rate of the whole call, activations in and outputs back
    # (8 MB + 25 MB), from pageable memory (through the library's pinned ring) and from memory of
    # the context's allocator (page-locked, by DMA as it is). Synchronous calls, wall clock.
    import ctypes
    a_host = a.cpu().numpy()
    c_host = np.empty((M, N), np.float32)
    pa, pc = capi.host_alloc(M * K * 4), capi.host_alloc(M * N * 4)
    a_pin = np.ctypeslib.as_array(ctypes.cast(pa, ctypes.POINTER(ctypes.c_float)), (M, K))
    a_pin[:] = a_host

    def host_call_ms(src, dst, reps=7):
        ts = []
        for i in range(reps + 2):
            t0 = time.perf_counter()
            capi.matmul(weights[i % n_copies], src, M, dst, mem=capi.MEM_HOST)
            ts.append((time.perf_counter() - t0) * 1e3)
        return sorted(ts[2:])[reps // 2]

    pageable_ms = host_call_ms(a_host, c_host)
    pinned_ms = host_call_ms(pa, pc)
    capi.host_free(pa)
    capi.host_free(pc)

    # ---- decode GEMV over the same matrix, weights rotating through HBM ----
    # One row against a matrix of this size is ONE launch (the workgroups quantize the row themselves
    # while their weights are on the way): kernel_ms is that kernel's own duration.
    a1 = a[:1].contiguous()
    c1 = torch.empty((1, N), device="cuda", dtype=torch.float32)
    gv_bytes = N * K * 144 // 256 + 4 * K + 4 * N
    gemv_all_ms, gemv_kern, gemv_ms, gemv_kernel_name = timed(weights, a1, 1, c1, 40 * n_copies)
    _, _, gemv_hot_ms, _ = timed(weights[:1], a1, 1, c1, 400)
    gemv_gbs = gv_bytes / (gemv_ms * 1e-3) / 1e9

    # ---- a batch of decode rows against the same matrices: Q4_K on the matrix cores with the
    # reference's bits up to sixteen rows (gemm_rows_q4k.hip), the prefill GEMM beyond ----
    rows_ms = {}
    for mr in (8, 4, 16, 64):
        ar = torch.randn((mr, K), generator=gen, device="cuda", dtype=torch.float32)
        cr_ = torch.empty((mr, N), device="cuda", dtype=torch.float32)
        call_, _, prod_, _ = timed(weights, ar, mr, cr_, 20 * n_copies)
        rows_ms[mr] = (prod_, call_)

    # ---- the Q4_K decode GEMV over widths from 4096 to the lm_head's: where the kernel meets the HBM
    # bound. Per width: copies that together exceed twice the last-level cache, the product kernel's own
    # duration against the algorithmic bytes (weights + 4K + 4N), and the whole call.
    sweep = []
    for n_ in (4096, 12288, 32768, 65536, 151936):
        w32_ = torch.randn((n_, K), generator=gen, device="cuda", dtype=torch.float32) * 0.02
        b_ = torch.empty(capi.weight_nbytes("q4_K", n_, K), dtype=torch.uint8, device="cuda")
        capi.quantize_weights("q4_K", w32_, n_, K, b_, stream=stream)
        torch.cuda.synchronize()
        del w32_
        by_ = n_ * K * 144 // 256 + 4 * K + 4 * n_
        copies_ = max(3, min(64, (600 << 20) // by_ + 1))
        ws_ = [capi.Weight("q4_K", n_, K, b_, mem=capi.MEM_DEVICE) for _ in range(copies_)]
        cn_ = torch.empty((1, n_), device="cuda")
        call_, _, prod_, name_ = timed(ws_, a1, 1, cn_, max(60, 6 * copies_))
        for w_ in ws_:
            w_.destroy()
        del b_
        sweep.append({"N": n_, "copies": copies_, "kernel": name_, "kernel_ms": round(prod_, 5),
                      "ms_per_call": round(call_, 5), "algorithmic_bytes": by_,
                      "kernel_gbs": round(by_ / (prod_ * 1e-3) / 1e9, 1),
                      "frac": round(by_ / (prod_ * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)})
    big_ms = sweep[-1]["kernel_ms"]
    big_bytes = sweep[-1]["algorithmic_bytes"]
    big_gbs = big_bytes / (big_ms * 1e-3) / 1e9
    big_kernel_name = sweep[-1]["kernel"]

    # ---- the other GEMV configurations: C1 (Q4_0, 4096 x 4096) and C3 (Q6_K lm_head) ----
    def gemv_case(kind, n, k, copies, bytes_per_weight_num, bytes_per_weight_den, prefill_rows=0):
        w32_ = torch.randn((n, k), generator=gen, device="cuda", dtype=torch.float32) * 0.02
        b_ = torch.empty(capi.weight_nbytes(kind, n, k), dtype=torch.uint8, device="cuda")
        capi.quantize_weights(kind, w32_, n, k, b_, stream=stream)
        torch.cuda.synchronize()
        del w32_
        ws_ = [capi.Weight(kind, n, k, b_, mem=capi.MEM_DEVICE) for _ in range(copies)]
        a_ = torch.randn((1, k), generator=gen, device="cuda")
        c_ = torch.empty((1, n), device="cuda")
        all_ms_, _, ms_, _ = timed(ws_, a_, 1, c_, max(60, 4 * copies))
        capi.matmul(ws_[0], a_, 1, c_, stream=stream)
        torch.cuda.synchronize()
        host_ = None if args.no_cpu else (b_.cpu().numpy(), a_.cpu().numpy(), c_.cpu().numpy())
        pre_ = None
        if prefill_rows:
            # the same weights against `prefill_rows` rows: the matrix-core product of the format
            ap_ = torch.randn((prefill_rows, k), generator=gen, device="cuda")
            cp_ = torch.empty((prefill_rows, n), device="cuda")
            runs_ = sorted((timed(ws_, ap_, prefill_rows, cp_, 6 * copies) for _ in range(3)), key=lambda r_: r_[2])
            pre_ = (runs_[1][2], runs_[1][0], runs_[1][3])
            del ap_, cp_
        for w_ in ws_:
            w_.destroy()
        by_ = n * k * bytes_per_weight_num // bytes_per_weight_den + 4 * k + 4 * n
        return ms_, all_ms_, by_, host_, pre_

    c1_ms, c1_all_ms, c1_bytes, c1_host, _ = gemv_case("q4_0", 4096, 4096, 60, 18, 32)
    c3_ms, c3_all_ms, c3_bytes, c3_host, c3_prefill = gemv_case("q6_K", 151936, 4096, 2, 210, 256, prefill_rows=512)

    # ---- the FC stack of one decoder layer of C5 (Qwen3-0.6B shapes, Q4_0), quantizer included ----
    def fc_stack(rows):
        shapes = [(2048, 1024), (1024, 1024), (1024, 1024), (1024, 2048), (3072, 1024), (3072, 1024), (1024, 3072)]
        total = 0.0
        for n_, k_ in shapes:
            w32_ = torch.randn((n_, k_), generator=gen, device="cuda", dtype=torch.float32) * 0.02
            b_ = torch.empty(capi.weight_nbytes("q4_0", n_, k_), dtype=torch.uint8, device="cuda")
            capi.quantize_weights("q4_0", w32_, n_, k_, b_, stream=stream)
            torch.cuda.synchronize()
            ws_ = [capi.Weight("q4_0", n_, k_, b_, mem=capi.MEM_DEVICE) for _ in range(8)]
            a_ = torch.randn((rows, k_), generator=gen, device="cuda")
            c_ = torch.empty((rows, n_), device="cuda")
            total += capi.matmul_loop(ws_, a_, rows, c_, 80, stream=stream)
            for w_ in ws_:
                w_.destroy()
        return total

    c5_prefill_ms, c5_decode_ms = fc_stack(512), fc_stack(1)
    c5_rows8_ms, c5_rows16_ms = fc_stack(8), fc_stack(16)
    # the same model's lm_head as a Q4_0 FC (151936 x 1024): one row and a batch of eight decode rows
    c5_head_ms, c5_head_all_ms, c5_head_bytes, _, c5_head_rows8 = gemv_case("q4_0", 151936, 1024, 4, 18, 32,
                                                                            prefill_rows=8)

    def decode_layer_graph(grouped, rows=1):
        """One step's FCs of 8 layers (8 weight copies) against `rows` rows captured in a graph and
        replayed: milliseconds per layer without the host's launch cost. grouped = 1: Q, K, V
        and gate, up each as one hipq_matmul_multi call (4 launches per layer, not 7).
        grouped = 2: Q, K, V as one call and up, gate and the SwiGLU between them and the down
        projection as one hipq_mlp_swiglu call (the qkv_layer and mlp_swiglu layers of the context)."""
        shapes = [(2048, 1024), (1024, 1024), (1024, 1024), (1024, 2048), (3072, 1024), (3072, 1024), (1024, 3072)]
        layers = []
        for _ in range(8):
            ws_ = []
            for n_, k_ in shapes:
                w32_ = torch.randn((n_, k_), generator=gen, device="cuda", dtype=torch.float32) * 0.02
                b_ = torch.empty(capi.weight_nbytes("q4_0", n_, k_), dtype=torch.uint8, device="cuda")
                capi.quantize_weights("q4_0", w32_, n_, k_, b_, stream=stream)
                torch.cuda.synchronize()
                ws_.append(capi.Weight("q4_0", n_, k_, b_, mem=capi.MEM_DEVICE))
            layers.append(ws_)
        xs_ = {k_: torch.randn((rows, k_), generator=gen, device="cuda") for k_ in (1024, 2048, 3072)}
        cs_ = [torch.empty((rows, n_), device="cuda") for n_, _ in shapes]

        def step(st):
            for ws_ in layers:
                if grouped == 2:
                    capi.matmul_multi(ws_[0:3], xs_[1024], rows, cs_[0:3], stream=st)
                    capi.matmul(ws_[3], xs_[2048], rows, cs_[3], stream=st)
                    capi.mlp_swiglu(ws_[4], ws_[5], xs_[1024], rows, cs_[4], stream=st)
                    capi.matmul(ws_[6], xs_[3072], rows, cs_[6], stream=st)
                elif grouped:
                    capi.matmul_multi(ws_[0:3], xs_[1024], rows, cs_[0:3], stream=st)
                    capi.matmul(ws_[3], xs_[2048], rows, cs_[3], stream=st)
                    capi.matmul_multi(ws_[4:6], xs_[1024], rows, cs_[4:6], stream=st)
                    capi.matmul(ws_[6], xs_[3072], rows, cs_[6], stream=st)
                else:
                    for w_, (n_, k_), c_ in zip(ws_, shapes, cs_):
                        capi.matmul(w_, xs_[k_], rows, c_, stream=st)

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step(side.cuda_stream)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step(side.cuda_stream)
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps = 20
        e0.record()
        for _ in range(reps):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / (reps * len(layers))
        del graph
        for ws_ in layers:
            for w_ in ws_:
                w_.destroy()
        return ms

    c5_graph_ms, c5_graph_grouped_ms = decode_layer_graph(0), decode_layer_graph(1)
    c5_graph_fused_ms = decode_layer_graph(2)
    c5_prefill_graph_ms, c5_prefill_grouped_ms = decode_layer_graph(0, 512), decode_layer_graph(1, 512)
    c5_rows8_grouped_ms = decode_layer_graph(1, 8)

    def whole_model(rows, with_head):
        """The FCs of all 28 decoder layers of configs[4] (Q, K, V as one call, the output projection,
        gate and up as one call, the down projection: what the context's qkv_layer and grouped FCs make
        of a layer) and, with_head, the model's lm_head as a Q4_0 FC on one row (the last one of a
        prompt), captured into ONE graph per model copy; two copies of the model (2 x 248 MB of FC
        weights) replayed in turn, so that a step does not find its weights in the last-level cache.
        Milliseconds per step."""
        shapes = [(2048, 1024), (1024, 1024), (1024, 1024), (1024, 2048), (3072, 1024), (3072, 1024), (1024, 3072)]
        models = []
        for _ in range(2):
            layers = []
            for _l in range(28):
                ws_ = []
                for n_, k_ in shapes:
                    w32_ = torch.randn((n_, k_), generator=gen, device="cuda", dtype=torch.float32) * 0.02
                    b_ = torch.empty(capi.weight_nbytes("q4_0", n_, k_), dtype=torch.uint8, device="cuda")
                    capi.quantize_weights("q4_0", w32_, n_, k_, b_, stream=stream)
                    torch.cuda.synchronize()
                    ws_.append(capi.Weight("q4_0", n_, k_, b_, mem=capi.MEM_DEVICE))
                layers.append(ws_)
            head = None
            if with_head:
                w32_ = torch.randn((151936, 1024), generator=gen, device="cuda", dtype=torch.float32) * 0.02
                b_ = torch.empty(capi.weight_nbytes("q4_0", 151936, 1024), dtype=torch.uint8, device="cuda")
                capi.quantize_weights("q4_0", w32_, 151936, 1024, b_, stream=stream)
                torch.cuda.synchronize()
                head = capi.Weight("q4_0", 151936, 1024, b_, mem=capi.MEM_DEVICE)
                del w32_, b_
            models.append((layers, head))
        xs_ = {k_: torch.randn((rows, k_), generator=gen, device="cuda") for k_ in (1024, 2048, 3072)}
        cs_ = [torch.empty((rows, n_), device="cuda") for n_, _ in shapes]
        logits_ = torch.empty((1, 151936), device="cuda")

        def step(st, model):
            layers, head = model
            for ws_ in layers:
                capi.matmul_multi(ws_[0:3], xs_[1024], rows, cs_[0:3], stream=st)
                capi.matmul(ws_[3], xs_[2048], rows, cs_[3], stream=st)
                capi.matmul_multi(ws_[4:6], xs_[1024], rows, cs_[4:6], stream=st)
                capi.matmul(ws_[6], xs_[3072], rows, cs_[6], stream=st)
            if head is not None:
                capi.matmul(head, xs_[1024][rows - 1:rows], 1, logits_, stream=st)

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for model in models:
                step(side.cuda_stream, model)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graphs = []
        for model in models:
            g_ = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g_, stream=side):
                step(side.cuda_stream, model)
            graphs.append(g_)
        for _ in range(2):
            for g_ in graphs:
                g_.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps = 10
        e0.record()
        for _ in range(reps):
            for g_ in graphs:
                g_.replay()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / (reps * len(graphs))
        del graphs
        for layers, head in models:
            for ws_ in layers:
                for w_ in ws_:
                    w_.destroy()
            if head is not None:
                head.destroy()
        return ms

    c5_model_decode_ms, c5_model_decode_head_ms = whole_model(1, False), whole_model(1, True)
    c5_model_prefill_ms = whole_model(512, True)

    # ---- one decode row through host memory (what the Layer API hands over): microseconds per call,
    # page-locked (memory of the context's allocator) and pageable, against the same call on device
    # memory, for the shapes of C1, C3 and the largest FC of C5
    def host_row_us(kind, n_, k_):
        w32_ = torch.randn((n_, k_), generator=gen, device="cuda", dtype=torch.float32) * 0.02
        b_ = torch.empty(capi.weight_nbytes(kind, n_, k_), dtype=torch.uint8, device="cuda")
        capi.quantize_weights(kind, w32_, n_, k_, b_, stream=stream)
        torch.cuda.synchronize()
        del w32_
        w_ = capi.Weight(kind, n_, k_, b_, mem=capi.MEM_DEVICE)
        xr = np.random.default_rng(5).standard_normal((1, k_)).astype(np.float32)
        yr = np.empty((1, n_), np.float32)
        px, py = capi.host_alloc(k_ * 4), capi.host_alloc(n_ * 4)
        np.ctypeslib.as_array(ctypes.cast(px, ctypes.POINTER(ctypes.c_float)), (1, k_))[:] = xr
        dx_, dy_ = torch.from_numpy(xr).cuda(), torch.empty((1, n_), device="cuda")

        def med(fn, reps=41):
            ts = []
            for _ in range(reps + 4):
                t0 = time.perf_counter()
                fn()
                ts.append((time.perf_counter() - t0) * 1e6)
            return sorted(ts[4:])[reps // 2]

        def dev_call():
            capi.matmul(w_, dx_, 1, dy_, stream=stream)
            torch.cuda.synchronize()

        out_ = {"page_locked": round(med(lambda: capi.matmul(w_, px, 1, py, mem=capi.MEM_HOST)), 2),
                "pageable": round(med(lambda: capi.matmul(w_, xr, 1, yr, mem=capi.MEM_HOST)), 2),
                "device_memory_call_and_synchronize": round(med(dev_call), 2)}
        capi.host_free(px)
        capi.host_free(py)
        w_.destroy()
        return out_

    decode_row_us = {"c1_q4_0_4096x4096": host_row_us("q4_0", 4096, 4096),
                     "c5_q4_0_3072x1024": host_row_us("q4_0", 3072, 1024),
                     "c3_q6_K_151936x4096": host_row_us("q6_K", 151936, 4096)}

    def q4k_qkv_rows(rows, copies=6):
        """Q, K, V of a 4096-wide layer with grouped-query attention (4096, 1024, 1024 x 4096, Q4_K) against
        `rows` rows as ONE hipq_matmul_multi call, replayed from a graph: milliseconds per call."""
        ns_ = (4096, 1024, 1024)
        sets_ = []
        for _ in range(copies):
            ws_ = []
            for n_ in ns_:
                w32_ = torch.randn((n_, K), generator=gen, device="cuda", dtype=torch.float32) * 0.02
                b_ = torch.empty(capi.weight_nbytes("q4_K", n_, K), dtype=torch.uint8, device="cuda")
                capi.quantize_weights("q4_K", w32_, n_, K, b_, stream=stream)
                torch.cuda.synchronize()
                ws_.append(capi.Weight("q4_K", n_, K, b_, mem=capi.MEM_DEVICE))
            sets_.append(ws_)
        x_ = torch.randn((rows, K), generator=gen, device="cuda")
        cs_ = [torch.empty((rows, n_), device="cuda") for n_ in ns_]

        def step(st):
            for ws_ in sets_:
                capi.matmul_multi(ws_, x_, rows, cs_, stream=st)

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step(side.cuda_stream)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step(side.cuda_stream)
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(20):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / (20 * copies)
        del graph
        for ws_ in sets_:
            for w_ in ws_:
                w_.destroy()
        return ms

    q4k_qkv_ms = {r_: q4k_qkv_rows(r_) for r_ in (1, 8, 16)}

    # ---- the MoE block of configs[3]: 64 tokens, 128 experts, top-8, Q4_K ----------
    mt, mh, me, mi, mk = 64, 2048, 128, 768, 8

    def mk_expert(n, k):
        e32 = torch.randn((n, k), generator=gen, device="cuda", dtype=torch.float32) * 0.02
        eb = torch.empty(capi.weight_nbytes("q4_K", n, k), dtype=torch.uint8, device="cuda")
        capi.quantize_weights("q4_K", e32, n, k, eb, stream=stream)
        torch.cuda.synchronize()
        return capi.Weight("q4_K", n, k, eb, mem=capi.MEM_DEVICE)

    # two sets of experts (2 x 340 MB) so that consecutive calls do not hit the last-level cache
    sets = [capi.Experts([mk_expert(mi, mh) for _ in range(me)], [mk_expert(mi, mh) for _ in range(me)],
                         [mk_expert(mh, mi) for _ in range(me)]) for _ in range(2)]
    mx = torch.randn((mt, mh), generator=gen, device="cuda")
    ml = torch.randn((mt, me), generator=gen, device="cuda")
    my = torch.empty((mt, mh), device="cuda")
    midx = torch.zeros((mt, mk), dtype=torch.int32, device="cuda")

    def moe_time(tokens, reps=40):
        """Milliseconds per block of `tokens` tokens, and the number of experts they reach."""
        x_, l_, y_, i_ = mx[:tokens], ml[:tokens], my[:tokens], midx[:tokens]
        for i in range(4):
            capi.moe_forward(tokens, mh, mi, me, mk, sets[i % 2], None, None, x_, y_, router_logits=l_,
                             topk_idx=i_, stream=stream)
        torch.cuda.synchronize()
        n_active = int(torch.unique(i_).numel())
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for i in range(reps):
            capi.moe_forward(tokens, mh, mi, me, mk, sets[i % 2], None, None, x_, y_, router_logits=l_,
                             stream=stream)
        ev1.record()
        torch.cuda.synchronize()
        return ev0.elapsed_time(ev1) / reps, n_active

    def moe_graph_time(tokens, reps=20):
        """The same from a captured graph of one call per expert set: the device's time
        without the host's share of the launches."""
        x_, l_, y_ = mx[:tokens], ml[:tokens], my[:tokens]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):   # the first call on a stream allocates its workspace
            capi.moe_forward(tokens, mh, mi, me, mk, sets[0], None, None, x_, y_, router_logits=l_,
                             stream=side.cuda_stream)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for st_ in sets:
                capi.moe_forward(tokens, mh, mi, me, mk, st_, None, None, x_, y_, router_logits=l_,
                                 stream=side.cuda_stream)
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for _ in range(reps):
            graph.replay()
        ev1.record()
        torch.cuda.synchronize()
        return ev0.elapsed_time(ev1) / (reps * len(sets))

    moe_ms, active = moe_time(mt)
    moe_graph_ms = moe_graph_time(mt)
    moe_decode_ms, decode_active = moe_time(1)
    moe_decode_graph_ms = moe_graph_time(1)

    def moe_router_time(tokens, reps=40):
        """The block given the router's weight instead of its logits (the layer API's case)."""
        wr = torch.randn((mh, me), generator=gen, device="cuda") * 0.05
        x_, y_ = mx[:tokens], my[:tokens]
        for i in range(4):
            capi.moe_forward(tokens, mh, mi, me, mk, sets[i % 2], None, None, x_, y_, router_weight=wr, stream=stream)
        torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for i in range(reps):
            capi.moe_forward(tokens, mh, mi, me, mk, sets[i % 2], None, None, x_, y_, router_weight=wr, stream=stream)
        ev1.record()
        torch.cuda.synchronize()
        return ev0.elapsed_time(ev1) / reps

    moe_router_ms, moe_router_decode_ms = moe_router_time(mt), moe_router_time(1)
    moe_bytes = active * 3 * (mi * mh * 144 // 256) + 2 * mt * mh * 4
    moe_gbs = moe_bytes / (moe_ms * 1e-3) / 1e9
    moe_decode_bytes = decode_active * 3 * (mi * mh * 144 // 256) + 2 * mh * 4
    for st_ in sets:
        for lst in st_.weights:
            for w_ in lst:
                w_.destroy()

    # ---- a plain device copy of known size: the yardstick the FETCH_SIZE / WRITE_SIZE
    # counters of a profiled run of this script are scaled by
    src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst

    # ---- the two ceilings, after everything else: for a second or two after milliseconds of nothing but matrix
    # instructions or reads the device serves host copies more slowly (the page-locked C2 call took 0.86-0.98 ms
    # instead of 0.62 ms when it was measured right behind them)
    # what the int8 matrix instruction sustains on this device with nothing else issued
    ceiling_tops, ceiling_ghz = capi.bench_mfma_ceiling(2.0, stream=stream)
    # what a kernel that only reads gets out of device memory (1 GiB, the GEMV kernels' access pattern)
    read_ceiling_gbs = max(capi.bench_hbm_read_ceiling(1 << 30, wps, stream=stream) for wps in (1, 2, 4)) * 1e3

    out = {
        "metric": METRIC, "value": round(value, 3), "unit": "TOPS", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(step_ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "Q4_K x Q8_K prefill GEMM, M=512 K=4096 N=12288 (BASELINE configs[1]); "
                               "step = activation quantizer + block-dot GEMM on HBM-resident inputs; inputs: the "
                               "repository's bit-reproducible generator, stream 1 (weights N(0, 0.02), activations "
                               "N(0, 1) behind them), the data of tests/test_gpu_configs.py::test_c2_q4_K_prefill_gemm",
                   "M": M, "K": K, "N": N, "weight_copies_rotated": n_copies, "input_digest": input_digest},
        "roofline": {"bound": "mfma", "kernel": gemm_kernel_name, "achieved": round(gemm_tops, 3),
                     "peak": INT8_PEAK_TOPS, "unit": "TOP/s", "frac": round(gemm_tops / INT8_PEAK_TOPS, 5),
                     "kernel_ms": round(gemm_ms, 5), "traffic": TRAFFIC_GEMM_C2,
                     "traffic_from": "profiles/gemm_q4k_prefill_m512_k4096_n12288.txt (counter runs; not live)",
                     "algorithmic_ops_per_launch": ops,
                     "mfma_ceiling_tops": round(ceiling_tops, 1), "mfma_ceiling_clock_ghz": round(ceiling_ghz, 3),
                     "frac_of_measured_ceiling": round(gemm_tops / ceiling_tops, 5)},
        "quantizer_ms": round(quant_ms, 5),
        "pcie_inclusive": {"workload": "the same step through hipq_matmul with HIPQ_MEM_HOST operands: 8.4 MB of "
                                       "activations in, 25.2 MB of outputs back, synchronous call, median of 7",
                           "pageable_ms_per_step": round(pageable_ms, 4),
                           "pageable_tops": round(ops / (pageable_ms * 1e-3) / 1e12, 2),
                           "page_locked_ms_per_step": round(pinned_ms, 4),
                           "page_locked_tops": round(ops / (pinned_ms * 1e-3) / 1e12, 2),
                           "decode_row_us": decode_row_us},
        "timing": {"method": "median of 5 blocks; a block is a C loop of `steps` calls of the public hipq_matmul "
                             "(hipq_bench_matmul_loop in libhipq_bench.so, which links libhipq.so) with two HIP "
                             "events on the launch stream around it (synchronize on both sides): ms_per_step; every "
                             "block is followed by the same loop under hipq_launch_timing_begin / _end, where every "
                             "launch carries its own start and stop event: roofline.kernel_ms and quantizer_ms are "
                             "the kernels' own mean durations (median block), ms_per_step - kernel_ms - quantizer_ms "
                             "the time between kernels",
                   "blocks_ms_per_step": [round(b[0], 5) for b in blocks_timed],
                   "blocks_wall_clock_ms_per_step": [round(b[1] * 1e3, 5) for b in blocks_timed],
                   "kernel_timing_blocks_quantizer_plus_kernel_ms": [round(b[0], 5) for b in blocks_instr],
                   "kernel_timing_blocks_kernel_ms": [round(b[2], 5) for b in blocks_instr],
                   "consistent": bool(gemm_ms + quant_ms <= step_ms)},
        "hbm_read_ceiling": {"value": round(read_ceiling_gbs, 1), "unit": "GB/s",
                             "method": "a kernel that only reads 1 GiB of device memory, each wavefront streaming its own "
                                       "consecutive share with four to eight non-temporal 128-bit loads a lane in "
                                       "flight (the next four asked for before the last four are used); the best of "
                                       "one, two and four wavefronts a SIMD, three launches each"},
        "decode_gemv": {"workload": "Q4_K GEMV M=1 K=4096 N=12288, %d weight copies rotated" % n_copies,
                        "value": round(gv_bytes / (gemv_all_ms * 1e-3) / 1e9, 2), "unit": "GB/s",
                        "ms_per_call": round(gemv_all_ms, 5),
                        "cache_hot_kernel_ms": round(gemv_hot_ms, 5),
                        "kernels": {k_: [v_[0], round(v_[1], 5)] for k_, v_ in gemv_kern.items()},
                        "roofline": {"bound": "hbm", "kernel": gemv_kernel_name,
                                     "achieved": round(gemv_gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                     "frac": round(gemv_gbs / HBM_PEAK_GBS, 5),
                                     "frac_of_measured_read_ceiling": round(gemv_gbs / read_ceiling_gbs, 5),
                                     "kernel_ms": round(gemv_ms, 5), "traffic": TRAFFIC_GEMV_C2,
                                     "algorithmic_bytes_per_launch": gv_bytes}},
        "decode_batch_rows": {
            "workload": "Q4_K, 8 and 4 activation rows (a batch of decode steps) against the same M=1 matrices "
                        "(K=4096 N=12288, %d copies rotated); outputs carry the reference's bits" % n_copies,
            "kernel": "gemm_rows_q4k_kernel",
            "rows_8_kernel_ms": round(rows_ms[8][0], 5), "rows_8_ms_per_call": round(rows_ms[8][1], 5),
            "rows_4_kernel_ms": round(rows_ms[4][0], 5), "rows_4_ms_per_call": round(rows_ms[4][1], 5),
            "rows_8_weight_gbs": round(gv_bytes / (rows_ms[8][0] * 1e-3) / 1e9, 2),
            "rows_16_kernel_ms": round(rows_ms[16][0], 5), "rows_16_ms_per_call": round(rows_ms[16][1], 5),
            "rows_64_kernel_ms": round(rows_ms[64][0], 5), "rows_64_ms_per_call": round(rows_ms[64][1], 5),
            "qkv_4096_1024_1024_as_one_call_in_a_graph_ms": {"rows_1": round(q4k_qkv_ms[1], 5),
                                                             "rows_8": round(q4k_qkv_ms[8], 5),
                                                             "rows_16": round(q4k_qkv_ms[16], 5)},
            "note": "16 rows: two passes of the same kernel, still the reference's bits; 64 rows: the prefill GEMM "
                    "in parts of K (one 64-row tile per 128 columns), within 1e-4; qkv: three Q4_K weights of a layer "
                    "through hipq_matmul_multi, one quantization and one launch of the few-rows kernel for all three"},
        "decode_gemv_size_sweep": {
            "workload": "Q4_K GEMV M=1 K=4096 over N = 4096 .. 151936, weight copies of more than twice the last-level "
                        "cache rotated; kernel_ms = the product kernel's own duration (one launch that quantizes the row "
                        "itself below 32768 columns; from there the quantizer is a launch of its own, counted in "
                        "ms_per_call only); frac = algorithmic bytes / kernel_ms / 8 TB/s",
            "points": sweep},
        "decode_gemv_lm_head_size": {
            "workload": "Q4_K GEMV M=1 K=4096 N=151936 (the last point of the sweep), %d weight copies rotated" % sweep[-1]["copies"],
            "roofline": {"bound": "hbm", "kernel": big_kernel_name,
                         "achieved": round(big_gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(big_gbs / HBM_PEAK_GBS, 5),
                         "frac_of_measured_read_ceiling": round(big_gbs / read_ceiling_gbs, 5),
                         "kernel_ms": round(big_ms, 5),
                         "traffic": TRAFFIC_GEMV_LM_HEAD, "algorithmic_bytes_per_launch": big_bytes}},
        "c1_q4_0_gemv": {
            "workload": "Q4_0 GEMV M=1 K=4096 N=4096 (BASELINE configs[0]), 60 weight copies rotated (566 MB)",
            "ms_per_call": round(c1_all_ms, 5),
            "roofline": {"bound": "hbm", "achieved": round(c1_bytes / (c1_ms * 1e-3) / 1e9, 2), "peak": HBM_PEAK_GBS,
                         "unit": "GB/s", "frac": round(c1_bytes / (c1_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 5),
                         "frac_of_measured_read_ceiling": round(c1_bytes / (c1_ms * 1e-3) / 1e9 / read_ceiling_gbs, 5),
                         "kernel_ms": round(c1_ms, 5), "traffic": None, "algorithmic_bytes_per_launch": c1_bytes}},
        "c3_q6_K_lm_head_gemv": {
            "workload": "Q6_K GEMV M=1 K=4096 N=151936 (BASELINE configs[2]), 2 weight copies rotated (1 GB)",
            "ms_per_call": round(c3_all_ms, 5),
            "roofline": {"bound": "hbm", "achieved": round(c3_bytes / (c3_ms * 1e-3) / 1e9, 2), "peak": HBM_PEAK_GBS,
                         "unit": "GB/s", "frac": round(c3_bytes / (c3_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 5),
                         "frac_of_measured_read_ceiling": round(c3_bytes / (c3_ms * 1e-3) / 1e9 / read_ceiling_gbs, 5),
                         "kernel_ms": round(c3_ms, 5), "traffic": None, "algorithmic_bytes_per_launch": c3_bytes}},
        "q6_K_prefill_lm_head_size": {
            "workload": "Q6_K x Q8_K prefill GEMM, M=512 K=4096 N=151936 (the C3 weights against 512 rows), "
                        "2 weight copies rotated",
            "ms_per_call": round(c3_prefill[1], 5),
            "roofline": {"bound": "mfma", "kernel": c3_prefill[2],
                         "achieved": round(2.0 * 512 * 151936 * 4096 / (c3_prefill[0] * 1e-3) / 1e12, 3),
                         "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                         "frac": round(2.0 * 512 * 151936 * 4096 / (c3_prefill[0] * 1e-3) / 1e12 / INT8_PEAK_TOPS, 5),
                         "kernel_ms": round(c3_prefill[0], 5), "traffic": 860.0e6 + 325.8e6,
                         "traffic_from": "profiles/gemm_q6k_prefill_m512_k4096_n151936.txt (counter runs; not live)",
                         "algorithmic_ops_per_launch": 2.0 * 512 * 151936 * 4096}},
        "c5_fc_stack_per_layer": {
            "workload": "the seven Q4_0 FCs of one Qwen3-0.6B-shaped decoder layer (BASELINE configs[4]) through "
                        "hipq_matmul, quantizers included, 8 weight copies rotated per FC",
            "prefill_512_rows_ms": round(c5_prefill_ms, 5),
            "prefill_512_rows_in_a_graph_ms": round(c5_prefill_graph_ms, 5),
            "prefill_512_rows_in_a_graph_qkv_and_gate_up_as_one_call_each_ms": round(c5_prefill_grouped_ms, 5),
            "decode_1_row_ms": round(c5_decode_ms, 5),
            "decode_batch_8_rows_ms": round(c5_rows8_ms, 5), "decode_batch_16_rows_ms": round(c5_rows16_ms, 5),
            "decode_batch_8_rows_in_a_graph_qkv_and_gate_up_as_one_launch_each_ms": round(c5_rows8_grouped_ms, 5),
            "lm_head_q4_0_n151936": {"kernel": "gemv_stream_kernel (one row, behind the quantizer's launch), gemm_rows_q40_kernel (eight rows)",
                                     "rows_1_kernel_ms": round(c5_head_ms, 5), "rows_1_ms_per_call": round(c5_head_all_ms, 5),
                                     "rows_8_kernel_ms": round(c5_head_rows8[0], 5),
                                     "rows_8_ms_per_call": round(c5_head_rows8[1], 5),
                                     "rows_8_weight_gbs": round(c5_head_bytes / (c5_head_rows8[0] * 1e-3) / 1e9, 2)},
            "decode_1_row_in_a_graph_ms": round(c5_graph_ms, 5),
            "decode_1_row_in_a_graph_qkv_and_gate_up_as_one_launch_each_ms": round(c5_graph_grouped_ms, 5),
            "decode_1_row_in_a_graph_qkv_one_launch_up_gate_swiglu_one_launch_ms": round(c5_graph_fused_ms, 5)},
        "c5_whole_model": {
            "workload": "the FCs of all 28 layers of the Qwen3-0.6B-shaped decoder of BASELINE configs[4] (Q4_0; Q, K, V "
                        "as one call, O, gate and up as one call, down), one graph per model copy, two copies replayed "
                        "in turn (the FC weights of one are 248 MB, about the last-level cache); lm_head = the model's "
                        "151936 x 1024 head as a Q4_0 FC on one row",
            "decode_ms_per_token_fcs": round(c5_model_decode_ms, 5),
            "decode_fc_gbs": round(247726080 / (c5_model_decode_ms * 1e-3) / 1e9, 1),
            "decode_roofline": {"bound": "hbm", "achieved": round(247726080 / (c5_model_decode_ms * 1e-3) / 1e9, 1),
                                "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                "frac": round(247726080 / (c5_model_decode_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 5),
                                "algorithmic_bytes_per_token": 247726080, "launches_per_token": 112},
            "decode_ms_per_token_fcs_and_lm_head": round(c5_model_decode_head_ms, 5),
            "decode_fcs_and_lm_head_gbs": round((247726080 + 151936 * 1024 * 18 // 32) / (c5_model_decode_head_ms * 1e-3) / 1e9, 1),
            "prefill_512_ms_fcs_and_lm_head": round(c5_model_prefill_ms, 5),
            "prefill_roofline": {"bound": "mfma", "achieved": round(450971566080 / (c5_model_prefill_ms * 1e-3) / 1e12, 1),
                                 "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                                 "frac": round(450971566080 / (c5_model_prefill_ms * 1e-3) / 1e12 / INT8_PEAK_TOPS, 5),
                                 "algorithmic_ops": 450971566080,
                                 "note": "the lm_head row's time is inside the figure, its ops are not"}},
        "c5_layer_through_plugin": plugin_layer,
        "moe_layer_through_plugin": plugin_moe,
        "moe_block": {
            "workload": "MoE FFN block (BASELINE configs[3]): 64 tokens, hidden 2048, 128 experts x "
                        "(gate/up 2048->768, down 768->2048) Q4_K, top-8; router, sort, experts, combine; "
                        "two expert sets alternated; whole call incl. launches",
            "ms_per_block": round(moe_ms, 5), "ms_per_block_in_a_graph": round(moe_graph_ms, 5),
            "active_experts": active,
            "roofline": {"bound": "hbm", "achieved": round(moe_gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(moe_gbs / HBM_PEAK_GBS, 5),
                         "frac_of_measured_read_ceiling": round(moe_gbs / read_ceiling_gbs, 5),
                         "algorithmic_bytes_per_block": moe_bytes,
                         "traffic": 232.4e6 + 133.2e6 + 11.3e6},
            "decode_token": {"ms_per_block": round(moe_decode_ms, 5),
                             "ms_per_block_in_a_graph": round(moe_decode_graph_ms, 5),
                             "active_experts": decode_active,
                             "gbs": round(moe_decode_bytes / (moe_decode_ms * 1e-3) / 1e9, 2)},
            "from_the_router_weight": {"note": "the same blocks given the router's weight [hidden x experts] instead of its "
                                               "logits: one more launch (router_logits_kernel)",
                                       "ms_per_block": round(moe_router_ms, 5),
                                       "decode_token_ms_per_block": round(moe_router_decode_ms, 5)}},
    }
    if not args.no_cpu:
        capi.matmul(weights[0], a, M, c, stream=stream)
        torch.cuda.synchronize()
        out["cpu_baseline"] = cpu_baseline(blocks.cpu().numpy(), a.cpu().numpy(), c.cpu().numpy())
        out["cpu_baseline_thread_pool"] = cpu_baseline_thread_pool(blocks.cpu().numpy(), a.cpu().numpy())
        out["cpu_baseline_gemv"] = {
            "c1_q4_0_m1_k4096_n4096": cpu_gemv_baseline("q4_0", 4096, 4096, c1_host, c1_bytes),
            "c3_q6_K_m1_k4096_n151936": cpu_gemv_baseline("q6_K", 151936, 4096, c3_host, c3_bytes)}
    for w in weights:
        w.destroy()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
