#!/usr/bin/env python3
"""Benchmark of the ternary BitLinear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--m M]

One "step" is one pass of the hot path over the BitLinear stack of a
BitNet-b1.58-2B decoder at M tokens (default 1): 30 layers x (wqkv, wo, w13,
w2), each call = BitLinearKernel.forward of the reference (gpu/model.py:73-75:
absmax quantizer, int8 x int2 product, scale epilogue), which the library runs
as ONE kernel per call at decode sizes.  Every layer has its own weights
(521 MB of packed weights per step, so the stream comes from HBM, not from
cache).  The 120 launches of a step are replayed from a HIP graph, as the
reference replays its decode step from a CUDA graph (gpu/generate.py:198-211).
Inputs are resident in HBM before timing starts.

Prints ONE JSON line.  `value` is packed-weight bytes (K*N/4 per product) per
second over the whole step.  `roofline` is for the kernel those launches run
(bitlinear_solo_kernel): the same timed region, measured with HIP events on
the stream the graph is replayed on, divided by the 120 launches of a step.
`cpu_baseline` is the C restatement of the reference's CPU I2_S kernel timed
on this host on a bounded sample of the same workload.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "M=1 ternary GEMV HBM GB/s (% of peak) + decode tokens/s, BitNet-2B shapes"
HBM_PEAK_GBPS = 8000.0


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def build_workload(M, device):
    """Weights of 30 layers (seeded, generated and packed on the GPU),
    per-shape weight scales and bf16 activations."""
    import numpy as np
    import torch

    from bitnet_amd import pack_weight, workload

    shapes = workload.shapes_2b()
    gen = torch.Generator(device=device)
    layers = []
    for layer in range(workload.N_LAYERS_2B):
        row = []
        for sh in shapes:
            gen.manual_seed(workload.SEED_W + sh.shape_id + 16 * layer)
            u = torch.rand(sh.N, sh.K, generator=gen, device=device)
            w = (u >= 0.7).to(torch.int8) - (u < 0.3).to(torch.int8)  # P(-1)=P(+1)=0.3
            row.append(pack_weight.convert_weight_int8_to_int2(w, keep_device=True))
            del u, w
        layers.append(row)
    scales, acts = [], []
    for sh in shapes:
        ws = workload.weight_scales(sh.K, sh.N, sh.shape_id, sh.parts)
        scales.append(torch.from_numpy(ws.view(np.int16).copy()).view(torch.bfloat16).to(device))
        xb = workload.activations_bf16(M, sh.K, sh.shape_id)
        acts.append(torch.from_numpy(xb.view(np.int16).copy()).view(torch.bfloat16).to(device))
    return shapes, layers, scales, acts


class GraphRun:
    """Captures `launch(stream_ptr)` into a HIP graph on its own stream and
    times replays with HIP events recorded on that stream."""

    def __init__(self, launch):
        import torch

        self.torch = torch
        self.stream = torch.cuda.Stream()
        self.stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(self.stream):
            sp = ctypes.c_void_p(self.stream.cuda_stream)
            launch(sp)  # eager once: first-use costs stay out of the graph
            self.stream.synchronize()
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph, stream=self.stream):
                launch(sp)
        self.stream.synchronize()

    def replay(self, n):
        with self.torch.cuda.stream(self.stream):
            for _ in range(n):
                self.graph.replay()

    def timed(self, n):
        """(wall seconds, event milliseconds) for n replays."""
        torch = self.torch
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        with torch.cuda.stream(self.stream):
            e0.record(self.stream)
            for _ in range(n):
                self.graph.replay()
            e1.record(self.stream)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        return t1 - t0, e0.elapsed_time(e1)


def per_shape_forward(lib, shapes, layers, scales, acts, q_buf, s_buf, o_buf, dev, M, reps=12):
    """The forward kernel per 2B shape, HBM-cold and cache-hot.  Cold: a graph of the 30 layers' calls of
    one shape (30 distinct weight matrices), every timed replay behind a pass that rewrites 768 MiB of
    other memory, so neither the 256 MB last-level cache nor the L2s hold any of the weights when the
    replay starts (the smaller shapes' 30 matrices would otherwise stay resident between replays).
    Hot: 30 calls on ONE layer's matrix (1.6-8.8 MB: it stays in the L2s).  HIP events on the replay
    stream, median and minimum over the replays, per launch."""
    import torch

    flush = torch.zeros(768 << 20, dtype=torch.uint8, device=dev)
    out = {}
    for i, sh in enumerate(shapes):
        def calls(rows, i=i, sh=sh):
            def fn(sp):
                for w in rows:
                    st = lib.bitlinear_forward_bf16(
                        _p(acts[i]), _p(w), _p(o_buf[i]), _p(scales[i]), _p(q_buf[i]), _p(s_buf[i]), M, sh.N, sh.K, 0, sp
                    )
                    assert st == 0, lib.bitlinear_status_string(st)
            return fn

        rows = [row[i] for row in layers]
        leg = {"K": sh.K, "N": sh.N, "bytes_per_launch": sh.weight_bytes}
        for tag, g, cold in (("hbm_cold", GraphRun(calls(rows)), True), ("cache_hot", GraphRun(calls([rows[0]] * len(rows))), False)):
            g.replay(3)
            times = []
            for _ in range(reps):
                if cold:
                    flush.add_(1)
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                with torch.cuda.stream(g.stream):
                    e0.record(g.stream)
                    g.graph.replay()
                    e1.record(g.stream)
                torch.cuda.synchronize()
                times.append(e0.elapsed_time(e1) * 1e3 / len(rows))
            times.sort()
            med = times[len(times) // 2]
            leg[tag] = {
                "us_per_launch": round(med, 3),
                "min_us_per_launch": round(times[0], 3),
                "achieved_GBps": round(sh.weight_bytes / (med * 1e-6) / 1e9, 1),
                "frac": round(sh.weight_bytes / (med * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
            }
            del g
        out[sh.name] = leg
    del flush
    return out


def cpu_baseline(shapes, M, budget_s=12.0):
    """C restatement of the reference's CPU I2_S path on this host, in the shape of the reference's own
    harness (utils/test_gemm_kernel.sh:338-348, 501-563: warm-ups, then the mean over timed iterations of one
    matrix product, built -O3 -march=native with OpenMP): per 2B shape at M tokens, 10 warm-ups and 200 timed
    calls, on one thread and on all the threads this job may use, rotating over 8 layers of distinct weights
    so that the stream comes from DRAM; one leg through the four-rows-at-a-time kernel (_Nx1) at 128 tokens;
    and the aggregate over the 8-layer sample that `value` reports."""
    import numpy as np

    from bitnet_amd import workload
    from oracle import bitlinear_oracle as o
    from oracle import i2s_cpu

    host_cpus = os.cpu_count() or 1
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = host_cpus
    threads = max(1, min(usable, 16))  # 16 = the CPU share of a one-GPU job on the measurement machines
    build = i2s_cpu.use_native_build()  # rebuilt here with -march=native when a compiler is present
    n_layers = 8  # distinct weights per layer: 139 MB of packed weights, streamed from DRAM like the GPU's from HBM
    cases = {sh.name: [] for sh in shapes}
    for layer in range(n_layers):
        for sh in shapes:
            w = workload.ternary_weight(sh.K, sh.N, sh.shape_id, layer)
            q, _ = o.quant_input(workload.activations_bf16(M, sh.K, sh.shape_id))
            cases[sh.name].append((i2s_cpu.pack(w), q, np.empty((M, sh.N), dtype=np.int32), np.empty((M, sh.N), dtype=np.float32)))
    layer_bytes = sum(sh.weight_bytes for sh in shapes) * n_layers

    def call(case, nt):
        packed, q, acc, tmp = case
        i2s_cpu.bitlinear_acc(packed, q, nt, tmp=tmp, acc=acc)

    # per shape, the reference harness's protocol
    per_shape = {}
    for sh in shapes:
        leg = {"K": sh.K, "N": sh.N}
        for tag, nt in (("threads_1", 1), (f"threads_{threads}", threads)):
            cs = cases[sh.name]
            for it in range(10):
                call(cs[it % n_layers], nt)
            ts = []
            for it in range(200):
                t0 = time.perf_counter()
                call(cs[it % n_layers], nt)
                ts.append(time.perf_counter() - t0)
            mean, mn = sum(ts) / len(ts), min(ts)
            leg[tag] = {"mean_us": round(mean * 1e6, 2), "min_us": round(mn * 1e6, 2), "iterations": len(ts),
                        "weight_GBps": round(sh.weight_bytes / mean / 1e9, 2)}
        per_shape[sh.name] = leg

    # M = 128 through the kernel that shares each decoded weight block between four activation rows
    nx1 = {}
    Mp = 128
    for sh in shapes:
        packed = cases[sh.name][0][0]
        q, _ = o.quant_input(workload.activations_bf16(Mp, sh.K, sh.shape_id, outliers=True))
        acc, tmp = np.empty((Mp, sh.N), dtype=np.int32), np.empty((Mp, sh.N), dtype=np.float32)
        i2s_cpu.bitlinear_acc(packed, q, threads, tmp=tmp, acc=acc)
        ts, t_start = [], time.perf_counter()
        while len(ts) < 20 and (len(ts) < 3 or time.perf_counter() - t_start < budget_s * 0.08):
            t0 = time.perf_counter()
            i2s_cpu.bitlinear_acc(packed, q, threads, tmp=tmp, acc=acc)
            ts.append(time.perf_counter() - t0)
        mean = sum(ts) / len(ts)
        nx1[sh.name] = {"mean_us": round(mean * 1e6, 1), "min_us": round(min(ts) * 1e6, 1), "iterations": len(ts),
                        "TOPS": round(2.0 * Mp * sh.N * sh.K / mean / 1e12, 3)}

    def one_pass(nt):  # one pass over the n_layers sample
        for layer in range(n_layers):
            for sh in shapes:
                call(cases[sh.name][layer], nt)

    out = {}
    for tag, nt, share in (("threads", threads, 0.35), ("single", 1, 0.25)):
        one_pass(nt)  # warm-up
        n, t0 = 0, time.perf_counter()
        while True:
            one_pass(nt)
            n += 1
            el = time.perf_counter() - t0
            if el > budget_s * share:
                break
        out[tag] = (layer_bytes * n / el / 1e9, n, el)
    return {
        "value": round(out["threads"][0], 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": (
            f"{n_layers} decoder layers with distinct weights (wqkv, wo, w13, w2 each; {layer_bytes} packed-weight "
            f"bytes per pass) at M={M}, {out['threads'][1]} passes in {out['threads'][2]:.1f} s on {threads} threads; "
            f"C/AVX2 restatement of ggml_vec_dot_i2_i8_s + explicit -sum(y) correction"
        ),
        "threads": {"single": 1, "all": threads, "host_cpu_count": host_cpus, "usable_by_this_process": usable,
                    "cap": "16 threads: the CPU share of a one-GPU job on the measurement machines"},
        "build": build,
        "single_thread_GBps": round(out["single"][0], 3),
        "tokens_per_s_bitlinear_only": round(out["threads"][0] * 1e9 / (layer_bytes / n_layers * 30), 2),
        "per_shape": per_shape,
        "per_shape_protocol": "per shape and thread count: 10 warm-up calls, then 200 timed calls of one BitLinear product "
                              "(_1x1 kernel per weight row, rows split over the threads), each on the next of 8 layers' weights",
        "M128_Nx1": nx1,
        "M128_Nx1_protocol": f"one product at 128 tokens (1 % outliers x20) on {threads} threads through the _Nx1 kernel "
                             "(PARALLEL_SIZE 4, tiles of 4 rows x 128 columns), 1 warm-up, 3 to 20 timed calls within the time budget",
    }


INT8_MFMA_PEAK_TOPS = 5000.0


def _acts(M, sh, dev, outliers=False):
    import numpy as np
    import torch

    from bitnet_amd import workload

    xb = workload.activations_bf16(M, sh.K, sh.shape_id, outliers=outliers)
    return torch.from_numpy(xb.view(np.int16).copy()).view(torch.bfloat16).to(dev)


def batched_and_prefill(lib, shapes, layers, scales, dev, decode_ms=(2, 4, 8, 16), prefill_ms=(128, 512, 2048)):
    """The other token counts the workload names, on the same 30 layers of
    weights: batched decode (every row its own absmax scale) through the whole
    forward call, and prefill with 1 % of the activations scaled x20, as the
    whole forward call (quantizer kernel + int8 MFMA GEMM) and as the GEMM alone."""
    import torch

    step_bytes = sum(sh.weight_bytes for sh in shapes) * len(layers)
    n_calls = len(shapes) * len(layers)
    out = {"batched_decode": {}, "prefill": {}}
    for M in decode_ms:
        acts = [_acts(M, sh, dev) for sh in shapes]
        o_buf = [torch.empty(M, sh.N, dtype=torch.bfloat16, device=dev) for sh in shapes]
        q_buf = [torch.empty(M, sh.K, dtype=torch.int8, device=dev) for sh in shapes]
        s_buf = [torch.empty(M, dtype=torch.bfloat16, device=dev) for sh in shapes]

        def launch(sp):
            for row in layers:
                for i, sh in enumerate(shapes):
                    st = lib.bitlinear_forward_bf16(
                        _p(acts[i]), _p(row[i]), _p(o_buf[i]), _p(scales[i]), _p(q_buf[i]), _p(s_buf[i]), M, sh.N, sh.K, 0, sp
                    )
                    assert st == 0, lib.bitlinear_status_string(st)

        g = GraphRun(launch)
        g.replay(5)
        _, ms = g.timed(50)
        us = ms * 1e3 / (50 * n_calls)
        out["batched_decode"][f"M{M}"] = {
            "us_per_call": round(us, 3),
            "weight_GBps": round(step_bytes / n_calls / (us * 1e-6) / 1e9, 1),
            "frac_of_hbm_peak": round(step_bytes / n_calls / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
            "bitlinear_tokens_per_s": round(M / (us * 1e-6 * n_calls), 1),
        }
        del g
    for M in prefill_ms:
        per = {}
        tot_ops, tot_us, tot_fwd_us = 0.0, 0.0, 0.0
        for i, sh in enumerate(shapes):
            x = _acts(M, sh, dev, outliers=True)
            q = torch.empty(M, sh.K, dtype=torch.int8, device=dev)
            s = torch.empty(M, dtype=torch.bfloat16, device=dev)
            o = torch.empty(M, sh.N, dtype=torch.bfloat16, device=dev)
            rows = [row[i] for row in layers]

            def fwd(sp):
                for w in rows:
                    st = lib.bitlinear_forward_bf16(_p(x), _p(w), _p(o), _p(scales[i]), _p(q), _p(s), M, sh.N, sh.K, 0, sp)
                    assert st == 0, lib.bitlinear_status_string(st)

            def gemm(sp):
                for w in rows:
                    lib.bitlinear_int8xint2(_p(q), _p(w), _p(o), _p(s), _p(scales[i]), M, sh.N, sh.K, sp)
                    assert lib.bitlinear_last_status() == 0

            res = []
            for fn in (fwd, gemm):  # fwd first: it fills q and s for the GEMM alone
                g = GraphRun(fn)
                g.replay(2)
                _, ms = g.timed(5)
                res.append(ms * 1e3 / (5 * len(rows)))
                del g
            ops = 2.0 * M * sh.N * sh.K
            per[sh.name] = {
                "forward_us": round(res[0], 2),
                "gemm_us": round(res[1], 2),
                "gemm_TOPS": round(ops / (res[1] * 1e-6) / 1e12, 1),
                "forward_TOPS": round(ops / (res[0] * 1e-6) / 1e12, 1),
            }
            tot_ops += ops
            tot_us += res[1]
            tot_fwd_us += res[0]
        tops = tot_ops / (tot_us * 1e-6) / 1e12
        vendor = vendor_int8_gemm(shapes, M, dev) if M >= 512 else None
        out["prefill"][f"M{M}"] = {
            **({"vendor_int8_gemm": vendor} if vendor else {}),
            "per_shape": per,
            "layer_gemm_TOPS": round(tops, 1),
            "layer_forward_TOPS": round(tot_ops / (tot_fwd_us * 1e-6) / 1e12, 1),
            "roofline": {"bound": "mfma", "achieved": round(tops, 1), "peak": INT8_MFMA_PEAK_TOPS, "unit": "TOP/s",
                         "frac": round(tops / INT8_MFMA_PEAK_TOPS, 4), "kernel": "gemm_i2_prefill_dma_kernel and gemm_i2_prefill_mix_kernel (gemm_i2_prefill_kernel for the small tiles with k-groups), the four 2B shapes of one layer"},
            "prefill_tokens_per_s_bitlinear_only": round(M / (tot_fwd_us * 1e-6 * len(layers)), 1),
        }
    return out


def vendor_int8_gemm(shapes, M, dev, reps=20):
    """For scale, not part of the product: the platform library's int8 x int8 -> int32 GEMM (torch._int_mm) on
    the same four shapes, with the ternary weights already expanded to one byte each (four times the weight
    bytes of the packed form, no 2-bit decode, no scaling epilogue, int32 outputs), the faster of its two
    operand layouts per shape.  Not fatal when the library refuses a shape."""
    import torch

    per, tot_us, tot_ops = {}, 0.0, 0.0
    try:
        for sh in shapes:
            a = torch.randint(-127, 128, (M, sh.K), dtype=torch.int8, device=dev)
            best = None
            for b in (torch.randint(-1, 2, (sh.K, sh.N), dtype=torch.int8, device=dev),
                      torch.randint(-1, 2, (sh.N, sh.K), dtype=torch.int8, device=dev).t()):
                for _ in range(3):
                    torch._int_mm(a, b)
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(reps):
                    torch._int_mm(a, b)
                e1.record()
                torch.cuda.synchronize()
                us = e0.elapsed_time(e1) * 1e3 / reps
                best = us if best is None else min(best, us)
            per[sh.name] = round(best, 2)
            tot_us += best
            tot_ops += 2.0 * M * sh.N * sh.K
    except Exception as e:  # a measurement for comparison only
        return {"error": f"{type(e).__name__}: {str(e)[:160]}"}
    return {"what": "torch._int_mm (int8 weights, int32 out), us per call, eager launches back to back", "per_shape_us": per,
            "layer_TOPS": round(tot_ops / (tot_us * 1e-6) / 1e12, 1)}


def mfma_ceiling(lib, dev, iters=20000):
    """What v_mfma_i32_32x32x32_i8 sustains on this machine in a register-only
    loop (bitlinear_probe_mfma_i8: three waves per SIMD, no memory traffic), for
    all-zero operands and for the operand values of this workload (random int8
    activations x random ternary codes, changing with every MFMA): the rate
    depends on the values, because switching activity decides the power the
    pipe draws and the clock it gets.  HIP events, best of 3 launches of about
    20 to 30 ms each."""
    import ctypes

    import torch

    out = {"how": "register-only loop of v_mfma_i32_32x32x32_i8, 3 waves per SIMD on every CU, HIP events, best of 3"}
    for mode, name in ((0, "zero_operands_TOPS"), (1, "random_int8_x_ternary_codes_TOPS")):
        ops = ctypes.c_longlong(0)
        best = None
        for _ in range(4):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            st = lib.bitlinear_probe_mfma_i8(mode, iters, None, ctypes.byref(ops), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
            e1.record()
            torch.cuda.synchronize()
            assert st == 0
            ms = e0.elapsed_time(e1)
            best = ms if best is None else min(best, ms)
        out[name] = round(ops.value / (best * 1e-3) / 1e12, 1)
    out["nominal_peak_TOPS"] = INT8_MFMA_PEAK_TOPS
    return out


def large_shapes(lib, dev, budget_bytes=1 << 30):
    """The other (N, K) of the reference's dispatch table (bitnet_kernels.cu:4-33:
    the 3B-class and the largest shapes) at M = 1 through the drop-in entry
    bitlinear_int8xint2: random packed bytes (timing only), rotating over about
    1 GiB of distinct weight copies so that nothing is cache-hot, 60 dependent
    launches replayed from a HIP graph."""
    import torch

    out = {}
    for (N, K) in ((4800, 3200), (3200, 3200), (20480, 3200), (3200, 10240), (5120, 27648), (55296, 5120)):
        nbytes = N * K // 4
        copies = max(2, min(64, budget_bytes // nbytes))
        w = torch.randint(0, 255, (copies, nbytes), dtype=torch.uint8, device=dev)
        a = torch.randint(-127, 128, (1, K), dtype=torch.int8, device=dev)
        s = torch.ones(1, dtype=torch.bfloat16, device=dev)
        ws = torch.ones(8, dtype=torch.bfloat16, device=dev)
        o = torch.empty(1, N, dtype=torch.bfloat16, device=dev)
        nl = 60

        def launch(sp):
            for i in range(nl):
                wp = ctypes.c_void_p(w.data_ptr() + (i % copies) * nbytes)
                lib.bitlinear_int8xint2(_p(a), wp, _p(o), _p(s), _p(ws), 1, N, K, sp)
                if lib.bitlinear_last_status() != 0:
                    raise RuntimeError(f"bitlinear_int8xint2 rejected N={N} K={K}")

        kernel_name = []

        def launch_and_name(sp):
            launch(sp)
            kernel_name[:] = [lib.bitlinear_last_kernel().decode()]

        sink = torch.zeros(4, dtype=torch.int32, device=dev)

        def launch_probe(sp):  # the same bytes, requested and dropped
            for i in range(nl):
                arr = (ctypes.c_void_p * 1)(w.data_ptr() + (i % copies) * nbytes)
                if lib.bitlinear_probe_weight_stream(arr, 1, N, K, _p(sink), sp) != 0:
                    raise RuntimeError(f"bitlinear_probe_weight_stream rejected N={N} K={K}")

        run = GraphRun(launch_and_name)
        run.replay(3)
        best = min(run.timed(5)[1] / 5 for _ in range(3)) * 1e3 / nl  # us per launch
        del run
        run = GraphRun(launch_probe)
        run.replay(3)
        floor = min(run.timed(5)[1] / 5 for _ in range(3)) * 1e3 / nl
        out[f"{N}x{K}"] = {
            "us_per_launch": round(best, 2),
            "weight_GBps": round(nbytes / best / 1e3, 1),
            "frac_of_hbm_peak": round(nbytes / best / 1e3 / HBM_PEAK_GBPS, 4),
            "weight_bytes": nbytes,
            "kernel": kernel_name[0],
            "load_only_us_per_launch": round(floor, 2),
            "load_only_frac_of_hbm_peak": round(nbytes / floor / 1e3 / HBM_PEAK_GBPS, 4),
            "frac_of_load_only": round(floor / best, 4),
        }
        del run, w
        torch.cuda.empty_cache()
    return {"large_shapes_product_only": out}


def latency_floor(lib, shapes, layers, dev, n_timed=20):
    """What a dependent launch costs on this machine before any BitLinear
    arithmetic, measured in the same run and the same way as the headline (a HIP
    graph of 120 launches on one stream, replayed; HIP events on that stream;
    the weights of 30 layers, so nothing is cache-hot): a kernel with an empty
    body (one wave, and with the product's grid), and a kernel that only
    requests one call's packed weights and drops them (per 2B shape)."""
    import torch

    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    n_layers = len(layers)

    def timed_us(fn, launches):
        g = GraphRun(fn)
        g.replay(3)
        us = min(g.timed(n_timed)[1] / n_timed for _ in range(3)) * 1e3 / launches
        del g
        return us

    def empty(blocks, threads):
        def fn(sp):
            for _ in range(4 * n_layers):
                assert lib.bitlinear_probe_empty(blocks, threads, sp) == 0
        return fn

    out = {
        "how": "HIP graph of 120 dependent launches on one stream (as the headline), HIP events, min of 3 x %d replays" % n_timed,
        "empty_kernel_us": {"1x64": round(timed_us(empty(1, 64), 4 * n_layers), 3)},
        "load_only_us": {},
        "hbm_time_at_peak_us": {},
    }
    for sh in shapes:
        out["empty_kernel_us"][f"{sh.N // 16}x512 ({sh.name} grid)"] = round(timed_us(empty(sh.N // 16, 512), 4 * n_layers), 3)
    tot_floor = 0.0
    for i, sh in enumerate(shapes):
        def fn(sp, i=i, sh=sh):
            for rep in range(4):
                for row in layers:
                    arr = (ctypes.c_void_p * 1)(row[i].data_ptr())
                    assert lib.bitlinear_probe_weight_stream(arr, 1, sh.N, sh.K, _p(sink), sp) == 0
        us = timed_us(fn, 4 * n_layers)
        tot_floor += us
        out["load_only_us"][sh.name] = round(us, 3)
        out["hbm_time_at_peak_us"][sh.name] = round(sh.weight_bytes / HBM_PEAK_GBPS / 1e3, 3)
    step_bytes = sum(sh.weight_bytes for sh in shapes) * n_layers
    out["load_only_us"]["mean_of_the_four"] = round(tot_floor / len(shapes), 3)
    out["load_only_chain_GBps"] = round(step_bytes / (tot_floor * n_layers) / 1e3, 1)
    out["load_only_chain_frac_of_hbm_peak"] = round(step_bytes / (tot_floor * n_layers) / 1e3 / HBM_PEAK_GBPS, 4)
    # what handing a flag from one workgroup to another inside a launch costs (two workgroups of one launch pass a
    # counter back and forth with relaxed device-scope accesses): the price of any producer -> consumer step that
    # would replace a kernel boundary
    flags = torch.zeros(128, dtype=torch.int32, device=dev)
    gave_up = torch.zeros(1, dtype=torch.int32, device=dev)
    rounds = 2000
    trips = {}
    for label, (wa, wb) in {"same_xcd (workgroups 0 and 8)": (0, 8), "next_xcd (0 and 1)": (0, 1), "far_xcd (0 and 4)": (0, 4)}.items():
        best, failed = None, None
        gave_up.zero_()  # per pair, so that a bounded wait that ran out is attributed to the pair it happened in
        for _ in range(3):
            flags.zero_()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            st = lib.bitlinear_probe_flag_roundtrip(_p(flags), wa, wb, rounds, _p(gave_up), None)
            e1.record()
            torch.cuda.synchronize()
            if st != 0:
                failed = f"probe refused: status {st}"
                break
            us = e0.elapsed_time(e1) * 1e3 / rounds
            best = us if best is None else min(best, us)
        if failed is None and int(gave_up[0]) != 0:
            failed = "a flag never arrived within the probe's bounded wait"
        trips[label] = {"error": failed} if failed else round(best, 3)
    out["flag_round_trip_us"] = trips
    out["note"] = (
        "flag_round_trip = bitlinear_probe_flag_roundtrip (launch duration / 2000 round trips, one launch: its own start "
        "and end weigh less than a nanosecond per trip); "
        "load_only = bitlinear_probe_weight_stream: the streaming kernel's grid, 16-byte loads and software pipeline with "
        "the activation operand, the decode, the MFMAs and the output removed; the chain figure is what 120 such launches "
        "per step would stream: the ceiling of any per-call kernel in a dependent chain on this machine"
    )
    return {"latency_floor": out}


def grouped_launches(lib, shapes, layers, scales, dev, M=1):
    """bitlinear_int8xint2_grouped: the 30 layers' products of one 2B shape in ONE
    launch (independent problems: their own int8 rows, scales and outputs), and
    the same bytes through the load-only probe.  What the kernels stream when
    the cost of starting a kernel is paid once per 49-265 MB instead of once per
    1.6-8.8 MB."""
    import torch

    from bitnet_amd import _lib

    out = {}
    L = len(layers)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    for i, sh in enumerate(shapes):
        a = torch.randint(-127, 128, (L, M, sh.K), dtype=torch.int8, device=dev)
        s = torch.full((L, M), 3.0, dtype=torch.bfloat16, device=dev)
        o = torch.empty(L, M, sh.N, dtype=torch.bfloat16, device=dev)
        nbytes = sh.weight_bytes * L
        # enough further sets of 30 weights (random bytes: timing only) that a replay streams at least 600 MB
        # of distinct weights: nothing is left in the 256 MB last-level cache when a set comes round again
        sets = max(1, -(-(600 << 20) // nbytes))
        extra = torch.randint(0, 255, (sets - 1, L, sh.weight_bytes), dtype=torch.uint8, device=dev) if sets > 1 else None

        def wptr(k, l):
            return layers[l][i].data_ptr() if k == 0 else extra[k - 1, l].data_ptr()

        arrs, ptrs = [], []
        for k in range(sets):
            arr = (_lib.Problem * L)()
            pp = (ctypes.c_void_p * L)()
            for l in range(L):
                arr[l] = _lib.Problem(a[l].data_ptr(), wptr(k, l), o[l].data_ptr(), s[l].data_ptr(), scales[i].data_ptr(),
                                      M, sh.N, sh.K)
                pp[l] = wptr(k, l)
            arrs.append(arr)
            ptrs.append(pp)
        name = []

        def fn(sp):
            for arr in arrs:
                st = lib.bitlinear_int8xint2_grouped(arr, L, sp)
                assert st == 0, lib.bitlinear_status_string(st)
            name[:] = [lib.bitlinear_last_kernel().decode()]

        def probe(sp):
            for pp in ptrs:
                assert lib.bitlinear_probe_weight_stream(pp, L, sh.N, sh.K, _p(sink), sp) == 0

        res = []
        for f in (fn, probe):
            g = GraphRun(f)
            g.replay(3)
            res.append(min(g.timed(10)[1] / 10 for _ in range(3)) * 1e3 / sets)
            del g
        out[sh.name] = {
            "problems_per_launch": L,
            "bytes_per_launch": nbytes,
            "us_per_launch": round(res[0], 2),
            "weight_GBps": round(nbytes / res[0] / 1e3, 1),
            "frac_of_hbm_peak": round(nbytes / res[0] / 1e3 / HBM_PEAK_GBPS, 4),
            "kernel": name[0],
            "load_only_us_per_launch": round(res[1], 2),
            "load_only_frac_of_hbm_peak": round(nbytes / res[1] / 1e3 / HBM_PEAK_GBPS, 4),
            "launches_per_replay": sets,
        }
        del extra
        torch.cuda.empty_cache()
    return {f"grouped_launch_M{M}": out}


def end_to_end_decode(batches=(1, 8), prompt_len=512, gen_len=128):
    """Random-init BitNet-b1.58-2B-shaped decoder (30 layers, dim 2560, ffn 6912,
    20/5 heads, vocab 128256, tied bf16 embedding / LM head): a seeded 512-token
    random-id prompt, then greedy decode steps replayed from a HIP graph;
    tokens/s over the decode phase (as gpu/generate.py:264-288 counts it)."""
    import torch

    from bitnet_amd import decoder

    dev = torch.device("cuda:0")
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(dev):
            model = decoder.Transformer(decoder.ModelArgs())
    finally:
        torch.set_default_dtype(prev)
    decoder.random_init_(model, seed=0)
    out = {}
    for B in batches:
        gen = decoder.Generator(model, B, prompt_len + gen_len + 1, use_graph=True)
        g = torch.Generator(device=dev).manual_seed(1234 + B)
        prompt = torch.randint(0, model.args.vocab_size, (B, prompt_len), generator=g, device=dev)
        gen.prefill(prompt)  # untimed: first use of every kernel and library involved
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        first = gen.prefill(prompt)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        gen.decode(first, prompt_len, 4)  # captures the graph, warms up
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        toks = gen.decode(first, prompt_len, gen_len - 1)
        torch.cuda.synchronize()
        t3 = time.perf_counter()
        a = model.args
        hd = a.dim // a.n_heads
        # bytes a decode step must move at least: every packed weight matrix once, the bf16 LM head (the tied
        # embedding) once, and the cache rows 0 .. position of every layer (k and v) for every sequence
        w_bytes = a.n_layers * ((a.dim + 2 * a.n_kv_heads * hd) * a.dim + a.dim * a.dim + 2 * a.ffn_dim * a.dim + a.dim * a.ffn_dim) // 4
        lm_bytes = a.vocab_size * a.dim * 2
        mean_pos = prompt_len + (gen_len - 1) / 2.0
        kv_bytes = int(B * a.n_layers * 2 * a.n_kv_heads * hd * 2 * mean_pos)
        step_s = (t3 - t2) / (gen_len - 1)
        step_gbps = (w_bytes + lm_bytes + kv_bytes) / step_s / 1e9
        out[f"batch{B}"] = {
            "decode_tokens_per_s": round(B * (gen_len - 1) / (t3 - t2), 1),
            "ms_per_decode_step": round((t3 - t2) * 1e3 / (gen_len - 1), 4),
            "roofline": {"bound": "hbm", "achieved": round(step_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": round(step_gbps / HBM_PEAK_GBPS, 4),
                         "bytes_per_step": {"packed_weights": w_bytes, "lm_head_bf16": lm_bytes, "kv_cache_mean": kv_bytes},
                         "what": "one whole decode step (all launches of the captured graph), wall clock over the decode phase"},
            "prefill_tokens_per_s": round(B * prompt_len / (t1 - t0), 1),
            "prompt_len": prompt_len,
            "generated": gen_len,
            "distinct_tokens_generated": int(torch.unique(toks).numel()),
        }
        del gen
    out["generation_latency_ms"] = generation_latency(model, dev)
    del model
    torch.cuda.empty_cache()
    return out


def generation_latency(model, dev, inputs=(64, 256, 512), outputs=(16, 32, 64)):
    """The reference's published end-to-end table (gpu/README.md:93-105: input length x output length,
    one sequence): wall-clock milliseconds from the prompt's token ids to the last generated token --
    prefill of the whole prompt, then output - 1 greedy decode steps replayed from the captured graph
    (the first token comes out of the prefill).  Same random-init 2B decoder as above; the graph is
    captured and every kernel has run once before anything is timed."""
    import torch

    from bitnet_amd import decoder

    table = {}
    gen = decoder.Generator(model, 1, max(inputs) + max(outputs) + 1, use_graph=True)
    g = torch.Generator(device=dev).manual_seed(4321)
    warm = torch.randint(0, model.args.vocab_size, (1, 8), generator=g, device=dev)
    gen.decode(gen.prefill(warm), 8, 2)  # captures the decode graph
    for P in inputs:
        prompt = torch.randint(0, model.args.vocab_size, (1, P), generator=g, device=dev)
        gen.prefill(prompt)  # first use of the prompt-size kernels at this length
        for G in outputs:
            best = None
            for _ in range(3):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                first = gen.prefill(prompt)
                gen.decode(first, P, G - 1)
                torch.cuda.synchronize()
                dt = (time.perf_counter() - t0) * 1e3
                best = dt if best is None else min(best, dt)
            table[f"in{P}_out{G}"] = round(best, 3)
    del gen
    return {"batch": 1, "how": "prefill + (output - 1) graph-replayed greedy steps, wall clock, best of 3", **table}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--m", type=int, default=1, help="tokens per step (decode batch), 1..16")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--no-e2e", action="store_true", help="skip the end-to-end 2B decode measurement")
    ap.add_argument("--e2e-only", action="store_true", help="only the end-to-end 2B decode measurement (for profiler runs)")
    ap.add_argument(
        "--prefill-probe",
        action="store_true",
        help="counter run for `rocprofv3 --pmc`: the prefill GEMM (drop-in entry, M=2048) once per 2B shape, then exit",
    )
    ap.add_argument("--no-sweeps", action="store_true", help="skip the batched-decode (M=2..16) and prefill (M=128..2048) figures")
    ap.add_argument(
        "--pmc-probe",
        action="store_true",
        help="counter run for `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE`: three plain 256 MiB device copies "
        "(calibration) and one eager pass of the 120 GEMV launches, then exit",
    )
    args = ap.parse_args()
    if args.gpus != 1:
        print(
            "bench.py: this build measures one GPU only (the BitLinear path needs no second GPU); "
            f"--gpus {args.gpus} is not supported",
            file=sys.stderr,
        )
        sys.exit(2)

    import torch

    from bitnet_amd import _lib

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path is the only path", file=sys.stderr)
        sys.exit(1)
    lib = _lib.load_library()  # raises if libbitlinear_hip.so is missing
    dev = torch.device("cuda:0")
    if args.e2e_only:
        print(json.dumps({"end_to_end_decode": end_to_end_decode()}))
        return
    M = args.m
    shapes, layers, scales, acts = build_workload(M, dev)

    q_buf = [torch.empty(M, sh.K, dtype=torch.int8, device=dev) for sh in shapes]
    s_buf = [torch.empty(M, dtype=torch.bfloat16, device=dev) for sh in shapes]
    o_buf = [torch.empty(M, sh.N, dtype=torch.bfloat16, device=dev) for sh in shapes]

    def launch_path(sp):  # quantizer + GEMV, the whole hot path
        for row in layers:
            for i, sh in enumerate(shapes):
                st = lib.bitlinear_forward_bf16(
                    _p(acts[i]), _p(row[i]), _p(o_buf[i]), _p(scales[i]), _p(q_buf[i]), _p(s_buf[i]), M, sh.N, sh.K, 0, sp
                )
                assert st == 0, lib.bitlinear_status_string(st)

    def launch_gemv_only(sp, only=None, passes=1):
        for row in layers * passes:
            for i, sh in enumerate(shapes):
                if only is not None and i != only:
                    continue
                lib.bitlinear_int8xint2(_p(q_buf[i]), _p(row[i]), _p(o_buf[i]), _p(s_buf[i]), _p(scales[i]), M, sh.N, sh.K, sp)
                assert lib.bitlinear_last_status() == 0

    def launch_quant_only(sp):
        for _ in layers:
            for i, sh in enumerate(shapes):
                lib.bitlinear_quant_absmax(_p(acts[i]), _p(q_buf[i]), _p(s_buf[i]), M, sh.K, 0, sp)

    if args.prefill_probe:
        Mp = 2048
        for i, sh in enumerate(shapes):
            q = torch.randint(-127, 128, (Mp, sh.K), dtype=torch.int8, device=dev)
            sc = torch.full((Mp,), 2.0, dtype=torch.bfloat16, device=dev)
            o = torch.empty(Mp, sh.N, dtype=torch.bfloat16, device=dev)
            for rep in range(3):
                lib.bitlinear_int8xint2(_p(q), _p(layers[rep][i]), _p(o), _p(sc), _p(scales[i]), Mp, sh.N, sh.K, None)
                assert lib.bitlinear_last_status() == 0
            torch.cuda.synchronize()
        print(json.dumps({"prefill_probe": "bitlinear_int8xint2 at M=2048, three launches per 2B shape (wqkv, wo, w13, w2)"}))
        return
    if args.pmc_probe:
        launch_quant_only(None)  # fills q_buf / s_buf
        src = torch.randint(0, 255, (256 << 20,), dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        launch_path(None)
        torch.cuda.synchronize()
        # and one grouped launch per 2B shape (the 30 layers' products of that shape in one launch of the streaming kernel)
        from bitnet_amd import _lib as _l

        L = len(layers)
        for i, sh in enumerate(shapes):
            o = torch.empty(L, M, sh.N, dtype=torch.bfloat16, device=dev)
            arr = (_l.Problem * L)()
            for l in range(L):
                arr[l] = _l.Problem(q_buf[i].data_ptr(), layers[l][i].data_ptr(), o[l].data_ptr(), s_buf[i].data_ptr(),
                                    scales[i].data_ptr(), M, sh.N, sh.K)
            assert lib.bitlinear_int8xint2_grouped(arr, L, None) == 0
            torch.cuda.synchronize()
        print(json.dumps({"pmc_probe": "3 copies of 268435456 B (read 256 MiB + write 256 MiB each), then the 120 launches of one "
                          "step, then one grouped launch per 2B shape (30 problems each)"}))
        return

    step_bytes = sum(sh.weight_bytes for sh in shapes) * len(layers)
    n_gemv = len(shapes) * len(layers)

    # ---- the timed region: K steps of the whole path ------------------------
    path = GraphRun(launch_path)
    path.replay(args.warmup)
    wall_s, ev_ms = path.timed(args.steps)
    ms_per_step = wall_s * 1e3 / args.steps
    value = step_bytes / (wall_s / args.steps) / 1e9

    # ---- the drop-in product entry alone (int8 activations already quantized) ----
    gemv = GraphRun(launch_gemv_only)
    gemv.replay(args.warmup)
    _, gemv_ms = gemv.timed(args.steps)
    gemv_us = gemv_ms * 1e3 / (args.steps * n_gemv)
    # the timed region holds nothing but the 120 launches of the fused kernel
    fused_us = ev_ms * 1e3 / (args.steps * n_gemv)
    achieved = (step_bytes / n_gemv) / (fused_us * 1e-6) / 1e9

    per_shape = {}
    for i, sh in enumerate(shapes):
        passes = 8  # 240 launches per graph, so the cost of starting a replay does not weigh on the figure
        g = GraphRun(lambda sp, i=i: launch_gemv_only(sp, only=i, passes=passes))
        g.replay(max(2, args.warmup // 4))
        nrep = max(1, args.steps // 4)
        _, ms = g.timed(nrep)
        us = ms * 1e3 / (nrep * len(layers) * passes)
        per_shape[sh.name] = {
            "K": sh.K,
            "N": sh.N,
            "us_per_launch": round(us, 3),
            "GBps": round(sh.weight_bytes / (us * 1e-6) / 1e9, 1),
            "note": "30 weight copies of this shape in a loop (49-265 MB): partly served by the 256 MB last-level cache",
        }
        del g
    # ---- the same 120 calls with the launch latencies overlapped: four graphs (one per shape, 30
    # layers each) replayed at the same time on four streams.  Not a decode step (no call waits
    # for another shape's result); it shows what the kernels move when starting them is hidden.
    def launch_shape_path(i):
        def fn(sp):
            sh = shapes[i]
            for row in layers:
                st = lib.bitlinear_forward_bf16(
                    _p(acts[i]), _p(row[i]), _p(o_buf[i]), _p(scales[i]), _p(q_buf[i]), _p(s_buf[i]), M, sh.N, sh.K, 0, sp
                )
                assert st == 0, lib.bitlinear_status_string(st)
        return fn

    lanes = [GraphRun(launch_shape_path(i)) for i in range(len(shapes))]
    for g in lanes:
        g.replay(2)
    torch.cuda.synchronize()
    nrep = max(4, args.steps // 4)
    t0 = time.perf_counter()
    for _ in range(nrep):
        for g in lanes:
            g.replay(1)
    torch.cuda.synchronize()
    overlapped_s = (time.perf_counter() - t0) / nrep
    del lanes

    quant = GraphRun(launch_quant_only)
    quant.replay(max(2, args.warmup // 4))
    _, q_ms = quant.timed(args.steps)
    quant_us = q_ms * 1e3 / (args.steps * n_gemv)

    traffic, traffic_source = None, None
    # HBM bytes per launch are NOT measured in this run (counters need the profiler): the figure is the one the
    # FETCH_SIZE / WRITE_SIZE counter runs gave for the same 120 launches, kept with its commands, date and commit
    # in profiles/; this run only repeats it
    tpath = os.path.join(ROOT, "profiles", "bitlinear_forward_m1_bitnet2b_hbm_traffic.txt")
    if M == 1 and os.path.exists(tpath):
        for line in open(tpath):
            if line.startswith("traffic_bytes_per_launch:"):
                traffic = int(float(line.split(":", 1)[1]))
            if line.startswith("measured:"):
                traffic_source = "profiles/bitlinear_forward_m1_bitnet2b_hbm_traffic.txt (rocprofv3 --pmc, " + line.split(":", 1)[1].strip() + "); not re-measured in this run"

    result = {
        "metric": METRIC,
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "dtype_detail": "int8 activations x 2-bit ternary weights, int32 accumulate, fp32 scale epilogue, bf16 out",
        "data": "synthetic",
        "config": {
            "workload": (
                f"BitNet-2B BitLinear stack, M={M}: 30 layers x (K,N) in (2560,3840) (2560,2560) (2560,13824) "
                "(6912,2560), BitLinearKernel.forward (quantizer + product + epilogue, one kernel) per call, 120 "
                "launches per step from a HIP graph, distinct weights per layer"
            ),
            "tokens_per_step": M,
            "packed_weight_bytes_per_step": step_bytes,
        },
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "bitlinear_tokens_per_s": round(M / (wall_s / args.steps), 1),
        "event_ms_per_step": round(ev_ms / args.steps, 5),
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 2),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "traffic_source": traffic_source,
            "kernel": "bitlinear_solo_kernel (BitLinearKernel.forward in one kernel: quantizer + int8 x int2 product + "
            "epilogue), mean over the 120 launches of a step, HIP events on the replay stream over the timed region",
            "bytes_per_launch": step_bytes // n_gemv,
            "us_per_launch": round(fused_us, 3),
        },
        "product_only_us_per_launch": round(gemv_us, 3),
        "per_shape_product_only": per_shape,
        "quantizer_us_per_launch": round(quant_us, 3),
        "overlapped_four_streams": {
            "GBps": round(step_bytes / overlapped_s / 1e9, 1),
            "frac_of_hbm_peak": round(step_bytes / overlapped_s / 1e9 / HBM_PEAK_GBPS, 4),
            "ms_per_120_calls": round(overlapped_s * 1e3, 5),
            "note": "the same 120 forward calls as four independent chains (one per shape) on four streams: "
            "launch latency overlapped, not a decode step; wall clock",
        },
    }
    if M == 1:
        result["roofline"]["per_shape"] = per_shape_forward(lib, shapes, layers, scales, acts, q_buf, s_buf, o_buf, dev, M)
        result["roofline"]["per_shape_note"] = (
            "BitLinearKernel.forward per 2B shape: hbm_cold = 30 layers' distinct matrices per replay behind a 768 MiB "
            "cache flush, cache_hot = one layer's matrix 30 times; frac = achieved / 8000 GB/s"
        )
    try:  # a diagnostic leg: whatever happens in it, the headline above is printed
        result.update(latency_floor(lib, shapes, layers, dev))
    except Exception as e:  # noqa: BLE001
        result["latency_floor"] = {"error": f"{type(e).__name__}: {e}"}
    if not args.no_sweeps:
        result.update(grouped_launches(lib, shapes, layers, scales, dev, 1))
        result.update(grouped_launches(lib, shapes, layers, scales, dev, 4))
        bp = batched_and_prefill(lib, shapes, layers, scales, dev)
        ceil = mfma_ceiling(lib, dev)
        for leg in bp["prefill"].values():  # the nominal peak prices the roofline; the measured ceiling stands beside it
            leg["roofline"]["frac_of_measured_ceiling"] = round(leg["layer_gemm_TOPS"] / ceil["random_int8_x_ternary_codes_TOPS"], 4)
        bp["prefill"]["mfma_ceiling"] = ceil
        result.update(bp)
        result.update(large_shapes(lib, dev))
    if not args.no_e2e:
        del path, gemv, quant, layers
        torch.cuda.empty_cache()
        result["end_to_end_decode"] = end_to_end_decode()
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(shapes, M, args.cpu_seconds)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
