#!/usr/bin/env python3
"""Headline benchmark: int8 weight-only GEMM HBM GB/s at LLaMA-7B decode shapes,
plus LLaMA-7B-shaped int8 decode tokens/s, on one MI355X.

A "step" is one pass of the fused dequant-GEMM over every int8 linear of a
32-layer LLaMA-7B-shaped decoder, launched as the decoder ops launch them (128
launches over 6.48 GB of distinct packed weights, so nothing is served from the
256 MB Infinity Cache) at M = 8 rows of fp16 activations.  `value` is
algorithmic bytes per step / time per step.

Prints ONE JSON line.  Synthetic, seeded data; weights live in HBM before the
timed region starts.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
LLAMA = dict(layers=32, hidden=4096, heads=32, d_ff=11008, vocab=32000, alibi=False)
BAICHUAN13B = dict(layers=40, hidden=5120, heads=40, d_ff=13696, vocab=64000, alibi=True)


def linear_shapes(hidden, d_ff):
    # (name, K, N) in the order a decoder layer calls them
    return [("qkv", hidden, 3 * hidden), ("o", hidden, hidden), ("gate", hidden, d_ff), ("up", hidden, d_ff),
            ("down", d_ff, hidden)]


# The launches the decoder ops actually make per layer (eet_amd/ops.py): gate and up are one
# launch over their tile-interleaved weights with the SwiGLU epilogue; O and down carry the
# residual add.  (name, K, N, epilogue)
EPI_NONE, EPI_RESIDUAL, EPI_SWIGLU = 0, 1, 2


def linear_bytes(M, K, N, epi=EPI_NONE):
    """Algorithmic bytes of one int8 linear: each operand once (weights, scales, activations,
    output; plus the residual rows read by that epilogue; the SwiGLU output is M x N/2)."""
    n_out = N // 2 if epi == EPI_SWIGLU else N
    return K * N + 2 * N + 2 * M * K + 2 * M * n_out + (2 * M * N if epi == EPI_RESIDUAL else 0)


def make_weights(torch, eet, dev, layers, hidden, d_ff, seed):
    """Per layer, per linear: (packed int8 [K, N], fp16 scales [N]) generated on
    the GPU: W ~ N(0, 0.02^2) in fp16, quantised per output channel (reference
    /128 rule) and permuted into the gfx950 layout."""
    g = torch.Generator(device=dev).manual_seed(seed)
    out = []
    for _ in range(layers):
        layer = {}
        for name, K, N in linear_shapes(hidden, d_ff):
            w = (torch.randn(K, N, generator=g, device=dev, dtype=torch.float32) * 0.02).half()
            p, s = eet.quant_weights_device(w, False, "ref128")     # the HIP packer
            layer[name] = (p, s)
            del w
        out.append(layer)
    return out


RMS_LAUNCHES = ("rmsnorm+qkv", "rmsnorm+gate|up+swiglu")     # the launches that carry the RMSnorm prologue
TIMELINE_READINGS = 24   # per workgroup in the bench-only build: 8 of the workgroup, then one per wavefront (up to 16)


def fused_launch_weights(eet_ops, weights):
    """Per layer, the operands of the four launches the decoder ops make (eet_amd/csrc/decode_ops.cc):
    RMSnorm + QKV, O + residual, RMSnorm + gate|up + SwiGLU, down + residual."""
    out = []
    for layer in weights:
        w01, s01 = eet_ops.interleave_gate_up(layer["gate"][0], layer["gate"][1], layer["up"][0], layer["up"][1])
        out.append({"rmsnorm+qkv": layer["qkv"] + (EPI_NONE,), "o+residual": layer["o"] + (EPI_RESIDUAL,),
                    "rmsnorm+gate|up+swiglu": (w01, s01, EPI_SWIGLU), "down+residual": layer["down"] + (EPI_RESIDUAL,)})
    return out


def bench_lib():
    """libeet_bench.so: the read-only streaming probe (measurement only, not part of the product ABI)."""
    import ctypes
    path = os.path.join(ROOT, "eet_amd", "libeet_bench.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build it with `python -m eet_amd.build`")
    h = ctypes.CDLL(path)
    vp, sz = ctypes.c_void_p, ctypes.c_size_t
    h.eet_hbm_stream_probe.restype = ctypes.c_int
    h.eet_hbm_stream_probe.argtypes = [vp, sz, ctypes.c_int, vp, sz, vp]
    h.eet_hbm_stream_probe_ring.restype = ctypes.c_int
    h.eet_hbm_stream_probe_ring.argtypes = [vp, sz, ctypes.c_int, vp, sz, vp]
    i, f = ctypes.c_int, ctypes.c_float
    h.eet_timeline_gemm_w8a16_fused.restype = i      # eet_gemm_w8a16_fused with clock readings in the kernel
    h.eet_timeline_gemm_w8a16_fused.argtypes = [vp, vp, vp, vp, i, i, i, i, vp, vp, f, vp, sz, vp]
    h.eet_timeline_begin.restype = i
    h.eet_timeline_begin.argtypes = [i]
    h.eet_timeline_launches.restype = i
    h.eet_timeline_read.restype = i
    h.eet_timeline_read.argtypes = [i, vp]
    h.eet_timeline_mmha_decode.restype = i           # eet_mmha_decode with clock readings in the kernel
    h.eet_timeline_mmha_decode.argtypes = [vp, vp, vp, ctypes.c_long, vp, vp, vp, vp, vp, i, i, i, i, i, vp, vp, sz, vp]
    h.eet_timeline_attn_begin.restype = i
    h.eet_timeline_attn_begin.argtypes = [i]
    h.eet_timeline_attn_read.restype = i
    h.eet_timeline_attn_read.argtypes = [i, vp]
    return h


def launch_timeline(torch, lib, weights, acts, outs, M):
    """Where the time of a launch goes, read inside the kernel: the GEMM pass through the bench-only build of the
    same source (eet_timeline_gemm_w8a16_fused), whose workgroups read the 100 MHz wall clock at entry, after their
    first multiplied batch, at the end of the k loop, after issuing their stores and after the stores are
    acknowledged.  Two passes are recorded; the second is analysed, by launch kind."""
    import ctypes
    import numpy as np
    B = bench_lib()
    st = torch.cuda.current_stream().cuda_stream
    ws_need = max([lib.eet_gemm_w8a16_workspace(M, w.shape[1], w.shape[0], epi)
                   for layer in weights for name, (w, s, epi) in layer.items() if name not in RMS_LAUNCHES] + [0])
    ws = torch.zeros(max(ws_need // 4, 1), dtype=torch.float32, device=outs["gamma"].device)
    calls, kinds = [], []
    for layer in weights:
        for name, (w, s, epi) in layer.items():
            K, N = w.shape
            n_out = N // 2 if epi == EPI_SWIGLU else N
            res = outs["residual"].data_ptr() if epi == EPI_RESIDUAL else None
            gam = outs["gamma"].data_ptr() if name in RMS_LAUNCHES else None
            calls.append((acts[K].data_ptr(), w.data_ptr(), s.data_ptr(), outs[n_out].data_ptr(), M, N, K, epi, res, gam, 1e-6,
                          None if gam or not ws_need else ws.data_ptr(), 0 if gam or not ws_need else ws.numel() * 4, st))
            kinds.append(name)
    n = len(calls)
    if B.eet_timeline_begin(2 * n):
        raise RuntimeError("eet_timeline_begin failed")
    torch.cuda.synchronize()
    for _ in range(2):
        for c in calls:
            if B.eet_timeline_gemm_w8a16_fused(*c):
                raise RuntimeError(lib.eet_last_error().decode())
    torch.cuda.synchronize()
    if B.eet_timeline_launches() != 2 * n:
        return {"error": f"{B.eet_timeline_launches()} launches recorded, {2 * n} made"}
    buf = np.zeros(1024 * TIMELINE_READINGS, dtype=np.uint64)
    stamps = []
    for l in range(n - 1, 2 * n):          # the last launch of the first pass, then the second pass
        wgs = B.eet_timeline_read(l, buf.ctypes.data_as(ctypes.c_void_p))
        if wgs <= 0:
            return {"error": f"eet_timeline_read({l}) returned {wgs}"}
        t = buf[: wgs * TIMELINE_READINGS].reshape(wgs, TIMELINE_READINGS)[:, :8].astype(np.int64)
        stamps.append(t[t[:, 0] > 0])
    out = {}
    for kind in dict.fromkeys(kinds):
        rows = []
        for i in range(1, n):              # launch i of the second pass; i - 1 is its predecessor (stamps[0] = last of pass 1)
            if kinds[i] != kind:
                continue
            prev, cur, nxt = stamps[i], stamps[i + 1], stamps[i + 2] if i + 2 < len(stamps) else None
            t0 = cur[:, 0].min()
            has1 = cur[:, 1] > 0
            rows.append([
                (nxt[:, 0].min() - t0) if nxt is not None else np.nan,      # period: entry to the next launch's entry
                t0 - prev[:, 4].max(),                                      # last acknowledged store of the predecessor -> first entry
                cur[:, 0].max() - t0,                                       # entry spread over the workgroups
                (cur[has1, 1] - cur[has1, 0]).mean() if has1.any() else np.nan,   # entry -> first batch multiplied
                (cur[:, 2] - t0).min(), (cur[:, 2] - t0).mean(), (cur[:, 2] - t0).max(),   # end of k loop after first entry
                (cur[:, 3] - cur[:, 2]).mean(),                             # reduction + epilogue until the stores are issued
                (cur[:, 4] - cur[:, 3]).mean(),                             # stores acknowledged
                cur[:, 4].max() - t0,                                       # first entry -> last acknowledged store
                (cur[:, 5] - cur[:, 6]).mean(),                             # first wavefront out of the k loop -> all out (barrier passed)
                (cur[:, 5] - cur[:, 7]).mean(),                             # mean wavefront out of the k loop -> all out
                (cur[:, 3] - cur[:, 5]).mean(),                             # barrier passed -> stores issued (the arithmetic of the epilogue)
                (cur[:, 5] - t0).max()])                                    # the last workgroup's barrier after the first entry
        a = np.nanmean(np.array(rows, dtype=np.float64), axis=0) / 100.0    # 100 MHz clock -> microseconds
        out[kind] = {"launches": len(rows), "period_us": round(a[0], 2), "idle_before_first_entry_us": round(a[1], 2),
                     "entry_spread_us": round(a[2], 2), "entry_to_first_batch_multiplied_us": round(a[3], 2),
                     "k_loop_end_after_first_entry_us": {"first": round(a[4], 2), "mean": round(a[5], 2), "last": round(a[6], 2)},
                     "reduce_and_epilogue_us": round(a[7], 2), "store_acknowledge_us": round(a[8], 2),
                     "first_entry_to_last_acknowledge_us": round(a[9], 2),
                     "wait_for_the_slowest_wavefront_us": {"from_the_first_wavefront_out": round(a[10], 2), "from_the_mean_wavefront_out": round(a[11], 2)},
                     "epilogue_after_the_barrier_us": round(a[12], 2), "last_workgroup_barrier_after_first_entry_us": round(a[13], 2)}
    out["what"] = ("clock readings inside the small-M kernel (bench-only build with -DEET_TIMELINE of the same source; thread 0 of "
                   "each workgroup, 100 MHz wall clock), second of two recorded passes, mean over the launches of a kind; "
                   "the instrumented kernel waits for its stores before its last reading, which the shipped one leaves to the "
                   "end of the kernel")
    return out


def time_gemm_pass(torch, lib, weights, acts, outs, M, steps, warmup, probe=False, probe_grid_scale=1, chained=False,
                   probe_ring=False):
    """Returns seconds per step (one pass over all linears), measured with
    events on the stream the kernels are launched on.  Launches named in
    RMS_LAUNCHES carry the RMSnorm prologue, as in the decoder.  probe=True
    replaces every GEMM by the read-only streaming probe over the same weight
    buffer with the same grid (the machine's ceiling for this launch chain).
    chained=True issues the pass as ONE chain (eet_gemm_w8a16_chained): every launch but the
    first of a pass is enqueued without the queue barrier and waits in the kernel for its
    predecessor's completion counter."""
    st = torch.cuda.current_stream()
    calls = []
    # the workspace the decoder ops hand to the launches without a prologue (the small-M kernel's k split):
    # one zero-initialised buffer shared by all launches of the stream, as in eet_amd/ops.py
    ws_need = max([lib.eet_gemm_w8a16_workspace(M, w.shape[1], w.shape[0], epi)
                   for layer in weights for name, (w, s, epi) in layer.items() if name not in RMS_LAUNCHES] + [0])
    if "k_split_ws" not in outs or outs["k_split_ws"].numel() * 4 < ws_need:
        outs["k_split_ws"] = torch.zeros(max(ws_need // 4, 1), dtype=torch.float32, device=outs["gamma"].device)
    wsp, wsb = (outs["k_split_ws"].data_ptr(), outs["k_split_ws"].numel() * 4) if ws_need else (None, 0)
    for layer in weights:
        for name, (w, s, epi) in layer.items():
            K, N = w.shape
            n_out = N // 2 if epi == EPI_SWIGLU else N
            res = outs["residual"].data_ptr() if epi == EPI_RESIDUAL else None
            gam = outs["gamma"].data_ptr() if name in RMS_LAUNCHES else None
            calls.append((acts[K].data_ptr(), w.data_ptr(), s.data_ptr(), outs[n_out].data_ptr(), M, N, K, epi, res, gam))
    f = lib.eet_gemm_w8a16_fused
    sp = st.cuda_stream

    if chained:
        fc = lib.eet_gemm_w8a16_chained

        def one_pass():
            mode = 1                       # EET_CHAIN_FIRST, then EET_CHAIN_NEXT
            for (a, w, s, c, m, n, k, epi, res, gam) in calls:
                rc = fc(a, w, s, c, m, n, k, epi, res, gam, 1e-6, mode, sp)
                if rc:
                    raise RuntimeError(lib.eet_last_error().decode())
                mode = 2
    elif probe:
        sink = outs["probe_sink"]
        g = bench_lib().eet_hbm_stream_probe_ring if probe_ring else bench_lib().eet_hbm_stream_probe

        def one_pass():
            for (a, w, s, c, m, n, k, epi, res, gam) in calls:
                # the grid the GEMM uses for this shape: 256 workgroups, 688 for the merged gate|up matrix
                rc = g(w, k * n, (688 if epi == EPI_SWIGLU and not probe_ring else 256) * probe_grid_scale, sink.data_ptr(),
                       sink.numel(), sp)
                if rc:
                    raise RuntimeError("eet_hbm_stream_probe failed")
    else:
        def one_pass():
            for (a, w, s, c, m, n, k, epi, res, gam) in calls:
                rc = f(a, w, s, c, m, n, k, epi, res, gam, 1e-6, None if gam else wsp, 0 if gam else wsb, sp)
                if rc:
                    raise RuntimeError(lib.eet_last_error().decode())
    for _ in range(warmup):
        one_pass()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(st)
    for _ in range(steps):
        one_pass()
    e1.record(st)
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    return e0.elapsed_time(e1) * 1e-3 / steps, wall, len(calls)


def cpu_info():
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as fh:
            for line in fh:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return model


def cpu_threads():
    """Threads the CPU legs run on: every core the process may use (the GPU boxes give a job
    16 cores whatever os.cpu_count() says)."""
    try:
        allowed = len(os.sched_getaffinity(0))
    except AttributeError:
        allowed = os.cpu_count() or 1
    return max(1, min(allowed, int(os.environ.get("OMP_NUM_THREADS", allowed))))


def cpu_baseline(torch, M, hidden, d_ff, seed, budget_s=10.0):
    """The reference CPU path, timed on the host cores: torch dequantise
    (int8 * scale -> fp32) + fp32 matmul -> fp16, for one layer's five linears
    (the same shapes as the GPU workload; a bounded sample of it).  Also timed:
    the matmul alone with the dequantised fp32 weights kept (the second number
    the reference path could be quoted on)."""
    from oracle import cpu_path
    threads = cpu_threads()
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(seed)
    layer = []
    for name, K, N in linear_shapes(hidden, d_ff):
        q = torch.randint(-128, 128, (K, N), generator=g, dtype=torch.int8)
        s = (torch.rand(N, generator=g) * 1e-3).half()
        x = torch.randn(M, K, generator=g).half()
        layer.append((x, q, s))
    nbytes = sum(linear_bytes(M, q.shape[0], q.shape[1]) for _, q, _ in layer)
    cpu_path.dequant_matmul_layer(layer)          # warm-up
    reps, t0 = 0, time.perf_counter()
    while True:
        cpu_path.dequant_matmul_layer(layer)
        reps += 1
        el = time.perf_counter() - t0
        if el > budget_s or reps >= 20:
            break
    per_layer = el / reps
    # matmul only: weights dequantised once, outside the timed region
    cached = [(x.float(), q.float() * s.float()[None, :]) for x, q, s in layer]
    for x32, wd in cached:
        (x32 @ wd).half()
    reps2, t0 = 0, time.perf_counter()
    while True:
        for x32, wd in cached:
            (x32 @ wd).half()
        reps2 += 1
        el2 = time.perf_counter() - t0
        if el2 > budget_s / 2 or reps2 >= 20:
            break
    per_layer_mm = el2 / reps2
    return {"value": round(nbytes / per_layer / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"one LLaMA-7B layer (5 int8 linears, M={M}, {nbytes / 1e6:.1f} MB algorithmic), "
                      f"{reps} reps, torch {torch.__version__} dequant+matmul fp32, "
                      f"{per_layer * 1e3:.1f} ms per layer",
            "matmul_only_value": round(nbytes / per_layer_mm / 1e9, 3),
            "matmul_only_sample": f"same layer, fp32 weights dequantised beforehand, {reps2} reps, "
                                  f"{per_layer_mm * 1e3:.1f} ms per layer",
            "os_cpu_count": os.cpu_count(), "torch_threads": torch.get_num_threads(), "cpu_model": cpu_info()}


def cpu_decode_baseline(torch, model, batch, step, layers_timed=2, steps_timed=2, seed=11):
    """One token step of the CPU oracle decoder (numpy fp32: dequantise + matmul, attention over
    the fp16 KV cache) at the decoder's real width, on `layers_timed` layers with KV caches
    filled with N(0,1) rows up to `step`, extrapolated to the full depth (labelled as such)."""
    import numpy as np

    from oracle import ops as O
    rng = np.random.default_rng(seed)
    H, heads, F = model["hidden"], model["heads"], model["d_ff"]
    dh = H // heads

    def lin(K, N):
        return rng.integers(-128, 128, (K, N), dtype=np.int8), (rng.random(N) * 1e-3 + 1e-4).astype(np.float16)
    layers = []
    for _ in range(layers_timed):
        gam = np.ones(H, np.float16)
        attn = O.OracleAttention(batch, heads, dh, step + steps_timed + 2, *lin(H, 3 * H), *lin(H, H), gam, 1e-6,
                                 rope=not model["alibi"])
        attn.k_cache[:, :, :step] = rng.standard_normal((batch, heads, step, dh), dtype=np.float32).astype(np.float16)
        attn.v_cache[:, :, :step] = rng.standard_normal((batch, heads, step, dh), dtype=np.float32).astype(np.float16)
        attn.step = step
        layers.append((attn, O.OracleFFN(*lin(H, F), *lin(H, F), *lin(F, H), gam, 1e-6)))
    x = rng.standard_normal((batch, 1, H), dtype=np.float32).astype(np.float16)
    t0 = time.perf_counter()
    for t in range(steps_timed):
        y = x
        for attn, ffn in layers:
            bias = O.alibi_bias(heads, attn.step + 1) if model["alibi"] else None
            y = ffn.forward(attn.forward(y, None, False, bias))
    per_layer = (time.perf_counter() - t0) / (steps_timed * layers_timed)
    step_s = per_layer * model["layers"]
    return {"tokens_per_s_extrapolated": round(batch / step_s, 3), "s_per_token_step_extrapolated": round(step_s, 3),
            "measured": f"{layers_timed} layers x {steps_timed} token steps of the numpy fp32 oracle decoder at hidden {H}, "
                        f"batch {batch}, cache length {step}: {per_layer * 1e3:.0f} ms per layer; multiplied by "
                        f"{model['layers']} layers (embedding, final norm and lm_head not included)",
            "cores": cpu_threads(), "kind": "port"}


def device_packer_bench(torch, eet, lib, dev, iters=3):
    """The packer on the GPU: eight distinct fp16 [11008, 4096] matrices (0.72 GB, more than the Infinity
    Cache) quantised and packed round-robin.  Algorithmic bytes per matrix: read 2*K*N once, write K*N
    packed + 2*N scales (the kernel pair reads the matrix twice: absmax first)."""
    K, N = 11008, 4096
    g = torch.Generator(device=dev).manual_seed(17)
    ws = [(torch.randn(K, N, generator=g, device=dev) * 0.02).half() for _ in range(8)]
    packed = torch.empty(K, N, dtype=torch.int8, device=dev)
    scale = torch.empty(N, dtype=torch.float16, device=dev)
    need = lib.eet_quantize_pack_device_workspace(N)
    work = torch.empty(need // 4, dtype=torch.int32, device=dev)
    st = torch.cuda.current_stream()

    def call(w):
        rc = lib.eet_quantize_pack_device(w.data_ptr(), 1, K, N, 0, None, packed.data_ptr(), scale.data_ptr(),
                                          work.data_ptr(), need, st.cuda_stream)
        if rc:
            raise RuntimeError(lib.eet_last_error().decode())
    for w in ws:
        call(w)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(st)
    for _ in range(iters):
        for w in ws:
            call(w)
    e1.record(st)
    torch.cuda.synchronize()
    t = e0.elapsed_time(e1) * 1e-3 / (iters * len(ws))
    nbytes = 3 * K * N + 2 * N
    return {"shape": f"K={K} N={N} fp16", "us": round(t * 1e6, 1), "Gweights_per_s": round(K * N / t / 1e9, 1),
            "GB/s": round(nbytes / t / 1e9, 1), "frac_of_hbm_peak": round(nbytes / t / 1e9 / HBM_PEAK_GBS, 4)}


def packer_bench(torch, eet):
    """The offline leg, on the host: fp16 [K, N] -> int8 (per-channel /128 quantiser) -> gfx950 tile layout,
    through the operator (`quant_weights`, threaded by column block), with the single-threaded plain-C
    restatement of the reference quantiser timed beside it on the same matrix (it quantises only: the
    reference's own layout pass is not restated in C).  One LLaMA-7B down-projection, K = 11008, N = 4096."""
    import ctypes

    import numpy as np
    K, N = 11008, 4096
    w = (torch.randn(K, N, generator=torch.Generator().manual_seed(3)) * 0.02).half()
    eet.quant_weights(w[:64].contiguous(), torch.int8, False)     # load the library, start the threads once
    t0 = time.perf_counter()
    eet.quant_weights(w, torch.int8, False)
    t_ours = time.perf_counter() - t0
    out = {"shape": f"K={K} N={N} fp16", "quantise_and_pack_s": round(t_ours, 3),
           "Mweights_per_s": round(K * N / t_ours / 1e6, 1), "threads": cpu_threads()}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "oracle", "liboracle.so")
    if os.path.exists(path):
        ref = ctypes.CDLL(path)
        ref.oracle_quantize_ref128.restype = ctypes.c_int
        ref.oracle_quantize_ref128.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_void_p,
                                               ctypes.c_void_p]
        w32 = w.float().numpy()
        q = np.empty((K, N), np.int8)
        sc = np.empty(N, np.float32)
        t0 = time.perf_counter()
        ref.oracle_quantize_ref128(w32.ctypes.data, K, N, q.ctypes.data, sc.ctypes.data)
        t_ref = time.perf_counter() - t0
        out["cpu_port_quantise_only_s"] = round(t_ref, 3)
        out["cpu_port_Mweights_per_s"] = round(K * N / t_ref / 1e6, 1)
    return out


def decode_bench(torch, eet, weights, dev, batch, prompt, gen, seed, model=LLAMA, graph_batch1=True):
    """Int8 decoder of the given shape, random init: prefill `prompt` tokens then
    greedy-decode `gen` tokens; tokens/s = batch * (gen - 1) / decode time."""
    from eet_amd import decoder as D
    cfg = D.DecoderConfig(num_layers=len(weights), hidden=model["hidden"], heads=model["heads"], d_ff=model["d_ff"],
                          vocab=model["vocab"], alibi=model["alibi"], max_batch=batch, max_prompt=prompt,
                          max_full_seq=prompt + gen + 10)
    g = torch.Generator(device=dev).manual_seed(seed)
    H = cfg.hidden
    sd = {}
    for i, layer in enumerate(weights):
        pre = f"layer.{i}."
        for key, name in (("qkv", "self_attn.qkv_proj"), ("o", "self_attn.out_proj"), ("gate", "ffn.intermediate_0"),
                          ("up", "ffn.intermediate_1"), ("down", "ffn.output")):
            sd[pre + name + ".weight"], sd[pre + name + ".scale"] = layer[key]
        sd[pre + "self_attn.layernorm.weight"] = (1 + 0.1 * torch.randn(H, generator=g, device=dev)).half()
        sd[pre + "ffn.layernorm.weight"] = (1 + 0.1 * torch.randn(H, generator=g, device=dev)).half()
    sd["embed_tokens.weight"] = (torch.randn(cfg.vocab, H, generator=g, device=dev) * 0.02).half()
    sd["norm.weight"] = (1 + 0.1 * torch.randn(H, generator=g, device=dev)).half()
    sd["lm_head.weight"] = (torch.randn(cfg.vocab, H, generator=g, device=dev) * 0.02).half()
    model = D.Int8Decoder(cfg, sd, device=str(dev))
    ids = torch.randint(0, cfg.vocab, (batch, prompt), generator=g, device=dev)
    with torch.no_grad():
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = model.logits(ids, True)
        torch.cuda.synchronize()
        t_prefill = time.perf_counter() - t0
        # the same prompt again: first_pass resets the step, and this time nothing is allocated
        t0 = time.perf_counter()
        logits = model.logits(ids, True)
        torch.cuda.synchronize()
        t_prefill_warm = time.perf_counter() - t0
        nxt = torch.argmax(logits[:, -1, :], dim=-1)
        # one untimed decode step (allocations, first-touch)
        logits = model.logits(nxt[:, None], False)
        nxt = torch.argmax(logits[:, -1, :], dim=-1)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(gen - 1):
            logits = model.logits(nxt[:, None], False)
            nxt = torch.argmax(logits[:, -1, :], dim=-1)
        torch.cuda.synchronize()
        t_dec = time.perf_counter() - t0
        # per-kernel breakdown from further steps of the same run: each launch issued on its own
        # and bracketed by events (the timed loop above used the one-call-per-op path)
        from eet_amd import ops as _ops
        timer = _ops.LaunchTimer()
        _ops.launch_timer = timer
        bd_steps = min(8, max(0, cfg.max_full_seq - (prompt + gen) - 1))
        try:
            for _ in range(bd_steps):
                logits = model.logits(nxt[:, None], False)
                nxt = timer.run("argmax (torch)", batch * cfg.vocab * 2, lambda: torch.argmax(logits[:, -1, :], dim=-1))
        finally:
            _ops.launch_timer = None
        raw = timer.summary() if bd_steps else {}

        # the same decode from HIP-graph replays of the incremental step, and both ways at batch 1
        def timed_decode(b, graph):
            lg = model.logits(ids[:b], True)
            tok = torch.argmax(lg[:, -1, :], dim=-1)
            if graph:
                replay = model.capture_decode_step(tok)
                replay()
                torch.cuda.synchronize()
                t = time.perf_counter()
                for _ in range(gen - 1):
                    replay()
            else:
                lg = model.logits(tok[:, None], False)
                tok = torch.argmax(lg[:, -1, :], dim=-1)
                torch.cuda.synchronize()
                t = time.perf_counter()
                for _ in range(gen - 1):
                    lg = model.logits(tok[:, None], False)
                    tok = torch.argmax(lg[:, -1, :], dim=-1)
            torch.cuda.synchronize()
            el = time.perf_counter() - t
            return {"tokens_per_s": round(b * (gen - 1) / el, 1), "ms_per_token_step": round(el / (gen - 1) * 1e3, 3)}
        eager_vs_graph = {f"batch {batch} graph": timed_decode(batch, True)}
        if graph_batch1:
            eager_vs_graph["batch 1 eager"] = timed_decode(1, False)
            eager_vs_graph["batch 1 graph"] = timed_decode(1, True)
    steps = gen - 1
    ms = t_dec / steps * 1e3
    # A bracket (event, launch, event) costs more than the launch does back to back -- the two event
    # records are packets of their own -- so the bracketed times are scaled to sum to the step time
    # measured without them; both are given.
    breakdown = {}
    tot = sum(r["us_total"] for r in raw.values()) / max(bd_steps, 1)
    for name, r in raw.items():
        us_raw = r["us_total"] / r["calls"]
        us = us_raw * (ms * 1e3 / tot)
        gbs = (r["bytes_total"] / r["calls"]) / us / 1e3
        breakdown[name] = {"calls_per_step": r["calls"] // bd_steps, "us_per_call": round(us, 2),
                           "us_per_call_bracketed": round(us_raw, 2),
                           "us_per_step": round(us * (r["calls"] // bd_steps), 1),
                           "share_of_step": round(r["us_total"] / bd_steps / tot, 4),
                           "bytes_per_call": r["bytes_total"] // r["calls"], "GB/s": round(gbs, 1),
                           "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
    # algorithmic HBM bytes of one token step: int8 weights + scales, KV cache read at mid length, fp16 lm_head
    wbytes = sum(w.numel() + 2 * s.numel() for layer in weights for (w, s) in layer.values())
    kv = len(weights) * 2 * (prompt + gen // 2) * batch * H * 2
    step_bytes = wbytes + kv + cfg.vocab * H * 2
    return {"tokens_per_s": round(batch * steps / t_dec, 1), "ms_per_token_step": round(ms, 3), "batch": batch,
            "prompt": prompt, "generated": gen, "layers": len(weights), "prefill_s": round(t_prefill, 3), "prefill_warm_s": round(t_prefill_warm, 3),
            "step_hbm_bytes": step_bytes,
            "step_roofline_frac": round(step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "hip_graph_replay": eager_vs_graph,
            "breakdown": breakdown,
            "breakdown_note": f"{bd_steps} further token steps with every launch issued on its own between two events; "
                              "us_per_call is the bracketed time scaled so that the kernels of a step sum to "
                              "ms_per_token_step (the brackets themselves cost time); bytes are algorithmic",
            "note": "greedy decode, random-init weights, random token ids; lm_head and embedding are fp16 torch ops"}


MFMA_FP16_PEAK_TFLOPS = 2500.0   # MI355X published dense fp16 MFMA peak


def prefill_gemm_bench(torch, eet, lib, dev, iters=10):
    """benchmark configuration 3: Baichuan-13B-shaped prefill GEMMs, M = 2048 tokens, on the MFMA kernel.
    Reports TFLOP/s = 2*M*N*K / t and the fraction of the fp16 MFMA peak."""
    M, hidden, d_ff = 2048, 5120, 13696
    g = torch.Generator(device=dev).manual_seed(21)
    out = {}
    st = torch.cuda.current_stream()
    for name, K, N in (("qkv", hidden, 3 * hidden), ("o", hidden, hidden), ("gate", hidden, d_ff),
                       ("down", d_ff, hidden)):
        w = (torch.randn(K, N, generator=g, device=dev) * 0.02).half()
        p, s = eet.quant_weights_device(w, False, "ref128")
        del w
        a = torch.randn(M, K, generator=g, device=dev).half()
        c = torch.empty(M, N, dtype=torch.float16, device=dev)
        args = (a.data_ptr(), p.data_ptr(), s.data_ptr(), c.data_ptr(), M, N, K, None, 0, st.cuda_stream)
        for _ in range(2):
            if lib.eet_gemm_w8a16(*args):
                raise RuntimeError(lib.eet_last_error().decode())
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(st)
        for _ in range(iters):
            lib.eet_gemm_w8a16(*args)
        e1.record(st)
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) * 1e-3 / iters
        tf = 2.0 * M * N * K / t / 1e12
        out[f"{name} M={M} K={K} N={N}"] = {"us": round(t * 1e6, 1), "TFLOP/s": round(tf, 1),
                                            "frac_of_fp16_mfma_peak": round(tf / MFMA_FP16_PEAK_TFLOPS, 4)}
    return out


def prefill_attention_bench(torch, lib, dev, iters=5):
    """Causal prefill attention (flash-style MFMA kernel) at the prompt shapes of configurations 4 and 5 (and one
    long prompt): TFLOP/s over the causal half of the work, 4 * B * H * (S^2 / 2) * dh."""
    out = {}
    st = torch.cuda.current_stream()
    for name, B, H, S, alibi in (("llama7b B=8 H=32 S=1024", 8, 32, 1024, False),
                                 ("baichuan13b B=8 H=40 S=2048 alibi", 8, 40, 2048, True),
                                 ("baichuan13b B=8 H=40 S=2048 no bias", 8, 40, 2048, False),
                                 # no configuration has a prompt this long: the kernel away from its diagonal chunks
                                 ("long prompt B=1 H=32 S=8192 no bias", 1, 32, 8192, False)):
        dh = 128
        g = torch.Generator(device=dev).manual_seed(S)
        q, kc, vc = [torch.randn(B, H, S, dh, generator=g, device=dev).half() for _ in range(3)]
        ctx = torch.empty(B, S, H * dh, dtype=torch.float16, device=dev)
        bias = (torch.rand(H, S, generator=g, device=dev) * 8).half() if alibi else None

        def call():
            rc = lib.eet_prefill_attention(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), ctx.data_ptr(),
                                           bias.data_ptr() if alibi else None, None, B, H, S, dh, S, st.cuda_stream)
            if rc:
                raise RuntimeError(lib.eet_last_error().decode())
        for _ in range(2):
            call()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(st)
        for _ in range(iters):
            call()
        e1.record(st)
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) * 1e-3 / iters
        tf = 4.0 * B * H * (S * S / 2) * dh / t / 1e12
        out[name] = {"us": round(t * 1e6, 1), "TFLOP/s_causal": round(tf, 1),
                     "frac_of_fp16_mfma_peak": round(tf / MFMA_FP16_PEAK_TFLOPS, 4)}
    return out


def attention_bench(torch, lib, dev, iters=20):
    """Isolated masked decode attention at the config 4 (LLaMA-7B, B=8) and config 5 (Baichuan-13B,
    B=32, ALiBi) shapes: GB/s over the algorithmic bytes 2*step*B*H*dh*2 + 6*B*H*dh*2 (+ 2*H*step)."""
    out = {}
    st = torch.cuda.current_stream()
    for name, B, H, step, alibi in (("llama7b B=8 step=1088", 8, 32, 1088, False),
                                    ("baichuan13b B=32 step=2176 alibi", 32, 40, 2176, True)):
        dh, cap = 128, step + 1
        g = torch.Generator(device=dev).manual_seed(step)
        # several caches in rotation so that the rows come from HBM, not the 256 MB Infinity Cache
        per = 2 * B * H * cap * dh * 2
        ncache = max(2, int(600e6 // per) + 1)
        caches = [(torch.randn(B, H, cap, dh, generator=g, device=dev).half(),
                   torch.randn(B, H, cap, dh, generator=g, device=dev).half()) for _ in range(ncache)]
        q, k, v = [torch.randn(B, H, dh, generator=g, device=dev).half() for _ in range(3)]
        ctx = torch.empty(B, H * dh, dtype=torch.float16, device=dev)
        bias = (torch.rand(H, step, generator=g, device=dev) * 8).half() if alibi else None
        need = lib.eet_mmha_decode_workspace(B, H, dh, step)
        ws = torch.empty(max(need // 4, 1), dtype=torch.float32, device=dev)

        def call(i):
            kc, vc = caches[i % ncache]
            rc = lib.eet_mmha_decode(q.data_ptr(), k.data_ptr(), v.data_ptr(), 0, kc.data_ptr(), vc.data_ptr(),
                                     ctx.data_ptr(), bias.data_ptr() if alibi else None, None, B, H, dh, step, cap,
                                     None, ws.data_ptr(), ws.numel() * 4, st.cuda_stream)
            if rc:
                raise RuntimeError(lib.eet_last_error().decode())
        for i in range(ncache):
            call(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(st)
        for i in range(iters):
            call(i)
        e1.record(st)
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) * 1e-3 / iters
        nbytes = 2 * step * B * H * dh * 2 + 6 * B * H * dh * 2 + (2 * H * step if alibi else 0)
        out[name] = {"us": round(t * 1e6, 1), "GB/s": round(nbytes / t / 1e9, 1),
                     "frac_of_hbm_peak": round(nbytes / t / 1e9 / HBM_PEAK_GBS, 4), "bytes": nbytes}
        del caches
    return out


def attention_timeline(torch, dev, launches=12):
    """Where the time of a decode-attention launch goes, read inside the kernel (bench-only build of the same
    source): back-to-back launches over caches in rotation at the two decoder shapes; the second of two recorded
    passes is analysed."""
    import ctypes
    import numpy as np
    B_ = bench_lib()
    st = torch.cuda.current_stream()
    out = {}
    for name, B, H, step, alibi in (("llama7b B=8 step=1088", 8, 32, 1088, False),
                                    ("baichuan13b B=32 step=2176 alibi", 32, 40, 2176, True)):
        dh, cap = 128, step + 1
        g = torch.Generator(device=dev).manual_seed(step)
        per = 2 * B * H * cap * dh * 2
        ncache = max(2, int(600e6 // per) + 1)
        caches = [(torch.randn(B, H, cap, dh, generator=g, device=dev).half(),
                   torch.randn(B, H, cap, dh, generator=g, device=dev).half()) for _ in range(ncache)]
        q, k, v = [torch.randn(B, H, dh, generator=g, device=dev).half() for _ in range(3)]
        ctx = torch.empty(B, H * dh, dtype=torch.float16, device=dev)
        bias = (torch.rand(H, step, generator=g, device=dev) * 8).half() if alibi else None
        if B_.eet_timeline_attn_begin(2 * launches):
            return {"error": "eet_timeline_attn_begin failed"}
        torch.cuda.synchronize()
        for i in range(2 * launches):
            kc, vc = caches[i % ncache]
            rc = B_.eet_timeline_mmha_decode(q.data_ptr(), k.data_ptr(), v.data_ptr(), 0, kc.data_ptr(), vc.data_ptr(),
                                             ctx.data_ptr(), bias.data_ptr() if alibi else None, None, B, H, dh, step,
                                             cap, None, None, 0, st.cuda_stream)
            if rc:
                return {"error": f"eet_timeline_mmha_decode returned {rc}"}
        torch.cuda.synchronize()
        buf = np.zeros(2048 * 8, dtype=np.uint64)
        stamps = []
        for l in range(launches - 1, 2 * launches):
            wgs = B_.eet_timeline_attn_read(l, buf.ctypes.data_as(ctypes.c_void_p))
            if wgs <= 0:
                return {"error": f"eet_timeline_attn_read({l}) returned {wgs}"}
            stamps.append(buf[: wgs * 8].reshape(wgs, 8).astype(np.int64).copy())
        rows = []
        for i in range(1, len(stamps) - 1):
            prev, cur, nxt = stamps[i - 1], stamps[i], stamps[i + 1]
            t0 = cur[:, 0].min()
            rows.append([nxt[:, 0].min() - t0,                    # period
                         t0 - prev[:, 6].max(),                   # idle: last acknowledged store of the predecessor -> first entry
                         cur[:, 0].max() - t0,                    # entry spread
                         (cur[:, 1] - cur[:, 0]).mean(),          # entry -> new token handled, ring requested
                         (cur[:, 2] - cur[:, 0]).mean(),          # entry -> first row consumed
                         (cur[:, 3] - t0).min(), (cur[:, 3] - t0).mean(), (cur[:, 3] - t0).max(),   # first wavefront through its rows
                         (cur[:, 4] - cur[:, 3]).mean(),          # ... -> all wavefronts of the workgroup through
                         (cur[:, 4] - t0).max(),                  # the last workgroup's barrier
                         (cur[:, 5] - cur[:, 4]).mean(),          # merge of the streams, result stores issued
                         (cur[:, 6] - cur[:, 5]).mean(),          # stores acknowledged
                         cur[:, 6].max() - t0])
        a = np.mean(np.array(rows, dtype=np.float64), axis=0) / 100.0
        out[name] = {"launches": len(rows), "workgroups": int(stamps[1].shape[0]), "period_us": round(a[0], 2),
                     "idle_before_first_entry_us": round(a[1], 2), "entry_spread_us": round(a[2], 2),
                     "entry_to_ring_requested_us": round(a[3], 2), "entry_to_first_row_consumed_us": round(a[4], 2),
                     "first_wavefront_through_after_first_entry_us": {"first": round(a[5], 2), "mean": round(a[6], 2), "last": round(a[7], 2)},
                     "wait_for_the_other_wavefronts_us": round(a[8], 2), "last_workgroup_barrier_after_first_entry_us": round(a[9], 2),
                     "merge_of_the_streams_us": round(a[10], 2), "store_acknowledge_us": round(a[11], 2),
                     "first_entry_to_last_acknowledge_us": round(a[12], 2)}
        del caches
    out["what"] = ("clock readings inside the decode-attention kernel (bench-only build with -DEET_TIMELINE of the same "
                   "source; thread 0 of each workgroup, 100 MHz wall clock), back-to-back launches over caches in rotation, "
                   "second of two recorded passes")
    return out


def recorded_traffic(M, layers):
    """HBM-side bytes per launch of the headline pass as recorded in profiles/ (a line
    'traffic_bytes_per_launch M=<M> layers=<n>: <bytes>' in the pmc summary), or None."""
    import glob
    import re
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*pmc*"))):
        try:
            text = open(path).read()
        except OSError:
            continue
        m = re.search(rf"traffic_bytes_per_launch M={M} layers={layers}: (\d+)", text)
        if m:
            return int(m.group(1)), os.path.relpath(path, ROOT)
    return None, None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--m", type=int, default=8, help="activation rows of the headline GEMM pass")
    ap.add_argument("--layers", type=int, default=LLAMA["layers"])
    ap.add_argument("--gen", type=int, default=128, help="tokens to greedy-decode in the decoder leg (0 = skip)")
    ap.add_argument("--prompt", type=int, default=1024)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-sweep", action="store_true", help="skip the M = 1..32 sweep")
    ap.add_argument("--no-chain", action="store_true", help="skip the chained-launch form of the GEMM pass")
    ap.add_argument("--no-timeline", action="store_true", help="skip the in-kernel clock readings of the GEMM pass")
    ap.add_argument("--no-baichuan", action="store_true",
                    help="skip benchmark configuration 5: Baichuan-13B-shaped decoder (40 layers, ALiBi), batch 32, "
                         "prompt 2048, 256 greedy tokens (needs ~85 GB of HBM and about a minute)")
    ap.add_argument("--only", default="",
                    help="comma-separated extra legs to run instead of all of them (for profiling one kernel): "
                         "prefill_gemm, prefill_attention, decode_attention, packer_device")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three 1 GiB device-to-device copies (a kernel of known traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; --gpus N with N > 1 is not supported (the path has no "
              "collectives: a linear would shard by output channels, or by input features with one all-reduce).",
              file=sys.stderr)
        sys.exit(2)

    import torch

    import eet_amd as eet
    from eet_amd._lib import lib
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP kernels have no CPU fallback.", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    L = lib()
    hidden, d_ff = LLAMA["hidden"], LLAMA["d_ff"]
    weights = make_weights(torch, eet, dev, args.layers, hidden, d_ff, seed=1234)
    g = torch.Generator(device=dev).manual_seed(99)
    acts = {K: torch.randn(32, K, generator=g, device=dev).half() for K in (hidden, d_ff)}
    outs = {N: torch.empty(32, N, dtype=torch.float16, device=dev) for N in (3 * hidden, hidden, d_ff)}
    outs["residual"] = torch.randn(32, hidden, generator=g, device=dev).half()
    outs["gamma"] = (1 + 0.1 * torch.randn(hidden, generator=g, device=dev)).half()
    outs["probe_sink"] = torch.empty(4 * 1024 * 1024, dtype=torch.uint8, device=dev)
    from eet_amd import ops as eet_ops
    fused = fused_launch_weights(eet_ops, weights)

    def pass_bytes(ws, m):
        return sum(linear_bytes(m, w.shape[0], w.shape[1], epi) for layer in ws for (w, _, epi) in layer.values())

    M = args.m
    sec, wall, launches = time_gemm_pass(torch, L, fused, acts, outs, M, args.steps, args.warmup)
    step_bytes = pass_bytes(fused, M)
    gbs = step_bytes / sec / 1e9
    per_launch_us = sec / launches * 1e6
    # the same chain of launches as pure reads of the same weight buffers: what the machine allows
    # (256 workgroups per launch, 688 for gate|up, and two and four times as many: the best of the three counts)
    weight_bytes = sum(w.numel() for layer in fused for (w, _, _) in layer.values())
    try:
        probe_sec = min([time_gemm_pass(torch, L, fused, acts, outs, M, max(3, args.steps // 2), 1, probe=True,
                                        probe_grid_scale=sc)[0] for sc in (1, 2, 4)] +
                        [time_gemm_pass(torch, L, fused, acts, outs, M, max(3, args.steps // 2), 1, probe=True,
                                        probe_grid_scale=sc, probe_ring=True)[0] for sc in (1, 2)])
        ceiling_gbs = weight_bytes / probe_sec / 1e9
        probe_error = None
    except (RuntimeError, OSError, AttributeError) as e:   # the measurement-only library is missing or stale: the headline stands without it
        probe_sec, ceiling_gbs, probe_error = float("nan"), float("nan"), str(e)
    traffic, traffic_file = recorded_traffic(M, args.layers)
    traffic_source = (f"{traffic_file}: FETCH_SIZE + WRITE_SIZE of this command under rocprofv3 --pmc, recorded when that "
                      "file was committed; NOT measured in this run (counters need the profiler)") if traffic_file else None
    if probe_error is None:
        stream_ceiling = {"GB/s": round(ceiling_gbs, 1), "frac_of_peak": round(ceiling_gbs / HBM_PEAK_GBS, 4),
                          "ms_per_step": round(probe_sec * 1e3, 4),
                          "what": "the same 128 launches per step as read-only streams of the same weight "
                                  "buffers (eet_hbm_stream_probe: two batches of four loads per lane in flight, 256 workgroups per launch, 688 "
                                  "for gate|up, also twice and four times as many; eet_hbm_stream_probe_ring: a ring of four loads "
                                  "per lane without a branch, 256 and 512 workgroups; the best of the five): the rate this machine "
                                  "allows a chain of dependent launches of these sizes"}
    else:
        stream_ceiling = {"error": probe_error}
    result = {
        "metric": "int8 W-only GEMM HBM GB/s (% peak) at M=1..16; LLaMA-7B int8 decode tokens/s, 1 GPU",
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp16 activations x int8 weights, fp32 accumulate", "data": "synthetic",
        "config": {"workload": f"LLaMA-7B-shaped decode linears, int8 per-channel weights: {args.layers} layers x "
                               f"(QKV 4096x12288, O 4096x4096, gate/up 4096x11008, down 11008x4096) at M={M}, "
                               "launched as the decoder ops launch them: RMSnorm prologue on QKV, gate and up in "
                               "one launch with the RMSnorm prologue and the SwiGLU epilogue, O and down with the "
                               "residual-add epilogue",
                   "launches_per_step": launches, "bytes_per_step": step_bytes,
                   "pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2)},
        "roofline": {"bound": "hbm", "kernel": "w8a16_small_m_kernel", "achieved": round(gbs, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "avg_launch_us": round(per_launch_us, 3),
                     "algorithmic_bytes_per_launch": round(step_bytes / launches),
                     # HBM-side bytes per launch, from the committed rocprofv3 --pmc summary of this workload
                     # (FETCH_SIZE and WRITE_SIZE scaled by a copy kernel of known size); null if none matches
                     "traffic": traffic, "traffic_source": traffic_source,
                     "stream_ceiling": stream_ceiling,
                     "frac_of_stream_ceiling": round(step_bytes / sec / (weight_bytes / probe_sec), 4) if probe_error is None else None},
        "host_wall_ms_per_step": round(wall * 1e3, 4),
    }

    # the same pass issued as one chain (eet_gemm_w8a16_chained): launches without the queue barrier that
    # wait in the kernel for their producer.  `value` stays the ordinary launch path.
    if not args.no_chain:
        import ctypes
        gave_up = ctypes.c_int(0)
        chain = {}
        for m in ((M,) if args.no_sweep else (1, 4, 8, 16, 32)):
            s_c, _, _ = time_gemm_pass(torch, L, fused, acts, outs, m, max(3, args.steps // 2), 1, chained=True)
            b = pass_bytes(fused, m)
            chain[f"M={m}"] = {"GB/s": round(b / s_c / 1e9, 1), "pct_peak": round(100 * b / s_c / 1e9 / HBM_PEAK_GBS, 2),
                               "avg_launch_us": round(s_c / launches * 1e6, 3)}
        if L.eet_chain_status(ctypes.byref(gave_up), 1, torch.cuda.current_stream().cuda_stream):
            raise RuntimeError(L.eet_last_error().decode())
        chain["a_wait_gave_up"] = bool(gave_up.value)
        chain["what"] = ("the same launches as one chain per pass: each launch after the first is enqueued without the "
                         "queue barrier (hipExtAnyOrderLaunch), requests its first weight batches and then waits in the "
                         "kernel (bounded) for the completion counter of the launch before it")
        result["chained_pass"] = chain

    if not args.no_timeline:
        try:
            result["launch_timeline"] = launch_timeline(torch, L, fused, acts, outs, M)
        except (RuntimeError, OSError, AttributeError) as e:
            result["launch_timeline"] = {"error": str(e)}

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(3)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if not args.no_sweep:
        sweep = {}
        for m in (1, 2, 4, 8, 16, 32):
            s, _, n = time_gemm_pass(torch, L, fused, acts, outs, m, max(3, args.steps // 4), 1)
            b = pass_bytes(fused, m)
            sweep[f"M={m}"] = {"GB/s": round(b / s / 1e9, 1), "pct_peak": round(100 * b / s / 1e9 / HBM_PEAK_GBS, 2)}
        per_shape = {}
        plain = [{k: v + (EPI_NONE,) for k, v in layer.items()} for layer in weights]
        for src, names in ((fused, list(fused[0].keys())), (plain, ["gate", "up"])):
            for name in names:
                sub = [{name: layer[name]} for layer in src]
                s, _, n = time_gemm_pass(torch, L, sub, acts, outs, M, max(3, args.steps // 4), 1)
                w, _, epi = sub[0][name]
                b = linear_bytes(M, w.shape[0], w.shape[1], epi)
                per_shape[f"{name} K={w.shape[0]} N={w.shape[1]}"] = {
                    "us": round(s / n * 1e6, 2), "GB/s": round(b * n / s / 1e9, 1),
                    "pct_peak": round(100 * b * n / s / 1e9 / HBM_PEAK_GBS, 2)}
        result["gemm_by_m"] = sweep
        result[f"gemm_by_shape_M{M}"] = per_shape

    only = [x for x in args.only.split(",") if x]
    if (not args.no_sweep and not only) or "prefill_gemm" in only:
        result["prefill_gemm_config3"] = prefill_gemm_bench(torch, eet, L, dev)
    if (not args.no_sweep and not only) or "prefill_attention" in only:
        result["prefill_attention"] = prefill_attention_bench(torch, L, dev)
    if (not args.no_sweep and not only) or "decode_attention" in only:
        result["decode_attention"] = attention_bench(torch, L, dev)
        if not args.no_timeline:
            try:
                result["decode_attention_timeline"] = attention_timeline(torch, dev)
            except (RuntimeError, OSError, AttributeError) as e:   # measurement only: never ends the run
                result["decode_attention_timeline"] = {"error": str(e)}
    if (not args.no_sweep and not only) or "packer_device" in only:
        result["packer_device"] = device_packer_bench(torch, eet, L, dev)

    if args.gen > 0:
        result["decode"] = decode_bench(torch, eet, weights, dev, args.batch, args.prompt, args.gen, seed=7)

    if not args.no_cpu and args.gen > 0:
        result["decode"]["cpu_baseline"] = cpu_decode_baseline(torch, LLAMA, args.batch, args.prompt + args.gen // 2)

    if not args.no_baichuan:
        del weights, fused
        torch.cuda.empty_cache()
        from eet_amd import ops as _ops
        _ops.workspaces.clear()
        _ops.spare_kv.clear()
        bw = make_weights(torch, eet, dev, BAICHUAN13B["layers"], BAICHUAN13B["hidden"], BAICHUAN13B["d_ff"], seed=4321)
        result["decode_baichuan13b"] = decode_bench(torch, eet, bw, dev, 32, 2048, 256, seed=9, model=BAICHUAN13B,
                                                    graph_batch1=False)
        del bw

    if not args.no_cpu:
        result["packer"] = packer_bench(torch, eet)
        result["cpu_baseline"] = cpu_baseline(torch, M, hidden, d_ff, seed=5)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
