#!/usr/bin/env python3
"""Headline benchmark: int8 weight-only GEMM HBM GB/s at LLaMA-7B decode shapes,
plus LLaMA-7B-shaped int8 decode tokens/s, on one MI355X.

A "step" is one pass of the fused dequant-GEMM over every int8 linear of a
32-layer LLaMA-7B-shaped decoder (160 launches over 6.48 GB of distinct packed
weights, so nothing is served from the 256 MB Infinity Cache) at M = 8 rows of
fp16 activations.  `value` is algorithmic bytes per step / time per step.

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


def launch_shapes(hidden, d_ff):
    return [("qkv", hidden, 3 * hidden, EPI_NONE), ("o+residual", hidden, hidden, EPI_RESIDUAL),
            ("gate|up+swiglu", hidden, 2 * d_ff, EPI_SWIGLU), ("down+residual", d_ff, hidden, EPI_RESIDUAL)]


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


def fused_launch_weights(eet_ops, weights):
    """Per layer, the operands of the four launches of launch_shapes()."""
    out = []
    for layer in weights:
        w01, s01 = eet_ops.interleave_gate_up(layer["gate"][0], layer["gate"][1], layer["up"][0], layer["up"][1])
        out.append({"qkv": layer["qkv"] + (EPI_NONE,), "o+residual": layer["o"] + (EPI_RESIDUAL,),
                    "gate|up+swiglu": (w01, s01, EPI_SWIGLU), "down+residual": layer["down"] + (EPI_RESIDUAL,)})
    return out


def time_gemm_pass(torch, lib, weights, acts, outs, M, steps, warmup):
    """Returns seconds per step (one pass over all linears), measured with
    events on the stream the kernels are launched on."""
    st = torch.cuda.current_stream()
    calls = []
    for layer in weights:
        for name, (w, s, epi) in layer.items():
            K, N = w.shape
            n_out = N // 2 if epi == EPI_SWIGLU else N
            res = outs["residual"].data_ptr() if epi == EPI_RESIDUAL else None
            calls.append((acts[K].data_ptr(), w.data_ptr(), s.data_ptr(), outs[n_out].data_ptr(), M, N, K, epi, res))
    f = lib.eet_gemm_w8a16_fused
    sp = st.cuda_stream

    def one_pass():
        for (a, w, s, c, m, n, k, epi, res) in calls:
            rc = f(a, w, s, c, m, n, k, epi, res, None, 0.0, None, 0, sp)
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


def cpu_baseline(torch, M, hidden, d_ff, seed, budget_s=12.0):
    """The reference CPU path, timed on the host cores: torch dequantise
    (int8 * scale -> fp32) + fp32 matmul -> fp16, for one layer's five linears
    (the same shapes as the GPU workload; a bounded sample of it)."""
    from oracle import cpu_path
    threads = min(os.cpu_count() or 1, 16)
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
    return {"value": round(nbytes / per_layer / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"one LLaMA-7B layer (5 int8 linears, M={M}, {nbytes / 1e6:.1f} MB algorithmic), "
                      f"{reps} reps, torch {torch.__version__} dequant+matmul fp32, "
                      f"{per_layer * 1e3:.1f} ms per layer"}


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
           "Mweights_per_s": round(K * N / t_ours / 1e6, 1), "threads": min(os.cpu_count() or 1, 16)}
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


def decode_bench(torch, eet, weights, dev, batch, prompt, gen, seed, model=LLAMA):
    """Int8 decoder of the given shape, random init: prefill `prompt` tokens then
    greedy-decode `gen` tokens; tokens/s = batch * (gen - 1) / decode time."""
    from eet_amd import decoder as D
    cfg = D.DecoderConfig(num_layers=len(weights), hidden=model["hidden"], heads=model["heads"], d_ff=model["d_ff"],
                          vocab=model["vocab"], alibi=model["alibi"], max_batch=batch, max_prompt=prompt,
                          max_full_seq=prompt + gen + 1)
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
    steps = gen - 1
    ms = t_dec / steps * 1e3
    # algorithmic HBM bytes of one token step: int8 weights + scales, KV cache read at mid length, fp16 lm_head
    wbytes = sum(w.numel() + 2 * s.numel() for layer in weights for (w, s) in layer.values())
    kv = len(weights) * 2 * (prompt + gen // 2) * batch * H * 2
    step_bytes = wbytes + kv + cfg.vocab * H * 2
    return {"tokens_per_s": round(batch * steps / t_dec, 1), "ms_per_token_step": round(ms, 3), "batch": batch,
            "prompt": prompt, "generated": gen, "layers": len(weights), "prefill_s": round(t_prefill, 3), "prefill_warm_s": round(t_prefill_warm, 3),
            "step_hbm_bytes": step_bytes,
            "step_roofline_frac": round(step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--m", type=int, default=8, help="activation rows of the headline GEMM pass")
    ap.add_argument("--layers", type=int, default=LLAMA["layers"])
    ap.add_argument("--gen", type=int, default=128, help="tokens to greedy-decode in the decoder leg (0 = skip)")
    ap.add_argument("--prompt", type=int, default=1024)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-sweep", action="store_true", help="skip the M = 1..32 sweep")
    ap.add_argument("--baichuan", action="store_true",
                    help="also run benchmark configuration 5: Baichuan-13B-shaped decoder (40 layers, ALiBi), batch 32, "
                         "prompt 2048, 256 greedy tokens (needs ~85 GB of HBM and about a minute)")
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
    from eet_amd import ops as eet_ops
    fused = fused_launch_weights(eet_ops, weights)

    def pass_bytes(ws, m):
        return sum(linear_bytes(m, w.shape[0], w.shape[1], epi) for layer in ws for (w, _, epi) in layer.values())

    M = args.m
    sec, wall, launches = time_gemm_pass(torch, L, fused, acts, outs, M, args.steps, args.warmup)
    step_bytes = pass_bytes(fused, M)
    gbs = step_bytes / sec / 1e9
    per_launch_us = sec / launches * 1e6
    result = {
        "metric": "int8 W-only GEMM HBM GB/s (% peak) at M=1..16; LLaMA-7B int8 decode tokens/s, 1 GPU",
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp16 activations x int8 weights, fp32 accumulate", "data": "synthetic",
        "config": {"workload": f"LLaMA-7B-shaped decode linears, int8 per-channel weights: {args.layers} layers x "
                               f"(QKV 4096x12288, O 4096x4096, gate/up 4096x11008, down 11008x4096) at M={M}, "
                               "launched as the decoder ops launch them: gate and up in one launch with the "
                               "SwiGLU epilogue, O and down with the residual-add epilogue",
                   "launches_per_step": launches, "bytes_per_step": step_bytes,
                   "pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2)},
        "roofline": {"bound": "hbm", "kernel": "w8a16_small_m_kernel", "achieved": round(gbs, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "avg_launch_us": round(per_launch_us, 3),
                     "algorithmic_bytes_per_launch": round(step_bytes / launches),
                     # HBM-side bytes per launch from rocprofv3 --pmc FETCH_SIZE (x2.000, calibrated on a
                     # 1 GiB copy) + WRITE_SIZE (x1.000) at the default workload (measured once, not per run)
                     "traffic": 51.73e6 if (M == 8 and args.layers == 32) else None},
        "host_wall_ms_per_step": round(wall * 1e3, 4),
    }

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(3)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if not args.no_sweep:
        sweep = {}
        for m in (1, 4, 8, 16, 32):
            s, _, n = time_gemm_pass(torch, L, fused, acts, outs, m, max(3, args.steps // 4), 1)
            b = pass_bytes(fused, m)
            sweep[f"M={m}"] = {"GB/s": round(b / s / 1e9, 1), "pct_peak": round(100 * b / s / 1e9 / HBM_PEAK_GBS, 2)}
        per_shape = {}
        plain = [{k: v + (EPI_NONE,) for k, v in layer.items()} for layer in weights]
        for src, names in ((fused, [n for n, _, _, _ in launch_shapes(hidden, d_ff)]), (plain, ["gate", "up"])):
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

    if not args.no_sweep:
        result["prefill_gemm_config3"] = prefill_gemm_bench(torch, eet, L, dev)
        result["decode_attention"] = attention_bench(torch, L, dev)
        result["packer_device"] = device_packer_bench(torch, eet, L, dev)

    if args.gen > 0:
        result["decode"] = decode_bench(torch, eet, weights, dev, args.batch, args.prompt, args.gen, seed=7)

    if args.baichuan:
        del weights, fused
        torch.cuda.empty_cache()
        from eet_amd import ops as _ops
        _ops.workspaces.clear()
        bw = make_weights(torch, eet, dev, BAICHUAN13B["layers"], BAICHUAN13B["hidden"], BAICHUAN13B["d_ff"], seed=4321)
        result["decode_baichuan13b"] = decode_bench(torch, eet, bw, dev, 32, 2048, 256, seed=9, model=BAICHUAN13B)
        del bw

    if not args.no_cpu:
        result["packer"] = packer_bench(torch, eet)
        result["cpu_baseline"] = cpu_baseline(torch, M, hidden, d_ff, seed=5)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
