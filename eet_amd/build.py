"""Builds libeet_hip.so (HIP kernels + C ABI + host packer) and libeet_bench.so (measurement only, no
part of the operator interface: the read-only streaming probe that bench.py times beside the GEMM
pass, and the dequant-GEMM and decode-attention sources compiled a second time with -DEET_TIMELINE, i.e.
with clock readings inside the kernels, under eet_timeline_* names) for gfx950 with hipcc.

Run as `python -m eet_amd.build`.  The libraries are built in-tree, next to this
file, so that they travel with the source tree.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libeet_hip.so")

BENCH_LIB = os.path.join(HERE, "libeet_bench.so")

SOURCES = ["packer.cc", "tuning.cc", "decode_ops.cc", "chain.hip", "packer_device.hip", "gemm_w8a16.hip",
           "gemm_w8a16_large.hip", "mmha_decode.hip", "prefill_attention.hip", "glue.hip"]
BENCH_SOURCES = ["probe.hip"]
# compiled again with -DEET_TIMELINE for libeet_bench.so
TIMELINE_SOURCES = {"gemm_w8a16.hip": "gemm_w8a16.timeline.o", "mmha_decode.hip": "mmha_decode.timeline.o"}

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def build(verbose=True):
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, "_obj"), exist_ok=True)
    for src in SOURCES + BENCH_SOURCES:
        obj = os.path.join(HERE, "_obj", src + ".o")
        if src.endswith(".hip"):
            cmd = [HIPCC] + [f for f in FLAGS if f != "-shared"] + ["-x", "hip", "-c"]
        else:   # host-only source: no device pass
            cmd = [HIPCC, "-x", "c++", "-O3", "-std=c++17", "-fPIC", "-pthread", "-c"] + [f for f in FLAGS if f.startswith("-I")]
        cmd += [os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for src, obj in TIMELINE_SOURCES.items():
        cmd = [HIPCC] + [f for f in FLAGS if f != "-shared"] + ["-DEET_TIMELINE", "-x", "hip", "-c", os.path.join(CSRC, src),
                                                               "-o", os.path.join(HERE, "_obj", obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src + " (timeline)", subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if out.strip() and verbose:
            print(out)
        if p.returncode != 0:
            print(f"[eet_amd.build] compiling {src} failed", file=sys.stderr)
            failed = True
    if failed:
        raise RuntimeError("hipcc failed")
    for lib, srcs in ((LIB, SOURCES), (BENCH_LIB, BENCH_SOURCES)):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + \
              [os.path.join(HERE, "_obj", src + ".o") for src in srcs]
        if lib == BENCH_LIB:   # the instrumented GEMM uses the operator library's dispatch tables and error slot
            cmd += [os.path.join(HERE, "_obj", obj) for obj in TIMELINE_SOURCES.values()]
            cmd += ["-L" + HERE, "-leet_hip", "-Wl,-rpath,$ORIGIN"]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build()
