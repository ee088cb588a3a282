"""Builds libforja_hip.so for gfx950 with hipcc (cross-compiles without a GPU)."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libforja_hip.so")
PROBES = os.path.join(HERE, "libforja_probes.so")
CONFORMANCE = os.path.join(HERE, "host", "conformance")

SOURCES = ["backend.cpp", "generic_ops.hip", "moe.hip", "paged_attention.hip", "qmm_fast.hip", "qmm_gemm.hip", "programs_fast.hip", "lane_fusion.hip", "sampling.hip", "qmm_valu.hip", "qmm_ksplit.hip"]

COMMON = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]
# The generic kernels follow the reference's mul-then-add order; no fused contraction there.
PER_FILE = {"generic_ops.hip": ["-ffp-contract=off"], "sampling.hip": ["-ffp-contract=off"],
            "qmm_valu.hip": ["-ffp-contract=off"]}


def build(verbose=False, jobs=8):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    objects = []
    for src in SOURCES:
        obj = os.path.join(objdir, src + ".o")
        objects.append(obj)
        cmd = [hipcc, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj] + COMMON + PER_FILE.get(src, [])
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    failed = False
    for src, proc in procs:
        out, _ = proc.communicate()
        out = "\n".join(line for line in out.splitlines() if "packed-fp32-ops" not in line)
        if proc.returncode != 0:
            failed = True
            print(f"[forja_amd.build] {src} failed:\n{out}", file=sys.stderr)
        elif verbose and out.strip():
            print(out)
    if failed:
        raise RuntimeError("hipcc failed")
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objects
    subprocess.run(link, check=True)
    build_probes()
    build_host()
    return LIB


def build_probes():
    """bench.py's measurement probes (sustained MFMA rate): a library of their own."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, "-x", "hip", os.path.join(CSRC, "bench_probes.hip"), "-shared", "-o", PROBES] + COMMON
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if out.returncode != 0:
        print(out.stdout, file=sys.stderr)
        raise RuntimeError("hipcc failed on bench_probes.hip")
    return PROBES


def build_host():
    """Compiles the C++ host interface's known-answer program against the built library."""
    host = os.path.join(HERE, "host")
    include = os.path.join(os.path.dirname(HERE), "include")
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-I" + include, "-I" + host,
           os.path.join(host, "conformance.cpp"), "-o", CONFORMANCE, "-L" + HERE, "-lforja_hip",
           "-Wl,-rpath,$ORIGIN/.."]
    subprocess.run(cmd, check=True)
    return CONFORMANCE


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
