"""Builds dsgx10_amd/csrc/libdsgx.so (the C ABI + every gfx950 kernel) with hipcc, in-tree.

    python -m dsgx10_amd.build [-j N] [--force]
"""
import argparse
import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
SO = os.path.join(CSRC, "libdsgx.so")
SOURCES = ["abi.hip", "route.hip", "gemv.hip", "moe_decode.hip", "moe_decode_fp8.hip", "moe_decode_int4.hip", "moe_decode_int4_mfma.hip", "moe_decode_mxfp4_mfma.hip",
           "moe_decode_bf16.hip", "moe_prefill.hip"]
# -packed-fp32-ops off: hipcc -O3 otherwise forms v_pk_*_f32 from scalar float code
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function"]


def _deps():
    return [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".cuh", ".h"))] + \
           [os.path.join(HERE, "..", "include", "dsgx.h")]


def _stale(out, srcs):
    if not os.path.exists(out):
        return True
    t = os.path.getmtime(out)
    return any(os.path.getmtime(s) > t for s in srcs)


def _compile(src, force, extra=(), suffix=""):
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + suffix + ".o")
    path = os.path.join(CSRC, src)
    if force or _stale(obj, [path] + _deps()):
        cmd = ["hipcc"] + FLAGS + list(extra) + ["-c", path, "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
        if r.returncode:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, err))
        if err.strip():
            sys.stderr.write(err + "\n")
    return obj


def build(jobs=None, force=False, extra=(), suffix=""):
    """extra / suffix: a diagnostic variant (e.g. extra=["-DDSGX_TRACE"], suffix="_trace" -> libdsgx_trace.so; DSGX_TRACE:
    the decode kernels' phase stamps, DSGX_PF_TRACE: the FP8 prefill GEMM's, eight wall-clock stamps a workgroup into the
    buffer whose address DSGX_PF_TRACE_PTR names; DSGX_LIB=libdsgx_trace.so loads the variant)"""
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    jobs = jobs or min(len(srcs), os.cpu_count() or 4)
    so = SO.replace(".so", suffix + ".so")
    with cf.ThreadPoolExecutor(jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force, extra, suffix), srcs))
    if force or _stale(so, objs):
        cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", so] + objs
        subprocess.check_call(cmd)
    if not suffix:
        build_mirror_run(force)
    return so


def build_mirror_run(force=False):
    """tests/mirror_run: the test program that drives the C++ mirror headers on the GPU (host code only; it links the
    library just built and finds it relative to its own place)"""
    root = os.path.dirname(HERE)
    inc = os.path.join(root, "include")
    hdrs = [os.path.join(dp, f) for dp, _, fs in os.walk(inc) for f in fs]
    exe = None
    for name in ("mirror_run", "mirror_run_dsk"):
        src, exe = os.path.join(root, "tests", name + ".cpp"), os.path.join(root, "tests", name)
        if not os.path.exists(src):
            continue
        if force or _stale(exe, [src, SO] + hdrs):
            subprocess.check_call(["hipcc", "-std=c++17", "-O1", "-Wall", "-I", inc, src, "-o", exe, "-L", CSRC, "-ldsgx",
                                   "-Wl,-rpath,$ORIGIN/../dsgx10_amd/csrc"])
    return exe


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("-j", type=int, default=None)
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--trace", action="store_true", help="the diagnostic variant libdsgx_trace.so (phase time stamps)")
    a = ap.parse_args()
    print(build(a.j, a.force, ["-DDSGX_TRACE", "-DDSGX_PF_TRACE"], "_trace") if a.trace else build(a.j, a.force))
