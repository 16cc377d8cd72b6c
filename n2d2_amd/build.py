"""Builds libn2d2hip.so (the C-ABI library of hand-written gfx950 kernels) with hipcc.

hipcc cross-compiles for gfx950 without a GPU.  The library is built in-tree
(n2d2_amd/lib/) so that it travels with the source tree.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libn2d2hip.so")
GLUE_LIB = os.path.join(LIBDIR, "libn2d2_frame_hip.so")
SOURCES = ["act.hip", "conv_igemm.hip", "conv_patch.hip", "conv_s2d.hip", "conv_chain.hip", "conv_pipe_w4.hip", "bottleneck.hip", "depthwise.hip", "dw_pw.hip", "conv_small.hip", "fc_chain.hip", "bandwidth.hip", "quantizer.hip", "train_f32.hip", "diag.hip"]

# -ffp-contract=off: float rescales must round the product and the sum
# separately, as the reference (built for baseline x86-64) does.
# The packed-fp32 target feature is switched off for all device code.
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


PROBE_LIB = os.path.join(LIBDIR, "libn2d2hip_probe.so")


def build_probe(verbose=False):
    """The same library with in-kernel phase probes (-DN2D2HIP_PROFILE, include/n2d2hip_probe.h) as
    lib/libn2d2hip_probe.so.  A measuring tool: N2D2HIP_LIB=<that file> selects it, bench.py --kernel-phases reads it."""
    os.makedirs(LIBDIR, exist_ok=True)
    objdir = os.path.join(LIBDIR, "obj_probe")
    os.makedirs(objdir, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "hipcc")
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in SOURCES]

    def compile_one(pair):
        src, obj = pair
        return _run([hipcc] + HIPCC_FLAGS + ["-DN2D2HIP_PROFILE", "-c", os.path.join(CSRC, src), "-o", obj])

    with ThreadPoolExecutor(max_workers=6) as ex:
        outs = list(ex.map(compile_one, zip(SOURCES, objs)))
    outs.append(_run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", PROBE_LIB] + objs))
    if verbose:
        for o in outs:
            if o.strip():
                print(o)
    return PROBE_LIB


def build(verbose=False):
    os.makedirs(LIBDIR, exist_ok=True)
    objdir = os.path.join(LIBDIR, "obj")
    os.makedirs(objdir, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "hipcc")
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in SOURCES]

    def compile_one(pair):
        src, obj = pair
        return _run([hipcc] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])

    with ThreadPoolExecutor(max_workers=6) as ex:
        outs = list(ex.map(compile_one, zip(SOURCES, objs)))
    outs.append(_run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs))
    # host cells ("Frame_HIP" model): plain C++ over the C ABI
    glue = os.path.join(CSRC, "frame_hip")
    outs.append(_run([os.environ.get("CXX", "g++"), "-std=c++14", "-O2", "-fPIC", "-Wall", "-Wextra", "-Wno-unused-parameter",
                      "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "include"), "-shared",
                      os.path.join(glue, "frame_hip.cpp"), os.path.join(glue, "quantization.cpp"), os.path.join(glue, "qat_fuse.cpp"),
                      os.path.join(glue, "frame_hip_capi.cpp"),
                      os.path.join(glue, "frame_hip_train.cpp"), os.path.join(glue, "frame_hip_train_capi.cpp"),
                      "-o", GLUE_LIB,
                      "-L" + LIBDIR, "-ln2d2hip", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,/opt/rocm/lib"]))
    if verbose:
        for o in outs:
            if o.strip():
                print(o)
    return LIB


if __name__ == "__main__":
    print(build_probe(verbose=True) if "--probe" in sys.argv[1:] else build(verbose=True))
