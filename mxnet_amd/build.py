"""Builds libmxq_hip.so (the C-ABI HIP launcher) in-tree with hipcc for gfx950."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmxq_hip.so")

HIP_SOURCES = ["mxq_capi.hip", "mxq_cast.hip", "mxq_fc.hip", "mxq_fc_plain.hip", "mxq_fc_f32.hip",
               "mxq_fc_sum.hip", "mxq_conv.hip", "mxq_conv_nchw.hip", "mxq_pool.hip",
               "mxq_eltwise.hip", "mxq_layout.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # one rounding per written float operation: no fused multiply-add
    "-ffp-contract=off",
    # packed FP32 instructions are not to be generated on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-command-line-argument",
    # the entry points of tests/mxq_test_hooks.h (pinned kernel variants): part of the build the
    # test-suite runs against, left out of a release build by dropping this definition
    "-DMXQ_TEST_HOOKS",
]


def build(verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    for src in HIP_SOURCES:
        obj = os.path.join(HERE, "build", src.replace(".hip", ".o"))
        cmd = [hipcc] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        text = out.decode()
        # hipcc's host pass does not know the packed-fp32 feature: harmless
        text = "\n".join(l for l in text.splitlines()
                         if "packed-fp32-ops" not in l and l.strip())
        if text:
            print(text)
        if p.returncode != 0:
            print("FAILED:", src)
            failed = True
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    subprocess.check_call(cmd)
    return LIB


ROOT = os.path.dirname(HERE)
PROBE_LIB = os.path.join(ROOT, "bench_probe.so")


def build_probe(verbose=False):
    """bench_probe.so: the register-only MFMA rate probe bench.py reports next to the FC
    figures.  A bench aid kept beside bench.py, not part of the operator library."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + HIPCC_FLAGS + ["-shared", os.path.join(ROOT, "bench_probe.hip"), "-o",
                                   PROBE_LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    text = "\n".join(l for l in out.stdout.decode().splitlines()
                     if "packed-fp32-ops" not in l and l.strip())
    if text:
        print(text)
    if out.returncode != 0:
        raise RuntimeError("hipcc failed: bench_probe.hip")
    return PROBE_LIB


OPS_LIB = os.path.join(HERE, "libmxq_ops.so")
HOST_SOURCES = ["mxq_registry.cc", "mxq_quantization_ops.cc", "mxq_quantized_tensor_ops.cc",
                "mxq_float_ops.cc", "mxq_graph.cc",
                "mxq_quantize_graph_pass.cc", "mxq_calibrate.cc", "mxq_ndarray_io.cc",
                "mxq_harness.cc"]


def build_ops(verbose=False):
    """libmxq_ops.so: the C++ operator host (registry + FCompute<gpu> functions).  Plain
    C++17, no HIP headers: it reaches the GPU only through libmxq_hip.so's C ABI."""
    cxx = os.environ.get("CXX", "g++")
    srcs = [os.path.join(CSRC, "host", s) for s in HOST_SOURCES]
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off", "-Wall", "-Wextra",
           "-Wno-unused-parameter", "-o", OPS_LIB] + srcs + \
          ["-L" + HERE, "-lmxq_hip", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return OPS_LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
    print(build_ops(verbose="-v" in sys.argv))
    print(build_probe(verbose="-v" in sys.argv))
