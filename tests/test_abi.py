"""The C-ABI libraries load without a GPU and export every symbol the headers
declare; the Python bindings declare a signature for each of them."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mxq_[a-z0-9_]+)\s*\(", text)))


def test_hip_library_exports_every_declared_symbol():
    import mxnet_amd
    names = declared_functions("mxq.h")
    assert len(names) >= 14
    lib = ctypes.CDLL(mxnet_amd._lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n
        assert n in mxnet_amd._lib.SIGNATURES, "no ctypes signature for " + n
    assert mxnet_amd._lib.lib.mxq_abi_version() == 3
    assert mxnet_amd._lib.last_error() == ""


def test_hip_library_has_no_tuning_state():
    """The launcher keeps no mutable process-wide configuration: the old tuning setter and
    its globals are gone; forced kernel variants are arguments of the test-only entry
    points (tests/mxq_test_hooks.h)."""
    import subprocess
    import mxnet_amd
    out = subprocess.run(["nm", "-C", "--defined-only", mxnet_amd._lib.LIB_PATH],
                         capture_output=True, text=True, check=True).stdout
    assert "mxq_set_tuning" not in out
    assert not re.findall(r"\bmxq::g_\w+", out)
    for hook in mxnet_amd._lib.TEST_HOOKS:
        assert hook in out
        assert hook not in declared_functions("mxq.h")
    hooks_h = open(os.path.join(ROOT, "tests", "mxq_test_hooks.h")).read()
    for hook in mxnet_amd._lib.TEST_HOOKS:
        assert hook in hooks_h


def test_ops_library_exports_every_declared_symbol():
    from mxnet_amd import operator as op
    names = declared_functions("mxq_ops.h")
    assert len(names) >= 12
    lib = ctypes.CDLL(op.OPS_LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n
        assert n in op.OPS_SIGNATURES, "no ctypes signature for " + n


def test_argument_validation_needs_no_gpu():
    """Checks that fail before any HIP call: return code + thread-local message."""
    import mxnet_amd
    lib = mxnet_amd._lib.lib
    buf = (ctypes.c_float * 4)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    rc = lib.mxq_quantize_v2(None, p, p, p, p, 4, 9, 1, -1.0, 1.0, None, 0)
    assert rc == -1 and "int8 and uint8" in mxnet_amd._lib.last_error()
    rc = lib.mxq_dequantize(None, p, 0, p, p, p, 4)
    assert rc == -1 and "int8 or uint8" in mxnet_amd._lib.last_error()
    rc = lib.mxq_quantized_fc(None, p, p, None, 4, 4, 16, p, p, p, p, None, None, None, p, p,
                              None, None, None, 0, 0.0, 0.0, None, 0)
    assert rc == -1 and "no output buffer" in mxnet_amd._lib.last_error()
    # the workspace queries are host arithmetic
    assert lib.mxq_quantized_fc_workspace(4, 4, 16, 0) == 0
    rc = lib.mxq_nhwc_to_nchw(None, p, p, 1, 1, 1, 1, 2)
    assert rc == -1 and "elem_bytes" in mxnet_amd._lib.last_error()
    assert lib.mxq_quantize_v2_workspace(1 << 26) >= 64
    # empty tensors are a no-op, like Kernel<gpu>::Launch with N == 0
    assert lib.mxq_dequantize(None, None, 5, p, p, None, 0) == 0


def test_no_fallback_without_library(tmp_path, monkeypatch):
    """The package refuses to import when the HIP library is missing."""
    import importlib.util
    import shutil
    import sys
    pkg = tmp_path / "mxnet_amd_copy"
    shutil.copytree(os.path.join(ROOT, "mxnet_amd"), pkg,
                    ignore=shutil.ignore_patterns("*.so", "build", "__pycache__", "csrc"))
    spec = importlib.util.spec_from_file_location("mxnet_amd_copy", pkg / "__init__.py",
                                                  submodule_search_locations=[str(pkg)])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["mxnet_amd_copy"] = mod
    try:
        try:
            spec.loader.exec_module(mod)
        except ImportError as e:
            assert "libmxq_hip.so is not built" in str(e)
        else:
            raise AssertionError("import succeeded without the HIP library")
    finally:
        sys.modules.pop("mxnet_amd_copy", None)
        for k in [k for k in sys.modules if k.startswith("mxnet_amd_copy.")]:
            sys.modules.pop(k)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU: any other --gpus value exits with a message."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "one GPU" in r.stderr


def test_fc_workspace_query_covers_both_epilogue_forms():
    """mxq_quantized_fc_workspace is host arithmetic: the fused-int8 figure is what both
    mxq_quantized_fc and mxq_quantized_fc_sum (which plans its own tile) may ask for, so it is
    never below the int32 form's figure where both split."""
    import mxnet_amd
    lib = mxnet_amd._lib.lib
    import random
    rnd = random.Random(5)
    for _ in range(200):
        M, N, K = rnd.choice([1, 64, 256, 4096, 50176]), rnd.choice([64, 256, 800, 4096]), \
            rnd.choice([64, 576, 4096, 8192, 25088])
        fused = lib.mxq_quantized_fc_workspace(M, N, K, 1)
        plain = lib.mxq_quantized_fc_workspace(M, N, K, 0)
        assert fused % 256 == 0 and plain % 256 == 0
        assert fused >= plain or plain == 0 or fused == 0
    assert lib.mxq_quantized_fc_workspace(4096, 4096, 4096, 1) == 0
