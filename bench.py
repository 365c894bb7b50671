#!/usr/bin/env python3
"""Benchmark of the MI355X int8 operator path (one GPU).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one pass of the hot path over one batch of synthetic input that is
already resident in HBM.  The defaults (2000 warm-up + 2000 timed steps, 0.26 s for the
default workload) are long enough for the clocks to settle: over the first ~100 ms after an
idle period the same kernels run 5-15 % slower.  The default workload is the quantized fully-connected
layer at M=K=N=4096 with the bias and the calibrated requantize-to-int8 fused in
the epilogue; --workload selects the other headline kernels (the 64M-element
quantize / requantize / dequantize casts, the 8192^3 FC, the ResNet-50 conv stacks).  One
JSON line is printed.  `roofline` describes the workload's kernel (algorithmic bytes or ops
per launch over the HIP-event-timed average launch; `traffic` is read from the rocprofv3
summary under profiles/ that `traffic_source` names); `other_kernels` lists the same
figures for the other kernels of the path and for the ResNet-50 conv stack and the BERT FC
chain (many small launches: captured into a HIP graph), measured in the same run;
`cpu_baseline` is the CPU oracle (the restatement of the reference's native CPU
operator) timed on a bounded sample on this host.  The last key, `targets`, repeats the
rows a reader looks for first (the casts, FC 8192^3, the two conv stacks) as
[us per step, achieved, fraction of peak], so that a truncated tail of the line still
holds them.
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

METRIC = "int8 FC TOPS (% MFMA peak) + quant/requant GB/s (% HBM peak), 1 GPU"
HBM_PEAK_GBS = 8000.0    # MI355X HBM3E
INT8_PEAK_TOPS = 5000.0  # MI355X dense int8 MFMA

# `roofline.traffic`: HBM bytes per step of the workload's kernels, read at run time from the
# rocprofv3 summary under profiles/ that holds the workload's `--pmc FETCH_SIZE` / `--pmc
# WRITE_SIZE` runs (KiB per dispatch; FETCH_SIZE x 2.00 per the copy-kernel calibration,
# profiles/copy_calibration_64M.md), so the figure cannot drift from the file it cites
# (`roofline.traffic_source`).  It is that profile's figure, not a counter read in this run;
# a workload without such a file reports null.
TRAFFIC_PROFILES = {
    "fc4096": "profiles/fc_dma_kernel_4096.md",
    "fc8192": "profiles/fc_dma_kernel_8192.md",
    "quantize": "profiles/quantize_kernel_64M.md",
    "quantize_uncal": "profiles/quantize_uncalibrated_64M.md",
    "requantize": "profiles/requantize_kernel_64M.md",
    "requantize_uncal": "profiles/requantize_uncalibrated_64M.md",
    "dequantize": "profiles/dequantize_chunk_kernel_64M.md",
    "elemwise_add": "profiles/add32_chunk_kernel_64M.md",
    "elemwise_add_int8": "profiles/add_kernel_int8_64M.md",
    "concat": "profiles/concat_kernel_64M.md",
    "quantized_act": "profiles/relu_chunk_kernel_64M.md",
    "maxpool": "profiles/pool_lds_kernel_maxpool.md",
    "avgpool": "profiles/pool_lds_kernel_global_avgpool.md",
    "resnet50_convs": "profiles/conv_stack_resnet50.md",
    "resnet50_convs_operator": "profiles/conv_stack_resnet50_operator_contract.md",
    "elemwise_mul_int8": "profiles/mul_kernel_int8_64M.md",
    "quantize_asym": "profiles/quantize_asym_kernel_64M.md",
    "batch_norm": "profiles/bn_rows_kernel_nchw_64M.md",
    "embedding": "profiles/embedding_kernel_bert_vocab.md",
    "transpose": "profiles/permute_elem_direct_kernel_attention_64M.md",
    "transpose_to_nhwc": "profiles/permute_tile16_kernel_to_nhwc_64M.md",
    "transpose_to_nchw": "profiles/permute_tile16_kernel_to_nchw_64M.md",
}


def profile_traffic(key):
    """(bytes per step, file) from the profile summary of workload `key`, or (None, None).
    A summary of many launches per step states `traffic_bytes_per_step: N`; one of a single
    launch (or of a two-launch step with one row per kernel and counter) is summed from its
    counter table."""
    import re
    rel = TRAFFIC_PROFILES.get(key)
    if rel is None or not os.path.exists(os.path.join(ROOT, rel)):
        return None, None
    text = open(os.path.join(ROOT, rel)).read()
    m = re.search(r"traffic_bytes_per_step:\s*([0-9.eE+]+)", text)
    if m:
        return float(m.group(1)), rel
    fetch = write = 0.0
    rows = re.findall(r"^\| `[^`]*` \| (FETCH_SIZE|WRITE_SIZE) \| \d+ \| ([0-9.]+) \|", text, re.M)
    for counter, kib in rows:
        if counter == "FETCH_SIZE":
            fetch += float(kib)
        else:
            write += float(kib)
    if not rows:
        return None, None
    return (2.0 * fetch + write) * 1024.0, rel


# What a default run measures besides the headline workload, in this order.  The operators
# outside the five the metric names keep their workloads (--workload) but are not part of
# the default run.
CAST_TARGETS = ["quantize", "quantize_laplace", "quantize_uint8", "quantize_uncal",
                "quantize_uint8_uncal", "requantize", "requantize_uncal", "dequantize"]
OTHER_WORKLOADS = CAST_TARGETS + [
    "quantize_v1", "quantized_act", "small_casts", "elemwise_add", "elemwise_add_int8", "concat",
    "maxpool", "avgpool", "fc8192", "resnet50_convs", "resnet50_convs_operator",
    "resnet50_chain_unfused", "resnet50_chain", "resnet50_chain_fused", "bert_fc_chain",
    "bert_fc_chain_fused", "bert_fc_chain_f32"]
SUMMARY_WORKLOADS = CAST_TARGETS + ["fc8192", "resnet50_convs", "resnet50_convs_operator",
                                    "resnet50_chain_fused", "bert_fc_chain",
                                    "bert_fc_chain_fused", "bert_fc_chain_f32"]


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=2000)
    ap.add_argument("--workload", default="fc4096",
                    choices=["fc4096", "fc8192", "quantize", "quantize_uncal", "quantize_uint8",
                             "quantize_v1", "quantized_act",
                             "quantize_laplace", "quantize_uint8_uncal", "small_casts",
                             "requantize", "requantize_uncal", "dequantize", "copy", "maxpool", "avgpool",
                             "elemwise_add", "elemwise_add_int8", "concat", "elemwise_mul_int8", "quantize_asym",
                             "batch_norm", "embedding", "transpose", "transpose_to_nhwc", "transpose_to_nchw",
                             "resnet50_convs", "resnet50_convs_operator",
                             "resnet50_convs_operator_adapters", "resnet50_chain",
                             "resnet50_chain_fused", "resnet50_chain_unfused",
                             "bert_fc_chain",
                             "bert_fc_chain_fused",
                             "bert_fc_chain_f32"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-cast-ops", action="store_true")
    return ap.parse_args()


class FcWorkload:
    """Benchmark configuration 3: data quantized from U(-1,1) with calib (-1,1), weight from
    N(0,0.02) with its own min/max, int8 bias, fused requantize with a calibrated range."""

    def __init__(self, S, torch, capi, lib):
        import numpy as np
        self.S = S
        self.name = "quantized_fully_connected M=K=N=%d, int8 bias + calibrated requantize " \
                    "fused in the epilogue" % S
        self.kernel = "fc_dma_kernel"
        self.bound = "mfma"
        self.ops = 2.0 * S * S * S
        g = torch.Generator(device="cuda").manual_seed(0)
        x = torch.rand((S, S), device="cuda", generator=g) * 2.0 - 1.0
        self.data, self.dmin, self.dmax = capi.quantize_v2(x, "int8", min_calib_range=-1.0,
                                                           max_calib_range=1.0)
        w = torch.randn((S, S), device="cuda", generator=g) * 0.02
        self.weight, self.wmin, self.wmax = capi.quantize(w, w.min().reshape(1),
                                                          w.max().reshape(1))
        b = torch.randn((S,), device="cuda", generator=g) * 0.02
        self.bias, self.bmin, self.bmax = capi.quantize(b, b.min().reshape(1), b.max().reshape(1))
        del x, w
        # calibration range of the output: max |fp32 output| over a 1-in-64 row sample
        rows = self.data[::64].to(torch.float32) @ self.weight.to(torch.float32).t()
        scale = (self.dmax.item() / 127.0) * (self.wmax.abs().item() / 127.0)
        r = float(rows.abs().max().item() * scale)
        self.calib = (-r, r)
        self.out8 = torch.empty((S, S), dtype=torch.int8, device="cuda")
        self.sc = [torch.empty(1, device="cuda") for _ in range(4)]
        self.ws = fc_workspace(torch, lib, S, S, S, True)
        self.lib = lib
        self.P = lambda t: ctypes.c_void_p(t.data_ptr())
        self.torch = torch

    def step(self):
        P, S = self.P, self.S
        st = ctypes.c_void_p(self.torch.cuda.current_stream().cuda_stream)
        rc = self.lib.mxq_quantized_fc(st, P(self.data), P(self.weight), P(self.bias), S, S, S,
                                       P(self.dmin), P(self.dmax), P(self.wmin), P(self.wmax),
                                       P(self.bmin), P(self.bmax), None, P(self.sc[0]),
                                       P(self.sc[1]), P(self.out8), P(self.sc[2]), P(self.sc[3]),
                                       0, self.calib[0], self.calib[1], *ws_args(self.ws))
        if rc != 0:
            raise RuntimeError(self.lib.mxq_last_error().decode())

    def value(self, sec_per_step):
        return self.ops / sec_per_step / 1e12, "TOPS"

    def cpu_baseline(self, oracle, budget_s=12.0):
        """Oracle FC on the first rows of the same operands, sized to ~budget_s."""
        import numpy as np
        S = self.S
        w = self.weight.cpu().numpy()
        d = self.data.cpu().numpy()
        t0 = time.perf_counter()
        oracle.fc_int32(d[:64], w)
        t64 = time.perf_counter() - t0
        rows = int(max(64, min(S, 64 * budget_s / max(t64, 1e-9))))
        reps, t0 = 0, time.perf_counter()
        while True:
            oracle.fc_int32(d[:rows], w)
            reps += 1
            dt = time.perf_counter() - t0
            if dt >= budget_s * 0.8 or reps >= 100:
                break
        tops = 2.0 * rows * S * S * reps / dt / 1e12
        return {"value": tops, "unit": "TOPS", "cores": oracle.num_threads(), "kind": "port",
                "sample": "oracle qref_fc (OpenMP) on the first %d of %d data rows against the "
                          "full [%d,%d] weight, %d repetitions, %.1f s" % (rows, S, S, S, reps,
                                                                           dt)}


def fc_workspace(torch, lib, M, N, K, fused):
    """The scratch mxq_quantized_fc asks for on this shape (None when it would not split)."""
    nbytes = lib.mxq_quantized_fc_workspace(M, N, K, int(fused))
    return torch.empty(nbytes, dtype=torch.uint8, device="cuda") if nbytes else None


def ws_args(ws):
    if ws is None:
        return None, 0
    return ctypes.c_void_p(ws.data_ptr()), ws.numel()


class CastWorkload:
    """Benchmark configuration 2: 64M-element flat tensors, buffers rotated so that the
    256 MB Infinity Cache cannot serve the reads."""
    N = 1 << 26
    NBUF = 3

    def __init__(self, kind, torch, capi, lib):
        import numpy as np
        self.kind = kind
        self.torch = torch
        self.lib = lib
        n = self.N
        self.bound = "hbm"
        self.P = lambda t: ctypes.c_void_p(t.data_ptr())
        g = torch.Generator(device="cuda").manual_seed(1)
        self.i = 0
        self.omin = torch.empty(1, device="cuda")
        self.omax = torch.empty(1, device="cuda")
        self.ws = torch.empty(lib.mxq_quantize_v2_workspace(n), dtype=torch.uint8, device="cuda")
        if kind in ("quantize", "quantize_uncal", "quantize_uint8", "quantize_laplace",
                    "quantize_uint8_uncal"):
            self.src = []
            for _ in range(self.NBUF):
                if kind == "quantize_laplace":
                    # Laplace(0, 1) by inversion of its distribution function
                    u = torch.rand(n, device="cuda", generator=g) - 0.5
                    x = -torch.sign(u) * torch.log1p(-2.0 * u.abs())
                    del u
                else:
                    x = torch.randn(n, device="cuda", generator=g)
                idx = torch.randint(0, n, (n // 10000,), device="cuda", generator=g)
                sign = torch.randint(0, 2, (n // 10000,), device="cuda", generator=g) * 2 - 1
                x[idx] = 50.0 * sign.to(torch.float32)
                self.src.append(x)
            self.dst = [torch.empty(n, dtype=torch.uint8, device="cuda")
                        for _ in range(self.NBUF)]
            uncal = kind in ("quantize_uncal", "quantize_uint8_uncal")
            self.bytes = (9.0 if uncal else 5.0) * n
            self.kernel = "quantize_kernel" + (" + minmax_f32_kernel" if uncal else "")
            self.name = {"quantize": "quantize_v2 fp32->int8 calibrated (-50,50), N(0,1) input "
                                     "with 0.01% outliers at +-50",
                         "quantize_uncal": "quantize_v2 fp32->int8 uncalibrated "
                                           "(on-device min/max)",
                         "quantize_uint8": "quantize_v2 fp32->uint8 calibrated (-50,50)",
                         "quantize_laplace": "quantize_v2 fp32->int8 calibrated (-50,50), "
                                             "Laplace(0,1) input with 0.01% outliers at +-50",
                         "quantize_uint8_uncal": "quantize_v2 fp32->uint8 uncalibrated "
                                                 "(on-device min/max)"}[kind]
        elif kind.startswith("requantize"):
            self.src = [torch.randint(-2 ** 28, 2 ** 28, (n,), device="cuda", generator=g,
                                      dtype=torch.int32) for _ in range(self.NBUF)]
            self.dst = [torch.empty(n, dtype=torch.int8, device="cuda")
                        for _ in range(self.NBUF)]
            self.imin = torch.tensor([-1.0], device="cuda")
            self.imax = torch.tensor([1.0], device="cuda")
            self.bytes = (9.0 if kind == "requantize_uncal" else 5.0) * n
            self.kernel = "requantize_kernel" + (" + minmax_i32_kernel"
                                                 if kind == "requantize_uncal" else "")
            self.name = ("requantize int32->int8 " +
                         ("uncalibrated (on-device min/max)" if kind == "requantize_uncal"
                          else "calibrated (-0.1,0.1)"))
        elif kind == "quantize_v1":
            self.src = [torch.randn(n, device="cuda", generator=g).clamp_(-4.0, 4.0)
                        for _ in range(self.NBUF)]
            self.dst = [torch.empty(n, dtype=torch.int8, device="cuda")
                        for _ in range(self.NBUF)]
            self.imin = torch.tensor([-4.0], device="cuda")
            self.imax = torch.tensor([4.0], device="cuda")
            self.bytes = 5.0 * n
            self.kernel = "quantize_kernel"
            self.name = "quantize (v1) fp32->int8, range (-4,4) given as inputs"
        elif kind == "quantized_act":
            self.src = [torch.randint(-127, 128, (n,), device="cuda", generator=g,
                                      dtype=torch.int8) for _ in range(self.NBUF)]
            self.dst = [torch.empty(n, dtype=torch.int8, device="cuda") for _ in range(self.NBUF)]
            self.imin = torch.tensor([-3.0], device="cuda")
            self.imax = torch.tensor([3.0], device="cuda")
            self.bytes = 2.0 * n
            self.kernel = "relu_chunk_kernel"
            self.name = "quantized_act relu int8->int8"
        elif kind == "dequantize":
            self.src = [torch.randint(-127, 128, (n,), device="cuda", generator=g,
                                      dtype=torch.int8) for _ in range(self.NBUF)]
            self.dst = [torch.empty(n, dtype=torch.float32, device="cuda")
                        for _ in range(self.NBUF)]
            self.imin = torch.tensor([-3.0], device="cuda")
            self.imax = torch.tensor([3.0], device="cuda")
            self.bytes = 5.0 * n
            self.kernel = "dequantize_chunk_kernel"
            self.name = "dequantize int8->fp32"
        elif kind in ("elemwise_add", "elemwise_add_int8"):
            self.src = [torch.randint(-127, 128, (n,), device="cuda", generator=g,
                                      dtype=torch.int8) for _ in range(self.NBUF)]
            self.rhs = [torch.randint(-127, 128, (n,), device="cuda", generator=g,
                                      dtype=torch.int8) for _ in range(self.NBUF)]
            out_dtype = torch.int32 if kind == "elemwise_add" else torch.int8
            self.dst = [torch.empty(n, dtype=out_dtype, device="cuda") for _ in range(self.NBUF)]
            self.imin = torch.tensor([-3.0], device="cuda")
            self.imax = torch.tensor([3.0], device="cuda")
            self.bytes = (6.0 if kind == "elemwise_add" else 3.0) * n
            self.kernel = "add32_chunk_kernel" if kind == "elemwise_add" else "add_kernel"
            self.name = ("quantized_elemwise_add int8+int8->" +
                         ("int32" if kind == "elemwise_add" else "int8 calibrated (-5,5)"))
        elif kind == "concat":
            half = n // 2
            self.src = [torch.randint(-127, 128, (half,), device="cuda", generator=g,
                                      dtype=torch.int8) for _ in range(self.NBUF)]
            self.rhs = [torch.randint(-127, 128, (half,), device="cuda", generator=g,
                                      dtype=torch.int8) for _ in range(self.NBUF)]
            self.dst = [torch.empty(n, dtype=torch.int8, device="cuda") for _ in range(self.NBUF)]
            self.ranges = [torch.tensor([v], device="cuda") for v in (-1.0, 1.0, -2.0, 2.0)]
            self.c_types = (ctypes.c_int * 2)(5, 5)
            self.c_mins = (ctypes.c_void_p * 2)(self.ranges[0].data_ptr(),
                                                self.ranges[2].data_ptr())
            self.c_maxs = (ctypes.c_void_p * 2)(self.ranges[1].data_ptr(),
                                                self.ranges[3].data_ptr())
            self.c_ext = (ctypes.c_int64 * 2)(half, half)
            self.bytes = 2.0 * n
            self.kernel = "concat_kernel"
            self.name = "quantized_concat of two int8 halves, ranges (-1,1) and (-2,2): " \
                        "one half rescaled, one copied"
        elif kind == "elemwise_mul_int8":
            self.src = [torch.randint(-127, 128, (n,), device="cuda", generator=g,
                                      dtype=torch.int8) for _ in range(self.NBUF)]
            self.rhs = [torch.randint(-127, 128, (n,), device="cuda", generator=g,
                                      dtype=torch.int8) for _ in range(self.NBUF)]
            self.dst = [torch.empty(n, dtype=torch.int8, device="cuda") for _ in range(self.NBUF)]
            self.imin = torch.tensor([-3.0], device="cuda")
            self.imax = torch.tensor([3.0], device="cuda")
            self.bytes = 3.0 * n
            self.kernel = "mul_kernel"
            self.name = "quantized_elemwise_mul int8*int8->int8 calibrated (-9,9)"
        elif kind == "quantize_asym":
            self.src = [torch.randn(n, device="cuda", generator=g) for _ in range(self.NBUF)]
            self.dst = [torch.empty(n, dtype=torch.uint8, device="cuda")
                        for _ in range(self.NBUF)]
            self.bytes = 5.0 * n
            self.kernel = "quantize_asym_kernel"
            self.name = "quantize_asym fp32->uint8 calibrated (-6,6)"
        elif kind == "batch_norm":
            # NCHW (64, 256, 64, 64) int8 -> int8, relu fused: one byte in, one out per element
            self.channels, self.inner = 256, 64 * 64
            self.outer = n // (self.channels * self.inner)
            self.src = [torch.randint(-127, 128, (n,), device="cuda", generator=g,
                                      dtype=torch.int8) for _ in range(self.NBUF)]
            self.dst = [torch.empty(n, dtype=torch.int8, device="cuda") for _ in range(self.NBUF)]
            self.gamma = torch.rand(self.channels, device="cuda", generator=g) + 0.5
            self.beta = torch.randn(self.channels, device="cuda", generator=g)
            self.mean = torch.randn(self.channels, device="cuda", generator=g)
            self.var = torch.rand(self.channels, device="cuda", generator=g) + 0.5
            self.imin = torch.tensor([-3.0], device="cuda")
            self.imax = torch.tensor([3.0], device="cuda")
            self.ws = torch.empty(lib.mxq_quantized_batch_norm_workspace(self.channels),
                                  dtype=torch.uint8, device="cuda")
            self.bytes = 2.0 * n
            self.kernel = "bn_rows_kernel"
            self.name = "quantized_batch_norm_relu int8->int8, NCHW (%d,256,64,64), calibrated " \
                        "(-6,6)" % self.outer
        elif kind == "embedding":
            # BERT-base vocabulary: 30522 rows of 768 int8; n / 768 token ids per launch
            self.rows = n // 768
            self.table = torch.randint(-127, 128, (30522, 768), device="cuda", generator=g,
                                       dtype=torch.int8)
            self.src = [torch.randint(0, 30522, (self.rows,), device="cuda", generator=g,
                                      dtype=torch.int32) for _ in range(self.NBUF)]
            self.dst = [torch.empty((self.rows, 768), dtype=torch.int8, device="cuda")
                        for _ in range(self.NBUF)]
            self.imin = torch.tensor([-1.0], device="cuda")
            self.imax = torch.tensor([1.0], device="cuda")
            # the gathered rows are read once each (the 23 MB table stays in cache) and
            # written once, plus 4 bytes of index per row
            self.bytes = (2.0 * 768 + 4.0) * self.rows
            self.kernel = "embedding_kernel"
            self.name = "quantized_embedding, 30522 x 768 int8 table, %d int32 ids" % self.rows
        elif kind in ("transpose", "transpose_to_nhwc", "transpose_to_nchw"):
            # attention layout change (batch, seq, heads, 64) -> (batch, heads, seq, 64), or
            # the layout change at a convolution's boundary, NCHW <-> NHWC of 256 x 64 x 64
            self.shape, self.axes = {
                "transpose": ((n // (512 * 16 * 64), 512, 16, 64), (0, 2, 1, 3)),
                "transpose_to_nhwc": ((n // (256 * 64 * 64), 256, 64, 64), (0, 2, 3, 1)),
                "transpose_to_nchw": ((n // (256 * 64 * 64), 64, 64, 256), (0, 3, 1, 2)),
            }[kind]
            self.src = [torch.randint(-127, 128, self.shape, device="cuda", generator=g,
                                      dtype=torch.int8) for _ in range(self.NBUF)]
            self.dst = [torch.empty(n, dtype=torch.int8, device="cuda") for _ in range(self.NBUF)]
            self.imin = torch.tensor([-1.0], device="cuda")
            self.imax = torch.tensor([1.0], device="cuda")
            self.c_shape = (ctypes.c_int64 * 4)(*self.shape)
            self.c_axes = (ctypes.c_int * 4)(*self.axes)
            self.bytes = 2.0 * n
            self.kernel = "permute_elem_direct_kernel" if kind == "transpose" else "permute_tile16_kernel"
            self.name = "quantized_transpose int8 %s axes (%s)" % (
                self.shape, ",".join(str(a) for a in self.axes))
        else:
            raise ValueError(kind)
        self.name += ", %d elements" % n

    def step(self):
        P, n, lib = self.P, self.N, self.lib
        k = self.i % self.NBUF
        self.i += 1
        st = ctypes.c_void_p(self.torch.cuda.current_stream().cuda_stream)
        kind = self.kind
        if kind in ("quantize", "quantize_laplace"):
            rc = lib.mxq_quantize_v2(st, P(self.src[k]), P(self.dst[k]), P(self.omin),
                                     P(self.omax), n, 5, 1, -50.0, 50.0, None, 0)
        elif kind == "quantize_uint8_uncal":
            rc = lib.mxq_quantize_v2(st, P(self.src[k]), P(self.dst[k]), P(self.omin),
                                     P(self.omax), n, 3, 0, 0.0, 0.0, P(self.ws),
                                     self.ws.numel())
        elif kind == "quantize_uint8":
            rc = lib.mxq_quantize_v2(st, P(self.src[k]), P(self.dst[k]), P(self.omin),
                                     P(self.omax), n, 3, 1, -50.0, 50.0, None, 0)
        elif kind == "quantize_uncal":
            rc = lib.mxq_quantize_v2(st, P(self.src[k]), P(self.dst[k]), P(self.omin),
                                     P(self.omax), n, 5, 0, 0.0, 0.0, P(self.ws),
                                     self.ws.numel())
        elif kind == "quantize_v1":
            rc = lib.mxq_quantize(st, P(self.src[k]), P(self.imin), P(self.imax), P(self.dst[k]),
                                  P(self.omin), P(self.omax), n, 5)
        elif kind == "quantized_act":
            rc = lib.mxq_quantized_relu(st, P(self.src[k]), P(self.imin), P(self.imax),
                                        P(self.dst[k]), P(self.omin), P(self.omax), n)
        elif kind == "requantize":
            rc = lib.mxq_requantize(st, P(self.src[k]), P(self.imin), P(self.imax),
                                    P(self.dst[k]), P(self.omin), P(self.omax), n, 1, -0.1, 0.1,
                                    None, 0)
        elif kind == "requantize_uncal":
            rc = lib.mxq_requantize(st, P(self.src[k]), P(self.imin), P(self.imax),
                                    P(self.dst[k]), P(self.omin), P(self.omax), n, 0, 0.0, 0.0,
                                    P(self.ws), self.ws.numel())
        elif kind == "concat":
            ptrs = (ctypes.c_void_p * 2)(self.src[k].data_ptr(), self.rhs[k].data_ptr())
            rc = lib.mxq_quantized_concat(st, 2, ptrs, self.c_types, self.c_mins, self.c_maxs,
                                          self.c_ext, 1, 1, P(self.dst[k]), 5, P(self.omin),
                                          P(self.omax))
        elif kind == "elemwise_add":
            rc = lib.mxq_quantized_elemwise_add(st, P(self.src[k]), 5, P(self.rhs[k]), 5,
                                                P(self.imin), P(self.imax), P(self.imin),
                                                P(self.imax), P(self.dst[k]), 4, P(self.omin),
                                                P(self.omax), n, 0, 0.0, 0.0)
        elif kind == "elemwise_add_int8":
            rc = lib.mxq_quantized_elemwise_add(st, P(self.src[k]), 5, P(self.rhs[k]), 5,
                                                P(self.imin), P(self.imax), P(self.imin),
                                                P(self.imax), P(self.dst[k]), 5, P(self.omin),
                                                P(self.omax), n, 1, -5.0, 5.0)
        elif kind == "elemwise_mul_int8":
            rc = lib.mxq_quantized_elemwise_mul(st, P(self.src[k]), P(self.rhs[k]), P(self.imin),
                                                P(self.imax), P(self.imin), P(self.imax),
                                                P(self.dst[k]), 5, P(self.omin), P(self.omax), n,
                                                1, -9.0, 9.0)
        elif kind == "quantize_asym":
            rc = lib.mxq_quantize_asym(st, P(self.src[k]), 0, P(self.dst[k]), P(self.omin),
                                       P(self.omax), n, 1, -6.0, 6.0, None, 0)
        elif kind == "batch_norm":
            rc = lib.mxq_quantized_batch_norm(st, P(self.src[k]), 5, P(self.gamma), P(self.beta),
                                              P(self.mean), P(self.var), P(self.imin),
                                              P(self.imax), P(self.dst[k]), P(self.omin),
                                              P(self.omax), self.outer, self.channels, self.inner,
                                              1e-3, -6.0, 6.0, 1, P(self.ws), self.ws.numel())
        elif kind == "embedding":
            rc = lib.mxq_quantized_embedding(st, P(self.src[k]), 4, P(self.table), P(self.imin),
                                             P(self.imax), P(self.dst[k]), P(self.omin),
                                             P(self.omax), self.rows, 30522, 768)
        elif kind.startswith("transpose"):
            rc = lib.mxq_quantized_transpose(st, P(self.src[k]), P(self.imin), P(self.imax),
                                             P(self.dst[k]), P(self.omin), P(self.omax), 4,
                                             self.c_shape, self.c_axes)
        else:
            rc = lib.mxq_dequantize(st, P(self.src[k]), 5, P(self.imin), P(self.imax),
                                    P(self.dst[k]), n)
        if rc != 0:
            raise RuntimeError(lib.mxq_last_error().decode())

    def value(self, sec_per_step):
        return self.bytes / sec_per_step / 1e9, "GB/s"

    def cpu_baseline(self, oracle, budget_s=12.0):
        import numpy as np
        n = 1 << 24
        kind = self.kind
        if kind == "embedding":
            n = (n // 768) * 768
            x = self.src[0][:n // 768].cpu().numpy()
            table = self.table.cpu().numpy()
        elif kind.startswith("transpose"):
            x = self.src[0][:n // (self.shape[1] * self.shape[2] * self.shape[3])].cpu().numpy()
        elif kind == "batch_norm":
            x = self.src[0][:n].cpu().numpy().reshape(-1, self.channels, self.inner)
            bn = [t.cpu().numpy() for t in (self.gamma, self.beta, self.mean, self.var)]
        else:
            x = self.src[0][:n].cpu().numpy()
        reps, t0 = 0, time.perf_counter()
        while True:
            if kind in ("quantize", "quantize_laplace"):
                oracle.quantize_v2(x, "int8", -50.0, 50.0)
            elif kind == "quantize_uint8_uncal":
                oracle.quantize_v2(x, "uint8")
            elif kind == "quantize_uint8":
                oracle.quantize_v2(x, "uint8", -50.0, 50.0)
            elif kind == "quantize_uncal":
                oracle.quantize_v2(x, "int8")
            elif kind == "quantize_v1":
                oracle.quantize(x, -4.0, 4.0)
            elif kind == "quantized_act":
                oracle.relu_i8(x)
            elif kind == "requantize":
                oracle.requantize(x, -1.0, 1.0, -0.1, 0.1)
            elif kind == "requantize_uncal":
                oracle.requantize(x, -1.0, 1.0)
            elif kind == "concat":
                oracle.quantized_concat([x[:n // 2], x[n // 2:]], [-1.0, -2.0], [1.0, 2.0], dim=0)
            elif kind == "elemwise_add":
                oracle.quantized_elemwise_add(x, x, -3.0, 3.0, -3.0, 3.0)
            elif kind == "elemwise_add_int8":
                oracle.quantized_elemwise_add(x, x, -3.0, 3.0, -3.0, 3.0, -5.0, 5.0)
            elif kind == "elemwise_mul_int8":
                oracle.quantized_elemwise_mul(x, x, -3.0, 3.0, -3.0, 3.0, -9.0, 9.0)
            elif kind == "quantize_asym":
                oracle.quantize_asym(x, -6.0, 6.0)
            elif kind == "batch_norm":
                oracle.quantized_batch_norm(x, *bn, -3.0, 3.0, -6.0, 6.0, relu=True)
            elif kind == "embedding":
                oracle.quantized_embedding(x, table, -1.0, 1.0)
            elif kind.startswith("transpose"):
                oracle.quantized_transpose(x, -1.0, 1.0, self.axes)
            else:
                oracle.dequantize(x, -3.0, 3.0)
            reps += 1
            dt = time.perf_counter() - t0
            if dt > budget_s / 2 or reps >= 2000:
                break
        gbs = self.bytes / self.N * n * reps / dt / 1e9
        return {"value": gbs, "unit": "GB/s", "cores": oracle.num_threads(), "kind": "port",
                "sample": "oracle (OpenMP) on the first %d elements, %d repetitions, %.1f s"
                          % (n, reps, dt)}


class PoolWorkload:
    """_contrib_quantized_pooling on NCHW int8, buffers rotated past the Infinity Cache.
    `maxpool`: the ResNet stem pool (3x3 / stride 2 / pad 1 on 112 x 112 x 64) at batch 256;
    `avgpool`: the ResNet global average pool (7 x 7 x 2048) at batch 4096.  Algorithmic
    bytes: input read once + output written once (1 B per element each)."""
    NBUF = 3

    def __init__(self, kind, torch, lib):
        self.kind, self.torch, self.lib = kind, torch, lib
        if kind == "maxpool":
            self.shape, self.k, self.s, self.p, self.pool = (256, 64, 112, 112), 3, 2, 1, 0
        else:
            self.shape, self.k, self.s, self.p, self.pool = (4096, 2048, 7, 7), 7, 1, 0, 1
        N, C, H, W = self.shape
        self.OH = (H + 2 * self.p - self.k) // self.s + 1
        g = torch.Generator(device="cuda").manual_seed(2)
        self.src = [torch.randint(-127, 128, self.shape, device="cuda", generator=g,
                                  dtype=torch.int8) for _ in range(self.NBUF)]
        self.dst = [torch.empty((N, C, self.OH, self.OH), dtype=torch.int8, device="cuda")
                    for _ in range(self.NBUF)]
        self.sc = [torch.tensor([v], device="cuda") for v in (-1.0, 1.0, 0.0, 0.0)]
        self.bytes = float(N * C * (H * W + self.OH * self.OH))
        self.bound = "hbm"
        self.kernel = "pool_lds_kernel"
        self.name = "quantized_pooling %s %dx%d/%d on int8 NCHW %s" % (
            "max" if self.pool == 0 else "avg", self.k, self.k, self.s, "x".join(map(str, self.shape)))
        self.i = 0
        self.P = lambda t: ctypes.c_void_p(t.data_ptr())

    def step(self):
        P = self.P
        k = self.i % self.NBUF
        self.i += 1
        N, C, H, W = self.shape
        st = ctypes.c_void_p(self.torch.cuda.current_stream().cuda_stream)
        rc = self.lib.mxq_quantized_pooling_nchw(st, P(self.src[k]), 5, N, C, H, W, self.k, self.k,
                                                 self.s, self.s, self.p, self.p, self.OH, self.OH,
                                                 self.pool, 1, P(self.sc[0]), P(self.sc[1]),
                                                 P(self.dst[k]), P(self.sc[2]), P(self.sc[3]))
        if rc != 0:
            raise RuntimeError(self.lib.mxq_last_error().decode())

    def value(self, sec_per_step):
        return self.bytes / sec_per_step / 1e9, "GB/s"


class CopyWorkload:
    """A plain device copy of known size (torch's copy kernel): the yardstick the
    FETCH_SIZE / WRITE_SIZE counters are scaled by, not a product kernel."""
    N = 1 << 26

    def __init__(self, torch):
        self.torch = torch
        self.bound = "hbm"
        self.kernel = "torch elementwise copy"
        self.name = "fp32 copy, %d elements (counter calibration)" % self.N
        self.bytes = 8.0 * self.N
        self.src = [torch.randn(self.N, device="cuda") for _ in range(2)]
        self.dst = torch.empty(self.N, device="cuda")
        self.i = 0

    def step(self):
        self.dst.copy_(self.src[self.i % 2])
        self.i += 1

    def value(self, sec_per_step):
        return self.bytes / sec_per_step / 1e9, "GB/s"

    def cpu_baseline(self, oracle, budget_s=0):
        return None


class GraphWorkload:
    """Many small launches per step: the step is captured once into a HIP graph and
    replayed, so that host-side call overhead (tens of microseconds per ctypes call)
    does not bound the measurement.  No memset nodes are recorded."""

    def capture(self, torch, body):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            body()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            body()

    def step(self):
        self.graph.replay()

    def value(self, sec_per_step):
        return self.ops / sec_per_step / 1e12, "TOPS"

    def time_alone(self, torch, body, reps=10, replays=30):
        """Average time of one pass of `body` when it is the only thing running: captured
        `reps` times into its own graph.  Its operands stay cache-warm between passes, so
        this is an upper bound on what the same launches reach inside the whole step."""
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            body()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(reps):
                body()
        for _ in range(5):
            g.replay()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(replays):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / 1e3 / (reps * replays)

    def cpu_baseline(self, oracle, budget_s=0):
        return None


class SmallCastsWorkload(GraphWorkload):
    """The cast operators at the sizes they have inside benchmark configurations 1 and 5:
    [128,1024] and [4096,768], [4096,2304], [4096,3072].  One step = calibrated quantize_v2,
    calibrated requantize and dequantize of every size (12 launches in one graph).  The
    operands of these sizes sit in the caches, so the table reports time per launch and the
    algorithmic GB/s it amounts to, not a fraction of HBM peak worth quoting."""
    SIZES = [(128, 1024), (4096, 768), (4096, 2304), (4096, 3072)]

    def __init__(self, torch, lib):
        self.kernel = "quantize_kernel / requantize_kernel / dequantize_kernel"
        self.bound = "hbm"
        self.name = "quantize_v2, requantize, dequantize at [128,1024], [4096,768], " \
                    "[4096,2304], [4096,3072] (calibrated), 12 launches per step"
        P = lambda t: ctypes.c_void_p(t.data_ptr())
        g = torch.Generator(device="cuda").manual_seed(6)
        self.bytes = 0.0
        self.items = []
        one = [torch.tensor([v], device="cuda") for v in (-1.0, 1.0)]
        sc = [torch.empty(1, device="cuda") for _ in range(2)]
        for (r, c) in self.SIZES:
            n = r * c
            x = torch.randn(n, device="cuda", generator=g)
            a = torch.randint(-2 ** 28, 2 ** 28, (n,), device="cuda", generator=g,
                              dtype=torch.int32)
            q = torch.randint(-127, 128, (n,), device="cuda", generator=g, dtype=torch.int8)
            o8 = torch.empty(n, dtype=torch.int8, device="cuda")
            of = torch.empty(n, dtype=torch.float32, device="cuda")
            self.items.append((n, x, a, q, o8, of))
            self.bytes += 15.0 * n
        self.keep = (one, sc)

        def body(only=None):
            st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            j = 0
            for (n, x, a, q, o8, of) in self.items:
                calls = [
                    lambda: lib.mxq_quantize_v2(st, P(x), P(o8), P(sc[0]), P(sc[1]), n, 5, 1,
                                                -4.0, 4.0, None, 0),
                    lambda: lib.mxq_requantize(st, P(a), P(one[0]), P(one[1]), P(o8), P(sc[0]),
                                               P(sc[1]), n, 1, -0.1, 0.1, None, 0),
                    lambda: lib.mxq_dequantize(st, P(q), 5, P(one[0]), P(one[1]), P(of), n)]
                for call in calls:
                    if only is None or only == j:
                        if call() != 0:
                            raise RuntimeError(lib.mxq_last_error().decode())
                    j += 1
        self.body = body
        self.capture(torch, body)

    def value(self, sec_per_step):
        return self.bytes / sec_per_step / 1e9, "GB/s"

    def per_layer(self, torch):
        rows, j = [], 0
        for (r, c) in self.SIZES:
            for op in ("quantize_v2", "requantize", "dequantize"):
                t = self.time_alone(torch, lambda: self.body(j), reps=20)
                rows.append({"launch": "%s [%d,%d]" % (op, r, c), "us": round(t * 1e6, 2),
                             "GB/s": round(5.0 * r * c / t / 1e9, 1)})
                j += 1
        return rows


# ResNet-50 v1 bottleneck convolutions, batch 64: (H, Cin, Cout, kernel, stride)
RESNET50_CONVS = [(56, 64, 64, 1, 1), (56, 64, 64, 3, 1), (56, 64, 256, 1, 1), (56, 256, 64, 1, 1),
                  (56, 256, 128, 1, 2), (28, 128, 128, 3, 1), (28, 128, 512, 1, 1),
                  (28, 512, 128, 1, 1), (56, 256, 512, 1, 2), (28, 512, 256, 1, 2),
                  (14, 256, 256, 3, 1), (14, 256, 1024, 1, 1), (14, 1024, 256, 1, 1),
                  (28, 512, 1024, 1, 2), (14, 1024, 512, 1, 2), (7, 512, 512, 3, 1),
                  (7, 512, 2048, 1, 1), (7, 2048, 512, 1, 1), (14, 1024, 2048, 1, 2)]


class ConvStackWorkload(GraphWorkload):
    """Benchmark configuration 4: the distinct 1x1 / 3x3 bottleneck convolutions of ResNet-50 v1 at
    batch 64 on NHWC int8, weights N(0, sqrt(2/fan_in)) quantized with their own min/max, each
    with the quantized ReLU and a calibrated requantize fused in the epilogue."""

    def __init__(self, torch, capi, lib):
        self.kernel = "conv_dma_kernel / fc_dma_kernel (1x1)"
        self.bound = "mfma"
        self.name = "ResNet-50 v1 bottleneck conv stack (19 distinct layers), batch 64, " \
                    "NHWC int8, fused relu + requantize, naive per-layer calibration " \
                    "(range = min/max of the layer's own fp32 output on a batch slice)"
        P = lambda t: ctypes.c_void_p(t.data_ptr())
        g = torch.Generator(device="cuda").manual_seed(4)
        N = 64
        self.layers, self.ops = [], 0.0
        for (H, C, O, k, s) in RESNET50_CONVS:
            pad = 1 if k == 3 else 0
            OH = (H + 2 * pad - k) // s + 1
            x = torch.randn((N, H, H, C), device="cuda", generator=g)
            d, dmin, dmax = capi.quantize_v2(x, "int8")
            w = torch.randn((O, k, k, C), device="cuda", generator=g) * (2.0 / (k * k * C)) ** 0.5
            wq, wmin, wmax = capi.quantize(w, w.min().reshape(1), w.max().reshape(1), "int8")
            b = torch.randn((O,), device="cuda", generator=g) * 0.1
            bq, bmin, bmax = capi.quantize(b, b.min().reshape(1), b.max().reshape(1), "int8")
            out8 = torch.empty((N, OH, OH, O), dtype=torch.int8, device="cuda")
            sc = [torch.empty(1, device="cuda") for _ in range(4)]
            nws = lib.mxq_quantized_conv_workspace(N, H, H, C, O, k, k, s, s, pad, pad, 1, 1, 1)
            ws = torch.empty(nws, dtype=torch.uint8, device="cuda") if nws else None
            # naive calibration: range of the fp32 output of this layer on a batch slice
            ref = torch.nn.functional.conv2d(x[:4].permute(0, 3, 1, 2), w.permute(0, 3, 1, 2), b,
                                             stride=s, padding=pad)
            r = float(ref.abs().max().item())
            self.layers.append((d, wq, bq, dmin, dmax, wmin, wmax, bmin, bmax, out8, sc,
                                (N, H, H, C, O, k, k, s, s, pad, pad), r, ws))
            self.ops += 2.0 * N * OH * OH * O * k * k * C
            del x, w, ref

        def body(only=None):
            st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            for i, (d, wq, bq, dmin, dmax, wmin, wmax, bmin, bmax, out8, sc, geo,
                    r, ws) in enumerate(self.layers):
                if only is not None and i != only:
                    continue
                rc = lib.mxq_quantized_conv_nhwc(st, P(d), P(wq), P(bq), *geo, 1, 1, P(dmin),
                                                 P(dmax), P(wmin), P(wmax), P(bmin), P(bmax),
                                                 None, P(sc[0]), P(sc[1]), P(out8), P(sc[2]),
                                                 P(sc[3]), 1, -r, r, *ws_args(ws))
                if rc != 0:
                    raise RuntimeError(lib.mxq_last_error().decode())
        self.body = body
        self.capture(torch, body)

    def per_layer(self, torch):
        rows = []
        for i, (H, C, O, k, s) in enumerate(RESNET50_CONVS):
            pad = 1 if k == 3 else 0
            OH = (H + 2 * pad - k) // s + 1
            ops = 2.0 * 64 * OH * OH * O * k * k * C
            t = self.time_alone(torch, lambda: self.body(i))
            rows.append({"layer": "%dx%d %d->%d k%d s%d" % (H, H, C, O, k, s),
                         "us": round(t * 1e6, 2), "TOPS": round(ops / t / 1e12, 1)})
        return rows


class ConvOperatorWorkload(GraphWorkload):
    """The same 19 ResNet-50 layers at batch 64 under the reference operator's own contract
    (quantized_conv.cu:101-219): NCHW int8 data and OIHW int8 weights in, NCHW int32 out,
    through mxq_quantized_conv_nchw, the one call the registered _contrib_quantized_conv
    makes.  `route` pins every layer to one route through the test-only entry point
    (1 = the layout adapters, as the reference's two TransposeImpl calls)."""

    def __init__(self, torch, capi, lib, route=0):
        self.kernel = "conv1x1_planes_kernel (NCHW 1x1) + adapters / conv_dma_kernel (3x3, small planes), int32 NCHW out"
        self.bound = "mfma"
        self.name = "ResNet-50 v1 bottleneck conv stack (19 distinct layers), batch 64, as the " \
                    "operator sees it: NCHW int8 in, NCHW int32 out (no requantize, so no " \
                    "calibration)" + \
                    (" (every layer through the layout adapters)" if route == 1 else "")
        P = lambda t: ctypes.c_void_p(t.data_ptr())
        g = torch.Generator(device="cuda").manual_seed(4)
        N = 64
        self.layers, self.ops = [], 0.0
        one = [torch.tensor([v], device="cuda") for v in (-1.0, 1.0)]
        for (H, C, O, k, s) in RESNET50_CONVS:
            pad = 1 if k == 3 else 0
            OH = (H + 2 * pad - k) // s + 1
            d = torch.randint(-127, 128, (N, C, H, H), device="cuda", generator=g, dtype=torch.int8)
            w = torch.randint(-127, 128, (O, C, k, k), device="cuda", generator=g, dtype=torch.int8)
            b = torch.randint(-127, 128, (O,), device="cuda", generator=g, dtype=torch.int8)
            out = torch.empty((N, O, OH, OH), dtype=torch.int32, device="cuda")
            sc = [torch.empty(1, device="cuda") for _ in range(2)]
            geo = (N, C, H, H, O, k, k, s, s, pad, pad, 1, 1)
            nws = lib.mxq_quantized_conv_nchw_workspace(*geo, 0 if route == 1 else 1)
            ws = torch.empty(nws, dtype=torch.uint8, device="cuda") if nws else None
            self.layers.append((d, w, b, out, sc, geo, ws))
            self.ops += 2.0 * N * OH * OH * O * k * k * C

        def body(only=None):
            st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            for i, (d, w, b, out, sc, geo, ws) in enumerate(self.layers):
                if only is not None and i != only:
                    continue
                args = [st, P(d), P(w), P(b)] + list(geo) + [
                    P(one[0]), P(one[1]), P(one[0]), P(one[1]), P(one[0]), P(one[1]), P(out),
                    P(sc[0]), P(sc[1])] + list(ws_args(ws))
                if route == 0:
                    rc = lib.mxq_quantized_conv_nchw(*args)
                else:
                    rc = lib.mxq_test_quantized_conv_nchw(*args, route)
                if rc != 0:
                    raise RuntimeError(lib.mxq_last_error().decode())
        self.body = body
        self.capture(torch, body)

    def per_layer(self, torch):
        rows = []
        for i, (H, C, O, k, s) in enumerate(RESNET50_CONVS):
            pad = 1 if k == 3 else 0
            OH = (H + 2 * pad - k) // s + 1
            ops = 2.0 * 64 * OH * OH * O * k * k * C
            t = self.time_alone(torch, lambda: self.body(i))
            rows.append({"layer": "%dx%d %d->%d k%d s%d" % (H, H, C, O, k, s),
                         "us": round(t * 1e6, 2), "TOPS": round(ops / t / 1e12, 1)})
        return rows


BERT_FCS = [(768, 2304), (768, 768), (768, 3072), (3072, 768)]


class ResNetChainWorkload(GraphWorkload):
    """The bottleneck body of ResNet-50 v1 at batch 64 as one producer -> consumer chain (the 19
    shapes of configuration 4 in the order and number a forward pass runs them): 16 blocks of
    conv1x1 (+relu) -> conv3x3 (+relu) -> conv1x1, a projection conv1x1 on the shortcut of the
    first block of each stage, quantized_elemwise_add of the two branches (int8 out, calibrated)
    and quantized ReLU; stride on the first 1x1 of a stage as in the reference's model zoo
    (python/mxnet/gluon/model_zoo/vision/resnet.py:108-123).  Every layer reads what the layer
    before it wrote.  NHWC int8, requantize fused into every convolution, calibration ranges
    from one pass with int32 outputs over the same synthetic input.  52 convolutions + 16 adds +
    16 relus per step; stem, pooling and the classifier are not part of it."""
    STAGES = [(3, 64, 256, 1), (4, 128, 512, 2), (6, 256, 1024, 2), (3, 512, 2048, 2)]

    def __init__(self, torch, capi, lib, fused_sum=False, unfused=False):
        self.kernel = "conv / fc kernels, add_kernel, relu"
        self.bound = "mfma"
        self.name = "ResNet-50 v1 bottleneck body as a chain (52 convolutions + 16 residual " \
                    "adds + relus), batch 64, NHWC int8, requantize fused, naive per-layer " \
                    "calibration (range = min/max of each layer's fp32 output on the chain's " \
                    "own data)"
        if unfused:
            # the operator sequence of the graph the reference's pass emits: every convolution
            # writes int32, a _contrib_requantize node narrows it, relu is a node of its own
            self.kernel = "conv / fc kernels (int32 out), requantize, relu, add_kernel"
            self.name = "ResNet-50 v1 bottleneck body as the reference's graph runs it: " \
                        "quantized_conv (int32) -> requantize -> quantized_act per layer, " \
                        "elemwise_add + act per block, batch 64, NHWC, naive per-layer " \
                        "calibration"
        if fused_sum:
            self.kernel = "conv / fc kernels, the residual sum and its relu in the epilogue of " \
                          "each block's last 1x1 convolution"
            self.name += ", residual add + relu fused into the block's last convolution " \
                         "(mxq_quantized_fc_sum)"
        P = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
        g = torch.Generator(device="cuda").manual_seed(44)
        N, H = 64, 56
        x = torch.randn((N, H, H, 64), device="cuda", generator=g).clamp_(min=0.0)
        cur, cmin, cmax = capi.quantize_v2(x, "int8")
        del x
        self.calls, self.ops, self.keep = [], 0.0, []
        f1 = lambda v: torch.tensor([v], dtype=torch.float32, device="cuda")

        def conv(inp, imin, imax, H, C, O, k, s, relu, record=True):
            """Adds one fused convolution to the chain; returns its int8 output and range
            (record=False: runs it once for the calibration of what follows, outside the
            chain, and also returns what a fused call needs)."""
            pad = 1 if k == 3 else 0
            OH = (H + 2 * pad - k) // s + 1
            w = torch.randn((O, k, k, C), device="cuda", generator=g) * (2.0 / (k * k * C)) ** 0.5
            wq, wmin, wmax = capi.quantize(w, w.min().reshape(1), w.max().reshape(1), "int8")
            b = torch.randn((O,), device="cuda", generator=g) * 0.1
            bq, bmin, bmax = capi.quantize(b, b.min().reshape(1), b.max().reshape(1), "int8")
            del w, b
            # calibration: the float range of this layer's int32 output on the chain's own data
            res = capi.quantized_conv_nhwc(inp, wq, bq, imin, imax, wmin, wmax, bmin, bmax,
                                           stride=(s, s), pad=(pad, pad), want_int32=True)
            r = float(res["out32"].abs().max().item()) * float(res["omax"].item()) / 2147483648.0
            r = max(r, 1e-6)
            del res
            out8 = torch.empty((N, OH, OH, O), dtype=torch.int8, device="cuda")
            sc = [torch.empty(1, device="cuda") for _ in range(4)]
            geo = (N, H, H, C, O, k, k, s, s, pad, pad)
            if unfused:
                acc = torch.empty((N, OH, OH, O), dtype=torch.int32, device="cuda")
                tmp8 = torch.empty_like(out8) if relu else out8
                sc += [torch.empty(1, device="cuda") for _ in range(2)]
                nws = lib.mxq_quantized_conv_workspace(*geo, 1, 1, 0)
                ws = torch.empty(nws, dtype=torch.uint8, device="cuda") if nws else None
                seq = [(lib.mxq_quantized_conv_nhwc,
                        (P(inp), P(wq), P(bq), *geo, 1, 1, P(imin), P(imax), P(wmin), P(wmax),
                         P(bmin), P(bmax), P(acc), P(sc[0]), P(sc[1]), None, None, None, 0, 0.0,
                         0.0, *ws_args(ws))),
                       (lib.mxq_requantize,
                        (P(acc), P(sc[0]), P(sc[1]), P(tmp8), P(sc[4] if relu else sc[2]),
                         P(sc[5] if relu else sc[3]), acc.numel(), 1, -r, r, None, 0))]
                if relu:
                    seq.append((lib.mxq_quantized_relu,
                                (P(tmp8), P(sc[4]), P(sc[5]), P(out8), P(sc[2]), P(sc[3]),
                                 out8.numel())))
                self.calls += seq
                self.keep.append((inp, wq, bq, imin, imax, wmin, wmax, bmin, bmax, out8, sc, ws,
                                  acc, tmp8))
                self.ops += 2.0 * N * OH * OH * O * k * k * C
                st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
                for fn, a_ in seq:
                    if fn(st, *a_):
                        raise RuntimeError(lib.mxq_last_error().decode())
                return out8, sc[2], sc[3], OH
            nws = lib.mxq_quantized_conv_workspace(*geo, 1, 1, 1)
            ws = torch.empty(nws, dtype=torch.uint8, device="cuda") if nws else None
            args = (P(inp), P(wq), P(bq), *geo, 1, 1, P(imin), P(imax), P(wmin), P(wmax), P(bmin),
                    P(bmax), None, P(sc[0]), P(sc[1]), P(out8), P(sc[2]), P(sc[3]), int(relu), -r,
                    r, *ws_args(ws))
            if record:
                self.calls.append((lib.mxq_quantized_conv_nhwc, args))
            self.keep.append((inp, wq, bq, imin, imax, wmin, wmax, bmin, bmax, out8, sc, ws))
            self.ops += 2.0 * N * OH * OH * O * k * k * C
            st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            if lib.mxq_quantized_conv_nhwc(st, *args):
                raise RuntimeError(lib.mxq_last_error().decode())
            if not record:
                return out8, sc[2], sc[3], OH, (wq, bq, wmin, wmax, bmin, bmax, r, ws)
            return out8, sc[2], sc[3], OH

        for (blocks, mid, out, stride) in self.STAGES:
            for bi in range(blocks):
                s = stride if bi == 0 else 1
                C = cur.shape[3]
                a, amin, amax, H1 = conv(cur, cmin, cmax, H, C, mid, 1, s, True)
                b, bmin_, bmax_, _ = conv(a, amin, amax, H1, mid, mid, 3, 1, True)
                if bi == 0:
                    sh, smin, smax, _ = conv(cur, cmin, cmax, H, C, out, 1, s, False)
                else:
                    sh, smin, smax = cur, cmin, cmax
                if fused_sum:
                    c, cmin_, cmax_, _, (wq3, bq3, w3min, w3max, b3min, b3max, r3, ws3) = conv(
                        b, bmin_, bmax_, H1, mid, out, 1, 1, False, record=False)
                else:
                    c, cmin_, cmax_, _ = conv(b, bmin_, bmax_, H1, mid, out, 1, 1, False)
                # residual sum, int8 out with a calibrated range, then the quantized ReLU
                fa = capi.dequantize(c, cmin_, cmax_) + capi.dequantize(sh, smin, smax)
                r = max(float(fa.abs().max().item()), 1e-6)
                del fa
                y = torch.empty_like(c)
                ysc = [torch.empty(1, device="cuda") for _ in range(4)]
                z = torch.empty_like(c)
                if fused_sum:
                    # the block's last 1x1 convolution is the FC of its flattened pixels
                    Mrows = N * H1 * H1
                    fargs = (P(b), P(wq3), P(bq3), Mrows, out, mid, P(bmin_), P(bmax_), P(w3min),
                             P(w3max), P(b3min), P(b3max), P(sh), P(smin), P(smax), P(z),
                             P(ysc[0]), P(ysc[1]), P(ysc[2]), P(ysc[3]), -r3, r3, -r, r, 1,
                             *ws_args(ws3))
                    self.calls.append((lib.mxq_quantized_fc_sum, fargs))
                    self.keep.append((c, sh, y, z, ysc))
                    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
                    if lib.mxq_quantized_fc_sum(st, *fargs):
                        raise RuntimeError(lib.mxq_last_error().decode())
                    # the three operators on the same tensors must give the same bytes
                    z3 = torch.empty_like(c)
                    zsc = [torch.empty(1, device="cuda") for _ in range(4)]
                    rcs = [lib.mxq_quantized_elemwise_add(st, P(c), 5, P(sh), 5, P(cmin_),
                                                          P(cmax_), P(smin), P(smax), P(y), 5,
                                                          P(zsc[0]), P(zsc[1]), c.numel(), 1,
                                                          -r, r),
                           lib.mxq_quantized_relu(st, P(y), P(zsc[0]), P(zsc[1]), P(z3),
                                                  P(zsc[2]), P(zsc[3]), y.numel())]
                    if any(rcs):
                        raise RuntimeError(lib.mxq_last_error().decode())
                    if not torch.equal(z, z3):
                        raise RuntimeError("fused residual sum differs from the three operators")
                    del z3
                    cur, cmin, cmax, H = z, ysc[2], ysc[3], H1
                    continue
                add_args = (P(c), 5, P(sh), 5, P(cmin_), P(cmax_), P(smin), P(smax), P(y), 5,
                            P(ysc[0]), P(ysc[1]), c.numel(), 1, -r, r)
                relu_args = (P(y), P(ysc[0]), P(ysc[1]), P(z), P(ysc[2]), P(ysc[3]), y.numel())
                self.calls.append((lib.mxq_quantized_elemwise_add, add_args))
                self.calls.append((lib.mxq_quantized_relu, relu_args))
                self.keep.append((c, sh, y, z, ysc))
                st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
                for fn, args in self.calls[-2:]:
                    if fn(st, *args):
                        raise RuntimeError(lib.mxq_last_error().decode())
                cur, cmin, cmax, H = z, ysc[2], ysc[3], H1
        torch.cuda.synchronize()
        self.images = N

        def body():
            st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            for fn, args in self.calls:
                if fn(st, *args):
                    raise RuntimeError(lib.mxq_last_error().decode())
        self.graph_body = body
        self.capture(torch, body)

    def per_layer(self, torch):
        t = self.time_alone(torch, self.graph_body, reps=1, replays=50)
        return [{"chain": "whole body", "us": round(t * 1e6, 1),
                 "images_per_s": round(self.images / t, 0), "launches": len(self.calls)}]


class BertChainWorkload(GraphWorkload):
    """Benchmark configuration 5: BERT-base FC shapes at M = 32 x 128 = 4096; per layer calibrated
    quantize_v2 -> quantized_fully_connected (+ int8 bias) -> requantize -> dequantize, as
    the unfused graph runs it.  Activations N(0,1) with 0.1% outliers at +-20."""

    def __init__(self, torch, capi, lib, fused=False):
        self.kernel = "quantize + fc_dma + requantize + dequantize kernels"
        self.bound = "mfma"
        self.name = "BERT-base FC chain M=4096: 768->2304, 768->768, 768->3072, 3072->768, " \
                    "quantize_v2 -> quantized_fc -> requantize -> dequantize per layer"
        if fused == "f32":
            self.kernel = "quantize + fc_dma (requantize and dequantize in the epilogue) kernels"
            self.name = self.name.replace("quantized_fc -> requantize -> dequantize",
                                          "quantized_fc with requantize and dequantize fused")
        elif fused:
            self.kernel = "quantize + fc_dma (requantize in the epilogue) + dequantize kernels"
            self.name = self.name.replace("quantized_fc -> requantize",
                                          "quantized_fc with the requantize fused")
        P = lambda t: ctypes.c_void_p(t.data_ptr())
        g = torch.Generator(device="cuda").manual_seed(5)
        M = 4096
        self.layers, self.ops = [], 0.0
        for (K, N) in BERT_FCS:
            x = torch.randn((M, K), device="cuda", generator=g)
            idx = torch.randint(0, M * K, (M * K // 1000,), device="cuda", generator=g)
            x.view(-1)[idx] = 20.0 * (torch.randint(0, 2, idx.shape, device="cuda",
                                                    generator=g) * 2 - 1).float()
            w = torch.randn((N, K), device="cuda", generator=g) * 0.02
            wq, wmin, wmax = capi.quantize(w, w.min().reshape(1), w.max().reshape(1), "int8")
            b = torch.randn((N,), device="cuda", generator=g) * 0.02
            bq, bmin, bmax = capi.quantize(b, b.min().reshape(1), b.max().reshape(1), "int8")
            r = float((x[:64] @ w.t() + b).abs().max().item())
            bufs = dict(x=x, q=torch.empty((M, K), dtype=torch.int8, device="cuda"),
                        acc=torch.empty((M, N), dtype=torch.int32, device="cuda"),
                        q8=torch.empty((M, N), dtype=torch.int8, device="cuda"),
                        y=torch.empty((M, N), dtype=torch.float32, device="cuda"),
                        sc=[torch.empty(1, device="cuda") for _ in range(6)],
                        ws=fc_workspace(torch, lib, M, N, K, fused is True))
            self.layers.append((K, N, wq, bq, wmin, wmax, bmin, bmax, r, bufs))
            self.ops += 2.0 * M * N * K
            del w

        def body(only=None):
            st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            for i, (K, N, wq, bq, wmin, wmax, bmin, bmax, r, B) in enumerate(self.layers):
                if only is not None and i != only:
                    continue
                sc = B["sc"]
                if fused == "f32":
                    rcs = [
                        lib.mxq_quantize_v2(st, P(B["x"]), P(B["q"]), P(sc[0]), P(sc[1]), M * K,
                                            5, 1, -20.0, 20.0, None, 0),
                        lib.mxq_quantized_fc_f32(st, P(B["q"]), P(wq), P(bq), M, N, K, P(sc[0]),
                                                 P(sc[1]), P(wmin), P(wmax), P(bmin), P(bmax),
                                                 P(B["y"]), P(sc[2]), P(sc[3]), P(sc[4]),
                                                 P(sc[5]), 0, -r, r, *ws_args(B["ws"]))]
                    if any(rcs):
                        raise RuntimeError(lib.mxq_last_error().decode())
                    continue
                if fused:
                    rcs = [
                        lib.mxq_quantize_v2(st, P(B["x"]), P(B["q"]), P(sc[0]), P(sc[1]), M * K,
                                            5, 1, -20.0, 20.0, None, 0),
                        lib.mxq_quantized_fc(st, P(B["q"]), P(wq), P(bq), M, N, K, P(sc[0]),
                                             P(sc[1]), P(wmin), P(wmax), P(bmin), P(bmax), None,
                                             P(sc[2]), P(sc[3]), P(B["q8"]), P(sc[4]), P(sc[5]),
                                             0, -r, r, *ws_args(B["ws"])),
                        lib.mxq_dequantize(st, P(B["q8"]), 5, P(sc[4]), P(sc[5]), P(B["y"]),
                                           M * N)]
                    if any(rcs):
                        raise RuntimeError(lib.mxq_last_error().decode())
                    continue
                rcs = [
                    lib.mxq_quantize_v2(st, P(B["x"]), P(B["q"]), P(sc[0]), P(sc[1]), M * K, 5, 1,
                                        -20.0, 20.0, None, 0),
                    lib.mxq_quantized_fc(st, P(B["q"]), P(wq), P(bq), M, N, K, P(sc[0]), P(sc[1]),
                                         P(wmin), P(wmax), P(bmin), P(bmax), P(B["acc"]),
                                         P(sc[2]), P(sc[3]), None, None, None, 0, 0.0, 0.0,
                                         *ws_args(B["ws"])),
                    lib.mxq_requantize(st, P(B["acc"]), P(sc[2]), P(sc[3]), P(B["q8"]), P(sc[4]),
                                       P(sc[5]), M * N, 1, -r, r, None, 0),
                    lib.mxq_dequantize(st, P(B["q8"]), 5, P(sc[4]), P(sc[5]), P(B["y"]), M * N)]
                if any(rcs):
                    raise RuntimeError(lib.mxq_last_error().decode())
        self.body = body
        self.capture(torch, body)

    def per_layer(self, torch):
        """One layer's launches (cast operators included) alone."""
        rows = []
        for i, (K, N) in enumerate(BERT_FCS):
            t = self.time_alone(torch, lambda: self.body(i))
            rows.append({"layer": "M=4096 K=%d N=%d" % (K, N), "us": round(t * 1e6, 2),
                         "TOPS": round(2.0 * 4096 * N * K / t / 1e12, 1)})
        return rows


def mfma_context(torch, S):
    """Context for the MFMA roofline fraction, measured in the same process: the
    register-only MFMA probe (what the matrix pipes sustain with no data movement at
    all, zero vs random operand bytes) and the vendor int8 GEMM (hipBLASLt through
    torch._int_mm, int32 output, no bias, no requantize) on the same operand shapes."""
    out = {}
    path = os.path.join(ROOT, "bench_probe.so")
    if os.path.exists(path):
        probe = ctypes.CDLL(path)
        probe.mxq_probe_mfma_i8.restype = ctypes.c_double
        probe.mxq_probe_mfma_i8.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                            ctypes.c_int, ctypes.c_void_p]
        cus = torch.cuda.get_device_properties(0).multi_processor_count
        blocks = 2 * cus  # 2 waves per SIMD, as the 256 x 256 FC tile runs
        sink = torch.zeros(blocks * 256, dtype=torch.int32, device="cuda")
        st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        for zero, key in ((1, "zero_operands"), (0, "random_operands")):
            best = None
            for rep in range(4):
                e0 = torch.cuda.Event(enable_timing=True)
                e1 = torch.cuda.Event(enable_timing=True)
                e0.record()
                ops = probe.mxq_probe_mfma_i8(st, blocks, 2000, zero, sink.data_ptr())
                e1.record()
                torch.cuda.synchronize()
                if ops < 0:
                    raise RuntimeError("MFMA probe launch failed")
                t = e0.elapsed_time(e1) / 1e3
                if rep > 0 and (best is None or t < best):
                    best = t
            out["mfma_probe_%s_TOPS" % key] = round(ops / best / 1e12, 1)
    try:
        g = torch.Generator(device="cuda").manual_seed(1)
        a = torch.randint(-127, 128, (S, S), device="cuda", dtype=torch.int8, generator=g)
        b = (torch.randn((S, S), device="cuda", generator=g) * 24).clamp(-127, 127).round() \
            .to(torch.int8)
        bt = b.t()
        reps = max(20, int(4e13 / (2.0 * S ** 3)))  # ~20 ms of work, as much again to warm up
        for _ in range(reps):
            torch._int_mm(a, bt)
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            torch._int_mm(a, bt)
        e1.record()
        torch.cuda.synchronize()
        out["vendor_gemm_int32_out_TOPS"] = round(2.0 * S ** 3 * reps /
                                                  (e0.elapsed_time(e1) / 1e3) / 1e12, 1)
    except Exception as e:  # informational only
        out["vendor_gemm_int32_out_TOPS"] = "unavailable: %s" % e
    return out


def make_workload(name, torch, capi, lib):
    if name == "resnet50_convs":
        return ConvStackWorkload(torch, capi, lib)
    if name == "resnet50_convs_operator":
        return ConvOperatorWorkload(torch, capi, lib)
    if name == "resnet50_convs_operator_adapters":
        return ConvOperatorWorkload(torch, capi, lib, route=1)
    if name == "resnet50_chain":
        return ResNetChainWorkload(torch, capi, lib)
    if name == "resnet50_chain_fused":
        return ResNetChainWorkload(torch, capi, lib, fused_sum=True)
    if name == "resnet50_chain_unfused":
        return ResNetChainWorkload(torch, capi, lib, unfused=True)
    if name == "bert_fc_chain":
        return BertChainWorkload(torch, capi, lib)
    if name == "bert_fc_chain_fused":
        return BertChainWorkload(torch, capi, lib, fused=True)
    if name == "bert_fc_chain_f32":
        return BertChainWorkload(torch, capi, lib, fused="f32")
    if name == "copy":
        return CopyWorkload(torch)
    if name == "small_casts":
        return SmallCastsWorkload(torch, lib)
    if name in ("maxpool", "avgpool"):
        return PoolWorkload(name, torch, lib)
    if name == "fc4096":
        return FcWorkload(4096, torch, capi, lib)
    if name == "fc8192":
        return FcWorkload(8192, torch, capi, lib)
    return CastWorkload(name, torch, capi, lib)


SETTLE_MS = 250.0


def settle(torch, wl, min_gpu_ms=SETTLE_MS):
    """Untimed steps of the same workload until at least `min_gpu_ms` of GPU time have
    passed: over the first ~100 ms after an idle period the clocks have not settled and
    every kernel here runs 5-15 % slower, whatever --warmup says.  Returns the GPU
    milliseconds spent."""
    spent, batch = 0.0, 8
    while spent < min_gpu_ms:
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(batch):
            wl.step()
        e1.record()
        torch.cuda.synchronize()
        spent += e0.elapsed_time(e1)
        batch = min(batch * 2, 4096)
    return spent


def timed_run(torch, wl, steps, warmup):
    """Returns (wall seconds for `steps` steps, HIP-event seconds for the same steps).
    The events are recorded on the stream the kernels are launched on (torch's current
    stream, whose handle every step passes to the C ABI)."""
    wl.settle_ms = settle(torch, wl)
    for _ in range(warmup):
        wl.step()
    torch.cuda.synchronize()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(steps):
        wl.step()
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, ev0.elapsed_time(ev1) / 1e3


def roofline_of(wl, event_s_per_launch, key=None):
    if wl.bound == "mfma":
        achieved = wl.ops / event_s_per_launch / 1e12
        peak, unit = INT8_PEAK_TOPS, "TOP/s"
    else:
        achieved = wl.bytes / event_s_per_launch / 1e9
        peak, unit = HBM_PEAK_GBS, "GB/s"
    return {"bound": wl.bound, "kernel": wl.kernel, "achieved": round(achieved, 1), "peak": peak,
            "unit": unit, "frac": round(achieved / peak, 4),
            "traffic": profile_traffic(key)[0],
            "traffic_source": profile_traffic(key)[1],
            "avg_launch_us": round(event_s_per_launch * 1e6, 2)}


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the operators "
              "shard without any exchange but one 8-byte min/max all-reduce); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the HIP path has no CPU fallback)", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    import mxnet_amd
    from mxnet_amd import capi
    lib = mxnet_amd._lib.lib

    wl = make_workload(args.workload, torch, capi, lib)
    wall, ev = timed_run(torch, wl, args.steps, args.warmup)
    sec_per_step = wall / args.steps
    value, unit = wl.value(sec_per_step)
    line = {
        "metric": METRIC,
        "value": round(value, 2),
        "unit": unit,
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(sec_per_step * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": wl.name},
        "device": torch.cuda.get_device_name(0),
        "settle_ms": round(wl.settle_ms, 1),
        "roofline": roofline_of(wl, ev / args.steps, args.workload),
    }

    if isinstance(wl, FcWorkload):
        line["roofline"]["context"] = mfma_context(torch, wl.S)
    if isinstance(wl, GraphWorkload):
        line["roofline"]["layers_alone"] = wl.per_layer(torch)

    if not args.no_cast_ops:
        rows = []
        for kind in OTHER_WORKLOADS:
            if kind == args.workload:
                continue
            w2 = make_workload(kind, torch, capi, lib)
            steps2 = 300
            wall2, ev2 = timed_run(torch, w2, steps2, 20)
            r = roofline_of(w2, ev2 / steps2, kind)
            r["workload"] = w2.name
            r["key"] = kind
            if isinstance(w2, GraphWorkload):
                r["layers_alone"] = w2.per_layer(torch)
            rows.append(r)
            del w2
            torch.cuda.empty_cache()
        line["other_kernels"] = rows

    if not args.no_cpu_baseline and not isinstance(wl, (GraphWorkload, CopyWorkload,
                                                       PoolWorkload)):
        import oracle
        line["cpu_baseline"] = wl.cpu_baseline(oracle)
        try:
            # the reference's timed CPU path is oneDNN; torch bundles a oneDNN int8 GEMM
            if isinstance(wl, FcWorkload):
                d = wl.data[:512].cpu()
                w = wl.weight.cpu()
                torch._int_mm(d, w.t())
                t0 = time.perf_counter()
                reps = 0
                while time.perf_counter() - t0 < 5.0:
                    torch._int_mm(d, w.t())
                    reps += 1
                dt = time.perf_counter() - t0
                line["cpu_baseline"]["onednn_via_torch_TOPS"] = round(
                    2.0 * 512 * wl.S * wl.S * reps / dt / 1e12, 4)
                line["cpu_baseline"]["onednn_threads"] = torch.get_num_threads()
        except Exception as e:  # informational only
            line["cpu_baseline"]["onednn_via_torch_TOPS"] = "unavailable: %s" % e
    # The rows the metric's two targets are read from, compact and last in the line: whoever
    # keeps only the end of this output still sees every cast kernel's share of the HBM peak
    # next to the FC's share of the MFMA peak.  [us per launch (or pass), achieved, frac]
    summary = {"unit": "[us, GB/s or TOP/s, frac of 8000 GB/s or 5000 TOP/s]"}
    head = line["roofline"]
    summary[args.workload] = [head["avg_launch_us"], head["achieved"], head["frac"]]
    for r in line.get("other_kernels", []):
        if r["key"] in SUMMARY_WORKLOADS:
            summary[r["key"]] = [r["avg_launch_us"], r["achieved"], r["frac"]]
    if "context" in head:
        summary["context"] = head["context"]
    line["targets"] = summary
    head["cast_ops"] = " ".join("%s=%.3f" % (k, summary[k][2]) for k in CAST_TARGETS
                                if k in summary)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
