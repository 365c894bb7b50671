"""Every kernel that writes its bytes with the 16-byte device-scope store helper
(stream_store16: inline assembly the compiler's hazard and wait-count passes do not see)
on sizes that drive its unrolled main loop, its remainder loop and its ragged tail in one
launch: several passes of a full grid (the loop-carried index arithmetic runs right behind
the stores), a remainder that is not a whole pass, and a length that is not a multiple of 16.
A store whose data registers are overwritten too early shows up as wrong bytes here."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

# more than four passes of the largest grid the launchers use (2 work-groups of 256 lanes
# per CU, 16 bytes per lane) plus a partial pass and a ragged tail
N_LOOP = 4 * 2 * 256 * 256 * 16 + 3 * 256 * 16 + 11


@pytest.fixture(scope="module")
def contrib():
    import mxnet_amd
    return mxnet_amd.contrib


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def scalar(v):
    return torch.tensor([v], dtype=torch.float32, device="cuda")


def host(t):
    return t.cpu().numpy()


def draw(rng, dtype, shape):
    lo, hi = (0, 256) if dtype == np.uint8 else (-128, 128)
    return rng.integers(lo, hi, shape).astype(dtype)


@pytest.mark.parametrize("ta,tb", [(np.int8, np.int8), (np.uint8, np.int8)])
def test_elemwise_add_bytes_loops(contrib, ta, tb):
    rng = np.random.default_rng(1)
    a, b = draw(rng, ta, N_LOOP), draw(rng, tb, N_LOOP)
    rngs = (-1.3, 0.9, -0.2, 2.2)
    out, mn, mx = contrib.quantized_elemwise_add(dev(a), dev(b), *[scalar(v) for v in rngs],
                                                 min_calib_range=-3.0, max_calib_range=2.5)
    ref, rmn, rmx = oracle.quantized_elemwise_add(a, b, *rngs, min_calib_range=-3.0,
                                                  max_calib_range=2.5)
    np.testing.assert_array_equal(host(out), ref)
    assert (host(mn)[0], host(mx)[0]) == (rmn, rmx)


def test_elemwise_add_int32_runs_and_tail(contrib):
    """The int32 output form: whole 4 KiB runs per wave, the partial last run, the tail."""
    rng = np.random.default_rng(2)
    a, b = draw(rng, np.int8, N_LOOP), draw(rng, np.int8, N_LOOP)
    rngs = (-1.3, 0.9, -0.2, 2.2)
    out, mn, mx = contrib.quantized_elemwise_add(dev(a), dev(b), *[scalar(v) for v in rngs])
    ref, rmn, rmx = oracle.quantized_elemwise_add(a, b, *rngs)
    np.testing.assert_array_equal(host(out), ref)


def test_elemwise_mul_bytes_loops(contrib):
    rng = np.random.default_rng(3)
    a, b = draw(rng, np.int8, N_LOOP), draw(rng, np.int8, N_LOOP)
    rngs = (-1.0, 1.0, -2.0, 2.0)
    out, mn, mx = contrib.quantized_elemwise_mul(dev(a), dev(b), *[scalar(v) for v in rngs],
                                                 min_calib_range=-2.5, max_calib_range=2.5)
    ref, rmn, rmx = oracle.quantized_elemwise_mul(a, b, *rngs, min_calib_range=-2.5,
                                                  max_calib_range=2.5)
    np.testing.assert_array_equal(host(out), ref)


@pytest.mark.parametrize("shape,axis", [((67, 48, 16 * 113), 1),      # rows of whole 16-byte pieces
                                        ((3, 5, N_LOOP // 15 // 16 * 16), 1),  # long rows
                                        ((N_LOOP // 96, 96), 1)])     # channel innermost: flat kernel
@pytest.mark.parametrize("relu", [False, True])
def test_batch_norm_loops(contrib, shape, axis, relu):
    rng = np.random.default_rng(4)
    C = shape[axis]
    d = draw(rng, np.int8, shape)
    gamma = rng.uniform(0.5, 1.5, C).astype(np.float32)
    beta = rng.normal(0, 1, C).astype(np.float32)
    mean = rng.normal(0, 1, C).astype(np.float32)
    var = rng.uniform(0.5, 1.5, C).astype(np.float32)
    out, mn, mx = contrib.quantized_batch_norm(
        dev(d), dev(gamma), dev(beta), dev(mean), dev(var), scalar(-2.7), scalar(3.1), eps=2e-5,
        axis=axis, min_calib_range=-6.5, max_calib_range=7.25, relu=relu)
    ref, rmn, rmx = oracle.quantized_batch_norm(d, gamma, beta, mean, var, -2.7, 3.1, -6.5, 7.25,
                                                eps=2e-5, axis=axis, relu=relu)
    np.testing.assert_array_equal(host(out), ref)


def test_concat_loops(contrib):
    """Three inputs of different ranges along the innermost axis (one copied, two rescaled),
    each several grid passes long, slab lengths that are and are not multiples of 16."""
    rng = np.random.default_rng(5)
    parts = [draw(rng, np.int8, (2, N_LOOP // 8 + off)) for off in (0, 16, 5)]
    mins, maxs = [-1.0, -2.0, -0.5], [1.0, 2.0, 0.25]
    args = [dev(p) for p in parts]
    for lo, hi in zip(mins, maxs):
        args += [scalar(lo), scalar(hi)]
    out, mn, mx = contrib.quantized_concat(*args, num_args=3, dim=1)
    ref, rmn, rmx = oracle.quantized_concat(parts, mins, maxs, dim=1)
    np.testing.assert_array_equal(host(out), ref)
    assert (host(mn)[0], host(mx)[0]) == (rmn, rmx)


@pytest.mark.parametrize("sa,sb", [((37, 64, 16 * 129), (1, 64, 1)),   # per-channel operand, long runs
                                   ((N_LOOP // 4096, 4096), (1, 4096)),  # a row added to every row
                                   ((611, 16 * 67), (611, 1))])        # a column: scalar per run
def test_broadcast_add_loops(contrib, sa, sb):
    rng = np.random.default_rng(6)
    a, b = draw(rng, np.int8, sa), draw(rng, np.int8, sb)
    rngs = (-1.3, 0.9, -0.2, 2.2)
    out, mn, mx = contrib.quantized_npi_add(dev(a), dev(b), *[scalar(v) for v in rngs],
                                            min_calib_range=-3.0, max_calib_range=2.5)
    ref, rmn, rmx = oracle.quantized_npi_add(a, b, *rngs, min_calib_range=-3.0,
                                             max_calib_range=2.5)
    np.testing.assert_array_equal(host(out), ref)
