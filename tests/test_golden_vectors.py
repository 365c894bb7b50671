"""The committed operator vectors (tests/golden/operator_vectors.npz, written by
tests/golden/make_fixtures.py): the oracle must still reproduce them on the CPU, and the
HIP operators, called through the operator host under the reference's operator names, must
reproduce them on the GPU — integers and bytes bit-exact, float32 within 1e-6 relative."""
import importlib.util
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("golden_fixtures",
                                               os.path.join(HERE, "golden", "make_fixtures.py"))
fixtures = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(fixtures)

CASES = fixtures.load()
IDS = ["%02d-%s" % (i, c[0].replace("_contrib_", "")) for i, c in enumerate(CASES)]


def check(got, want, what):
    got = np.asarray(got)
    assert got.dtype == want.dtype, "%s: dtype %s, expected %s" % (what, got.dtype, want.dtype)
    assert got.shape == want.shape, "%s: shape %s, expected %s" % (what, got.shape, want.shape)
    if want.dtype == np.float32 and want.size > 1:
        np.testing.assert_allclose(got, want, rtol=1e-6, atol=0, err_msg=what)
    else:
        np.testing.assert_array_equal(got, want, err_msg=what)


def test_file_covers_every_registered_quantized_operator():
    from mxnet_amd import operator as op
    have = {c[0] for c in CASES}
    for name in op.list_operators():
        if name.startswith("_contrib_quant") or name in ("_contrib_requantize",
                                                         "_contrib_dequantize"):
            assert name in have, "no committed vector for " + name


def test_generator_is_deterministic():
    fresh = fixtures.cases()
    assert len(fresh) == len(CASES)
    for (op, attrs, ins), (op2, attrs2, ins2, _) in zip(fresh, CASES):
        assert op == op2
        assert {k: list(v) if isinstance(v, tuple) else v for k, v in attrs.items()} == attrs2
        for a, b in zip(ins, ins2):
            np.testing.assert_array_equal(a, b)


@pytest.mark.parametrize("case", CASES, ids=IDS)
def test_oracle_reproduces_the_vectors(case):
    op, attrs, ins, outs = case
    got = fixtures.run_oracle(op, attrs, ins)
    assert len(got) == len(outs)
    for j, (g, w) in enumerate(zip(got, outs)):
        np.testing.assert_array_equal(np.asarray(g), w, err_msg="%s output %d" % (op, j))


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=IDS)
def test_operators_reproduce_the_vectors(case):
    import torch
    from mxnet_amd.operator import invoke
    op, attrs, ins, outs = case
    dev = [torch.from_numpy(np.require(a, requirements="C")).cuda() for a in ins]
    attrs = {k: tuple(v) if isinstance(v, list) else v for k, v in attrs.items()}
    got = invoke(op, *dev, **attrs)
    if not isinstance(got, (tuple, list)):
        got = [got]
    assert len(got) == len(outs)
    for j, (g, w) in enumerate(zip(got, outs)):
        check(g.cpu().numpy(), w, "%s output %d" % (op, j))
