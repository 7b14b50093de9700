"""The one numeric network output the reference holds that can be used offline: `toy_parallel_conv`
(golden of its benchmark tool, checked there with rtol 5e-4 / atol 1e-6, plaidbench/core.py:395-399).
Fixture: tests/golden/toy_parallel_conv.npz, written by tests/golden/make_toy_parallel_conv.py.

Tolerance here: rtol 5e-4 as in the reference, atol 2e-4 instead of 1e-6.  The stored output was produced
by another fp32 implementation with its own summation order; a float64 evaluation of the definition differs
from it by at most 5e-5 absolute (activations reach 128), and 0.007 % of the elements -- small values next to
the ReLU cut -- miss atol 1e-6 for that reason alone.
"""
import numpy as np
import pytest

import programs
from oracle import tile_oracle as E
from oracle import tile_oplib as op

RTOL, ATOL = 5e-4, 2e-4


def thinned(out, fx):
    pos = fx['positions']
    return np.asarray(out)[0][np.ix_(pos, pos)]


def test_oracle_matches_reference_golden():
    prog, vals, fx = programs.toy_parallel_conv(E, op)
    out, = E.run(prog, vals)
    assert out.shape == (1, 56, 56, 256)
    got = thinned(out, fx)
    np.testing.assert_allclose(got, fx['expected'], rtol=RTOL, atol=ATOL)
    # and nearly everywhere to the reference's own bar
    assert np.isclose(got, fx['expected'], rtol=5e-4, atol=1e-6).mean() > 0.999


@pytest.mark.gpu
@pytest.mark.parametrize('target', ['hip', 'hip{specialise=0,fuse=0}'])
def test_hip_matches_reference_golden(target):
    from plaidml_amd import edsl as P
    from plaidml_amd import op as Pop
    prog, vals, fx = programs.toy_parallel_conv(P, Pop)
    out, = P.run(prog, vals, target=target)
    assert out.shape == (1, 56, 56, 256)
    # fp32 MFMA accumulates in another order again: the fp32 bar of this build (rtol 1e-3) with the same atol
    np.testing.assert_allclose(thinned(out, fx), fx['expected'], rtol=1e-3, atol=ATOL)
