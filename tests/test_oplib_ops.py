"""Data-movement and simple-arithmetic operations of the op library: the oracle against numpy closed forms and
the reference's exact cases (CPU), the HIP path against the same expectations (GPU)."""
import numpy as np
import pytest

import oplib_cases
from oracle import tile_oracle as E
from oracle import tile_oplib as op


def check(outs, refs, exact):
    if not isinstance(refs, list):
        refs = [refs]
    assert len(outs) == len(refs)
    for out, ref in zip(outs, refs):
        check_one(out, ref, exact)


def check_one(out, ref, exact):
    assert np.asarray(out).shape == np.asarray(ref).shape
    if exact:
        np.testing.assert_array_equal(out, ref)
    else:
        np.testing.assert_allclose(out, ref, rtol=1e-3, atol=1e-5)


@pytest.mark.parametrize('name', sorted(oplib_cases.CASES))
def test_oracle(name):
    prog, ins, ref, exact = oplib_cases.CASES[name](E, op)
    check(E.run(prog, ins), ref, exact)


@pytest.mark.gpu
@pytest.mark.parametrize('target', ['hip', 'hip{specialise=0,fuse=0}'])
@pytest.mark.parametrize('name', sorted(oplib_cases.CASES))
def test_hip(name, target):
    from plaidml_amd import edsl as P
    from plaidml_amd import op as Pop
    prog, ins, ref, exact = oplib_cases.CASES[name](P, Pop)
    check(P.run(prog, ins, target=target), ref, exact)
