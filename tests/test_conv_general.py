"""The convolution operation in its general form (layouts, dilations, groups, derivative modes): the oracle and the
hip device against direct numpy evaluations (tests/conv_cases.py)."""
import numpy as np
import pytest

import conv_cases
from oracle import tile_oracle as OE
from oracle import tile_oplib as Oop

NAMES = sorted(conv_cases.CASES)


def check(outs, refs):
    assert len(outs) == len(refs)
    for out, ref in zip(outs, refs):
        assert out.shape == ref.shape
        np.testing.assert_allclose(out, ref, rtol=1e-3, atol=1e-4)   # fp32 bar


@pytest.mark.parametrize('name', NAMES)
def test_oracle(name):
    prog, ins, refs = conv_cases.CASES[name](OE, Oop)
    check(OE.run(prog, ins), refs)


def test_oracle_rejects_inconsistent_requests():
    X = OE.Placeholder(OE.DType.FLOAT32, [1, 5, 5, 4])
    F = OE.Placeholder(OE.DType.FLOAT32, [3, 3, 4, 8])
    with pytest.raises(ValueError, match='UNGROUPED requires groups == 1'):
        Oop.convolution(X, F, groups=2)
    with pytest.raises(ValueError, match='GroupLayout not specified'):
        Oop.convolution(X, F, groups=2, autogroup_mode=Oop.AUTOGROUP_EXPLICIT)
    with pytest.raises(ValueError, match='require specifying the result_shape'):
        Oop.convolution(X, F, deriv_mode=Oop.DERIV_DATA)
    with pytest.raises(ValueError, match='separate groups'):
        Oop.convolution(X, F, filter_layout=Oop.LAYOUT_XGCK)
    with pytest.raises(ValueError, match='Autopadding and manual padding'):
        Oop.convolution(X, F, manual_padding=[1, 1])


@pytest.mark.gpu
@pytest.mark.parametrize('target', ['hip', 'hip{specialise=0,fuse=0}'])
@pytest.mark.parametrize('name', NAMES)
def test_hip(name, target):
    from plaidml_amd import edsl as P
    from plaidml_amd import op as Pop
    print('conv case', name, 'target', target, flush=True)
    prog, ins, refs = conv_cases.CASES[name](P, Pop)
    outs = P.run(prog, ins, target=target)
    check(outs, refs)
    oprog, oins, _ = conv_cases.CASES[name](OE, Oop)
    for got, want in zip(outs, OE.run(oprog, oins)):
        np.testing.assert_allclose(got, want, rtol=1e-3, atol=1e-5)


@pytest.mark.gpu
def test_hip_rejects_inconsistent_requests():
    from plaidml_amd import edsl as P
    from plaidml_amd import op as Pop
    X = P.Placeholder(P.DType.FLOAT32, [1, 5, 5, 4])
    F = P.Placeholder(P.DType.FLOAT32, [3, 3, 4, 8])
    with pytest.raises(P.PlaidMLError, match='UNGROUPED requires groups == 1'):
        Pop.convolution(X, F, groups=2)
    with pytest.raises(P.PlaidMLError, match='GroupLayout not specified for grouped convolution'):
        Pop.convolution(X, F, groups=2, autogroup_mode=Pop.AUTOGROUP_EXPLICIT)
    with pytest.raises(P.PlaidMLError, match='require specifying the result_shape'):
        Pop.convolution(X, F, deriv_mode=Pop.DERIV_DATA)
    F5 = P.Placeholder(P.DType.FLOAT32, [3, 3, 2, 2, 4])
    with pytest.raises(P.PlaidMLError, match="isn't SEPARATE"):
        Pop.convolution(X, F5, filter_layout=Pop.LAYOUT_XGCK)
    with pytest.raises(P.PlaidMLError, match='expected spatial rank 2 but filter tensor has 4 dimensions'):
        Pop.convolution(X, F, filter_layout=Pop.LAYOUT_XGCK, group_layout=Pop.GROUP_SEPARATE)
