"""The benchmark harness (plaidml_amd/plaidbench.py): the correctness arithmetic of the reference's tool
(plaidbench/plaidbench/core.py:395-416) on hand-computed cases, argument checks, and on the GPU one golden-checked
network and one synthetic network through the whole warm-up / timed loop."""
import numpy as np
import pytest

from plaidml_amd import plaidbench as pb


def test_correctness_arithmetic_by_hand():
    # |base - cur| = 1e-3 at cur = 2: relative error p * 1e-3 / (1e-6 + p * 2) with p = 5e-4
    base, cur = np.array([2.001, 1.0, 0.0]), np.array([2.0, 1.0, 0.0])
    correct, max_error, max_abs_error, fail_ratio = pb.check_correctness(base, cur, 5e-4)
    assert max_error == pytest.approx(5e-4 * 1e-3 / (1e-6 + 5e-4 * 2.0), rel=1e-9)
    assert max_abs_error == pytest.approx(1e-3, rel=1e-9)
    assert fail_ratio == 0.0          # 4.995e-4 is just inside the precision
    assert correct                    # 1e-3 <= 1e-6 + 5e-4 * 2
    # a mismatch next to zero: passes neither allclose (atol 1e-6) nor the relative bar
    correct, max_error, max_abs_error, fail_ratio = pb.check_correctness(np.array([1e-4, 1.0]), np.array([0.0, 1.0]), 5e-4)
    assert not correct
    assert max_error == pytest.approx(5e-4 * 1e-4 / 1e-6, rel=1e-9)
    assert fail_ratio == 0.5
    # the same under a wider absolute tolerance: `correct` changes, fail_ratio keeps the reference's definition
    correct, _, _, fail_ratio = pb.check_correctness(np.array([1e-4, 1.0]), np.array([0.0, 1.0]), 5e-4, atol=2e-4)
    assert correct and fail_ratio == 0.5


def test_correctness_is_not_symmetric():
    # allclose scales the tolerance by |cur| (its second argument), as in the reference's call
    assert pb.check_correctness(np.array([1.0]), np.array([1000.0]), 0.5)[0] is False
    assert pb.check_correctness(np.array([600.0]), np.array([1000.0]), 0.5)[0] is True
    assert pb.check_correctness(np.array([1000.0]), np.array([600.0]), 0.5)[0] is False


def test_empty_output():
    assert pb.check_correctness(np.zeros(0), np.zeros(0), 5e-4) == (True, 0.0, 0.0, 'Undefined')


def test_argument_checks():
    with pytest.raises(ValueError, match='divisible by the batch size'):
        pb.run('resnet50', batch_size=3, examples=10)
    with pytest.raises(ValueError, match='unknown network'):
        pb.run('no_such_network')


def test_report_text():
    r = {'model': 'toy', 'backend': 'hip', 'batch_size': 1, 'examples': 4, 'compile_duration': 0.5, 'execution_duration': 0.004,
         'duration_per_example': 0.001, 'tile_duration_per_example': 0.0005, 'correct': True, 'max_error': 1e-5,
         'max_abs_error': 2e-5, 'fail_ratio': 0.0}
    text = pb.format_report(r)
    assert '1.00 ms / 1000.00 fps' in text and 'Correctness: PASS' in text
    r['correct'] = 'untested'
    assert 'Could not find golden data' in pb.format_report(r)


def test_toy_network_builds_and_has_golden_only_at_batch_one():
    program, inputs = pb._toy_parallel_conv(2)
    assert [tuple(s.sizes) for s in program.inputs] == [(2, 224, 224, 3)]
    assert [tuple(s.sizes) for s in program.outputs] == [(2, 56, 56, 256)]
    assert inputs[0].shape == (2, 224, 224, 3) and (inputs[0][0] == inputs[0][1]).all()
    assert pb._toy_golden(2) is None
    g = pb._toy_golden(1)
    assert g.expected.shape == (16, 16, 256) and g.precision == 5e-4
    assert g.select(np.zeros((1, 56, 56, 256))).shape == (16, 16, 256)


@pytest.mark.gpu
def test_toy_parallel_conv_through_the_harness():
    r = pb.run('toy_parallel_conv', batch_size=1, examples=8, warmups=2)
    assert r['correct'] is True
    assert r['fail_ratio'] < 1e-3 and r['max_abs_error'] < 2e-3
    assert r['examples'] == 8 and r['batch_size'] == 1 and r['model'] == 'toy_parallel_conv' and r['backend'] == 'hip'
    assert 0 < r['tile_duration_per_example'] <= r['duration_per_example']
    assert r['compile_duration'] > 0
    assert 'Correctness: PASS' in pb.format_report(r)


@pytest.mark.gpu
def test_toy_parallel_conv_batched_is_untested_but_runs():
    r = pb.run('toy_parallel_conv', batch_size=4, examples=8, warmups=4)
    assert r['correct'] == 'untested' and r['tile_duration_per_example'] > 0


@pytest.mark.gpu
def test_resnet50_through_the_harness():
    r = pb.run('resnet50', batch_size=2, examples=4, warmups=2)
    assert r['correct'] == 'untested'       # synthetic weights; the harness has checked the softmax rows
    assert 0 < r['tile_duration_per_example'] <= r['duration_per_example']
    assert pb.main(['resnet50', '--batch-size', '2', '--examples', '2', '--warmups', '0', '--json']) == 0
