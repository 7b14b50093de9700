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


@pytest.mark.gpu
def test_toy_gemms_through_the_harness_and_against_float64():
    """Four dense layers with ReLU: the harness runs and reports; the output equals a float64 evaluation with the same
    weights (the builder's random streams, restated here) to the fp32 bar."""
    from plaidml_amd import edsl as P
    r = pb.run('toy_gemms', batch_size=8, examples=16, warmups=8)
    assert r['correct'] == 'untested' and 0 < r['tile_duration_per_example'] <= r['duration_per_example']
    program, inputs = pb._NETWORKS['toy_gemms'].build(8)
    got, = P.run(program, inputs, target='hip')
    rng = np.random.default_rng(5)
    weights, width = [], 256
    for units in (512, 1024, 2048, 1000):
        limit = np.sqrt(6.0 / (width + units))
        weights.append(rng.uniform(-limit, limit, (width, units)).astype(np.float32))
        width = units
    x = rng.uniform(0, 1, (8, 256)).astype(np.float32)
    np.testing.assert_array_equal(x, inputs[0])
    ref = x.astype(np.float64)
    for W in weights:
        ref = np.maximum(ref @ W.astype(np.float64), 0)
    np.testing.assert_allclose(got, ref, rtol=1e-3, atol=1e-5)


@pytest.mark.gpu
def test_toy_xcp_through_the_harness_and_against_float64_samples():
    """ReLU -> 3x3 convolution 64 -> 128 (SAME) -> max-pool 3x3 / 2 (SAME) on 149x149: 400 sampled outputs against a
    float64 evaluation of their windows."""
    from plaidml_amd import edsl as P
    r = pb.run('toy_xcp', batch_size=2, examples=4, warmups=2)
    assert r['correct'] == 'untested' and 0 < r['tile_duration_per_example'] <= r['duration_per_example']
    program, inputs = pb._NETWORKS['toy_xcp'].build(2)
    got, = P.run(program, inputs, target='hip')
    assert got.shape == (2, 75, 75, 128)
    rng = np.random.default_rng(6)
    limit = np.sqrt(6.0 / (9 * 64 + 9 * 128))
    W = rng.uniform(-limit, limit, (3, 3, 64, 128)).astype(np.float32).astype(np.float64)
    x = rng.uniform(0, 1, (2, 149, 149, 64)).astype(np.float32)
    np.testing.assert_array_equal(x, inputs[0])
    xr = np.maximum(x, 0).astype(np.float64)

    def conv_at(n, y, xx, c):  # SAME, stride 1: pad 1
        acc = 0.0
        for ky in range(3):
            for kx in range(3):
                iy, ix = y + ky - 1, xx + kx - 1
                if 0 <= iy < 149 and 0 <= ix < 149:
                    acc += float(xr[n, iy, ix] @ W[ky, kx, :, c])
        return acc

    pick = np.random.default_rng(1)
    for _ in range(400):
        n, oy, ox, c = int(pick.integers(2)), int(pick.integers(75)), int(pick.integers(75)), int(pick.integers(128))
        if _ < 8:
            oy, ox = (0, 74)[_ & 1], (0, 74)[(_ >> 1) & 1]  # corners
        best = -np.inf
        for ky in range(3):          # SAME_UPPER with stride 2 on 149 -> 75: pad_before 0... (75 - 1) * 2 + 3 - 149 = 2 -> 1 before
            for kx in range(3):
                y, xx = 2 * oy + ky - 1, 2 * ox + kx - 1
                if 0 <= y < 149 and 0 <= xx < 149:
                    best = max(best, conv_at(n, y, xx, c))
        np.testing.assert_allclose(got[n, oy, ox, c], best, rtol=1e-3, atol=1e-5)
