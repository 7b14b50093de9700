"""A benchmark harness in the manner of the reference's plaidbench, over the ctypes front end.

What it keeps of `plaidbench/plaidbench/core.py`: a network is set up and compiled (timed), run once for its output,
run again for `warmups` examples, then timed over `examples` examples in batches (:220-268); the report carries the
reference's keys -- `compile_duration`, `duration_per_example`, `tile_duration_per_example`, `examples`, `batch_size`,
`model`, `backend` -- and, where a golden output exists, `correct`, `max_error`, `max_abs_error` and `fail_ratio`
computed as `Runner._check_correctness` computes them (:395-416).  A network is a function that builds a Tile
program.  Registered here: `resnet50` (v1.5, bf16, synthetic weights: no golden, so "untested" as in the reference
when the golden file is missing; the softmax rows are checked to sum to one) and `toy_parallel_conv` (fp32, the
reference tool's own weights, input and golden output at batch size 1, from the fixture file named by
PLAIDBENCH_GOLDEN or found beside the tests), `toy_gemms` and `toy_xcp` (the reference tool's two other toy
networks, randomly initialised there as here); `register` adds others.

    python -m plaidml_amd.plaidbench resnet50 --batch-size 128 --examples 1024
"""
import argparse
import json
import os
import time

import numpy as np

from . import edsl as P
from . import op as Pop

DEFAULT_WARMUPS = 32      # examples, as in the reference (plaidbench/core.py:116-121)
DEFAULT_EXAMPLES = 1024


INFERENCE_PRECISION = 5e-04   # plaidbench/core.py Precision.INFERENCE
TRAINING_PRECISION = 2e-03    # plaidbench/core.py Precision.TRAINING


class Golden:
    """The expected value of output 0 (after `select`, which cuts the part of the output the file holds),
    the relative precision, and the absolute tolerance of the PASS / FAIL result (the reference's is 1e-6)."""

    def __init__(self, expected, precision=INFERENCE_PRECISION, atol=1e-06, select=None):
        self.expected, self.precision, self.atol, self.select = expected, precision, atol, select or (lambda out: out)


class Network:
    """build(batch_size) -> (program, [input arrays]); golden(batch_size) -> Golden, or None when there is no
    golden output for that batch size; sanity(outputs) may raise when the outputs are implausible (used where no
    golden exists)."""

    def __init__(self, name, build, golden=None, sanity=None):
        self.name, self.build, self.golden, self.sanity = name, build, golden, sanity


_NETWORKS = {}


def register(network):
    _NETWORKS[network.name] = network
    return network


def check_correctness(base_output, cur_output, precision, atol=1e-06):
    """(correct, max_error, max_abs_error, fail_ratio) with the reference's definitions: allclose at
    rtol = precision, atol = 1e-6 (unless given); relative error precision * |base - cur| / (1e-6 + precision * |cur|);
    an entry fails when that exceeds the precision."""
    base_output, cur_output = np.asarray(base_output, np.float64), np.asarray(cur_output, np.float64)
    correct = bool(np.allclose(base_output, cur_output, rtol=precision, atol=atol))
    relative_error = (precision * np.absolute(base_output - cur_output)) / (1e-06 + precision * np.absolute(cur_output))
    max_error = float(np.amax(relative_error)) if relative_error.size else 0.0
    max_abs_error = float(np.amax(np.absolute(base_output - cur_output))) if relative_error.size else 0.0
    total = relative_error.size
    fail_ratio = float((relative_error > precision).sum()) / total if total else 'Undefined'
    return correct, max_error, max_abs_error, fail_ratio


def run(network_name, batch_size=1, examples=DEFAULT_EXAMPLES, warmups=DEFAULT_WARMUPS, target='hip', device=''):
    """Benchmarks one network; returns the report dictionary."""
    if network_name not in _NETWORKS:
        raise ValueError('unknown network %r (known: %s)' % (network_name, ', '.join(sorted(_NETWORKS))))
    if examples % batch_size != 0:
        raise ValueError('The number of examples must be divisible by the batch size.')
    net = _NETWORKS[network_name]
    results = {'model': network_name, 'backend': target, 'batch_size': batch_size, 'examples': examples}
    program, inputs = net.build(batch_size)
    t0 = time.perf_counter()
    runner = P.Runner(program, device=device, target=target)
    results['compile_duration'] = time.perf_counter() - t0
    outputs = runner.run(inputs)                                   # the run whose output is checked
    staged = runner.stage(inputs)                                  # conversion to the device's types happens once
    for _ in range((warmups + batch_size - 1) // batch_size):
        runner.run_staged(staged)
    t0 = time.perf_counter()
    kernel_ms = 0.0
    for _ in range(examples // batch_size):
        runner.run_staged(staged)                                  # upload, kernels, download of every output
        kernel_ms += P.last_run_stats()['kernel_ms']
    execution_duration = time.perf_counter() - t0
    results['execution_duration'] = execution_duration
    results['duration_per_example'] = execution_duration / examples            # wall time, transfers included
    results['tile_duration_per_example'] = kernel_ms * 1e-3 / examples         # device time of the kernels alone
    golden = net.golden(batch_size) if net.golden else None
    if golden is not None:
        correct, max_error, max_abs_error, fail_ratio = check_correctness(golden.expected, golden.select(outputs[0]),
                                                                          golden.precision, golden.atol)
        results.update(correct=correct, max_error=max_error, max_abs_error=max_abs_error, fail_ratio=fail_ratio,
                       precision=golden.precision, atol=golden.atol)
    else:
        results['correct'] = 'untested'
        if net.sanity:
            net.sanity(outputs)
    return results


def format_report(results):
    per = results['duration_per_example']
    lines = ['Example finished, elapsed: %.3fs (compile), %.3fs (execution)' % (results['compile_duration'], results['execution_duration']),
             '-' * 89, '%-20s %-25s %-20s' % ('Network Name', 'Inference Latency', 'Time / FPS'), '-' * 89,
             '%-20s %-25s %-20s' % (results['model'], '%.2f ms' % (per * 1000), '%.2f ms / %.2f fps' % (per * 1000, 1.0 / per)),
             'Device time per example: %.4f ms (%.1f examples/s)' % (results['tile_duration_per_example'] * 1000,
                                                                     1.0 / results['tile_duration_per_example'])]
    if results['correct'] == 'untested':
        lines.append('Correctness: untested. Could not find golden data to compare against.')
    else:
        lines.append('Correctness: %s, max_error: %s, max_abs_error: %s, fail_ratio: %s' % (
            'PASS' if results['correct'] else 'FAIL', results['max_error'], results['max_abs_error'], results['fail_ratio']))
    return '\n'.join(lines)


def _resnet50(batch_size):
    from . import resnet50
    program, _, _ = resnet50.build(P, Pop, batch=batch_size, round_fn=P.round_bf16)
    x = np.random.default_rng(11).uniform(0, 1, (batch_size, 224, 224, 3)).astype(np.float32)
    return program, [x]


def _softmax_rows(outputs):
    out = np.asarray(outputs[0], np.float64)
    if not (np.isfinite(out).all() and (out >= 0).all() and np.allclose(out.sum(axis=1), 1.0, atol=2e-2)):
        raise RuntimeError('the output rows are not probability distributions')


register(Network('resnet50', _resnet50, sanity=_softmax_rows))


def _toy_fixture():
    here = os.path.dirname(os.path.abspath(__file__))
    for path in (os.environ.get('PLAIDBENCH_GOLDEN', ''), os.path.join(here, '..', 'tests', 'golden', 'toy_parallel_conv.npz')):
        if path and os.path.exists(path):
            return np.load(path)
    raise FileNotFoundError('toy_parallel_conv.npz not found: set PLAIDBENCH_GOLDEN to its path')


def _toy_parallel_conv(batch_size):
    """plaidbench/plaidbench/networks/keras/toy_parallel_conv.py:18-41 -- conv 7x7/2 3->64 + ReLU, then
    relu(relu(conv 1x1/2 64->256) + relu(conv 3x3/2 64->256)), SAME padding, fp32; the image is the 32x32 input
    of the fixture repeated 7 times along both axes (values 0..255, unscaled)."""
    fx = _toy_fixture()
    f32 = P.DType.FLOAT32
    image = np.repeat(np.repeat(fx['image'][None].astype(np.float32), 7, axis=1), 7, axis=2)
    image = np.ascontiguousarray(np.broadcast_to(image, (batch_size,) + image.shape[1:]))
    X = P.Placeholder(f32, list(image.shape))

    def conv(x, i):
        W, B = P.Constant(fx['kernel%d' % i], f32), P.Constant(fx['bias%d' % i], f32)
        return Pop.relu(Pop.convolution(x, W, strides=[2, 2], autopad=Pop.SAME_UPPER) + B)

    first = conv(X, 1)
    out = Pop.relu(conv(first, 2) + conv(first, 3))
    return P.Program('toy_parallel_conv', [X], [out]), [image]


def _toy_golden(batch_size):
    if batch_size != 1:  # the reference keeps one golden file per batch size and has this one only
        return None
    fx = _toy_fixture()
    pos = fx['positions']
    # The file holds the output at `positions` x `positions` of the 56x56 plane.  Its values come from another fp32
    # implementation with its own summation order: a float64 evaluation of the definition differs from them by up to
    # 5e-5 (activations reach 128), so PASS / FAIL uses atol 2e-4; fail_ratio keeps the reference's definition.
    return Golden(fx['expected'], INFERENCE_PRECISION, atol=2e-04, select=lambda out: np.asarray(out)[0][np.ix_(pos, pos)])


register(Network('toy_parallel_conv', _toy_parallel_conv, golden=_toy_golden))


def _finite(outputs):
    if not all(np.isfinite(np.asarray(o, np.float64)).all() for o in outputs):
        raise RuntimeError('the output holds values that are not finite')


def _toy_gemms(batch_size):
    """plaidbench/plaidbench/networks/keras/toy_gemms.py:22-38 -- four dense layers 256 -> 512 -> 1024 -> 2048 -> 1000,
    each followed by ReLU, fp32; randomly initialised as there (Glorot-uniform weights, zero biases), so no golden."""
    rng = np.random.default_rng(5)
    f32 = P.DType.FLOAT32
    X = P.Placeholder(f32, [batch_size, 256])
    x, width = X, 256
    for units in (512, 1024, 2048, 1000):
        limit = np.sqrt(6.0 / (width + units))
        W = P.Constant(rng.uniform(-limit, limit, (width, units)).astype(np.float32), f32)
        b = P.Constant(np.zeros(units, np.float32), f32)
        x, width = Pop.relu(Pop.dot(x, W) + b), units
    return P.Program('toy_gemms', [X], [x]), [rng.uniform(0, 1, (batch_size, 256)).astype(np.float32)]


def _toy_xcp(batch_size):
    """plaidbench/plaidbench/networks/keras/toy_xcp.py:25-50 (the internal form): ReLU of a 149x149x64 input, a 3x3
    convolution to 128 channels (SAME, no bias), max-pool 3x3 / 2 (SAME); fp32, random initialisation, no golden."""
    rng = np.random.default_rng(6)
    f32 = P.DType.FLOAT32
    X = P.Placeholder(f32, [batch_size, 149, 149, 64])
    limit = np.sqrt(6.0 / (9 * 64 + 9 * 128))
    W = P.Constant(rng.uniform(-limit, limit, (3, 3, 64, 128)).astype(np.float32), f32)
    y = Pop.convolution(Pop.relu(X), W, autopad=Pop.SAME_UPPER)
    y = Pop.pool(y, 'max', [3, 3], [2, 2], autopad=Pop.SAME_UPPER)
    return P.Program('toy_xcp', [X], [y]), [rng.uniform(0, 1, (batch_size, 149, 149, 64)).astype(np.float32)]


register(Network('toy_gemms', _toy_gemms, sanity=_finite))
register(Network('toy_xcp', _toy_xcp, sanity=_finite))


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split('\n')[0])
    ap.add_argument('network', choices=sorted(_NETWORKS))
    ap.add_argument('--batch-size', type=int, default=1)
    ap.add_argument('--examples', type=int, default=DEFAULT_EXAMPLES)
    ap.add_argument('--warmups', type=int, default=DEFAULT_WARMUPS)
    ap.add_argument('--target', default='hip')
    ap.add_argument('--json', action='store_true', help='print the report as one JSON object')
    args = ap.parse_args(argv)
    results = run(args.network, args.batch_size, args.examples, args.warmups, args.target)
    print(json.dumps(results, sort_keys=True) if args.json else format_report(results))
    return 0


if __name__ == '__main__':
    raise SystemExit(main())
