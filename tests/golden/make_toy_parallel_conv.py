"""Writes tests/golden/toy_parallel_conv.npz from data files the reference holds (run once, in a checkout
that has /root/reference; the result is committed).

The reference's benchmark tool checks its `toy_parallel_conv` network (plaidbench/networks/keras/
toy_parallel_conv.py:23-41: conv 7x7/2 SAME 3->64 + ReLU, then relu(relu(conv 1x1/2 64->256) +
relu(conv 3x3/2 SAME 64->256))) against a stored output with rtol 5e-4 / atol 1e-6
(plaidbench/core.py:395-399).  This script copies the three data files that check needs and nothing else:
  * the layer weights, read from networks/keras/toy_parallel_conv.h5 with tests/golden/h5min.py,
  * the input: image 0 of cifar16.npy (uint8 32x32x3; the tool repeats every pixel 7x7 times and feeds the
    values unscaled, toy_parallel_conv.py:18-20),
  * the expected output golden/toy_parallel_conv/infer,bs-1.npy (1x56x56x256 fp32), thinned to the 16 x 16
    output positions ROWS x ROWS (all 256 channels; the borders, where padding acts, are kept densely)
    to keep the fixture below 1 MB.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import h5min  # noqa: E402

REF = '/root/reference/plaidbench/plaidbench'
ROWS = [0, 1, 2, 3, 8, 16, 24, 27, 28, 32, 40, 48, 52, 53, 54, 55]


def main():
    ds = h5min.H5File(os.path.join(REF, 'networks/keras/toy_parallel_conv.h5')).datasets()
    out = {}
    for i in (1, 2, 3):
        out['kernel%d' % i] = ds['/conv2d_%d/conv2d_%d/kernel:0' % (i, i)]
        out['bias%d' % i] = ds['/conv2d_%d/conv2d_%d/bias:0' % (i, i)]
    out['image'] = np.load(os.path.join(REF, 'cifar16.npy'))[0]
    full = np.load(os.path.join(REF, 'golden/toy_parallel_conv/infer,bs-1.npy'))
    assert full.shape == (1, 56, 56, 256)
    out['positions'] = np.array(ROWS, np.int32)
    out['expected'] = full[0][np.ix_(ROWS, ROWS)]
    path = os.path.join(HERE, 'toy_parallel_conv.npz')
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), 'bytes;', {k: (v.shape, str(v.dtype)) for k, v in out.items()})


if __name__ == '__main__':
    main()
