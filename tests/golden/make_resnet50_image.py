"""Writes tests/golden/resnet50_v1_5_image_probs.npz: the class probabilities and the logits the CPU oracle computes for one
224 x 224 image through the full-width ResNet-50 v1.5 program of plaidml_amd/resnet50.py (bf16, the builder's
seeded weights).  The oracle needs about five minutes for the image, too long for a test; the GPU test runs the
batch-128 program with this image in slot 0 and compares that row.

    python tests/golden/make_resnet50_image.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import tile_oracle as E          # noqa: E402
from oracle import tile_oplib as Eop         # noqa: E402
from plaidml_amd import resnet50             # noqa: E402

IMAGE_SEED = 11


def image():
    return E.round_bf16(np.random.default_rng(IMAGE_SEED).uniform(0, 1, (1, 224, 224, 3)).astype(np.float32))


if __name__ == '__main__':
    prog, _, _ = resnet50.build(E, Eop, batch=1, round_fn=E.round_bf16, with_logits=True)
    probs, logits = E.run(prog, [image()])
    out = os.path.join(ROOT, 'tests', 'golden', 'resnet50_v1_5_image_probs.npz')
    np.savez(out, probs=probs.astype(np.float32), logits=logits.astype(np.float32), image_seed=np.int64(IMAGE_SEED))
    print('wrote', out, probs.shape, int(probs.argmax()), float(logits.min()), float(logits.max()), float(np.abs(logits).mean()))
