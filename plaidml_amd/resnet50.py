"""ResNet-50 v1.5 as a Tile program, built through the edsl / op API.

Topology of the reference's op-library network (networks/oplib/resnet50.cc:26-57 bottleneck block,
:222-331 network) with the stride of a down-sampling block moved from the first 1x1 convolution to
the 3x3 one (v1.5).  Batch norm is folded into (weight, bias) of every convolution, so a layer is
`relu(convolution(x, W) + b)`; weights and biases are program constants (uploaded once), the image
batch is the only input.

`build(E, op, ...)` works with any module pair that offers the edsl / op surface: the product
binding (plaidml_amd.edsl, plaidml_amd.op) or the CPU oracle used by the tests.
"""
import numpy as np

STAGES = [(3, 64), (4, 128), (6, 256), (3, 512)]  # (blocks, bottleneck width); output channels = 4 x width


def _he(rng, shape, fan_in):
    return (rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)).astype(np.float32)


def build(E, op, batch=128, image=224, classes=1000, dtype_name='BFLOAT16', seed=12, base=64, stages=None,
          round_fn=None, with_logits=False):
    """Returns (program, weights) where weights is the list of host arrays in creation order.

    base scales every width (64 = the real network); stages overrides the (blocks, width) list;
    round_fn maps fp32 arrays to the values representable in dtype_name (identity for FLOAT32);
    with_logits adds the values before the softmax as a second program output.
    """
    dt = getattr(E.DType, dtype_name)
    round_fn = round_fn or (lambda a: a)
    stages = stages or [(n, w * base // 64) for n, w in STAGES]
    layer = [0]
    weights = []
    flops = [0.0]

    def constant(arr):
        arr = round_fn(arr)
        weights.append(arr)
        return E.Constant(arr, dt)

    def conv(x, kh, ci, co, stride=1, autopad=op.SAME_UPPER, pad=None, bias_scale=0.0):
        rng = np.random.default_rng(seed + layer[0])
        layer[0] += 1
        W = constant(_he(rng, (kh, kh, ci, co), kh * kh * ci))
        b = constant((rng.standard_normal(co) * bias_scale).astype(np.float32))
        y = op.convolution(x, W, strides=[stride, stride], autopad=autopad, manual_padding=pad)
        flops[0] += 2.0 * np.prod(y.shape) * kh * kh * ci  # full box; edge taps are discounted by the planner
        return y + b

    X = E.Placeholder(dt, [batch, image, image, 3])
    x = op.relu(conv(X, 7, 3, stages[0][1], stride=2, autopad=op.EXPLICIT, pad=[3, 3]))
    x = op.pool(x, 'max', [3, 3], [2, 2], autopad=op.EXPLICIT, manual_padding=[1, 1])
    ci = stages[0][1]
    for si, (blocks, width) in enumerate(stages):
        for bi in range(blocks):
            stride = 2 if (bi == 0 and si > 0) else 1
            y = op.relu(conv(x, 1, ci, width, autopad=op.VALID))
            y = op.relu(conv(y, 3, width, width, stride=stride))
            y = conv(y, 1, width, 4 * width, autopad=op.VALID)
            if bi == 0:
                y = y + conv(x, 1, ci, 4 * width, stride=stride, autopad=op.VALID)
            else:
                y = y + x
            x = op.relu(y)
            ci = 4 * width
    x = op.mean(x, axes=[1, 2])
    rng = np.random.default_rng(seed + 1000)
    Wd = constant(_he(rng, (ci, classes), ci))
    bd = constant(np.zeros(classes, np.float32))
    logits = op.dot(x, Wd) + bd
    flops[0] += 2.0 * batch * ci * classes
    probs = op.softmax(logits, axis=1)
    program = E.Program('resnet50_v1_5', [X], [probs, logits] if with_logits else [probs])
    return program, weights, flops[0]
