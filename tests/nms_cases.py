"""Non-maximum suppression cases, built twice like tests/programs.py: with the oracle's op library and with
the product's.  The reference holds no test of plaidml::op::nms (plaidml/op/lib/ops.cc:2157-2417), so the
oracle's restatement is pinned here against an independent, loop-written greedy suppression -- the textbook
algorithm the operation unrolls -- for the NMS box formats and the three styles; the SSD box decoding is pinned
in tests/test_nms.py by hand-computed boxes."""
import numpy as np

CAFFE, MXNET, OV = range(3)


def inputs(seed, B=2, C=3, N=8, centered=False):
    r = np.random.default_rng(seed)
    ctr, size = r.uniform(0.2, 0.8, (B, N, 2)), r.uniform(0.1, 0.4, (B, N, 2))
    if centered:
        boxes = np.concatenate([ctr[..., ::-1], size[..., ::-1]], -1)  # x, y, width, height
    else:
        lo, hi = ctr - size / 2, ctr + size / 2
        flip = r.integers(0, 2, (B, N, 1)).astype(bool)  # either corner may come first
        boxes = np.concatenate([np.where(flip, hi, lo), np.where(flip, lo, hi)], -1)  # y, x, y, x
    scores = r.permutation(B * C * N).reshape(B, C, N) / float(B * C * N) + 0.01  # all different
    return boxes.astype(np.float32), scores.astype(np.float32)


def build(E, op, boxes, scores, iou_thr, score_thr, k, **kw):
    B, N, _ = boxes.shape
    C = scores.shape[1]
    Bx = E.Placeholder(E.DType.FLOAT32, [B, N, 4])
    Sc = E.Placeholder(E.DType.FLOAT32, [B, C, N])
    It = E.Placeholder(E.DType.FLOAT32, [1])
    St = E.Placeholder(E.DType.FLOAT32, [1])
    outs = op.nms(Bx, Sc, It, St, k, **kw)
    return E.Program('nms', [Bx, Sc, It, St], outs), [boxes, scores, np.array([iou_thr], np.float32),
                                                      np.array([score_thr], np.float32)]


def _edges(box, centered):
    if centered:
        x, y, w, h = (np.float32(v) for v in box)
        return y - h / np.float32(2), x - w / np.float32(2), y + h / np.float32(2), x + w / np.float32(2)
    return min(box[0], box[2]), min(box[1], box[3]), max(box[0], box[2]), max(box[1], box[3])


def _iou(a, b):
    ih = np.float32(min(a[2], b[2])) - np.float32(max(a[0], b[0]))
    iw = np.float32(min(a[3], b[3])) - np.float32(max(a[1], b[1]))
    inter = (ih if ih > 0 else np.float32(0)) * (iw if iw > 0 else np.float32(0))
    union = (a[2] - a[0]) * (a[3] - a[1]) + (b[2] - b[0]) * (b[3] - b[1]) - inter
    return inter * (np.float32(1) / union) if union > 0 else np.float32(0)


def greedy(boxes, scores, iou_thr, score_thr, k, style=OV, hard=True, sigma=0.0, centered=False, descending=False):
    """Loop-written suppression: [(batch, class, box, score)] in the order the operation reports them."""
    B, C, N = scores.shape
    per_class = min(N, k) if k else N
    s = np.where(scores > np.float32(score_thr), scores, np.float32(0)).astype(np.float32)
    if style == CAFFE:
        for b in range(B):
            for c in range(C):
                keep = np.argsort(-s[b, c], kind='stable')[:per_class]
                t = np.zeros(N, np.float32)
                t[keep] = s[b, c, keep]
                s[b, c] = t
    elif style == MXNET:
        for b in range(B):
            best_class, best = s[b].argmax(0), s[b].max(0)
            keep = np.argsort(-best, kind='stable')[:per_class]
            t = np.zeros((C, N), np.float32)
            t[best_class[keep], keep] = best[keep]
            s[b] = t
    found = []
    for b in range(B):
        e = [_edges(boxes[b, j], centered) for j in range(N)]
        for c in range(C):
            cur = s[b, c].copy()
            for _ in range(per_class):
                j = int(np.argmax(cur))
                if not cur[j] > 0:
                    break
                found.append((b, c, j, cur[j]))
                cur[j] = 0
                for m in range(N):
                    v = _iou(e[j], e[m])
                    if (v >= np.float32(iou_thr)) if hard else (v > np.float32(iou_thr)):
                        cur[m] = 0
                    elif sigma != 0:
                        cur[m] = cur[m] * np.exp(v * v * np.float32(-0.5 / sigma), dtype=np.float32)
                        if not cur[m] > np.float32(score_thr):
                            cur[m] = 0
    if descending:
        found.sort(key=lambda t: -t[3])
    return found


def expected(found, rows):
    boxes = -np.ones((rows, 3), np.int32)
    scores = -np.ones((rows, 3), np.float32)
    for i, (b, c, j, v) in enumerate(found):
        boxes[i] = (b, c, j)
        scores[i] = (b, c, v)
    return boxes, scores, np.array([len(found)], np.int32)


# name -> (input kwargs, iou threshold, score threshold, boxes per class, operation kwargs, greedy kwargs)
CASES = {
    'ov': (dict(seed=1), 0.3, 0.25, 4, {}, {}),
    'ov_all_boxes': (dict(seed=2, B=1, C=2, N=6), 0.1, 0.0, 0, {}, {}),
    'ov_strict_compare': (dict(seed=3), 0.2, 0.1, 3, dict(hard_suppression=False), dict(hard=False)),
    'ov_high_score_threshold': (dict(seed=4), 0.4, 0.8, 5, {}, {}),
    'ov_centered': (dict(seed=5, centered=True), 0.3, 0.2, 4, dict(center_point_box=True), dict(centered=True)),
    'ov_sorted': (dict(seed=6), 0.3, 0.3, 3, dict(sort_result_descending=True), dict(descending=True)),
    'ov_soft': (dict(seed=7), 0.6, 0.2, 4, dict(soft_nms_sigma=0.5), dict(sigma=0.5)),
    'caffe': (dict(seed=8), 0.3, 0.2, 3, dict(nms_style=CAFFE), dict(style=CAFFE)),
    'mxnet': (dict(seed=9), 0.3, 0.2, 4, dict(nms_style=MXNET), dict(style=MXNET)),
}
