"""plaidml::op::nms: the oracle against a loop-written greedy suppression (CPU), the device against the oracle."""
import numpy as np
import pytest

import nms_cases
from oracle import tile_oracle as OE, tile_oplib as Oop


def _run_oracle(name):
    kw, iou_thr, score_thr, k, op_kw, greedy_kw = nms_cases.CASES[name]
    boxes, scores = nms_cases.inputs(**kw)
    prog, vals = nms_cases.build(OE, Oop, boxes, scores, iou_thr, score_thr, k, **op_kw)
    return OE.run(prog, vals), (boxes, scores, iou_thr, score_thr, k, greedy_kw)


@pytest.mark.parametrize('name', sorted(nms_cases.CASES))
def test_oracle_matches_greedy_suppression(name):
    (rb, rs, rv), (boxes, scores, iou_thr, score_thr, k, greedy_kw) = _run_oracle(name)
    found = nms_cases.greedy(boxes, scores, iou_thr, score_thr, k, **greedy_kw)
    assert 0 < len(found) <= rb.shape[0]
    eb, es, ev = nms_cases.expected(found, rb.shape[0])
    np.testing.assert_array_equal(rb, eb)
    np.testing.assert_array_equal(rv.astype(np.int32), ev)
    np.testing.assert_array_equal(rs[:, :2], es[:, :2])
    np.testing.assert_allclose(rs[:, 2], es[:, 2], rtol=1e-6)


def test_some_rows_stay_unused():
    """A case is only telling if suppression removes something: the selections must not fill every row."""
    for name in ('ov_all_boxes', 'ov_high_score_threshold'):  # removed by overlap / by the score threshold
        (rb, _, rv), _ = _run_oracle(name)
        assert int(rv[0]) < rb.shape[0] and (rb[int(rv[0]):] == -1).all(), name


def test_argument_checks():
    from plaidml_amd import edsl as E, op
    boxes, scores = nms_cases.inputs(seed=1)
    with pytest.raises(E.PlaidMLError):
        nms_cases.build(E, op, boxes, scores, 0.3, 0.2, 3, nms_style=7)
    with pytest.raises(E.PlaidMLError):
        nms_cases.build(E, op, boxes, scores, 0.3, 0.2, 3, boxes_decode_mode=5)
    prog, _ = nms_cases.build(E, op, boxes, scores, 0.3, 0.2, 3)
    shapes = [tuple(s.sizes) for s in prog.output_shapes] if hasattr(prog, 'output_shapes') else None
    assert shapes is None or shapes == [(18, 3), (18, 3), (1,)]


def _ssd_case(E, op, with_arm, share, style):
    B, C, N = 1, 3, 6
    r = np.random.default_rng(17)
    lo = r.uniform(10, 60, (B, N, 2))
    priors = np.concatenate([lo, lo + r.uniform(10, 40, (B, N, 2))], -1).astype(np.float32)  # pixels of a 100 x 100 image
    L = 1 if share else C
    var = np.full((B, N, 4), 0.1, np.float32)
    loc = r.uniform(-0.5, 0.5, (B, L, N, 4)).astype(np.float32)
    arm = r.uniform(-0.3, 0.3, (B, L, N, 4)).astype(np.float32)
    scores = (r.permutation(B * C * N).reshape(B, C, N) / float(B * C * N) + 0.01).astype(np.float32)
    f32 = E.DType.FLOAT32
    Bx, Sc = E.Placeholder(f32, [B, N, 4]), E.Placeholder(f32, [B, C, N])
    It, St = E.Placeholder(f32, [1]), E.Placeholder(f32, [1])
    Va, Lo, Ar = E.Placeholder(f32, [B, N, 4]), E.Placeholder(f32, [B, L, N, 4]), E.Placeholder(f32, [B, L, N, 4])
    outs = op.nms(Bx, Sc, It, St, 3, boxes_decode_mode=1, ssd_input_height=100, ssd_input_width=100, ssd_variances=Va,
                  ssd_location=Lo, ssd_with_arm_loc=with_arm, ssd_arm_location=Ar if with_arm else None,
                  clip_before_nms=True, clip_after_nms=True, center_point_box=with_arm, share_location=share,
                  nms_style=style)
    ins, vals = [Bx, Sc, It, St, Va, Lo], [priors, scores, np.array([0.4], np.float32), np.array([0.1], np.float32), var, loc]
    if with_arm:
        ins.append(Ar)
        vals.append(arm)
    return E.Program('nms_ssd', ins, outs), vals


@pytest.mark.parametrize('with_arm,share,style', [(False, True, 2), (True, True, 2), (False, False, 2), (False, True, 1)])
def test_ssd_decoding_runs_in_the_oracle(with_arm, share, style):
    prog, vals = _ssd_case(OE, Oop, with_arm, share, style)
    rb, rs, rv = OE.run(prog, vals)
    assert rb.shape == (9, 3) and rs.shape == (9, 7) and 0 < int(rv[0]) <= 9
    live = rs[:int(rv[0]), 3:]
    assert ((live >= 0) & (live <= 1)).all()  # clipped corners of the selected boxes


@pytest.mark.gpu
@pytest.mark.parametrize('name', sorted(nms_cases.CASES))
def test_device_matches_oracle(name):
    from plaidml_amd import edsl as E, op
    print('nms case', name, flush=True)
    (rb, rs, rv), (boxes, scores, iou_thr, score_thr, k, _) = _run_oracle(name)
    prog, vals = nms_cases.build(E, op, boxes, scores, iou_thr, score_thr, k, **nms_cases.CASES[name][4])
    gb, gs, gv = E.run(prog, vals, target='hip')
    np.testing.assert_array_equal(gb, rb)
    np.testing.assert_array_equal(gv, rv)
    np.testing.assert_allclose(gs, rs, rtol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize('with_arm,share,style', [(False, True, 2), (True, True, 2), (False, False, 2), (False, True, 1)])
def test_device_matches_oracle_ssd(with_arm, share, style):
    from plaidml_amd import edsl as E, op
    print('nms ssd case', with_arm, share, style, flush=True)
    oprog, vals = _ssd_case(OE, Oop, with_arm, share, style)
    rb, rs, rv = OE.run(oprog, vals)
    prog, vals = _ssd_case(E, op, with_arm, share, style)
    gb, gs, gv = E.run(prog, vals, target='hip')
    np.testing.assert_array_equal(gb, rb)
    np.testing.assert_array_equal(gv, rv)
    np.testing.assert_allclose(gs, rs, rtol=1e-4, atol=1e-6)


# --- SSD box decoding (decode_boxes, plaidml/op/lib/ops.cc:2034-2117) pinned by hand-computed boxes -------------
# Two priors in pixels of a 100 (wide) x 200 (high) image, variances (0.1, 0.1, 0.2, 0.2).  The numbers below
# were worked out by hand from the reference's formulas, not produced by this repository's code:
#   centred form, prior (20, 30, 60, 50), location (1, -2, 0.5, -0.5):
#     normalised prior x 0.2 .. 0.6, y 0.15 .. 0.25 (x by the width, y by the height), size 0.4 x 0.1
#     centre x = 0.1 * 1 * 0.4 + 0.4 = 0.44, centre y = 0.1 * -2 * 0.1 + 0.2 = 0.18
#     half width = exp(0.2 * 0.5) * 0.4 / 2 = 0.2210342, half height = exp(0.2 * -0.5) * 0.1 / 2 = 0.0452419
#   centred form, location 0: the normalised prior itself
#   corner form: every coordinate is divided by the WIDTH (also y), then + variance * location
_SSD_PRIORS = np.array([[[[20, 30, 60, 50], [10, 10, 30, 90], [70, 20, 95, 40]]]], np.float32)
_SSD_VAR = np.array([[[[0.1, 0.1, 0.2, 0.2]] * 3]], np.float32)
_SSD_LOC = np.array([[[[1, -2, 0.5, -0.5], [0, 0, 0, 0], [-9, -3, 1, 2]]]], np.float32)
_SSD_WANT = {  # (centred, clip) -> rows of (y1, x1, y2, x2)
    (True, False): [[0.1347581, 0.2189658, 0.2252419, 0.6610342], [0.05, 0.1, 0.45, 0.3],
                    [0.12 - 0.0745912, 0.6 - 0.1526753, 0.12 + 0.0745912, 0.6 + 0.1526753]],
    (False, False): [[0.1, 0.3, 0.4, 0.7], [0.1, 0.1, 0.9, 0.3], [-0.1, -0.2, 0.8, 1.15]],
    (False, True): [[0.1, 0.3, 0.4, 0.7], [0.1, 0.1, 0.9, 0.3], [0.0, 0.0, 0.8, 1.0]],
}
# third prior, centred: x 0.7 .. 0.95 (size 0.25), y 0.1 .. 0.2 (size 0.1); centre x = 0.1 * -9 * 0.25 + 0.825 = 0.6,
# centre y = 0.1 * -3 * 0.1 + 0.15 = 0.12; half width exp(0.2) * 0.125 = 0.1526753, half height exp(0.4) * 0.05 = 0.0745912


@pytest.mark.parametrize('centered,clip', sorted(_SSD_WANT))
def test_ssd_box_decoding_hand_computed(centered, clip):
    f32 = OE.DType.FLOAT32
    Bx, Va, Lo = (OE.Placeholder(f32, [1, 1, 3, 4]) for _ in range(3))
    corners = Oop._box_corners(Bx, Va, Lo, Oop.BOXES_SSD, 200, 100, clip, centered)
    got = OE.run(OE.Program('decode', [Bx, Va, Lo], corners), [_SSD_PRIORS, _SSD_VAR, _SSD_LOC])
    got = np.stack([g.reshape(3) for g in got], axis=1)  # rows of (y1, x1, y2, x2)
    np.testing.assert_allclose(got, np.array(_SSD_WANT[(centered, clip)], np.float32), rtol=2e-6, atol=2e-7)


@pytest.mark.parametrize('with_arm,share,style', [(False, True, 2), (True, True, 2), (False, False, 2), (False, True, 1)])
def test_ssd_result_rows_carry_the_decoded_boxes(with_arm, share, style):
    """The four extra columns of the score rows are (x1, y1, x2, y2) of the selected box, decoded here box by box
    with scalar arithmetic (twice for the refined priors of the ARM variant) and clipped to the unit square."""
    prog, vals = _ssd_case(OE, Oop, with_arm, share, style)
    rb, rs, rv = OE.run(prog, vals)
    priors, var, loc = vals[0], vals[4], vals[5]
    arm = vals[6] if with_arm else None
    W = H = np.float32(100)
    f = np.float32

    def decode(box, v, l, centred):  # -> (x1, y1, x2, y2)
        if centred:
            x1, y1, x2, y2 = box[0] / W, box[1] / H, box[2] / W, box[3] / H
            pw, ph = x2 - x1, y2 - y1
            xc, yc = v[0] * l[0] * pw + (x1 + x2) / f(2), v[1] * l[1] * ph + (y1 + y2) / f(2)
            hw, hh = np.exp(v[2] * l[2]) * pw / f(2), np.exp(v[3] * l[3]) * ph / f(2)
            out = [xc - hw, yc - hh, xc + hw, yc + hh]
        else:
            out = [box[k] / W + v[k] * l[k] for k in range(4)]
        return [min(max(t, f(0)), f(1)) for t in out]  # clip_before_nms

    for row in range(int(rv[0])):
        b, c, j = (int(t) for t in rb[row])
        cls = c + 1 if style == 1 else c  # the MXNET style reports the class without the background id
        lc = 0 if share else cls
        if with_arm:
            refined = decode(priors[b, j], var[b, j], arm[b, lc, j], True)
            want = decode(refined, var[b, j], loc[b, lc, j], True)
        else:
            want = decode(priors[b, j], var[b, j], loc[b, lc, j], False)
        np.testing.assert_allclose(rs[row, 3:], np.array(want, np.float32), rtol=1e-5, atol=1e-6, err_msg=str((row, b, c, j)))
