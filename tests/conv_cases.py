"""Convolution beyond the NXC / XCK forward form: the other tensor layouts, dilations and data dilations, the
four group layouts, and the two derivative modes (DATA is the transposed convolution).  Expected values come from
a direct numpy evaluation of the definition on zero-dilated, zero-padded data (np_conv) and, for the derivative
modes, from the adjoint identities  <conv(I, F), O> = <I, conv_data(O, F)> = <F, conv_filter(I, O)>  evaluated
element by element through linearity."""
import numpy as np


def _rng(seed=5):
    return np.random.default_rng(seed)


def same_pad(in_size, f_eff, stride, lower=False):
    out = -(-in_size // stride)
    return (max(0, (out - 1) * stride + f_eff - in_size) + (1 if lower else 0)) // 2, out


def np_conv(x, f, strides, dilations, data_dilations, pad_before, out_sizes, groups=1):
    """x [N, H, W, CI], f [KH, KW, CI / G, CO] with the output channels of group g at g * CO/G ...; float64."""
    n, h, w, ci = x.shape
    kh, kw, cig, co = f.shape
    cog = co // groups
    dh, dw = data_dilations
    xd = np.zeros((n, (h - 1) * dh + 1, (w - 1) * dw + 1, ci))
    xd[:, ::dh, ::dw, :] = x
    oh, ow = out_sizes
    need_h = (oh - 1) * strides[0] + (kh - 1) * dilations[0] + 1
    need_w = (ow - 1) * strides[1] + (kw - 1) * dilations[1] + 1
    xp = np.zeros((n, pad_before[0] + max(need_h, xd.shape[1]) + 1, pad_before[1] + max(need_w, xd.shape[2]) + 1, ci))
    xp[:, pad_before[0]:pad_before[0] + xd.shape[1], pad_before[1]:pad_before[1] + xd.shape[2], :] = xd
    out = np.zeros((n, oh, ow, co))
    for a in range(kh):
        for b in range(kw):
            win = xp[:, a * dilations[0]:a * dilations[0] + (oh - 1) * strides[0] + 1:strides[0],
                     b * dilations[1]:b * dilations[1] + (ow - 1) * strides[1] + 1:strides[1], :]
            for g in range(groups):
                out[..., g * cog:(g + 1) * cog] += win[..., g * cig:(g + 1) * cig] @ f[a, b, :, g * cog:(g + 1) * cog]
    return out


def _f32(E, shape):
    return E.Placeholder(E.DType.FLOAT32, list(shape))


def dilated_strided_ncx_kcx(E, op):
    """NCX data with KCX filters, stride 2, dilation 2, explicit padding (1, 2) before and (2, 0) after."""
    r = _rng(1)
    x = r.standard_normal((2, 9, 11, 3)).astype(np.float32)
    f = r.standard_normal((3, 2, 3, 4)).astype(np.float32)
    oh = (9 + 1 + 2 - 5 + 2) // 2
    ow = (11 + 2 + 0 - 3 + 2) // 2
    ref = np_conv(x.astype(np.float64), f.astype(np.float64), (2, 2), (2, 2), (1, 1), (1, 2), (oh, ow))
    X, F = _f32(E, (2, 3, 9, 11)), _f32(E, (4, 3, 3, 2))
    O = op.convolution(X, F, strides=[2, 2], dilations=[2, 2], autopad=op.EXPLICIT, manual_padding=[1, 2, 2, 0],
                       input_layout=op.LAYOUT_NCX, filter_layout=op.LAYOUT_KCX)
    return E.Program('conv', [X, F], [O]), [x.transpose(0, 3, 1, 2).copy(), f.transpose(3, 2, 0, 1).copy()], [ref.transpose(0, 3, 1, 2)]


def data_dilation(E, op):
    """Input seen through a zero-stuffing of 2 (fractionally strided convolution), SAME_LOWER padding."""
    r = _rng(2)
    x = r.standard_normal((1, 5, 4, 3)).astype(np.float32)
    f = r.standard_normal((4, 3, 3, 2)).astype(np.float32)
    ph, oh = same_pad(9, 4, 1, True)
    pw, ow = same_pad(7, 3, 1, True)
    ref = np_conv(x.astype(np.float64), f.astype(np.float64), (1, 1), (1, 1), (2, 2), (ph, pw), (oh, ow))
    X, F = _f32(E, x.shape), _f32(E, f.shape)
    O = op.convolution(X, F, data_dilations=[2, 2], autopad=op.SAME_LOWER)
    return E.Program('conv', [X, F], [O]), [x, f], [ref]


def _grouped(E, op, group_layout, filter_layout, depthwise=False):
    r = _rng(3)
    G = 6 if depthwise else 3
    CI, CO = 6, 12
    x = r.standard_normal((2, 7, 6, CI)).astype(np.float32)
    fs = r.standard_normal((3, 3, CI // G, CO)).astype(np.float32)   # standard form: [k, k, CI/G, CO]
    ph, oh = same_pad(7, 3, 2)
    pw, ow = same_pad(6, 3, 2)
    ref = np_conv(x.astype(np.float64), fs.astype(np.float64), (2, 2), (1, 1), (1, 1), (ph, pw), (oh, ow), G)
    cig, cog = CI // G, CO // G
    per_group = fs.reshape(3, 3, cig, G, cog).transpose(0, 1, 3, 2, 4)          # [k, k, G, CI/G, CO/G]
    if group_layout == op.GROUP_IN_C:
        f = per_group.reshape(3, 3, CI, cog)                                      # F[k, k, g*CI/G + ci, co]
    elif group_layout == op.GROUP_IN_K:
        f = fs                                                                    # F[k, k, ci, g*CO/G + co]
    elif filter_layout == op.LAYOUT_XGCK:
        f = per_group
    else:
        f = per_group.transpose(2, 4, 3, 0, 1)                                    # GKCX
    f = np.ascontiguousarray(f)
    X, F = _f32(E, x.shape), _f32(E, f.shape)
    O = op.convolution(X, F, strides=[2, 2], groups=1 if depthwise else G, filter_layout=filter_layout, group_layout=group_layout,
                       autogroup_mode=op.AUTOGROUP_DEPTHWISE if depthwise else op.AUTOGROUP_EXPLICIT)
    return E.Program('conv', [X, F], [O]), [x, f], [ref]


def grouped_in_c(E, op):
    return _grouped(E, op, op.GROUP_IN_C, op.LAYOUT_XCK)


def grouped_in_k(E, op):
    return _grouped(E, op, op.GROUP_IN_K, op.LAYOUT_XCK)


def grouped_separate_xgck(E, op):
    return _grouped(E, op, op.GROUP_SEPARATE, op.LAYOUT_XGCK)


def grouped_separate_gkcx(E, op):
    return _grouped(E, op, op.GROUP_SEPARATE, op.LAYOUT_GKCX)


def depthwise_in_k(E, op):
    return _grouped(E, op, op.GROUP_IN_K, op.LAYOUT_XCK, depthwise=True)


def depthwise_separate(E, op):
    return _grouped(E, op, op.GROUP_SEPARATE, op.LAYOUT_XGCK, depthwise=True)


def auto_separate(E, op):
    """AutoGroupMode AUTO: the group count is read off the filter tensor's own group dimension."""
    p, ins, ref = _grouped(E, op, op.GROUP_SEPARATE, op.LAYOUT_XGCK)
    x, f = ins
    X, F = _f32(E, x.shape), _f32(E, f.shape)
    O = op.convolution(X, F, strides=[2, 2], filter_layout=op.LAYOUT_XGCK, group_layout=op.GROUP_SEPARATE,
                       autogroup_mode=op.AUTOGROUP_AUTO)
    return E.Program('conv', [X, F], [O]), ins, ref


def _deriv_setup(seed, stride, dilation, autopad_name):
    r = _rng(seed)
    x = r.standard_normal((2, 8, 7, 3)).astype(np.float32)
    f = r.standard_normal((3, 2, 3, 4)).astype(np.float32)
    fe = ((3 - 1) * dilation + 1, (2 - 1) * dilation + 1)
    if autopad_name == 'valid':
        pads, outs = (0, 0), tuple((s - e + stride) // stride for s, e in zip((8, 7), fe))
    else:
        (ph, oh), (pw, ow) = same_pad(8, fe[0], stride), same_pad(7, fe[1], stride)
        pads, outs = (ph, pw), (oh, ow)
    o = r.standard_normal((2,) + outs + (4,)).astype(np.float32)
    return x, f, o, pads, outs


def _adjoint(x, f, o, stride, dilation, pads, outs, wrt):
    """Gradient of <conv(I, F), O> with respect to I or F, one element at a time through linearity."""
    x64, f64, o64 = x.astype(np.float64), f.astype(np.float64), o.astype(np.float64)
    target = x64 if wrt == 'data' else f64
    grad = np.zeros_like(target)
    for idx in np.ndindex(target.shape):
        e = np.zeros_like(target)
        e[idx] = 1.0
        y = np_conv(e if wrt == 'data' else x64, f64 if wrt == 'data' else e, (stride, stride), (dilation, dilation), (1, 1), pads, outs)
        grad[idx] = (y * o64).sum()
    return grad


def _deriv_data(E, op, seed, stride, dilation, autopad_name):
    x, f, o, pads, outs = _deriv_setup(seed, stride, dilation, autopad_name)
    ref = _adjoint(x, f, o, stride, dilation, pads, outs, 'data')
    Ot, F = _f32(E, o.shape), _f32(E, f.shape)
    R = op.convolution(Ot, F, strides=[stride] * 2, dilations=[dilation] * 2, autopad=getattr(op, autopad_name.upper()),
                       deriv_mode=op.DERIV_DATA, result_shape=[8, 7])
    return E.Program('conv_data', [Ot, F], [R]), [o, f], [ref]


def deriv_data_same_stride2(E, op):
    return _deriv_data(E, op, 11, 2, 1, 'same_upper')


def deriv_data_valid_dilated(E, op):
    return _deriv_data(E, op, 12, 1, 2, 'valid')


def _deriv_filter(E, op, seed, stride, dilation, autopad_name):
    x, f, o, pads, outs = _deriv_setup(seed, stride, dilation, autopad_name)
    ref = _adjoint(x, f, o, stride, dilation, pads, outs, 'filter')
    X, Ot = _f32(E, x.shape), _f32(E, o.shape)
    R = op.convolution(X, Ot, strides=[stride] * 2, dilations=[dilation] * 2, autopad=getattr(op, autopad_name.upper()),
                       deriv_mode=op.DERIV_FILTER, result_shape=[3, 2])
    return E.Program('conv_filter', [X, Ot], [R]), [x, o], [ref]


def deriv_filter_same_stride2(E, op):
    return _deriv_filter(E, op, 13, 2, 1, 'same_upper')


def deriv_filter_valid_dilated(E, op):
    return _deriv_filter(E, op, 14, 1, 2, 'valid')


def deriv_data_inferred_shape(E, op):
    """Without result_shape the smallest input that yields the given output is assumed: out*s + F_eff - s (VALID)."""
    r = _rng(15)
    o = r.standard_normal((1, 3, 4, 2)).astype(np.float32)
    f = r.standard_normal((3, 3, 5, 2)).astype(np.float32)
    h, w = 3 * 2 + 3 - 2, 4 * 2 + 3 - 2
    x0 = np.zeros((1, h, w, 5), np.float32)
    ref = _adjoint(x0, f, o, 2, 1, (0, 0), (3, 4), 'data')
    Ot, F = _f32(E, o.shape), _f32(E, f.shape)
    R = op.convolution(Ot, F, strides=[2, 2], autopad=op.VALID, deriv_mode=op.DERIV_DATA, infer_result_shape=True)
    return E.Program('conv_data', [Ot, F], [R]), [o, f], [ref]


CASES = {f.__name__: f for f in (
    dilated_strided_ncx_kcx, data_dilation, grouped_in_c, grouped_in_k, grouped_separate_xgck, grouped_separate_gkcx,
    depthwise_in_k, depthwise_separate, auto_separate, deriv_data_same_stride2, deriv_data_valid_dilated,
    deriv_filter_same_stride2, deriv_filter_valid_dilated, deriv_data_inferred_shape)}
