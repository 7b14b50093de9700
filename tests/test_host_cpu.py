"""Host-side logic that needs no GPU: building programs through the plaidml_* C ABI, shape / dtype
inference, error texts, bounds, and the kernel plan the `hip` target chooses."""
import numpy as np
import pytest

import programs
from oracle import tile_oracle as OE
from oracle import tile_oplib as Oop
from plaidml_amd import edsl as E
from plaidml_amd import op

D = E.DType


def plan_of(program, target=''):
    program.compile(target)
    return dict(program.passes)['hip-plan']


@pytest.mark.parametrize('name', sorted(programs.ALL))
def test_shapes_and_dtypes_match_the_oracle(name):
    prog, vals, _ = programs.ALL[name](E, op)
    oprog, ovals, _ = programs.ALL[name](OE, Oop)
    outs = OE.run(oprog, ovals)
    shapes = prog.outputs
    assert len(shapes) == len(outs)
    for s, o, ot in zip(shapes, outs, oprog.outputs):
        assert tuple(s.sizes) == tuple(o.shape), name
        assert int(s.dtype) == int(ot.dt), name
    text = plan_of(prog)
    assert text.startswith('hip plan:')


def test_plan_choices_for_the_workload_configs():
    t = plan_of(programs.config0_gemm_f32(E, op)[0])
    assert 'gemm f32 m=128 n=128 k=128' in t and t.count('\n') == 2
    t = plan_of(programs.config1_conv(E, op, 'BFLOAT16')[0])
    assert 'conv2d bf16' in t and '+init' in t and 'tail=[relu]' in t and t.count('\n') == 2
    t = plan_of(programs.config2_int8_gemm(E, op)[0])
    # int8 MFMA on the un-cast operands, si32 result stored mid-tail, requantisation fused
    assert 'gemm si8' in t and 'store' in t and 'cast:si8' in t and t.count('\n') == 2, t
    t = plan_of(programs.config3_xception_block(E, op)[0])
    assert 'dwconv2d bf16' in t and 'gemm bf16' in t and 'pool2d max' in t and '+window argmax' in t, t
    assert 'contract (general)' not in t
    t = plan_of(programs.residual_block(E, op)[0])
    assert t.count('conv2d bf16') + t.count('gemm bf16') == 2 and 'constant' in t and 'add(t' in t, t


def test_depthwise_temporary_gets_a_pitch_of_whole_lines():
    """728 bf16 channels are 1456 bytes: the depthwise result that only the pointwise product reads is laid out with
    768 elements per pixel; 64 channels (128 bytes) need nothing, and a depthwise result that is a program output
    keeps its dense layout."""
    t = plan_of(programs.config3_xception_block(E, op, N=2, C=728)[0])
    assert '(row pitch 768)' in t and '(lda 768)' in t, t
    t = plan_of(programs.config3_xception_block(E, op, N=2, C=64)[0])
    assert 'row pitch' not in t and 'lda' not in t, t
    dt = E.DType.BFLOAT16
    I, F = E.Placeholder(dt, [1, 9, 9, 328]), E.Placeholder(dt, [3, 3, 328, 1])
    t = plan_of(E.Program('dw', [I, F], [op.convolution(I, F, depthwise=True)]))
    assert 'dwconv2d' in t and 'row pitch' not in t, t
    t = plan_of(programs.config3_xception_block(E, op, N=2, C=728)[0], 'hip{specialise=0}')
    assert 'row pitch' not in t


def test_output_coordinates_that_are_sums_are_solved_for_one_index():
    """O[n, 2x + i - 1, 2y + j - 1, co]: the planner solves each such coordinate for its widest index (x, y), so the
    kernel's threads walk the taps and input channels only -- 7 indices (4 output coordinates + i, j, ci), not 11;
    an output access with a fraction keeps the full enumeration."""
    t = plan_of(programs.scatter_form_transposed_conv(E, op)[0])
    assert 'contract (general) add/mul idx=7 out_idx=4 (output enumerated per element; solved for' in t, t
    solved = t.split('solved for ')[1].split(')')[0].split()
    assert len(solved) == 4, t  # n and co trivially, x and y from the sums
    t = plan_of(programs.flatten_by_contraction(E, op)[0])
    assert 'idx=2 out_idx=1 (output enumerated per element; solved for' in t, t
    t = plan_of(programs.mirrored_sum_of_indices(E, op)[0])
    assert 'idx=3 out_idx=2 (output enumerated per element; solved for' in t, t
    A = E.Placeholder(D.FLOAT32, [8])
    i, j = E.TensorIndexes(2)
    O = E.Contraction().outShape(8).outAccess((i + j) // 2).sum(A[i] * A[j]).build()
    t = plan_of(E.Program('halved', [A], [O]))
    assert 'idx=3 out_idx=1 (output enumerated per element)' in t, t


def test_one_image_keeps_the_window_kernels():
    """At batch 1 the batch index is a constant; depthwise, pooling, window argmax and the pooling over the whole
    image must still be matched (the reference tool benchmarks at batch 1 by default)."""
    t = plan_of(programs.config3_xception_block(E, op, N=1)[0])
    assert 'dwconv2d bf16' in t and 'pool2d max' in t and '+window argmax' in t and 'contract (general)' not in t, t
    t = plan_of(programs.classifier_tail(E, op, N=1, dtype_name='BFLOAT16')[0])
    assert 'pool2d add bf16 1x7x7x64xbf16 over the whole image' in t, t


def test_softmax_is_one_launch():
    """The op library's softmax (max, sub, exp, sum, div) is recognised as a whole when nothing else reads its
    intermediate values; an intermediate that is also a program output keeps the five operations apart."""
    X = E.Placeholder(E.DType.BFLOAT16, [4, 1000])
    t = plan_of(E.Program('sm', [X], [op.softmax(X, axis=1)]))
    assert 'hip plan: 1 launches' in t and 'softmax bf16 over the last axis of 4x1000xbf16' in t, t
    X = E.Placeholder(E.DType.FLOAT32, [2, 3, 10])
    t = plan_of(E.Program('sm3', [X], [op.softmax(X, axis=2)]))
    assert 'hip plan: 1 launches' in t and 'softmax f32' in t, t
    X = E.Placeholder(E.DType.FLOAT32, [4, 10])
    i, j = E.TensorIndexes(2)
    M = E.Contraction().outShape(4, 1).outAccess(i, 0).max(X[i, j]).build()
    Ex = E.exp(X - M)
    S = E.Contraction().outShape(4, 1).outAccess(i, 0).sum(Ex[i, j]).build()
    t = plan_of(E.Program('sm_visible', [X], [Ex / S, Ex]))
    assert 'softmax' not in t and 'hip plan: 4 launches' in t, t
    X = E.Placeholder(E.DType.BFLOAT16, [4, 1000])
    prog = E.Program('sm', [X], [op.softmax(X, axis=1)])
    prog.compile('hip{fuse=0}')
    assert 'softmax' not in dict(prog.passes)['hip-plan']


def test_mean_over_the_image_is_one_launch():
    """mean = sum / count: the division by the literal rides in the launch that sums whole images (49 pixels: the
    kernel that shares an image's taps among threads); a 3x3 image (the plain window kernel) keeps it apart, and so
    does `fuse=0`."""
    def program(h):
        X = E.Placeholder(E.DType.BFLOAT16, [2, h, h, 64])
        return E.Program('mean', [X], [op.mean(X, axes=[1, 2])])
    t = plan_of(program(7))
    assert 'over the whole image tail=[div(49)]' in t and 'hip plan: 1 launches' in t, t
    t = plan_of(program(3))
    assert 'hip plan: 2 launches' in t and 'eltwise div' in t, t
    prog = program(7)
    prog.compile('hip{fuse=0}')
    t = dict(prog.passes)['hip-plan']
    assert 'hip plan: 2 launches' in t, t


def test_stem_convolution_pools_inside_its_launch():
    """relu(conv 7x7x3 stride 2 + b) followed by a 3x3 stride-2 max-pool that alone reads it: the pooling step goes and
    the convolution writes the pooled tensor (the kernel library is asked first).  Not when the convolution's result is
    also a program output, not with a window argmax beside the pool, not under `fuse=0` or a program-wide `conv=`."""
    bf = E.DType.BFLOAT16
    def program(also_output=False):
        X = E.Placeholder(bf, [2, 64, 64, 3])
        F = E.Constant(np.zeros((7, 7, 3, 64), np.float32), bf)
        B = E.Constant(np.zeros(64, np.float32), bf)
        C = op.relu(op.convolution(X, F, strides=[2, 2], autopad=op.SAME_UPPER) + B)
        M = op.pool(C, 'max', [3, 3], [2, 2], autopad=op.SAME_UPPER)
        return E.Program('stem', [X], [M, C] if also_output else [M])
    t = plan_of(program())
    assert 'hip plan: 1 launches' in t and '+ max-pool 3x3 stride 2 -> 2x16x16x64xbf16' in t, t
    t = plan_of(program(also_output=True))
    assert 'hip plan: 2 launches' in t and 'max-pool 3x3 stride 2' not in t, t
    for target in ('hip{fuse=0}', 'hip{conv=igemm}'):
        prog = program()
        prog.compile(target)
        t = dict(prog.passes)['hip-plan']
        assert 'max-pool 3x3 stride 2' not in t and 'pool2d max' in t, t


def test_projection_shortcut_and_main_path_share_one_launch():
    """relu(conv1x1(y) + b + conv1x1(x) + b') of a residual block with a projection shortcut is one GEMM with two
    products (plain rows, or the pixel rows of the stride-2 shortcut); `fuse=0` keeps the contractions apart."""
    prog = programs.resnet50_tiny(E, op)[0]
    t = plan_of(prog)
    assert t.count('+ second product') == 4 and t.count('pixel rows of a 1x1 convolution, stride 2') == 2, t
    assert '+init +init2 tail=[relu]' in t
    prog = programs.resnet50_tiny(E, op)[0]
    assert 'second product' not in plan_of(prog, 'hip{fuse=0}')


def test_operand_of_two_gib_takes_the_general_kernel():
    """The matrix-core kernels address an operand with 32-bit byte offsets; a contraction over a larger one must
    be planned onto the general kernel at compile time instead of failing at every run."""
    A = E.Placeholder(D.FLOAT32, [32768, 16384], name='A')      # exactly 2 GiB
    B = E.Placeholder(D.FLOAT32, [16384, 8], name='B')
    t = plan_of(E.Program('big_dot', [A, B], [op.dot(A, B)]))
    assert 'contract (general)' in t and 'gemm' not in t, t
    A = E.Placeholder(D.FLOAT32, [32768, 8192], name='A')       # 1 GiB: the GEMM kernel
    B = E.Placeholder(D.FLOAT32, [8192, 8], name='B')
    assert 'gemm f32' in plan_of(E.Program('dot', [A, B], [op.dot(A, B)]))


def test_target_option_fp32_as_three_bf16_products():
    prog = programs.config1_conv(E, op, 'FLOAT32')[0]
    assert 'as 3 bf16 products' not in plan_of(prog)
    prog = programs.config1_conv(E, op, 'FLOAT32')[0]
    assert 'conv2d f32 (as 3 bf16 products)' in plan_of(prog, 'hip{fp32=bf16x3}')
    prog = programs.config1_conv(E, op, 'BFLOAT16')[0]
    assert 'as 3 bf16 products' not in plan_of(prog, 'hip{fp32=bf16x3}')   # bf16 programs are not touched
    prog = programs.config0_gemm_f32(E, op)[0]
    assert 'gemm f32 (as 3 bf16 products)' in plan_of(prog, 'hip{fp32=bf16x3}')
    with pytest.raises(E.PlaidMLError, match='Invalid target option fp32'):
        programs.config0_gemm_f32(E, op)[0].compile('hip{fp32=tf32}')


def test_schedule_overrides_by_option_and_by_file(tmp_path, monkeypatch):
    """Tiling overrides: `hip{tile=...,conv=...}` for a whole program, a schedule file for single steps (the reference
    loads one from PLAIDML_SCHEDULE_PATH, pmlc/target/x86/pipeline.cc:267-272).  The plan dump shows the override and
    an edited dump is itself a schedule file."""
    from plaidml_amd import hipkernels as hk
    L = hk.lib()
    for t, name in enumerate(hk.TILE_NAMES):  # the Python names are the library's
        assert L.pml_hip_tile_name(t) == name.encode() and L.pml_hip_tile_by_name(name.encode()) == t
    assert L.pml_hip_tile_name(len(hk.TILE_NAMES)) is None and L.pml_hip_tile_by_name(b'1x1') == -1
    plain = plan_of(programs.residual_block(E, op)[0])
    assert '{' not in plain
    t = plan_of(programs.residual_block(E, op)[0], 'hip{tile=128x128w8,conv=igemm}')
    for a, b in zip(plain.splitlines()[1:], t.splitlines()[1:]):
        if 'conv2d' in a:
            assert b == a + ' {tile=128x128w8,conv=igemm}'
        elif 'gemm' in a:
            assert b == a + ' {tile=128x128w8}'
        else:
            assert b == a
    with pytest.raises(E.PlaidMLError, match="Invalid tile '3x3'"):
        programs.residual_block(E, op)[0].compile('hip{tile=3x3}')
    with pytest.raises(E.PlaidMLError, match="Invalid convolution path"):
        programs.residual_block(E, op)[0].compile('hip{conv=winograd}')
    # a schedule file: the plain dump with one step's line marked
    lines = plain.splitlines()
    k = next(i for i, l in enumerate(lines) if 'gemm' in l or 'conv2d' in l)
    lines[k] += ' {tile=64x64}'
    sched = tmp_path / 'schedule.txt'
    sched.write_text('\n'.join(lines) + '\n')
    monkeypatch.setenv('PLAIDML_SCHEDULE_PATH', str(sched))
    t = plan_of(programs.residual_block(E, op)[0])
    assert t.splitlines() == lines          # only that step changed, and the dump reproduces the file
    t2 = plan_of(programs.residual_block(E, op)[0], 'hip{tile=128x64}')   # the file's entry wins over the program-wide option
    assert t2.splitlines()[k] == lines[k] and t2.count('{tile=128x64}') >= 1
    monkeypatch.setenv('PLAIDML_SCHEDULE_PATH', str(tmp_path / 'missing.txt'))
    with pytest.raises(E.PlaidMLError, match='Cannot read the schedule file'):
        programs.residual_block(E, op)[0].compile('')


def test_target_options_switch_specialisation_off():
    prog = programs.config1_conv(E, op, 'BFLOAT16')[0]
    t = plan_of(prog, 'hip{specialise=0,fuse=0}')
    assert 'contract (general)' in t and 'conv2d' not in t
    with pytest.raises(E.PlaidMLError, match='Could not find compiler target'):
        prog.compile('llvm_cpu')


def test_tensor_shape_strings_and_dtype_inference():
    # plaidml/core/core_test.py / pmlc/util/shape.cc:69-91
    assert str(E.TensorShape(D.FLOAT32, [8, 32])) == '8x32xf32'
    assert str(E.TensorShape(D.INT8, [])) == 'si8'
    assert str(E.TensorShape(D.BFLOAT16, [4])) == '4xbf16'
    A = E.Placeholder(D.INT8, [3, 3])
    B = E.Placeholder(D.INT8, [3, 3])
    i, j, k = E.TensorIndexes(3)
    C = E.Contraction().outShape(3, 3).outAccess(i, j).sum(A[i, k] * B[k, j]).build()
    assert C.dtype == D.INT8  # no widening: plaidml/edsl/tests/edsl_test.cc:1195-1208
    F = E.Placeholder(D.FLOAT32, [3, 3])
    assert (F + E.cast(E.Constant(1), D.UINT64)).dtype == D.FLOAT32
    assert (F + E.cast(E.Constant(2.0), D.FLOAT64)).dtype == D.FLOAT64
    assert (F < 1.0).dtype == D.BOOLEAN
    assert E.index([3, 4], 1).dtype == D.INT32 and E.index([3, 4], 1).shape == (3, 4)


def test_error_texts():
    A = E.Placeholder(D.FLOAT32, [3, 4])
    with pytest.raises(E.PlaidMLError, match='Rank mismatch in bind_dims'):
        A.bind_dims(*E.TensorDims(3))
    X, Y = E.TensorDim(5), E.TensorDim()
    with pytest.raises(E.PlaidMLError, match=r'bind dims mismatch: shape=\[3, 4\] != dims=\[5, 4\]'):
        A.bind_dims(X, Y)
    with pytest.raises(E.PlaidMLError, match='Incompatible types'):
        A + E.Placeholder(D.FLOAT32, [5])
    i, = E.TensorIndexes(1)
    with pytest.raises(E.PlaidMLError, match='ambiguous'):
        E.Contraction().outShape(3).outAccess(i).sum(E.Constant(1)[()] * E.Constant(2)[()]).build()
    with pytest.raises(E.PlaidMLError, match='unmatched operand types'):
        E.select(A < 0.0, A, E.cast(A, D.FLOAT64))
    k, = E.TensorIndexes(1)
    P = E.Program('unbounded', [A], [E.Contraction().outShape(3).outAccess(i - k).sum(A[i - k, 0]).build()])
    with pytest.raises(E.PlaidMLError, match="Unbounded index"):
        P.compile()


def test_bounds_of_same_conv_and_pool():
    prog = programs.config1_conv(E, op, 'FLOAT32', N=1, H=5, W=5, CI=32, CO=48)[0]
    prog.compile()
    text = dict(prog.passes)['tile-compute-bounds']
    # n, x0, x1, co, k0, k1, ci (first-seen order over sink, sources): pmlc/ast/builder.cc:311-323
    assert 'idxs = [n, x0, x1, co, k0, k1, ci]' in text
    assert 'lowerBounds = (0, 0, 0, 0, 0, 0, 0), upperBounds = (0, 4, 4, 47, 2, 2, 31)' in text
    assert 'x0 + k0 - 1' in text


def test_run_without_a_device_fails_loudly():
    if E.list_devices():
        pytest.skip('a GPU is present')
    prog = programs.dot_f32(E, op)[0]
    prog.compile()
    with pytest.raises(E.PlaidMLError, match='Unable to find hip runtime'):
        E.Executable(prog)
    with pytest.raises(E.PlaidMLError, match='Invalid device name'):
        E.Executable(prog, 'not a device')


def test_cpp_cases_fail_loudly_without_a_device():
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'cpp', 'edsl_cases')
    if not os.path.exists(exe):
        pytest.skip('tests/cpp/edsl_cases is built by __graft_entry__.build()')
    import torch
    if torch.cuda.is_available():
        pytest.skip('a GPU is present')
    res = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert res.returncode != 0
    assert 'hip' in res.stderr.lower()


def test_placeholder_shapes_and_collected_passes():
    """test_placeholder and test_collect_passes, plaidml/edsl/tests/edsl_test.py:534-571."""
    from plaidml_amd import edsl as E, op
    assert str(E.Placeholder(E.DType.INT32).compute_shape()) == 'si32'
    assert str(E.Placeholder(E.DType.INT32, [1, 1]).compute_shape()) == '1x1xsi32'
    assert str(E.Placeholder(E.DType.INT32, [1, 1], name='I').compute_shape()) == '1x1xsi32'
    A, B = E.Placeholder(E.DType.FLOAT32, [10, 10]), E.Placeholder(E.DType.FLOAT32, [10, 10])
    program = E.Program('collect_passes', [A, B], [op.dot(A, B)])
    program.compile(debug=True)
    assert program.passes[0][0] == 'tile'


def test_lens_rejects_mismatched_layouts():
    """TensorLens, plaidml/edsl/__init__.py:292-309."""
    from plaidml_amd import edsl as E
    with pytest.raises(ValueError):
        E.TensorLens('NHWC', 'NCH')
    with pytest.raises(ValueError):
        E.TensorLens('NHWC', 'NCHX')
    assert E.TensorLens('NCHW', 'NHWC').apply(list('abcd')) == ['a', 'd', 'b', 'c']
    with pytest.raises(ValueError):
        E.TensorLens('MN', 'MN').apply([1, 2, 3])
