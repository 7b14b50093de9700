"""Parity of whole Tile programs: built through the plaidml_* C ABI and run on the `hip` device,
against the CPU oracle on the same seeded inputs.

Bars (from this build's north-star statement): bit-exact for integer and index outputs, rtol 1e-3 for
fp32, rtol 2e-2 for bf16.  Each program also runs with `hip{specialise=0,fuse=0}` (every contraction
through the general kernel, every elementwise operation on its own), which must agree as well."""
import numpy as np
import pytest

import programs
from oracle import tile_oracle as OE
from oracle import tile_oplib as Oop
from plaidml_amd import edsl as E
from plaidml_amd import op

pytestmark = pytest.mark.gpu


def check(name, got, ref, tol):
    assert len(got) == len(ref)
    for k, (g, r) in enumerate(zip(got, ref)):
        assert g.shape == r.shape, (name, k)
        if tol == programs.EXACT or r.dtype.kind in 'iub':
            np.testing.assert_array_equal(g, r, err_msg='%s output %d' % (name, k))
        elif tol == programs.FP32:
            np.testing.assert_allclose(g, r, rtol=1e-3, atol=1e-5, err_msg='%s output %d' % (name, k))
        else:
            np.testing.assert_allclose(g, r, rtol=2e-2, atol=2e-2, err_msg='%s output %d' % (name, k))


@pytest.mark.parametrize('target', ['hip', 'hip{specialise=0,fuse=0}'])
@pytest.mark.parametrize('name', sorted(programs.ALL))
def test_program_matches_oracle(name, target):
    print('program', name, 'target', target, flush=True)
    oprog, ovals, tol = programs.ALL[name](OE, Oop)
    ref = OE.run(oprog, ovals)
    prog, vals, _ = programs.ALL[name](E, op)
    got = E.run(prog, vals, target=target)
    if name.startswith('config3') and tol == programs.BF16:
        # The pooled bf16 values may differ from the oracle's by one rounding step upstream, and with them the
        # winning tap.  Every index is therefore checked, bit for bit, against the device's own pool input (a
        # third program output); the comparison with the oracle's indices covers the positions whose pooled values
        # agree.
        prog3, vals3, _ = programs.config3_xception_block(E, op, with_pool_input=True)
        M3, AM3, R3 = E.run(prog3, vals3, target=target)
        np.testing.assert_array_equal(M3, got[0])
        np.testing.assert_array_equal(AM3, got[1])
        np.testing.assert_array_equal(AM3, programs.window_argmax_of(R3, M3))
        same = got[0] == ref[0]
        assert same.mean() > 0.98
        np.testing.assert_array_equal(got[1][same], ref[1][same])
        check(name, got[:1], ref[:1], tol)
        return
    check(name, got, ref, tol)


@pytest.mark.parametrize('name', sorted(n for n in programs.ALL if programs.ALL[n](OE, Oop)[2] == programs.FP32))
def test_fp32_program_as_three_bf16_products(name):
    """Every fp32 program again with `hip{fp32=bf16x3}`: GEMMs and convolutions multiply on the bf16 matrix cores
    (operands split into head + remainder), everything else is unchanged; the fp32 bar holds."""
    print('program', name, 'target hip{fp32=bf16x3}', flush=True)
    oprog, ovals, tol = programs.ALL[name](OE, Oop)
    ref = OE.run(oprog, ovals)
    prog, vals, _ = programs.ALL[name](E, op)
    got = E.run(prog, vals, target='hip{fp32=bf16x3}')
    assert len(got) == len(ref)
    for k, (g, r) in enumerate(zip(got, ref)):
        if r.dtype.kind in 'iub':
            np.testing.assert_array_equal(g, r, err_msg='%s output %d' % (name, k))
        else:
            np.testing.assert_allclose(g, r, rtol=1e-3, atol=1e-4, err_msg='%s output %d' % (name, k))


def test_domain_bounded_only_by_combinations_of_accesses():
    """O[i + j] += A[i - j] over 10-element vectors: neither access bounds i or j by itself (i in [0, 9], j in [-4, 4]
    follow from the pair), so the index box has a negative corner and most of its points are invalid.  Expected result
    by direct enumeration."""
    i, j = E.TensorIndex('i'), E.TensorIndex('j')
    A = E.Placeholder(E.DType.FLOAT32, [10], name='A')
    O = E.Contraction().outShape(10).outAccess(i + j).sum(A[i - j]).build()
    a = np.arange(1, 11, dtype=np.float32)
    want = np.zeros(10, np.float32)
    for ii in range(-20, 21):
        for jj in range(-20, 21):
            if 0 <= ii + jj < 10 and 0 <= ii - jj < 10:
                want[ii + jj] += a[ii - jj]
    for target in ('hip', 'hip{specialise=0,fuse=0}'):
        got, = E.run(E.Program('skewed', [A], [O]), [a], target=target)
        np.testing.assert_array_equal(got, want)


def test_config2_full_size_properties():
    """BASELINE configs[2] at full size through the plaidml API: int8 4096^3 -> int32 (bit-exact by a checksum of
    checksums: row sums of C against A . rowsum(B) in int64) and the per-column requantised int8 output (exact
    elementwise restatement of the Tile program on the GPU's own C)."""
    prog, vals, _ = programs.config2_int8_gemm(E, op, 4096, 4096, 4096)
    runner = E.Runner(prog, target='hip')
    C, Q = runner.run(vals)
    A, B, S = vals
    assert C.dtype == np.int32 and Q.dtype == np.int8
    np.testing.assert_array_equal(C.astype(np.int64).sum(axis=1), A.astype(np.int64) @ B.astype(np.int64).sum(axis=1))
    np.testing.assert_array_equal(C.astype(np.int64).sum(axis=0), A.astype(np.int64).sum(axis=0) @ B.astype(np.int64))
    cols = [0, 1, 777, 4095]
    np.testing.assert_array_equal(C[:, cols], (A.astype(np.int32) @ B[:, cols].astype(np.int32)))
    x = C.astype(np.float32) * S[None, :]
    x = np.where(x > np.float32(-127.0), x, np.float32(-127.0))   # op::clip: select(O > min, O, min), then select(O < max, O, max)
    x = np.where(x < np.float32(127.0), x, np.float32(127.0))
    q = (np.sign(x) * np.floor(np.abs(x) + np.float32(0.5))).astype(np.int8)   # C roundf: half away from zero
    np.testing.assert_array_equal(Q, q)
    runner.run(vals)
    print('configs[2] run stats (second run)', E.last_run_stats(), flush=True)


def test_config3_full_size_against_oracle_on_a_slice():
    """BASELINE configs[3] at full size (N64 19x19x728 bf16: depthwise 3x3 -> pointwise -> scale/shift + ReLU ->
    max-pool 3x3/2 + window argmax) through the plaidml API.  Images do not interact, so the first two images of the
    batch-64 run must equal what the oracle computes for a batch of those two with the same weights."""
    prog, vals, _ = programs.config3_xception_block(E, op, N=64, C=728, with_pool_input=True)
    M, AM, R = E.run(prog, vals, target='hip')
    assert M.shape == (64, 10, 10, 728) and AM.shape == (64, 10, 10, 728) and R.shape == (64, 19, 19, 728)
    # every index of the whole batch, bit for bit, from the device's own pool input; and the pooled values exactly
    np.testing.assert_array_equal(AM, programs.window_argmax_of(R, M))
    padded = np.zeros((64, 21, 21, 728), np.float32)   # ReLU outputs: zero padding never wins over a window's maximum
    padded[:, 1:20, 1:20] = R
    np.testing.assert_array_equal(M, np.max([padded[:, a:a + 20:2, b:b + 20:2] for a in range(3) for b in range(3)], axis=0))
    M2, AM2 = E.run(programs.config3_xception_block(E, op, N=64, C=728)[0], vals, target='hip')
    np.testing.assert_array_equal(M2, M)               # the two-output program of the benchmark gives the same
    np.testing.assert_array_equal(AM2, AM)
    oprog, ovals, _ = programs.config3_xception_block(OE, Oop, N=2, C=728)
    ovals[0] = vals[0][:2]
    for a, b in zip(ovals[1:], vals[1:]):
        np.testing.assert_array_equal(a, b)          # the same seeded weights
    rM, rAM = OE.run(oprog, ovals)
    np.testing.assert_allclose(M[:2], rM, rtol=2e-2, atol=2e-2)
    same = M[:2] == rM                                # the argmax is exact wherever the pooled bf16 values agree
    assert same.mean() > 0.98
    np.testing.assert_array_equal(AM[:2][same], rAM[same])
    # the pooled value is the value at the reported window position: checked for the whole batch on the GPU's own
    # output by recomputing position -> value for a sample of channels is the oracle's job above; here the
    # structural facts that hold for every image
    assert AM.min() >= 0 and AM.max() <= 8
    assert (M >= 0).all()                             # max over ReLU outputs


@pytest.mark.parametrize('target', ['hip', 'hip{fp32=bf16x3}'])
def test_config0_full_size_against_float64(target):
    """BASELINE configs[0] at full size through the plaidml API: fp32 1024^3, U(-1, 1), against float64 numpy; with
    fp32 MFMAs and with the operands split for the bf16 matrix cores (three products per term)."""
    prog, vals, _ = programs.config0_gemm_f32(E, op, n=1024)
    C, = E.run(prog, vals, target=target)
    assert ('as 3 bf16 products' in dict(prog.passes)['hip-plan']) == ('bf16x3' in target)
    want = vals[0].astype(np.float64) @ vals[1].astype(np.float64)
    # rtol 1e-3 on the scale of a result row (entries are sums of 1024 terms of either sign: those near zero are
    # compared through atol = 1e-3 x the typical magnitude sqrt(1024 / 9))
    np.testing.assert_allclose(C, want, rtol=1e-3, atol=1e-3 * np.sqrt(1024 / 9.0))
    assert np.abs(C - want).max() < 1e-3                  # measured: a few 1e-5 (fp32 accumulation over 1024 terms)


@pytest.mark.parametrize('dtype_name,target', [('FLOAT32', 'hip'), ('BFLOAT16', 'hip'), ('FLOAT32', 'hip{fp32=bf16x3}')])
def test_config1_full_size_through_exec(dtype_name, target):
    """BASELINE configs[1] at full size (N128 56x56x64, 3x3x64x64, SAME, + bias + ReLU) through the plaidml API, in
    fp32 and in bf16: images do not interact, so images 0 and 127 must equal the oracle's result for a batch of
    those two; sampled pixels of every image are checked against float64 arithmetic on the same values."""
    print('configs[1] full size', dtype_name, flush=True)
    prog, vals, tol = programs.config1_conv(E, op, dtype_name, N=128, H=56, W=56)
    O, = E.run(prog, vals, target=target)
    assert O.shape == (128, 56, 56, 64)
    plan = dict(prog.passes)['hip-plan']
    assert 'conv2d' in plan and 'contract (general)' not in plan, plan
    oprog, ovals, _ = programs.config1_conv(OE, Oop, dtype_name, N=2, H=56, W=56)
    ovals[0] = vals[0][[0, 127]]
    np.testing.assert_array_equal(ovals[1], vals[1])
    ref, = OE.run(oprog, ovals)
    rtol, atol = (2e-2, 2e-2) if dtype_name == 'BFLOAT16' else (1e-3, 1e-4 if 'bf16x3' in target else 1e-5)
    np.testing.assert_allclose(O[[0, 127]], ref, rtol=rtol, atol=atol)
    Iv, Fv, Bv = (v.astype(np.float64) for v in vals)
    r = np.random.default_rng(12)
    pix = [(int(n), int(y), int(x)) for n, y, x in zip(r.integers(0, 128, 300), r.integers(0, 56, 300), r.integers(0, 56, 300))]
    pix += [(n, y, x) for n in (0, 64, 127) for y in (0, 55) for x in (0, 55)]     # corners: padding on two sides
    for n, y, x in pix:
        acc = Bv.copy()
        for ky in range(3):
            for kx in range(3):
                yy, xx = y + ky - 1, x + kx - 1
                if 0 <= yy < 56 and 0 <= xx < 56:
                    acc += Iv[n, yy, xx] @ Fv[ky, kx]
        np.testing.assert_allclose(O[n, y, x], np.maximum(acc, 0), rtol=rtol, atol=atol if dtype_name == 'BFLOAT16' else 1e-4,
                                   err_msg=str((n, y, x)))


def test_config4_full_size_image_against_golden():
    """BASELINE configs[4] at full size: ResNet-50 v1.5, batch 128, 224 x 224, bf16, through the plaidml API.  Row 0
    of the result is compared with the probabilities the oracle computed for that image alone
    (tests/golden/resnet50_v1_5_image_probs.npz, written by tests/golden/make_resnet50_image.py: five minutes of
    CPU, too long to run here); every row must be a probability distribution, and a second copy of the image in
    another slot must give the same row."""
    import os
    from plaidml_amd import resnet50
    fx = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'resnet50_v1_5_image_probs.npz'))
    from oracle.tile_oracle import round_bf16
    prog, _, _ = resnet50.build(E, op, batch=128, round_fn=round_bf16, with_logits=True)
    x = round_bf16(np.random.default_rng(5).uniform(0, 1, (128, 224, 224, 3)).astype(np.float32))
    img = round_bf16(np.random.default_rng(int(fx['image_seed'])).uniform(0, 1, (1, 224, 224, 3)).astype(np.float32))
    x[0] = img[0]
    x[77] = img[0]
    probs, logits = E.run(prog, [x], target='hip')
    assert probs.shape == (128, 1000) and np.isfinite(probs).all() and np.isfinite(logits).all()
    np.testing.assert_allclose(probs.sum(axis=1), 1.0, rtol=2e-2)
    np.testing.assert_array_equal(logits[0], logits[77])
    # 53 bf16 layers deep, every layer rounding its output: the logits (spread about 2400, one bf16 step there is 16)
    # are compared on the scale of their spread.  Measured: 8 (0.33 % of the spread) against the oracle, while the
    # row of a different image is 24 away, so the bound separates the two.
    ref = fx['logits'].reshape(1000)
    spread = float(np.abs(ref).max())
    np.testing.assert_allclose(logits[0], ref, rtol=1e-2, atol=5e-3 * spread)
    assert np.abs(logits[1] - ref).max() > 5e-3 * spread
    assert np.corrcoef(logits[0], ref)[0, 1] > 0.9999
    assert int(probs[0].argmax()) == int(fx['probs'].reshape(1000).argmax())
    print('configs[4] run stats', E.last_run_stats(), flush=True)


def test_transposed_convolution_from_the_input_side_at_size():
    """O[n, 2x + i - 1, 2y + j - 1, co] += I[n, x, y, ci] K[i, j, ci, co] on 2 x 32 x 32 x 16 -> 64 x 64 x 16: 131072
    output elements over a box of 4.7 million index tuples.  Each thread walks the 144 (tap, channel) tuples of its
    element, the two sums being solved for x and y; exact on small-integer data against loops over the input."""
    print('transposed convolution, input side, 32x32x16', flush=True)
    prog, vals, _ = programs.scatter_form_transposed_conv(E, op, N=2, H=32, CI=16, CO=16)
    want = programs.scatter_form_transposed_conv_answer(*vals)
    got, = E.run(prog, vals, target='hip')
    np.testing.assert_array_equal(got, want.astype(np.float32))
    assert E.last_run_stats()['kernel_ms'] < 50.0


@pytest.mark.parametrize('out_name', ['INT8', 'UINT8', 'INT16'])
@pytest.mark.parametrize('R,C', [(64, 48), (33, 40), (5, 37), (256, 1024)])
def test_requantisation_chain_as_its_own_launch(R, C, out_name):
    """int32 -> fp32 -> scale per column -> clamp -> round -> narrow integer as an element-wise launch of its own
    (what a large int8 GEMM leaves to a second launch): the typed-chain kernel (rows of whole 16-byte output
    vectors), the vector kernel with a narrower output (rows of whole 16-byte input vectors) and the interpreter
    (anything else) must give the bits of the same fp32 arithmetic in numpy; values beyond the clamp included."""
    print('requantisation chain', (R, C, out_name), flush=True)
    lo, hi = {'INT8': (-127.0, 127.0), 'UINT8': (0.0, 255.0), 'INT16': (-32767.0, 32767.0)}[out_name]
    X = E.Placeholder(E.DType.INT32, [R, C])
    S = E.Placeholder(E.DType.FLOAT32, [C])
    Q = E.cast(E.round(op.clip(E.cast(X, E.DType.FLOAT32) * S, lo, hi)), getattr(E.DType, out_name))
    prog = E.Program('requant', [X, S], [Q])
    rng = np.random.default_rng(R * 131 + C)
    x = rng.integers(-60000, 60001, (R, C)).astype(np.int32)
    x[0, :4] = [0, 1, -1, 2 ** 31 - 1]
    sc = rng.uniform(0.001, 0.01, C).astype(np.float32) * (100.0 if out_name == 'INT16' else 1.0)
    got, = E.run(prog, [x, sc], target='hip')
    y = np.minimum(np.maximum(x.astype(np.float32) * sc, np.float32(lo)), np.float32(hi)).astype(np.float32)
    want = np.where(y >= 0, np.floor(y + np.float32(0.5)), np.ceil(y - np.float32(0.5))).astype(np.float32)
    np.testing.assert_array_equal(got, want.astype(got.dtype))
    assert got.min() == lo and got.max() == hi  # both clamps bite


def test_large_int8_gemm_keeps_its_requantisation_and_leaves_other_chains_to_a_second_launch():
    """4096^3 int8: the clip-and-round requantisation chain runs as straight code behind the large tile and stays fused
    (one launch); a chain that only the step-wise tail can run (here floor instead of clip and round) would cost
    that tile, so the planner, having asked the kernel library, leaves it to an element-wise launch of its own."""
    prog = programs.config2_int8_gemm(E, op, M=4096, N=4096, K=4096)[0]
    prog.compile('hip')
    plan = dict(prog.passes)['hip-plan']
    assert '1 launches' in plan and 'tail=[store cast:f32 mul(t0) maxgt(-127) min(127) round cast:si8]' in plan, plan
    M = N = K = 4096
    A, B, S = E.Placeholder(E.DType.INT8, [M, K]), E.Placeholder(E.DType.INT8, [K, N]), E.Placeholder(E.DType.FLOAT32, [N])
    i, j, k = E.TensorIndexes(3)
    C = E.Contraction().outShape(M, N).outAccess(i, j).sum(E.cast(A, E.DType.INT32)[i, k] * E.cast(B, E.DType.INT32)[k, j]).build()
    Q = E.cast(E.floor(E.cast(C, E.DType.FLOAT32) * S), E.DType.INT8)
    prog = E.Program('int8_gemm_floor', [A, B, S], [C, Q])
    prog.compile('hip')
    plan = dict(prog.passes)['hip-plan']
    assert '2 launches' in plan and 'gemm si8 m=4096 n=4096 k=4096 B=[k][n] -> 4096x4096xsi32' in plan, plan
    assert 'eltwise cast tail=[cast:f32 mul(t0) floor' in plan, plan
    prog = programs.config2_int8_gemm(E, op)[0]
    prog.compile('hip')
    assert '1 launches' in dict(prog.passes)['hip-plan']


def test_run_checks_arity_and_shapes():
    prog, vals, _ = programs.dot_f32(E, op)
    prog.compile()
    exe = E.Executable(prog)
    a = E.Buffer(E.TensorShape(E.DType.FLOAT32, [8, 16]))
    b = E.Buffer(E.TensorShape(E.DType.FLOAT32, [16, 32]))
    o = E.Buffer(E.TensorShape(E.DType.FLOAT32, [8, 32]))
    with pytest.raises(E.PlaidMLError, match='Program expects 2 inputs, but 1 were specified'):
        exe.run([a], [o])
    bad = E.Buffer(E.TensorShape(E.DType.FLOAT32, [16, 16]))
    with pytest.raises(E.PlaidMLError, match="Shape mismatch for input buffer #0, expected '8x16xf32' but '16x16xf32' was specified"):
        exe.run([bad, b], [o])
    assert exe.run([a, b], [o]) >= 0.0
    assert 'hip.0' in E.list_devices()


def test_cpp_header_api_cases():
    """User C++ against include/plaidml/* (tests/cpp/edsl_cases.cc, built by __graft_entry__.build) on the hip device."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'cpp', 'edsl_cases')
    assert os.path.exists(exe), 'run __graft_entry__.build() first'
    res = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(res.stdout, res.stderr, flush=True)
    assert res.returncode == 0, res.stderr
    assert 'all cases passed' in res.stdout


@pytest.mark.gpu
@pytest.mark.parametrize('dtype_name', ['FLOAT32', 'BFLOAT16'])
def test_row_reductions_at_size(dtype_name):
    """Row sum / max / min of a 2048 x 3000 matrix and the sum of everything, against numpy: the maxima exactly, the
    sums to the accumulation tolerance (fp32 partial sums per lane, folded across the wavefront)."""
    print('row reductions at size', dtype_name, flush=True)
    from oracle.tile_oracle import round_bf16
    rows, cols = 2048, 3000
    x = np.random.default_rng(51).standard_normal((rows, cols)).astype(np.float32)
    if dtype_name == 'BFLOAT16':
        x = round_bf16(x)
    X = E.Placeholder(getattr(E.DType, dtype_name), [rows, cols])
    i, j = E.TensorIndexes(2)
    outs = [E.Contraction().outShape(rows).outAccess(i).sum(X[i, j]).build(),
            E.Contraction().outShape(rows).outAccess(i).max(X[i, j]).build(),
            E.Contraction().outShape(rows).outAccess(i).min(X[i, j]).build(),
            E.Contraction().sum(X[i, j]).build()]
    s, mx, mn, total = E.run(E.Program('rows', [X], outs), [x], target='hip')
    np.testing.assert_array_equal(mx, x.max(1))
    np.testing.assert_array_equal(mn, x.min(1))
    exact = x.astype(np.float64).sum(1)
    if dtype_name == 'BFLOAT16':
        np.testing.assert_allclose(s, exact, rtol=1e-2, atol=0.5)      # one bf16 rounding of a sum of magnitude ~55
        np.testing.assert_allclose(total, exact.sum(), rtol=1e-2, atol=16)
    else:
        np.testing.assert_allclose(s, exact, rtol=1e-4, atol=1e-3)
        np.testing.assert_allclose(total, exact.sum(), rtol=1e-4, atol=0.5)


@pytest.mark.parametrize('name', sorted(programs.ALL))
def test_replayed_graph_equals_one_by_one_launches(name):
    """From its third run on an executable replays its launches as one recorded HIP graph.  Six runs on inputs that
    change from run to run, each compared bit for bit with an executable compiled with `hip{graph=0}` that runs (its
    own launches, its own synchronisations) between the replays.  Programs with a sort, gather, scatter, index or
    random-number step are never recorded and pass trivially."""
    print('program', name, flush=True)
    prog, vals, _ = programs.ALL[name](E, op)
    replaying = E.Runner(prog, target='hip')
    prog0, _, _ = programs.ALL[name](E, op)
    one_by_one = E.Runner(prog0, target='hip{graph=0}')
    replays = 0
    for r in range(6):
        # (rolled, not re-drawn: index operands stay in range)
        ins = [np.roll(np.asarray(v), r, axis=-1) if np.asarray(v).ndim else np.asarray(v) for v in vals]
        got = replaying.run(ins)
        replays += bool(E.last_run_stats()['graph'])
        note = E.last_run_stats()['graph_note']
        ref = one_by_one.run(ins)
        assert not E.last_run_stats()['graph']
        for k, (g, x) in enumerate(zip(got, ref)):
            np.testing.assert_array_equal(g, x, err_msg='%s run %d output %d' % (name, r, k))
    assert replays in (0, 4), replays
    if name in ('config3_xception_block_bf16', 'resnet50_tiny_bf16', 'residual_block_bf16', 'mnist_cnn'):
        assert replays == 4, 'a program of plain kernel launches was not recorded: ' + note
