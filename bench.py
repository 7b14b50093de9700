#!/usr/bin/env python3
"""Benchmark of the Tile contraction hot path on one MI355X.

Workload (BASELINE.json configs[1]): conv2d NHWC via the contraction
  O[n,y,x,co] += I[n,y+ky-1,x+kx-1,ci] * F[ky,kx,ci,co]   (N128, 56x56x64, 3x3x64x64, stride 1, SAME)
followed by the fused bias + ReLU tail, bf16 (fp32 accumulate).  One step = one pass over one
batch, inputs (image, HWCK filter, bias) resident in HBM: a single launch of the resident-filter
convolution kernel, which re-lays the filter out on its way into LDS.  Consecutive steps take five
input / output buffer pairs in turn, so that no step finds its input in the last-level cache.

Prints ONE JSON line.  `value` is TFLOP/s over the algorithmic FLOPs (2 x valid index tuples:
SAME-padding taps that fall outside the image are not counted).  `roofline` describes the
dominant kernel (the convolution kernel with a pre-packed filter) timed with HIP events on the
launch stream; `roofline.traffic` is the HBM bytes per launch taken from the committed rocprofv3
counter summary (profiles/), null when that file is absent; `cpu_baseline` is the
OpenMP restatement (oracle/cpu_baseline.c) on a bounded sample of the same workload.
`extra` carries the other configs (each kernel alone, and the whole programs through the plaidml API), all on
the data the configs name (N(0,1) activations, uniform int8), and the rate the matrix cores sustain on LDS-resident
operands with constant and with random values (the clock the chip holds under real data bounds every GEMM here).
`--only a,b` runs just those legs of `extra` (for profiling runs); ResNet-50 img/s is repeated at the top level.

`--copy-calibration` runs only a plain device copy of a known size (the factor that scales the
FETCH_SIZE / WRITE_SIZE counters) and prints its byte count.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK = {'bf16': 2500.0, 'f32': 157.3, 'i8': 5000.0}  # dense MFMA TFLOP/s (TOP/s), MI355X
HBM_PEAK_GBS = 8000.0


def conv_plan(hk, in_dt, N, H, W, CI, CO, KH, KW, relu=True, flags=0):
    d = hk.Conv2dDesc()
    d.in_dtype, d.out_dtype, d.c_dtype = in_dt, in_dt, in_dt
    d.flags = flags
    d.n, d.h, d.w, d.ci, d.kh, d.kw, d.co, d.oh, d.ow = N, H, W, CI, KH, KW, CO, H, W
    d.stride_h = d.stride_w = d.dil_h = d.dil_w = 1
    d.pad_h, d.pad_w = (KH - 1) // 2, (KW - 1) // 2
    d.init_kind, d.init_dtype = 1, in_dt
    d.init_row_stride, d.init_col_stride = 0, 1
    if relu:
        d.tail = hk.make_tail(ops=[(hk.EPI_RELU, in_dt, 0, 0, 0.0)])
    plan = hk.lib().pml_hip_conv2d_dispatch(ctypes.byref(d))
    if not plan:
        raise RuntimeError(hk.lib().pml_hip_last_error().decode())
    return plan


# A device that has been idle runs its first tens of milliseconds of work at a lower clock than it then settles at
# (a 1024^3 fp32 GEMM: 28.0 us per launch over the first 2 ms, 24.9 us once half a second has passed).  Every timed
# loop is therefore preceded, after its warm-up steps, by further untimed steps of the same call until this much
# wall time has passed since the loop began: the figure is the one a device under sustained load shows.
SETTLE_MS = 100.0


def time_loop(hk, fn, steps, warmup, settle_ms=SETTLE_MS):
    began = time.perf_counter()
    for _ in range(warmup):
        fn()
    hk.check(hk.lib().pml_hip_stream_sync(None))
    while (time.perf_counter() - began) * 1e3 < settle_ms:
        for _ in range(32):
            fn()
        hk.check(hk.lib().pml_hip_stream_sync(None))
    t = hk.Timer()
    wall0 = time.perf_counter()
    t.start()
    for _ in range(steps):
        fn()
    ms = t.stop()
    hk.check(hk.lib().pml_hip_stream_sync(None))
    wall = (time.perf_counter() - wall0) * 1e3
    return ms / steps, wall / steps


def fp32_fraction(tflops, flags):
    """fp32 work against the pipe it runs on: fp32 MFMAs against their own peak; as three bf16 products per term against
    a third of the bf16 peak (that pipe does three multiplications per useful one)."""
    if flags:
        return {'frac_of_bf16_peak_over_3': round(tflops / (PEAK['bf16'] / 3), 4), 'peak_TFLOP/s': round(PEAK['bf16'] / 3, 1)}
    return {'frac_mfma_f32': round(tflops / PEAK['f32'], 4)}


def valid_taps(size, k, pad):
    return sum(1 for x in range(size) for t in range(k) if 0 <= x + t - pad < size)


def cpu_model():
    try:
        for line in open('/proc/cpuinfo'):
            if line.startswith('model name'):
                return line.split(':', 1)[1].strip()
    except OSError:
        pass
    return 'unknown'


def cpu_baseline_conv(N_sample, H, W, CI, CO, seed_i, seed_f, flops_per_image):
    """The only leg that touches oracle/: the OpenMP restatement, timed on a bounded sample (threads pinned to cores,
    median of the timed runs)."""
    # the OpenMP runtime reads its placement when the library is loaded
    os.environ.setdefault('OMP_PROC_BIND', 'close')
    os.environ.setdefault('OMP_PLACES', 'cores')
    from oracle import tile_oracle as E  # checker (test infrastructure), never the thing measured
    lib = ctypes.CDLL(os.path.join(ROOT, 'oracle', 'libcpu_baseline.so'))
    lib.cpu_baseline_threads.restype = ctypes.c_int
    threads = lib.cpu_baseline_threads()
    rng = np.random.default_rng(seed_i)
    Iv = E.round_bf16(rng.standard_normal((N_sample, H, W, CI)).astype(np.float32))
    Fv = E.round_bf16((np.random.default_rng(seed_f).standard_normal((3, 3, CI, CO)) * np.sqrt(2.0 / (9 * CI))).astype(np.float32))
    bias = np.zeros(CO, np.float32)
    out = np.empty((N_sample, H, W, CO), np.float32)
    fp = ctypes.POINTER(ctypes.c_float)

    def run():
        lib.cpu_conv2d_nhwc_f32(Iv.ctypes.data_as(fp), Fv.ctypes.data_as(fp), bias.ctypes.data_as(fp),
                                out.ctypes.data_as(fp), N_sample, H, W, CI, 3, 3, CO, H, W, 1, 1, 1)

    run()  # warm-up
    times, total = [], 0.0
    while (total < 10.0 and len(times) < 50) or len(times) < 5:
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
        total += times[-1]
    sec = float(np.median(times))
    return {
        'value': round(flops_per_image * N_sample / sec / 1e12, 5), 'unit': 'TFLOP/s', 'cores': threads, 'kind': 'port',
        'sample': '%d of 128 images of the same conv (fp32 arithmetic on bf16-valued inputs), median of %d runs (fastest %.1f ms, '
                  'slowest %.1f ms), OMP_NUM_THREADS=%s OMP_PROC_BIND=%s OMP_PLACES=%s'
                  % (N_sample, len(times), min(times) * 1e3, max(times) * 1e3, os.environ.get('OMP_NUM_THREADS', 'unset'),
                     os.environ.get('OMP_PROC_BIND'), os.environ.get('OMP_PLACES')),
        'cpu': cpu_model(),
    }, E.round_bf16(out), Iv, Fv


def staged_runs(runner, staged, P, runs, settle_ms):
    """Runs a staged program back to back -- at least `runs` times and until `settle_ms` have passed -- and returns the
    statistics of the run whose device time is the median of those after the first, with the fastest beside it."""
    stats, began = [], time.perf_counter()
    while len(stats) < runs + 1 or (time.perf_counter() - began) * 1e3 < settle_ms:
        wall = runner.run_staged(staged)
        stats.append(dict(P.last_run_stats(), wall_ms=wall))
    timed = sorted(stats[1:], key=lambda t: t['kernel_ms'])
    return dict(timed[len(timed) // 2], kernel_ms_min=timed[0]['kernel_ms'], runs=len(timed))


def copy_calibration(hk, steps):
    """A plain copy kernel of known size: out[i] = in[i] over 256 MiB of fp32."""
    n = 64 << 20
    d = hk.EltwiseDesc()
    d.rank, d.in_dtype, d.out_dtype = 1, hk.F32, hk.F32
    d.sizes[0] = n
    d.in_strides[0] = 1
    plan = hk.lib().pml_hip_eltwise_dispatch(ctypes.byref(d))
    if not plan:
        raise RuntimeError(hk.lib().pml_hip_last_error().decode())
    src, dst = hk.DeviceBuffer(n * 4), hk.DeviceBuffer(n * 4)
    hk.check(hk.lib().pml_hip_fill_u32(src.ptr, 0x3f800000, n, None))
    none = hk.ptr_array([])
    ms, _ = time_loop(hk, lambda: hk.check(hk.lib().pml_hip_eltwise_invoke(plan, src.ptr, dst.ptr, none, none, None)), steps, 2)
    return {'copy_kernel': hk.describe(plan), 'bytes_read_per_launch': n * 4, 'bytes_written_per_launch': n * 4,
            'ms': round(ms, 4), 'GBps': round(2 * n * 4 / ms / 1e6, 1)}


def int8_program_leg(n=4096, runs=5):
    from plaidml_amd import edsl as P, op as Pop
    A = P.Placeholder(P.DType.INT8, [n, n])
    B = P.Placeholder(P.DType.INT8, [n, n])
    S = P.Placeholder(P.DType.FLOAT32, [n])
    i, j, k = P.TensorIndexes(3)
    C = P.Contraction().outShape(n, n).outAccess(i, j).sum(P.cast(A, P.DType.INT32)[i, k] * P.cast(B, P.DType.INT32)[k, j]).build()
    Q = P.cast(P.round(Pop.clip(P.cast(C, P.DType.FLOAT32) * S, -127.0, 127.0)), P.DType.INT8)
    runner = P.Runner(P.Program('int8_gemm', [A, B, S], [C, Q]), target='hip')
    a = np.random.default_rng(4).integers(-127, 128, (n, n), dtype=np.int8)
    b = np.random.default_rng(5).integers(-127, 128, (n, n), dtype=np.int8)
    sc = np.random.default_rng(6).uniform(0.001, 0.01, n).astype(np.float32)
    runner.run([a, b, sc])  # one whole run for the transfer times
    first = P.last_run_stats()
    staged = runner.stage([a, b, sc])  # then back to back on staged inputs (B is still transposed in every run)
    mid = staged_runs(runner, staged, P, runs, SETTLE_MS)
    ops = 2.0 * n ** 3
    plan = [l.strip() for l in dict(runner.program.passes)['hip-plan'].splitlines()[1:]]
    return {'kernel_ms': round(mid['kernel_ms'], 4), 'kernel_ms_min': round(mid['kernel_ms_min'], 4), 'runs': mid['runs'],
            'launches': int(mid['launches']), 'TOP/s': round(ops / mid['kernel_ms'] / 1e9, 1),
            'frac_mfma_i8': round(ops / mid['kernel_ms'] / 1e9 / PEAK['i8'], 4), 'h2d_ms': round(first['h2d_ms'], 3),
            'd2h_ms': round(first['d2h_ms'], 3), 'b_layout': '[K][N] as the config states it (program input, re-laid per run)', 'plan': plan}


def xception_leg(hk, L, none, N=64, H=19, W=19, C=728):  # noqa: C901
    """Depthwise 3x3, pointwise 728->728 with the fused scale/shift + ReLU tail, max-pool 3x3/2 with window argmax."""
    out = {}
    px = N * H * W
    from plaidml_amd import edsl as P
    rng = np.random.default_rng(7)
    dI = hk.DeviceBuffer.from_numpy(P.to_bf16_bits(rng.standard_normal((N, H, W, C)).astype(np.float32)))  # N(0,1) as the config says
    # the depthwise result is a temporary: like the planner, give its rows a pitch of whole 128-byte lines
    pitch = (C * 2 + 127) // 128 * 128 // 2
    dD, dP = hk.DeviceBuffer(px * pitch * 2), hk.DeviceBuffer(px * C * 2)
    # depthwise
    d = hk.Dwconv2dDesc()
    d.dtype = hk.BF16
    d.out_pitch = pitch
    d.n, d.h, d.w, d.c, d.kh, d.kw, d.oh, d.ow = N, H, W, C, 3, 3, H, W
    d.stride_h = d.stride_w = d.dil_h = d.dil_w = 1
    d.pad_h = d.pad_w = 1
    plan = L.pml_hip_dwconv2d_dispatch(ctypes.byref(d))
    dF = hk.DeviceBuffer.from_numpy(P.to_bf16_bits((rng.standard_normal((3, 3, C, 1)) * np.sqrt(2.0 / 9)).astype(np.float32)))
    nbytes = 2 * px * C * 2
    ms, _ = time_loop(hk, lambda: hk.check(L.pml_hip_dwconv2d_invoke(plan, dI.ptr, dF.ptr, dD.ptr, none, none, None)), 20, 3)
    out['depthwise3x3_filter_per_call'] = {'ms': round(ms, 4), 'GB/s': round(nbytes / ms / 1e6, 1), 'frac_hbm': round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
    # the block's weights are constants: the filter is handed over once, as the planner does for a program constant
    hk.check(L.pml_hip_dwconv2d_pack_filter(plan, dF.ptr, None))
    ms, _ = time_loop(hk, lambda: hk.check(L.pml_hip_dwconv2d_invoke(plan, dI.ptr, None, dD.ptr, none, none, None)), 20, 3)
    out['depthwise3x3'] = {'ms': round(ms, 4), 'GB/s': round(nbytes / ms / 1e6, 1), 'frac_hbm': round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4),
                           'filter': 'constant, packed once'}
    # pointwise + scale/shift + relu
    g = hk.GemmDesc()
    g.in_dtype = g.out_dtype = g.c_dtype = hk.BF16
    g.m, g.n, g.k, g.lda, g.ldb, g.ldc = px, C, C, pitch, C, C
    g.tail = hk.make_tail(ops=[(hk.EPI_MUL, hk.BF16, hk.OPND_TENSOR, 0, 0.0), (hk.EPI_ADD, hk.BF16, hk.OPND_TENSOR, 1, 0.0),
                               (hk.EPI_RELU, hk.BF16, 0, 0, 0.0)], operands=[(hk.BF16, 0, 1), (hk.BF16, 0, 1)])
    pg = L.pml_hip_gemm_dispatch(ctypes.byref(g))
    dW = hk.DeviceBuffer.from_numpy(P.to_bf16_bits((rng.standard_normal((C, C)) * np.sqrt(2.0 / C)).astype(np.float32)))
    dS = hk.DeviceBuffer.from_numpy(P.to_bf16_bits(rng.uniform(0.5, 1.5, C).astype(np.float32)))
    dT = hk.DeviceBuffer.from_numpy(P.to_bf16_bits(rng.uniform(-0.5, 0.5, C).astype(np.float32)))
    hk.check(L.pml_hip_gemm_pack_b(pg, dW.ptr, None))
    ops = hk.ptr_array([dS.ptr, dT.ptr])
    ms, _ = time_loop(hk, lambda: hk.check(L.pml_hip_gemm_invoke(pg, dD.ptr, None, dP.ptr, None, ops, none, None)), 20, 3)
    fl = 2.0 * px * C * C
    out['pointwise_scale_shift_relu'] = {'ms': round(ms, 4), 'TFLOP/s': round(fl / ms / 1e9, 1),
                                         'frac_mfma_bf16': round(fl / ms / 1e9 / PEAK['bf16'], 4), 'plan': hk.describe(pg)}
    # max-pool 3x3/2 SAME + window argmax
    p = hk.Pool2dDesc()
    p.dtype, p.agg = hk.BF16, hk.AGG_MAX
    p.n, p.h, p.w, p.c, p.kh, p.kw, p.oh, p.ow = N, H, W, C, 3, 3, 10, 10
    p.stride_h = p.stride_w = 2
    p.pad_h = p.pad_w = 1
    p.with_index = 1
    pp = L.pml_hip_pool2d_dispatch(ctypes.byref(p))
    dM, dX = hk.DeviceBuffer(N * 100 * C * 2), hk.DeviceBuffer(N * 100 * C * 4)
    ms, _ = time_loop(hk, lambda: hk.check(L.pml_hip_pool2d_invoke(pp, dP.ptr, dM.ptr, dX.ptr, None)), 20, 3)
    nbytes = px * C * 2 + N * 100 * C * 6
    out['maxpool3x3s2_argmax'] = {'ms': round(ms, 4), 'GB/s': round(nbytes / ms / 1e6, 1), 'frac_hbm': round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
    for b in (dI, dD, dP, dF, dW, dS, dT, dM, dX):
        b.free()
    out['block_through_exec'] = xception_program_leg(N, H, W, C)
    return out


def xception_program_leg(N, H, W, C, runs=5):
    """The same block as one Tile program through libplaidml.so: what the planner makes of it, device time of a run."""
    from plaidml_amd import edsl as P, op as Pop
    dt = P.DType.BFLOAT16
    rng = np.random.default_rng(7)
    image = rng.standard_normal((N, H, W, C)).astype(np.float32)
    # the block's weights are program constants, as a network's are (uploaded and re-laid-out once)
    I = P.Placeholder(dt, [N, H, W, C])
    Fdw = P.Constant(P.round_bf16((rng.standard_normal((3, 3, C, 1)) * np.sqrt(2.0 / 9)).astype(np.float32)), dt)
    Fpw = P.Constant(P.round_bf16((rng.standard_normal((1, 1, C, C)) * np.sqrt(2.0 / C)).astype(np.float32)), dt)
    scale = P.Constant(P.round_bf16(rng.uniform(0.5, 1.5, C).astype(np.float32)), dt)
    shift = P.Constant(P.round_bf16(rng.uniform(-0.5, 0.5, C).astype(np.float32)), dt)
    R = Pop.relu(Pop.convolution(Pop.convolution(I, Fdw, depthwise=True), Fpw) * scale + shift)
    M = Pop.pool(R, 'max', [3, 3], [2, 2], autopad=Pop.SAME_UPPER)
    n, x0, x1, c, k0, k1 = P.TensorIndexes(6)
    IX = P.index([3, 3], 0) * 3 + P.index([3, 3], 1)
    AM = P.Contraction().outShape(M.shape).outAccess(n, x0, x1, c).max(
        P.cond(R[n, 2 * x0 + k0 - 1, 2 * x1 + k1 - 1, c], M[n, x0, x1, c], IX[k0, k1])).build()
    prog = P.Program('xception_block', [I], [M, AM])
    runner = P.Runner(prog, target='hip')
    staged = runner.stage([image])
    mid = staged_runs(runner, staged, P, runs, SETTLE_MS)
    plan = [l.strip() for l in dict(prog.passes)['hip-plan'].splitlines()[1:]]
    return {'kernel_ms': round(mid['kernel_ms'], 4), 'kernel_ms_min': round(mid['kernel_ms_min'], 4), 'runs': mid['runs'],
            'launches': int(mid['launches']), 'plan': plan}


def resnet50_leg(batch=128, runs=5):
    """Whole-network forward through libplaidml.so: device time between the first and the last kernel of a run."""
    from plaidml_amd import edsl as P, op as Pop, resnet50
    prog, _, flops_full_box = resnet50.build(P, Pop, batch=batch, round_fn=P.round_bf16)
    runner = P.Runner(prog, target='hip')
    x = np.random.default_rng(11).uniform(0, 1, (batch, 224, 224, 3)).astype(np.float32)
    out, = runner.run([x])
    first = P.last_run_stats()
    if not (np.isfinite(out).all() and np.allclose(out.sum(axis=1), 1.0, atol=2e-2)):
        raise SystemExit('bench: ResNet-50 output is not a probability distribution')
    # the timed runs follow one another without the 77 MB upload between them (during which the device idles and
    # its clock falls back): the input is staged once
    staged = runner.stage([x])
    best = staged_runs(runner, staged, P, runs, 2 * SETTLE_MS)   # the median run
    best = dict(best, h2d_ms=first['h2d_ms'], d2h_ms=first['d2h_ms'])
    return {'img_per_s': round(batch / (best['kernel_ms'] * 1e-3), 1), 'kernel_ms': round(best['kernel_ms'], 3),
            'replayed_as_graph': bool(best['graph']), 'wall_ms': round(best['wall_ms'], 3),
            'kernel_ms_min': round(best['kernel_ms_min'], 3), 'img_per_s_fastest_run': round(batch / (best['kernel_ms_min'] * 1e-3), 1),
            'runs': best['runs'],
            'h2d_ms': round(best['h2d_ms'], 3), 'd2h_ms': round(best['d2h_ms'], 3), 'launches': int(best['launches']),
            'device_MB': round(best['device_bytes'] / 1e6, 1), 'arena_MB': round(best['arena_bytes'] / 1e6, 1),
            'temporaries_unshared_MB': round(best['unshared_temp_bytes'] / 1e6, 1),
            'TFLOP/s_full_box': round(flops_full_box / (best['kernel_ms'] * 1e-3) / 1e12, 1),
            'frac_mfma_bf16': round(flops_full_box / (best['kernel_ms'] * 1e-3) / 1e12 / PEAK['bf16'], 4)}


def committed_traffic():
    """HBM bytes per launch of the bench kernel from the committed counter summary, or None."""
    path = os.path.join(ROOT, 'profiles', 'conv_regfilter3x3_bf16_configs1_hbm_traffic.md')
    try:
        for line in open(path):
            if line.startswith('traffic_bytes_per_launch'):
                return float(line.split('=')[1].split()[0])
    except OSError:
        pass
    return None


def gemm_leg(hk, kind, n=4096, b_nk=True):
    """A square GEMM on the data its config names: int8 uniform in [-127, 127], bf16 N(0,1).  b_nk: B is handed over as
    [N][K] (K contiguous, what the matrix instructions read); otherwise as the row-major [K][N] the configs describe,
    which every run first re-lays (or reads through transposing LDS reads, where the library finds that cheaper)."""
    from plaidml_amd import edsl as P
    L, none = hk.lib(), hk.ptr_array([])
    g = hk.GemmDesc()
    rng = np.random.default_rng(4)
    if kind == 'i8':
        g.in_dtype, g.out_dtype, g.c_dtype = hk.I8, hk.I32, hk.I32
        a, b = rng.integers(-127, 128, (n, n), dtype=np.int8), rng.integers(-127, 128, (n, n), dtype=np.int8)
        out_bytes, peak, unit = 4, PEAK['i8'], 'TOP/s'
    else:
        g.in_dtype = g.out_dtype = g.c_dtype = hk.BF16
        a, b = (P.to_bf16_bits(rng.standard_normal((n, n)).astype(np.float32)) for _ in range(2))
        out_bytes, peak, unit = 2, PEAK['bf16'], 'TFLOP/s'
    g.m = g.n = g.k = g.lda = g.ldb = g.ldc = n
    g.b_layout = 1 if b_nk else 0
    plan = L.pml_hip_gemm_dispatch(ctypes.byref(g))
    dA, dB, dC = hk.DeviceBuffer.from_numpy(a), hk.DeviceBuffer.from_numpy(b), hk.DeviceBuffer(n * n * out_bytes)
    ms, _ = time_loop(hk, lambda: hk.check(L.pml_hip_gemm_invoke(plan, dA.ptr, dB.ptr, dC.ptr, None, none, none, None)), 20, 5)
    res = {'ms': round(ms, 4), unit: round(2.0 * n ** 3 / ms / 1e9, 2), 'frac_mfma': round(2.0 * n ** 3 / ms / 1e9 / peak, 4),
           'plan': hk.describe(plan), 'data': 'uniform int8 [-127, 127]' if kind == 'i8' else 'N(0,1) bf16',
           'b_layout': '[N][K], K contiguous (pre-transposed by the caller)' if b_nk else '[K][N] row-major as the config states it (re-laid by every run)'}
    for buf in (dA, dB, dC):
        buf.free()
    L.pml_hip_plan_free(plan)
    return res


def mfma_ceiling_leg(hk):
    """pml_hip_probe_mfma: bf16 MFMA stream on LDS-resident operands, constant against random operand values."""
    out = {}
    for name, rnd in (('constant_operands', 0), ('random_operands', 1)):
        tf, mhz = ctypes.c_double(), ctypes.c_double()
        hk.check(hk.lib().pml_hip_probe_mfma(rnd, 2000, ctypes.byref(tf), ctypes.byref(mhz)))
        out[name] = {'TFLOP/s': round(tf.value, 1), 'frac_of_2500': round(tf.value / PEAK['bf16'], 4), 'core_clock_MHz': round(mhz.value)}
    return out


def conv_through_exec(N, H, W, CI, CO, Iv, Fv, runs=6):
    """configs[1] bf16 as a Tile program through plaidml::exec: the planner's own choice of kernel, device ms per run."""
    from plaidml_amd import edsl as P, op as Pop
    I = P.Placeholder(P.DType.BFLOAT16, [N, H, W, CI])
    F = P.Placeholder(P.DType.BFLOAT16, [3, 3, CI, CO])
    B = P.Placeholder(P.DType.BFLOAT16, [CO])
    prog = P.Program('conv', [I, F, B], [Pop.relu(Pop.convolution(I, F) + B)])
    runner = P.Runner(prog, target='hip')
    bias = np.zeros(CO, np.float32)
    times = []
    for _ in range(runs):  # whole runs: upload, launch, download (the launch finds an idle device)
        runner.run([Iv, Fv, bias])
        times.append(P.last_run_stats())
    cold = sorted(times[1:], key=lambda t: t['kernel_ms'])[(len(times) - 1) // 2]
    staged = runner.stage([Iv, Fv, bias])  # and back to back on staged inputs, as a stream of batches arrives
    warm = staged_runs(runner, staged, P, runs, SETTLE_MS)
    plan = [v for k, v in prog.passes if k == 'hip-plan']
    return {'kernel_ms': round(warm['kernel_ms'], 5), 'kernel_ms_min': round(warm['kernel_ms_min'], 5), 'runs': warm['runs'],
            'kernel_ms_after_an_upload': round(cold['kernel_ms'], 5),
            'launches': int(warm['launches']), 'h2d_ms': round(cold['h2d_ms'], 3), 'd2h_ms': round(cold['d2h_ms'], 3),
            'plan': plan[0].splitlines()[1].strip() if plan else ''}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=10)
    ap.add_argument('--no-extra', action='store_true')
    ap.add_argument('--no-cpu', action='store_true')
    ap.add_argument('--copy-calibration', action='store_true')
    ap.add_argument('--only', default='', help='comma-separated legs of `extra` to run (default: all)')
    args = ap.parse_args()
    if args.gpus != 1:
        print('bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)' % args.gpus, file=sys.stderr)
        sys.exit(2)

    from plaidml_amd import edsl as P
    from plaidml_amd import hipkernels as hk

    hk.init(0)
    L = hk.lib()
    if args.copy_calibration:
        print(json.dumps(copy_calibration(hk, args.steps)))
        return
    N, H, W, CI, CO = 128, 56, 56, 64, 64
    taps = valid_taps(H, 3, 1) * valid_taps(W, 3, 1)          # valid (y,ky) x (x,kx) pairs
    flops = 2.0 * N * taps * CI * CO
    flops_full_box = 2.0 * N * H * W * 9 * CI * CO
    bytes_alg = (N * H * W * CI + N * H * W * CO) * 2 + 9 * CI * CO * 2 + CO * 2

    rng = np.random.default_rng(2)
    Iv = P.round_bf16(rng.standard_normal((N, H, W, CI)).astype(np.float32))
    Fv = P.round_bf16((np.random.default_rng(3).standard_normal((3, 3, CI, CO)) * np.sqrt(2.0 / (9 * CI))).astype(np.float32))
    # Five input / output pairs taken in turn (514 MB): a loop over one pair re-reads a 51 MB input that the 256 MB
    # last-level cache in front of HBM can hold between launches; in turn, every launch reads from HBM.
    n_pairs = 5
    bits = P.to_bf16_bits(Iv)
    pairs = [(hk.DeviceBuffer.from_numpy(bits), hk.DeviceBuffer(N * H * W * CO * 2)) for _ in range(n_pairs)]
    dI, dO = pairs[0]
    dF = hk.DeviceBuffer.from_numpy(P.to_bf16_bits(Fv))
    dB = hk.DeviceBuffer.from_numpy(np.zeros(CO, np.uint16))
    plan = conv_plan(hk, hk.BF16, N, H, W, CI, CO, 3, 3)
    none = hk.ptr_array([])
    turn = {'k': 0}

    def step():  # one batch through the convolution, filter as the caller holds it (HWCK)
        turn['k'] = (turn['k'] + 1) % n_pairs
        i_buf, o_buf = pairs[turn['k']]
        hk.check(L.pml_hip_conv2d_invoke(plan, i_buf.ptr, dF.ptr, o_buf.ptr, dB.ptr, none, none, None))

    def kernel_only():  # the same with the filter packed once, as a network's constant weights are
        turn['k'] = (turn['k'] + 1) % n_pairs
        i_buf, o_buf = pairs[turn['k']]
        hk.check(L.pml_hip_conv2d_invoke(plan, i_buf.ptr, None, o_buf.ptr, dB.ptr, none, none, None))

    def one_pair():
        hk.check(L.pml_hip_conv2d_invoke(plan, dI.ptr, None, dO.ptr, dB.ptr, none, none, None))

    ms_step, wall_step = time_loop(hk, step, args.steps, args.warmup)
    hk.check(L.pml_hip_conv2d_pack_filter(plan, dF.ptr, None))
    ms_kernel, _ = time_loop(hk, kernel_only, args.steps, args.warmup)

    result = {
        'metric': 'contraction TFLOP/s & % MFMA peak (GEMM/conv); ResNet-50 b128 fwd img/s',
        'value': round(flops / (ms_step * 1e-3) / 1e12, 3),
        'unit': 'TFLOP/s',
        'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'ms_per_step': round(ms_step, 5),
        'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'bf16', 'data': 'synthetic',
        'config': {'workload': 'configs[1]: conv2d NHWC N128 56x56x64 (*) 3x3x64x64 stride 1 SAME + bias + ReLU, bf16, fp32 accumulate',
                   'plan': hk.describe(plan), 'device': hk.device_name(),
                   'input_output_pairs_in_turn': n_pairs, 'algorithmic_gflop': round(flops / 1e9, 3), 'full_box_gflop': round(flops_full_box / 1e9, 3),
                   'host_wall_ms_per_step': round(wall_step, 5), 'settle_ms_before_timing': SETTLE_MS},
        'roofline': {'bound': 'mfma', 'achieved': round(flops / (ms_kernel * 1e-3) / 1e12, 3), 'peak': PEAK['bf16'],
                     'unit': 'TFLOP/s', 'frac': round(flops / (ms_kernel * 1e-3) / 1e12 / PEAK['bf16'], 4),
                     'traffic': committed_traffic(), 'kernel': hk.describe(plan).split('tile=')[-1], 'kernel_ms': round(ms_kernel, 5),
                     'hbm_GBps_at_algorithmic_bytes': round(bytes_alg / (ms_kernel * 1e-3) / 1e9, 1),
                     'hbm_frac': round(bytes_alg / (ms_kernel * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
    }

    # what the matrix cores of this device sustain on random bf16 operands that never leave LDS (the clock the chip holds
    # under real data): the same achieved figure against that ceiling, beside the fraction of the published peak
    probe = mfma_ceiling_leg(hk)
    sustained = probe['random_operands']['TFLOP/s']
    result['roofline']['frac_of_sustained'] = round(result['roofline']['achieved'] / sustained, 4)
    result['roofline']['sustained_peak'] = {'TFLOP/s': sustained, 'core_clock_MHz': probe['random_operands']['core_clock_MHz'],
                                            'what': 'pml_hip_probe_mfma, random bf16 operands resident in LDS'}

    # spot check of the timed output against the CPU baseline on the sampled images
    if not args.no_cpu:
        n_s = 4
        cb, ref, _, _ = cpu_baseline_conv(n_s, H, W, CI, CO, 2, 3, flops / N)
        got = P.from_bf16_bits(dO.to_numpy(np.uint16, (N, H, W, CO)))[:n_s]
        if not np.allclose(got, ref, rtol=2e-2, atol=2e-2):
            raise SystemExit('bench: GPU output disagrees with the CPU baseline on the sampled images')
        result['cpu_baseline'] = cb
    else:
        result['cpu_baseline'] = None

    if not args.no_extra:
        only = set(x for x in args.only.split(',') if x)
        want = lambda name: not only or name in only  # noqa: E731
        extra = {}
        if want('conv_one_pair'):
            # the same kernel over ONE input / output pair (what the last-level cache can hold): the cache-resident figure
            ms, _ = time_loop(hk, one_pair, args.steps, args.warmup)
            extra['conv_bf16_configs1_one_buffer_pair'] = {
                'ms': round(ms, 5), 'TFLOP/s': round(flops / ms / 1e9, 2), 'frac_mfma_bf16': round(flops / ms / 1e9 / PEAK['bf16'], 4),
                'hbm_GBps_at_algorithmic_bytes': round(bytes_alg / (ms * 1e-3) / 1e9, 1)}
        if want('conv_exec'):
            extra['conv_bf16_configs1_through_exec'] = conv_through_exec(N, H, W, CI, CO, Iv, Fv)
            e = extra['conv_bf16_configs1_through_exec']
            e['TFLOP/s'] = round(flops / e['kernel_ms'] / 1e9, 2)
        if want('conv_f32'):
            # configs[1] in fp32: with fp32 MFMAs, and with every operand value split into a bf16 head + remainder in
            # registers (three bf16 MFMAs per term, rtol 1e-3 kept: tests/test_kernels_gpu.py)
            dI32 = hk.DeviceBuffer.from_numpy(Iv)
            dF32 = hk.DeviceBuffer.from_numpy(Fv)
            dB32 = hk.DeviceBuffer.from_numpy(np.zeros(CO, np.float32))
            dO32 = hk.DeviceBuffer(N * H * W * CO * 4)
            for name, flags in (('conv_f32_configs1', 0), ('conv_f32_as_bf16x3_configs1', hk.FP32_AS_BF16X3)):
                p32 = conv_plan(hk, hk.F32, N, H, W, CI, CO, 3, 3, flags=flags)
                ms, _ = time_loop(hk, lambda: hk.check(L.pml_hip_conv2d_invoke(p32, dI32.ptr, dF32.ptr, dO32.ptr, dB32.ptr, none, none, None)),
                                  max(5, args.steps // 5), 3)
                extra[name] = dict({'ms': round(ms, 4), 'TFLOP/s': round(flops / ms / 1e9, 2)}, **fp32_fraction(flops / ms / 1e9, flags),
                                   plan=hk.describe(p32))
                L.pml_hip_plan_free(p32)
            for b in (dI32, dF32, dB32, dO32):
                b.free()
        if want('gemm_f32'):
            # configs[0]: fp32 GEMM 1024^3, B as the program gives it ([K][N], re-laid per run); both fp32 modes
            A = np.random.default_rng(1).uniform(-1, 1, (1024, 1024)).astype(np.float32)
            dA, dBm, dC = hk.DeviceBuffer.from_numpy(A), hk.DeviceBuffer.from_numpy(A.T.copy()), hk.DeviceBuffer(4 << 20)
            for name, flags in (('gemm_f32_1024_configs0', 0), ('gemm_f32_as_bf16x3_1024_configs0', hk.FP32_AS_BF16X3)):
                g = hk.GemmDesc()
                g.in_dtype = g.out_dtype = g.c_dtype = hk.F32
                g.m = g.n = g.k = g.lda = g.ldb = g.ldc = 1024
                g.flags = flags
                pg = L.pml_hip_gemm_dispatch(ctypes.byref(g))
                ms, _ = time_loop(hk, lambda: hk.check(L.pml_hip_gemm_invoke(pg, dA.ptr, dBm.ptr, dC.ptr, None, none, none, None)), 50, 10)
                extra[name] = dict({'ms': round(ms, 4), 'TFLOP/s': round(2 * 1024 ** 3 / ms / 1e9, 2)},
                                   **fp32_fraction(2 * 1024 ** 3 / ms / 1e9, flags), plan=hk.describe(pg))
                L.pml_hip_plan_free(pg)
            for b in (dA, dBm, dC):
                b.free()
        if want('gemm_i8'):
            extra['gemm_i8_4096_b_as_nk'] = gemm_leg(hk, 'i8')
            extra['gemm_i8_4096_configs2_b_as_kn'] = gemm_leg(hk, 'i8', b_nk=False)
        if want('gemm_bf16'):
            extra['gemm_bf16_4096_b_as_nk'] = gemm_leg(hk, 'bf16')
            extra['gemm_bf16_4096_b_as_kn'] = gemm_leg(hk, 'bf16', b_nk=False)
        if want('mfma_ceiling'):
            extra['mfma_ceiling_bf16'] = probe
        if want('int8_program'):
            # configs[2] as a Tile program through the plaidml API: cast -> contraction (si32, first output) with the
            # fused per-column requantisation tail (si8, second output); B is a program input, so it is re-laid per run
            extra['int8_gemm_requant_program_configs2'] = int8_program_leg()
        if want('xception'):
            extra['xception_block_configs3'] = xception_leg(hk, L, none)
        if want('resnet50'):
            # configs[4]: ResNet-50 v1.5, batch 128, bf16, through the plaidml API (weights are program constants)
            extra['resnet50_v1_5_b128_bf16'] = resnet50_leg()
            result['resnet50_b128_img_per_s'] = extra['resnet50_v1_5_b128_bf16']['img_per_s']
        if want('resnet50_b1'):
            # the same network on one image: latency (few tiles per layer: the K loops of the long-K layers are split
            # over workgroups, the launches replayed as one graph)
            extra['resnet50_v1_5_b1_bf16'] = resnet50_leg(batch=1, runs=20)
        result['extra'] = extra

    print(json.dumps(result))


if __name__ == '__main__':
    main()
