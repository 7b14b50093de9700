// Bandwidth-bound window kernels over NHWC tensors: depthwise convolution and
// pooling (with the optional window-argmax output).  One thread owns 16 bytes
// of channels (8 bf16 / 4 fp32) of one output pixel; consecutive threads walk
// the channel vectors of a pixel, then the next pixel, so every global access
// of a wavefront is a run of contiguous 16-byte pieces.  The KHxKW taps of
// neighbouring outputs overlap and are served by L1/L2, so HBM sees each input
// byte about once.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "device_common.h"
#include "plans.h"

namespace pml {

namespace {

template <int ES>
struct VecIO;
template <>
struct VecIO<2> {
  static constexpr int V = 8;
  __device__ static void load(const void* p, int64_t elem_off, float* f) {
    i32x4_t raw = *(const i32x4_t*)((const uint16_t*)p + elem_off);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(((uint32_t)raw[i]) << 16);
      f[2 * i + 1] = __uint_as_float(((uint32_t)raw[i]) & 0xffff0000u);
    }
  }
};
template <>
struct VecIO<4> {
  static constexpr int V = 4;
  __device__ static void load(const void* p, int64_t elem_off, float* f) {
    f32x4_t raw = *(const f32x4_t*)((const float*)p + elem_off);
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = raw[i];
  }
};

// Eight fp32 values to eight bf16 (hardware conversion: round to nearest even, NaN quieted), one 16-byte vector.
__device__ __forceinline__ i32x4_t pack_bf16_rne(const float* v) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  i32x4_t o;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const bf16x2 h = __builtin_convertvector(f32x2{v[2 * q], v[2 * q + 1]}, bf16x2);
    uint32_t w;
    __builtin_memcpy(&w, &h, 4);
    o[q] = (int)w;
  }
  return o;
}

template <int ES>
__global__ __launch_bounds__(256) void dwconv2d_kernel(DwconvArgs a, int64_t total_vecs) {
  constexpr int V = VecIO<ES>::V;
  const pml_hip_dwconv2d_desc& d = a.d;
  const int dt = d.dtype;
  const int64_t cvecs = d.c / V;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t g = (int64_t)xcd_contiguous_block(blockIdx.x, gridDim.x) * blockDim.x + threadIdx.x; g < total_vecs; g += stride) {
    const int64_t cv = g % cvecs;
    const int64_t pix = g / cvecs;
    const int ox = (int)(pix % d.ow);
    const int64_t t = pix / d.ow;
    const int oy = (int)(t % d.oh);
    const int64_t n = t / d.oh;
    const int64_t c0 = cv * V;
    float acc[V];
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = 0.f;
    // The taps are walked in groups of kGroup: all loads of a group (input and filter; taps outside
    // the image read the tensor's first vector and are ignored) are issued before the first product.
    constexpr int kGroup = 9;
    const int taps = (int)(d.kh * d.kw);
    const int64_t iy0 = (int64_t)oy * d.stride_h - d.pad_h, ix0 = (int64_t)ox * d.stride_w - d.pad_w;
    int ky = 0, kx = 0;
    for (int k0 = 0; k0 < taps; k0 += kGroup) {
      float x[kGroup][V], w[kGroup][V];
      bool ok[kGroup];
#pragma unroll
      for (int u = 0; u < kGroup; ++u) {
        const int64_t iy = iy0 + (int64_t)ky * d.dil_h, ix = ix0 + (int64_t)kx * d.dil_w;
        ok[u] = k0 + u < taps && iy >= 0 && iy < d.h && ix >= 0 && ix < d.w;
        VecIO<ES>::load(a.in, ok[u] ? ((n * d.h + iy) * d.w + ix) * d.c + c0 : 0, x[u]);
        VecIO<ES>::load(a.filter, ok[u] ? (int64_t)(k0 + u) * d.c + c0 : 0, w[u]);
        if (++kx == d.kw) {
          kx = 0;
          ++ky;
        }
      }
#pragma unroll
      for (int u = 0; u < kGroup; ++u) {
        if (!ok[u]) continue;
#pragma unroll
        for (int i = 0; i < V; ++i) acc[i] += x[u][i] * w[u][i];
      }
    }
    const int64_t o0 = pix * (d.out_pitch ? (int64_t)d.out_pitch : d.c) + c0;  // a pitch other than c comes without a tail
    if (d.tail.n_ops == 0 && (dt == PML_HIP_BF16 || dt == PML_HIP_F32)) {
      // no tail: one 16-byte store of the rounded values
      if constexpr (ES == 2) {
        i32x4_t o;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          o[i] = (int)((uint32_t)f32_to_bf16_bits(acc[2 * i]) | ((uint32_t)f32_to_bf16_bits(acc[2 * i + 1]) << 16));
        *(i32x4_t*)((uint16_t*)a.out + o0) = o;
      } else {
        const f32x4_t o = {acc[0], acc[1], acc[2], acc[3]};
        *(f32x4_t*)((float*)a.out + o0) = o;
      }
      continue;
    }
#pragma unroll
    for (int i = 0; i < V; ++i) {
      Scalar<float, int> v;
      v.i = 0;
      v.f = round_float_to<float>(dt, acc[i]);
      int cur = dt;
      int64_t off[PML_HIP_MAX_EPI_OPERANDS];
#pragma unroll
      for (int q = 0; q < PML_HIP_MAX_EPI_OPERANDS; ++q)
        off[q] = q < d.tail.n_operands ? pix * d.tail.operand_row_stride[q] + (c0 + i) * d.tail.operand_col_stride[q] : 0;
      v = run_tail<float, int>(d.tail, v, &cur, a.operands, off, a.outs, o0 + i);
      store_scalar<float, int>(a.out, o0 + i, cur, v);
    }
  }
}

// 3x3 depthwise convolution, unit stride and dilation, no tail: a thread computes kDwPx neighbouring
// output pixels of a row for one 16-byte channel vector, so the three rows of kDwPx + 2 input vectors
// it loads serve all of them and the nine filter vectors are loaded once (27 loads for 4 outputs
// instead of 72).  A tap outside the image takes no part in the sum (it is not multiplied by zero).
constexpr int kDwPx = 4;
// IT: the integer type of the index arithmetic.  Element counts below 2^31 (checked by the launcher) take
// 32-bit arithmetic: a thread's three divisions and its address sums are a fifth of the 64-bit cost, and on a
// 19x19x728 image the kernel is bound by its instruction count, not by memory.
// (165 registers, three wavefronts per SIMD: capping the registers for four or more made the compiler spill and the
// kernel two to four times slower.)
template <int ES, typename IT>
__global__ __launch_bounds__(256) void dwconv3x3_kernel(DwconvArgs a, int64_t total) {
  constexpr int V = VecIO<ES>::V;
  const pml_hip_dwconv2d_desc& d = a.d;
  const IT cvecs = (IT)(d.c / V);
  const IT xblocks = (IT)((d.ow + kDwPx - 1) / kDwPx);
  const IT oh = (IT)d.oh, H = (IT)d.h, W = (IT)d.w, C = (IT)d.c;
  const IT CO = d.out_pitch ? (IT)d.out_pitch : C;  // elements between two output pixels
  const int pad_h = (int)d.pad_h, pad_w = (int)d.pad_w;
  const IT stride = (IT)gridDim.x * blockDim.x;
  for (IT g = (IT)xcd_contiguous_block(blockIdx.x, gridDim.x) * blockDim.x + threadIdx.x; g < (IT)total; g += stride) {
    const IT cv = g % cvecs;
    IT t = g / cvecs;
    const int ox0 = (int)(t % xblocks) * kDwPx;
    t /= xblocks;
    const int oy = (int)(t % oh);
    const IT n = t / oh;
    const IT c0 = cv * V;
    const int iy0 = oy - pad_h, ix0 = ox0 - pad_w;
    i32x4_t xr[3][kDwPx + 2], wr[9];
    bool ok[3][kDwPx + 2];
#pragma unroll
    for (int k = 0; k < 9; ++k) wr[k] = *(const i32x4_t*)((const unsigned char*)a.filter + ((int64_t)((IT)k * C + c0)) * ES);
    // the whole 3 x (kDwPx + 2) window inside the image: one base offset, constant steps, no per-tap checks
    const bool all_ok = iy0 >= 0 && iy0 + 2 < (int)H && ix0 >= 0 && ix0 + kDwPx + 1 < (int)W;
    if (all_ok) {
      const IT base = ((n * H + (IT)iy0) * W + (IT)ix0) * C + c0;
#pragma unroll
      for (int ky = 0; ky < 3; ++ky)
#pragma unroll
        for (int c = 0; c < kDwPx + 2; ++c)
          xr[ky][c] = *(const i32x4_t*)((const unsigned char*)a.in + (int64_t)(base + ((IT)ky * W + (IT)c) * C) * ES);
    } else {
#pragma unroll
      for (int ky = 0; ky < 3; ++ky) {
        const int iy = iy0 + ky;
#pragma unroll
        for (int c = 0; c < kDwPx + 2; ++c) {
          const int ix = ix0 + c;
          ok[ky][c] = iy >= 0 && iy < (int)H && ix >= 0 && ix < (int)W;
          const IT off = ok[ky][c] ? ((n * H + (IT)iy) * W + (IT)ix) * C + c0 : 0;
          xr[ky][c] = *(const i32x4_t*)((const unsigned char*)a.in + (int64_t)off * ES);
        }
      }
    }
    auto unpack = [](const i32x4_t& raw, float* f) {
      if constexpr (ES == 2) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          f[2 * i] = __uint_as_float(((uint32_t)raw[i]) << 16);
          f[2 * i + 1] = __uint_as_float(((uint32_t)raw[i]) & 0xffff0000u);
        }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = __int_as_float(raw[i]);
      }
    };
    float acc[kDwPx][V];
#pragma unroll
    for (int px = 0; px < kDwPx; ++px)
#pragma unroll
      for (int i = 0; i < V; ++i) acc[px][i] = 0.f;
    // taps in the reference's order (ky outer, kx inner) for every pixel
    auto accumulate = [&](auto checked) {
#pragma unroll
      for (int ky = 0; ky < 3; ++ky) {
        float w[3][V];
#pragma unroll
        for (int kx = 0; kx < 3; ++kx) unpack(wr[ky * 3 + kx], w[kx]);
#pragma unroll
        for (int c = 0; c < kDwPx + 2; ++c) {
          if (decltype(checked)::value && !ok[ky][c]) continue;
          float x[V];
          unpack(xr[ky][c], x);
#pragma unroll
          for (int kx = 0; kx < 3; ++kx) {
            const int px = c - kx;
            if (px < 0 || px >= kDwPx) continue;
#pragma unroll
            for (int i = 0; i < V; ++i) acc[px][i] += x[i] * w[kx][i];
          }
        }
      }
    };
    if (all_ok)
      accumulate(std::false_type());
    else
      accumulate(std::true_type());
    const IT orow = ((n * oh + (IT)oy) * (IT)d.ow + (IT)ox0) * CO + c0;
#pragma unroll
    for (int px = 0; px < kDwPx; ++px) {
      if (ox0 + px >= (int)d.ow) break;
      const int64_t o0 = (int64_t)(orow + (IT)px * CO);
      if constexpr (ES == 2) {
        *(i32x4_t*)((uint16_t*)a.out + o0) = pack_bf16_rne(acc[px]);
      } else {
        const f32x4_t o = {acc[px][0], acc[px][1], acc[px][2], acc[px][3]};
        *(f32x4_t*)((float*)a.out + o0) = o;
      }
    }
  }
}

// The same work for tensors below 2 GiB, as one straight line of code for interior and border pixels alike.
// The input is read through a buffer descriptor: a tap outside the image gets an offset beyond the buffer and
// arrives as zeros, so no lane branches around it and a wavefront whose lanes sit on both sides of an image border
// does not run two code paths one after the other.  A zero times a finite weight adds nothing, which is what
// leaving the tap out means; only a weight that is infinite or NaN would turn such a zero into NaN.  Every lane
// therefore looks at its nine filter vectors once, and the (rare) lanes that hold such a weight and sit on a border
// redo their sums from the same registers with the outside taps left out.  Indices come from multiply-and-shift
// divisions prepared on the host.
struct DwFlatArgs {
  unsigned total;      // threads with work: images x rows x pixel blocks x channel vectors
  unsigned cvecs, xblocks, oh;
  unsigned cv_magic, xb_magic, oh_magic;
  int cv_shift, xb_shift, oh_shift;
  unsigned in_bytes;
};

template <int ES>
__global__ __launch_bounds__(256, 3) void dwconv3x3_flat_kernel(DwconvArgs a, DwFlatArgs f) {
  constexpr int V = VecIO<ES>::V;
  constexpr int kCols = kDwPx + 2;
  const pml_hip_dwconv2d_desc& d = a.d;
  const unsigned g = xcd_contiguous_block(blockIdx.x, gridDim.x) * 256u + threadIdx.x;
  if (g >= f.total) return;
  const unsigned t1 = fast_div(g, f.cv_magic, f.cv_shift), cv = g - t1 * f.cvecs;
  const unsigned t2 = fast_div(t1, f.xb_magic, f.xb_shift), xb = t1 - t2 * f.xblocks;
  const unsigned n = fast_div(t2, f.oh_magic, f.oh_shift), oy = t2 - n * f.oh;
  const int H = (int)d.h, W = (int)d.w;
  const unsigned pix_bytes = (unsigned)d.c * ES, c0b = cv * 16u;
  const int ox0 = (int)xb * kDwPx, iy0 = (int)oy - (int)d.pad_h, ix0 = ox0 - (int)d.pad_w;
  constexpr unsigned kOutside = 0x80000000u;  // beyond any buffer this kernel is launched for

  i32x4_t wr[9];
#pragma unroll
  for (int k = 0; k < 9; ++k) wr[k] = *(const i32x4_t*)((const unsigned char*)a.filter + (unsigned)k * pix_bytes + c0b);

  const __amdgpu_buffer_rsrc_t rin = __builtin_amdgcn_make_buffer_rsrc((void*)a.in, 0, (int)f.in_bytes, 0x00020000u);
  bool row_ok[3], col_ok[kCols];
  unsigned col_off[kCols];
#pragma unroll
  for (int c = 0; c < kCols; ++c) {
    col_ok[c] = (unsigned)(ix0 + c) < (unsigned)W;
    col_off[c] = col_ok[c] ? (unsigned)(ix0 + c) * pix_bytes + c0b : kOutside;
  }
  i32x4_t xr[3][kCols];
  auto load_row = [&](int ky) {
    const unsigned row = row_ok[ky] ? (n * (unsigned)H + (unsigned)(iy0 + ky)) * (unsigned)W * pix_bytes : kOutside;
#pragma unroll
    for (int c = 0; c < kCols; ++c)  // an offset with the top bit set lies beyond the buffer
      xr[ky][c] = __builtin_amdgcn_raw_buffer_load_b128(rin, (int)(row | col_off[c]) < 0 ? (int)kOutside : (int)(row + col_off[c]), 0, 0);
  };
#pragma unroll
  for (int ky = 0; ky < 3; ++ky) row_ok[ky] = (unsigned)(iy0 + ky) < (unsigned)H;
  // The third window row is requested after the first has been used, into the registers the first leaves free; it
  // arrives during the second row's arithmetic.  With all three up front the kernel needs more than the 168
  // registers that let three wavefronts share a SIMD.
  load_row(0);
  load_row(1);

  // does this lane hold a weight that is infinite or NaN (all exponent bits set)?
  unsigned odd = 0;
#pragma unroll
  for (int k = 0; k < 9; ++k)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const unsigned w = (unsigned)wr[k][i];
      if constexpr (ES == 2)
        odd |= ((w & 0x7f807f80u) + 0x00800080u) & 0x80008000u;  // a carry out of either exponent field
      else
        odd |= ((w & 0x7f800000u) + 0x00800000u) & 0x80000000u;
    }

  auto unpack = [](const i32x4_t& raw, float* o) {
    if constexpr (ES == 2) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        o[2 * i] = __uint_as_float(((uint32_t)raw[i]) << 16);
        o[2 * i + 1] = __uint_as_float(((uint32_t)raw[i]) & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = __int_as_float(raw[i]);
    }
  };
  float acc[kDwPx][V];
  // taps in the reference's order (ky outer, kx inner) for every pixel
  auto accumulate = [&](auto checked) {
#pragma unroll
    for (int px = 0; px < kDwPx; ++px)
#pragma unroll
      for (int i = 0; i < V; ++i) acc[px][i] = 0.f;
#pragma unroll
    for (int ky = 0; ky < 3; ++ky) {
      // (the second pass reads its operands through an empty asm: shared subexpressions of the two passes would
      // otherwise keep every unpacked value of the first alive for the second)
      auto fresh = [](i32x4_t v) {
        if (decltype(checked)::value) asm volatile("" : "+v"(v));
        return v;
      };
      float w[3][V];
#pragma unroll
      for (int kx = 0; kx < 3; ++kx) unpack(fresh(wr[ky * 3 + kx]), w[kx]);
#pragma unroll
      for (int c = 0; c < kCols; ++c) {
        if (decltype(checked)::value && !(row_ok[ky] && col_ok[c])) continue;
        float x[V];
        unpack(fresh(xr[ky][c]), x);
#pragma unroll
        for (int kx = 0; kx < 3; ++kx) {
          const int px = c - kx;
          if (px < 0 || px >= kDwPx) continue;
#pragma unroll
          for (int i = 0; i < V; ++i) acc[px][i] += x[i] * w[kx][i];
        }
      }
      // one filter row at a time: unpacked values of later rows would only take registers
      __builtin_amdgcn_sched_barrier(0);
      if (!decltype(checked)::value && ky == 0) {
        load_row(2);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  accumulate(std::false_type());
  const bool border = !(row_ok[0] && row_ok[2] && col_ok[0] && col_ok[kCols - 1]);
  if (odd != 0 && border) {
    // everything again from memory (the registers of the first pass have been given up by now)
#pragma unroll
    for (int k = 0; k < 9; ++k) wr[k] = *(const i32x4_t*)((const unsigned char*)a.filter + (unsigned)k * pix_bytes + c0b);
    load_row(0);
    load_row(1);
    load_row(2);
    accumulate(std::true_type());
  }

  const unsigned opix_bytes = (d.out_pitch ? (unsigned)d.out_pitch : (unsigned)d.c) * ES;
  const unsigned orow = ((n * f.oh + oy) * (unsigned)d.ow + (unsigned)ox0) * opix_bytes + c0b;
#pragma unroll
  for (int px = 0; px < kDwPx; ++px) {
    if (ox0 + px >= (int)d.ow) break;
    unsigned char* o = (unsigned char*)a.out + orow + (unsigned)px * opix_bytes;
    if constexpr (ES == 2) {
      *(i32x4_t*)o = pack_bf16_rne(acc[px]);
    } else {
      const f32x4_t v = {acc[px][0], acc[px][1], acc[px][2], acc[px][3]};
      *(f32x4_t*)o = v;
    }
  }
}

// The same arithmetic with the window rows kept in registers while a thread walks down the image: a thread owns two
// neighbouring output pixels (16 bytes of channels each) of a run of output rows.  Every step fetches one input row of
// four vectors and uses it for the three output rows it touches -- filter row 0 of the row below it, 1 of its own, 2
// of the row above -- so an input vector is fetched 2 to 2.4 times over the walk where the kernels above fetch it 4.5
// times, is unpacked once for nine taps, and the weights are unpacked once per thread.  Three sets of sums are in
// flight; a set gets its taps in the reference's order (filter row 0 first, columns rising), so the sums are the
// ones dwconv3x3_flat_kernel forms, bit for bit.  Rows are fetched three steps ahead.  Lanes that hold an infinite or
// NaN weight take a plain loop with the outside taps left out (see above); the others rely on outside taps reading
// zeros.
struct DwWalkArgs {
  unsigned total;  // threads with work: images x row segments x pixel pairs x channel vectors
  unsigned cvecs, xblocks, ysegs, seg_rows;
  unsigned cv_magic, xb_magic, ys_magic;
  int cv_shift, xb_shift, ys_shift;
  unsigned in_bytes;
};

template <int ES>
__global__ __launch_bounds__(256, 2) void dwconv3x3_walk_kernel(DwconvArgs a, DwWalkArgs f) {
  constexpr int V = VecIO<ES>::V;
  constexpr int kPx = 2, kCols = kPx + 2;
  const pml_hip_dwconv2d_desc& d = a.d;
  const unsigned g = xcd_contiguous_block(blockIdx.x, gridDim.x) * 256u + threadIdx.x;
  if (g >= f.total) return;
  const unsigned t1 = fast_div(g, f.cv_magic, f.cv_shift), cv = g - t1 * f.cvecs;
  const unsigned t2 = fast_div(t1, f.xb_magic, f.xb_shift), xb = t1 - t2 * f.xblocks;
  const unsigned n = fast_div(t2, f.ys_magic, f.ys_shift), ys = t2 - n * f.ysegs;
  const int H = (int)d.h, W = (int)d.w, OH = (int)d.oh, OW = (int)d.ow;
  const unsigned pix_bytes = (unsigned)d.c * ES, c0b = cv * 16u;
  const int oy0 = (int)(ys * f.seg_rows), ox0 = (int)xb * kPx;
  const int iy0 = oy0 - (int)d.pad_h, ix0 = ox0 - (int)d.pad_w;
  const int rows = OH - oy0 < (int)f.seg_rows ? OH - oy0 : (int)f.seg_rows;  // output rows of this thread
  const unsigned opix_bytes = (d.out_pitch ? (unsigned)d.out_pitch : (unsigned)d.c) * ES;
  unsigned char* const out0 = (unsigned char*)a.out + ((n * (unsigned)OH + (unsigned)oy0) * (unsigned)OW + (unsigned)ox0) * opix_bytes + c0b;
  const unsigned orow_bytes = (unsigned)OW * opix_bytes;

  i32x4_t wr[9];
#pragma unroll
  for (int k = 0; k < 9; ++k) wr[k] = *(const i32x4_t*)((const unsigned char*)a.filter + (unsigned)k * pix_bytes + c0b);
  unsigned odd = 0;  // a weight that is infinite or NaN (all exponent bits set)?
#pragma unroll
  for (int k = 0; k < 9; ++k)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const unsigned w = (unsigned)wr[k][i];
      if constexpr (ES == 2)
        odd |= ((w & 0x7f807f80u) + 0x00800080u) & 0x80008000u;  // a carry out of either exponent field
      else
        odd |= ((w & 0x7f800000u) + 0x00800000u) & 0x80000000u;
    }
  auto unpack = [](const i32x4_t& raw, float* o) {
    if constexpr (ES == 2) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        o[2 * i] = __uint_as_float(((uint32_t)raw[i]) << 16);
        o[2 * i + 1] = __uint_as_float(((uint32_t)raw[i]) & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = __int_as_float(raw[i]);
    }
  };
  auto store = [&](int r, int px, const float* v) {
    unsigned char* o = out0 + (unsigned)r * orow_bytes + (unsigned)px * opix_bytes;
    if constexpr (ES == 2) {
      *(i32x4_t*)o = pack_bf16_rne(v);
    } else {
      *(f32x4_t*)o = f32x4_t{v[0], v[1], v[2], v[3]};
    }
  };
  float w[9][V];
#pragma unroll
  for (int k = 0; k < 9; ++k) unpack(wr[k], w[k]);

  if (odd != 0) {
    // pixel by pixel, every tap checked
    for (int r = 0; r < rows; ++r)
      for (int px = 0; px < kPx; ++px) {
        if (ox0 + px >= OW) break;
        float acc[V];
#pragma unroll
        for (int i = 0; i < V; ++i) acc[i] = 0.f;
#pragma unroll
        for (int ky = 0; ky < 3; ++ky)
#pragma unroll
          for (int kx = 0; kx < 3; ++kx) {
            const int iy = iy0 + r + ky, ix = ix0 + px + kx;
            if ((unsigned)iy >= (unsigned)H || (unsigned)ix >= (unsigned)W) continue;
            float x[V];
            unpack(*(const i32x4_t*)((const unsigned char*)a.in + ((n * (unsigned)H + (unsigned)iy) * (unsigned)W + (unsigned)ix) * pix_bytes + c0b), x);
#pragma unroll
            for (int i = 0; i < V; ++i) acc[i] += x[i] * w[ky * 3 + kx][i];
          }
        store(r, px, acc);
      }
    return;
  }

  // A tap outside the image must read zeros: its offset is made to lie beyond the buffer.  Rows and columns carry
  // different marks, so that their plain sum is beyond the buffer whenever either is marked and never wraps around
  // (the input is smaller than 1 GiB here).
  constexpr unsigned kRowOutside = 0x80000000u, kColOutside = 0x40000000u;
  const __amdgpu_buffer_rsrc_t rin = __builtin_amdgcn_make_buffer_rsrc((void*)a.in, 0, (int)f.in_bytes, 0x00020000u);
  unsigned col_off[kCols];
#pragma unroll
  for (int c = 0; c < kCols; ++c) col_off[c] = (unsigned)(ix0 + c) < (unsigned)W ? (unsigned)(ix0 + c) * pix_bytes + c0b : kColOutside;
  const unsigned in_row_bytes = (unsigned)W * pix_bytes;
  i32x4_t xr[3][kCols];
  auto load_row = [&](int slot, int k) {  // input row iy0 + k
    const int iy = iy0 + k;
    const unsigned row = (unsigned)iy < (unsigned)H ? (n * (unsigned)H + (unsigned)iy) * in_row_bytes : kRowOutside;
#pragma unroll
    for (int c = 0; c < kCols; ++c) xr[slot][c] = __builtin_amdgcn_raw_buffer_load_b128(rin, (int)(row + col_off[c]), 0, 0);
  };
  const int seg_rows = (int)f.seg_rows, steps = seg_rows + 2;  // the same for every thread
  load_row(0, 0);
  load_row(1, 1);
  load_row(2, 2);
  float acc[3][kPx][V];
  // filter row KY of the input row in x, added to one set of sums
  auto taps = [&](auto ky_tag, float (&sum)[kPx][V], const float (&x)[kCols][V]) {
    constexpr int KY = decltype(ky_tag)::value;
    if (KY == 0) {
#pragma unroll
      for (int px = 0; px < kPx; ++px)
#pragma unroll
        for (int i = 0; i < V; ++i) sum[px][i] = 0.f;
    }
#pragma unroll
    for (int c = 0; c < kCols; ++c)
#pragma unroll
      for (int kx = 0; kx < 3; ++kx) {
        const int px = c - kx;
        if (px < 0 || px >= kPx) continue;
#pragma unroll
        for (int i = 0; i < V; ++i) sum[px][i] += x[c][i] * w[KY * 3 + kx][i];
      }
  };
  for (int k = 0; k < steps; k += 3) {
#pragma unroll
    for (int u = 0; u < 3; ++u) {
      const int kk = k + u;  // the step: input row iy0 + kk, in slot u
      if (kk >= steps) break;
      float x[kCols][V];
#pragma unroll
      for (int c = 0; c < kCols; ++c) unpack(xr[u][c], x[c]);
      if (kk + 3 < steps) load_row(u, kk + 3);
      // output row kk starts its sums, row kk - 1 goes on, row kk - 2 ends
      if (kk < seg_rows) taps(std::integral_constant<int, 0>(), acc[u], x);
      if (kk >= 1 && kk - 1 < seg_rows) taps(std::integral_constant<int, 1>(), acc[(u + 2) % 3], x);
      if (kk >= 2) {
        taps(std::integral_constant<int, 2>(), acc[(u + 1) % 3], x);
        if (kk - 2 < rows) {
#pragma unroll
          for (int px = 0; px < kPx; ++px)
            if (ox0 + px < OW) store(kk - 2, px, acc[(u + 1) % 3][px]);
        }
      }
    }
  }
}

// The bf16 case with a filter packed once (dw_pack_filter below), all of whose weights are finite.  Two things go
// away: the look at the weights for infinities (made once, when the filter is packed: a filter that has one keeps the
// kernel above), and most of the bf16 -> fp32 unpacking, which was half of the arithmetic.  The taps of filter rows 0
// and 1 that lie above each other are multiplied as a pair: one byte-permute puts a channel's two input values (row
// y, row y + 1, same column) side by side in a register, the packed filter holds that channel's two weights the same
// way, and v_dot2_f32_bf16 adds both products to the fp32 sum in one instruction.  Filter row 2 is kept as fp32
// weights and multiplied the plain way.  Per thread (8 channels x 4 pixels): 48 permutes + 96 paired multiply-adds +
// 48 unpacks + 96 multiply-adds, against 216 unpacks + 288 multiply-adds + 108 for the weight check before.
// Packed filter: 12 vectors of 16 bytes per channel vector cv, vector j at (j * cvecs + cv) * 16 --
//   j = 2 kx + h      (kx = 0..2, h = 0..1): words {w[0][kx][c], w[1][kx][c]} as bf16 pairs, channels 8 cv + 4 h .. + 3
//   j = 6 + 2 kx + h: w[2][kx][c] as fp32, the same channels.
// WLDS: the workgroups stay (the grid is what the device holds at once) and walk over their share of the work
// blocks; the packed filter is copied into LDS once per workgroup and every thread takes its twelve vectors from
// there.  The vector memory path, which moves 64 bytes per clock and CU, then carries the 18 input vectors of a
// thread only, not 30; it is what this kernel waits for once the arithmetic is halved.
template <bool WLDS>
__global__ __launch_bounds__(256, 3) void dwconv3x3_flat_paired_kernel(DwconvArgs a, DwFlatArgs f, const i32x4_t* __restrict__ pw_global,
                                                                       unsigned nblocks) {
  constexpr int V = 8, ES = 2;
  constexpr int kCols = kDwPx + 2;
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  const pml_hip_dwconv2d_desc& d = a.d;
  extern __shared__ __attribute__((aligned(16))) unsigned char dw_smem[];
  const i32x4_t* pw = pw_global;
  if constexpr (WLDS) {
    for (unsigned q = threadIdx.x; q < 12u * f.cvecs; q += 256u) ((i32x4_t*)dw_smem)[q] = pw_global[q];
    __syncthreads();
    pw = (const i32x4_t*)dw_smem;
  }
  for (unsigned vb = blockIdx.x; vb < nblocks; vb += gridDim.x) {
  const unsigned g = xcd_contiguous_block(vb, nblocks) * 256u + threadIdx.x;
  if (g >= f.total) continue;
  const unsigned t1 = fast_div(g, f.cv_magic, f.cv_shift), cv = g - t1 * f.cvecs;
  const unsigned t2 = fast_div(t1, f.xb_magic, f.xb_shift), xb = t1 - t2 * f.xblocks;
  const unsigned n = fast_div(t2, f.oh_magic, f.oh_shift), oy = t2 - n * f.oh;
  const int H = (int)d.h, W = (int)d.w;
  const unsigned pix_bytes = (unsigned)d.c * ES, c0b = cv * 16u;
  const int ox0 = (int)xb * kDwPx, iy0 = (int)oy - (int)d.pad_h, ix0 = ox0 - (int)d.pad_w;
  // A tap outside the image must read zeros: its offset is made to lie beyond the buffer.  Rows and columns carry
  // different marks, so that their plain sum is beyond the buffer whenever either is marked and never wraps around
  // (the input is smaller than 1 GiB here): no select per load.
  constexpr unsigned kRowOutside = 0x80000000u, kColOutside = 0x40000000u;

  const __amdgpu_buffer_rsrc_t rin = __builtin_amdgcn_make_buffer_rsrc((void*)a.in, 0, (int)f.in_bytes, 0x00020000u);
  unsigned col_off[kCols];
#pragma unroll
  for (int c = 0; c < kCols; ++c) col_off[c] = (unsigned)(ix0 + c) < (unsigned)W ? (unsigned)(ix0 + c) * pix_bytes + c0b : kColOutside;
  i32x4_t xr[3][kCols];
#pragma unroll
  for (int ky = 0; ky < 3; ++ky) {
    const unsigned row = (unsigned)(iy0 + ky) < (unsigned)H ? (n * (unsigned)H + (unsigned)(iy0 + ky)) * (unsigned)W * pix_bytes : kRowOutside;
#pragma unroll
    for (int c = 0; c < kCols; ++c) xr[ky][c] = __builtin_amdgcn_raw_buffer_load_b128(rin, (int)(row + col_off[c]), 0, 0);
  }
  i32x4_t wp[3][2];
#pragma unroll
  for (int j = 0; j < 6; ++j) wp[j >> 1][j & 1] = pw[(unsigned)j * f.cvecs + cv];

  float acc[kDwPx][V];
#pragma unroll
  for (int px = 0; px < kDwPx; ++px)
#pragma unroll
    for (int i = 0; i < V; ++i) acc[px][i] = 0.f;
  // filter rows 0 and 1, a column of the window at a time
#pragma unroll
  for (int c = 0; c < kCols; ++c) {
    unsigned pair[V];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pair[2 * i] = __builtin_amdgcn_perm((unsigned)xr[1][c][i], (unsigned)xr[0][c][i], 0x05040100u);      // the even channel of both rows
      pair[2 * i + 1] = __builtin_amdgcn_perm((unsigned)xr[1][c][i], (unsigned)xr[0][c][i], 0x07060302u);  // the odd one
    }
#pragma unroll
    for (int kx = 0; kx < 3; ++kx) {
      const int px = c - kx;
      if (px < 0 || px >= kDwPx) continue;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        bf16x2 x2, w2;
        const unsigned wbits = (unsigned)wp[kx][i >> 2][i & 3];
        __builtin_memcpy(&x2, &pair[i], 4);
        __builtin_memcpy(&w2, &wbits, 4);
        acc[px][i] = __builtin_amdgcn_fdot2_f32_bf16(x2, w2, acc[px][i], false);
      }
    }
  }
  __builtin_amdgcn_sched_barrier(0);  // the fp32 weights of row 2 are fetched only now: they would only take registers before
  f32x4_t w2[3][2];
#pragma unroll
  for (int j = 0; j < 6; ++j) {
    const i32x4_t raw = pw[(unsigned)(6 + j) * f.cvecs + cv];
    w2[j >> 1][j & 1] = __builtin_bit_cast(f32x4_t, raw);
  }
#pragma unroll
  for (int c = 0; c < kCols; ++c) {
    float x[V];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[2 * i] = __uint_as_float(((uint32_t)xr[2][c][i]) << 16);
      x[2 * i + 1] = __uint_as_float(((uint32_t)xr[2][c][i]) & 0xffff0000u);
    }
#pragma unroll
    for (int kx = 0; kx < 3; ++kx) {
      const int px = c - kx;
      if (px < 0 || px >= kDwPx) continue;
#pragma unroll
      for (int i = 0; i < V; ++i) acc[px][i] += x[i] * w2[kx][i >> 2][i & 3];
    }
  }

  const unsigned opix_bytes = (d.out_pitch ? (unsigned)d.out_pitch : (unsigned)d.c) * ES;
  const unsigned orow = ((n * f.oh + oy) * (unsigned)d.ow + (unsigned)ox0) * opix_bytes + c0b;
#pragma unroll
  for (int px = 0; px < kDwPx; ++px) {
    if (ox0 + px >= (int)d.ow) break;
    *(i32x4_t*)((unsigned char*)a.out + orow + (unsigned)px * opix_bytes) = pack_bf16_rne(acc[px]);
  }
  }
}

// IT: the integer type of the index arithmetic (32 bits where every element offset stays below 2^31).
// AGG: the aggregation (PML_HIP_AGG_*), a compile-time constant so that the tap loop is straight-line code.
template <int ES, bool WITH_INDEX, typename IT, int AGG>
__global__ __launch_bounds__(256) void pool2d_kernel(PoolArgs a, int64_t total_vecs) {
  constexpr int V = VecIO<ES>::V;
  const pml_hip_pool2d_desc& d = a.d;
  const int dt = d.dtype;
  const IT cvecs = (IT)(d.c / V), ow = (IT)d.ow, oh = (IT)d.oh, H = (IT)d.h, W = (IT)d.w, C = (IT)d.c;
  const IT stride = (IT)gridDim.x * blockDim.x;
  for (IT g = (IT)xcd_contiguous_block(blockIdx.x, gridDim.x) * blockDim.x + threadIdx.x; g < (IT)total_vecs; g += stride) {
    const IT cv = g % cvecs;
    const IT pix = g / cvecs;
    const int ox = (int)(pix % ow);
    const IT t = pix / ow;
    const int oy = (int)(t % oh);
    const IT n = t / oh;
    const IT c0 = cv * V;
    float acc[V];
    int best[V];  // with_index: largest window index whose (in-range) tap equals the pooled value; 0 if none
    const float ident = AGG == PML_HIP_AGG_MAX ? -INFINITY : (AGG == PML_HIP_AGG_MIN ? INFINITY : 0.f);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      acc[i] = ident;
      best[i] = 0;
    }
    // The window is walked in groups of kGroup taps: all loads of a group are issued (taps outside the
    // image read the tensor's first vector and are ignored) before the first value is used, so a
    // thread has kGroup loads in flight instead of one.
    constexpr int kGroup = 9;
    const int taps = (int)(d.kh * d.kw);
    const int iy0 = oy * (int)d.stride_h - (int)d.pad_h, ix0 = ox * (int)d.stride_w - (int)d.pad_w;
    // the whole window inside the image: the taps' offsets are the first one's plus steps that are the same for
    // every thread
    const bool inside = iy0 >= 0 && iy0 + (int)d.kh <= (int)H && ix0 >= 0 && ix0 + (int)d.kw <= (int)W;
    const IT base = inside ? ((n * H + (IT)iy0) * W + (IT)ix0) * C + c0 : 0;
    int ky = 0, kx = 0;
    for (int k0 = 0; k0 < taps; k0 += kGroup) {
      float x[kGroup][V];
      bool ok[kGroup];
#pragma unroll
      for (int u = 0; u < kGroup; ++u) {
        const int iy = iy0 + ky, ix = ix0 + kx;
        IT off;
        if (inside) {
          ok[u] = k0 + u < taps;
          off = ok[u] ? base + ((IT)ky * W + (IT)kx) * C : 0;
        } else {
          ok[u] = k0 + u < taps && iy >= 0 && iy < (int)H && ix >= 0 && ix < (int)W;
          off = ok[u] ? ((n * H + (IT)iy) * W + (IT)ix) * C + c0 : 0;
        }
        VecIO<ES>::load(a.in, (int64_t)off, x[u]);
        if (++kx == (int)d.kw) {
          kx = 0;
          ++ky;
        }
      }
      // (a tap outside the image takes no part: its comparisons are masked, not branched around)
#pragma unroll
      for (int u = 0; u < kGroup; ++u) {
        const bool live = ok[u];
#pragma unroll
        for (int i = 0; i < V; ++i) {
          if constexpr (AGG == PML_HIP_AGG_MAX) {
            // taps come in rising window index, so ">=" leaves the largest index among equal values
            if (WITH_INDEX) best[i] = (live & (x[u][i] >= acc[i])) ? k0 + u : best[i];
            acc[i] = (live & (x[u][i] > acc[i])) ? x[u][i] : acc[i];
          } else if constexpr (AGG == PML_HIP_AGG_MIN) {
            if (WITH_INDEX) best[i] = (live & (x[u][i] <= acc[i])) ? k0 + u : best[i];
            acc[i] = (live & (x[u][i] < acc[i])) ? x[u][i] : acc[i];
          } else {
            acc[i] += live ? x[u][i] : 0.f;
          }
        }
      }
    }
    const int64_t o0 = (int64_t)(pix * C + c0);
    if (dt == PML_HIP_BF16 || dt == PML_HIP_F32) {
      // one 16-byte store of the rounded values
      if constexpr (ES == 2) {
        store_streaming((i32x4_t*)((uint16_t*)a.out + o0), pack_bf16_rne(acc));
      } else {
        const f32x4_t o = {acc[0], acc[1], acc[2], acc[3]};
        store_streaming((f32x4_t*)((float*)a.out + o0), o);
      }
    } else {
#pragma unroll
      for (int i = 0; i < V; ++i) {
        Scalar<float, int> v;
        v.i = 0;
        v.f = round_float_to<float>(dt, acc[i]);
        store_scalar<float, int>(a.out, o0 + i, dt, v);
      }
    }
    if (WITH_INDEX) {
      int32_t* ip = (int32_t*)a.idx + o0;
#pragma unroll
      for (int i = 0; i < V; i += 4) {
        i32x4_t w = {best[i], best[i + 1], best[i + 2], best[i + 3]};
        store_streaming((i32x4_t*)(ip + i), w);
      }
    }
  }
}

// Pooling windows of up to 3 x 3 taps over tensors below 2 GiB as one straight line of code: indices from
// multiply-and-shift divisions, the taps read through a buffer descriptor (a tap outside the image gets an offset
// beyond the buffer; what arrives for it is never looked at: its comparisons are masked), no loop over the window
// and no second code path for windows that cross the image border.
struct PoolFlatArgs {
  unsigned total;  // output pixels x channel vectors
  unsigned cvecs, ow, oh;
  unsigned cv_magic, ow_magic, oh_magic;
  int cv_shift, ow_shift, oh_shift;
  unsigned in_bytes;
};

template <int ES, bool WITH_INDEX, int AGG, int KH, int KW>
__global__ __launch_bounds__(256) void pool_flat_kernel(PoolArgs a, PoolFlatArgs f) {
  constexpr int V = VecIO<ES>::V;
  const pml_hip_pool2d_desc& d = a.d;
  const unsigned g = xcd_contiguous_block(blockIdx.x, gridDim.x) * 256u + threadIdx.x;
  if (g >= f.total) return;
  const unsigned pix = fast_div(g, f.cv_magic, f.cv_shift), cv = g - pix * f.cvecs;
  const unsigned t = fast_div(pix, f.ow_magic, f.ow_shift), ox = pix - t * f.ow;
  const unsigned n = fast_div(t, f.oh_magic, f.oh_shift), oy = t - n * f.oh;
  const int H = (int)d.h, W = (int)d.w;
  const unsigned pix_bytes = (unsigned)d.c * ES, c0b = cv * 16u;
  const int iy0 = (int)oy * (int)d.stride_h - (int)d.pad_h, ix0 = (int)ox * (int)d.stride_w - (int)d.pad_w;
  constexpr unsigned kOutside = 0x80000000u;
  const __amdgpu_buffer_rsrc_t rin = __builtin_amdgcn_make_buffer_rsrc((void*)a.in, 0, (int)f.in_bytes, 0x00020000u);
  bool row_ok[KH], col_ok[KW];
  unsigned col_off[KW];
#pragma unroll
  for (int kx = 0; kx < KW; ++kx) {
    col_ok[kx] = (unsigned)(ix0 + kx) < (unsigned)W;
    col_off[kx] = col_ok[kx] ? (unsigned)(ix0 + kx) * pix_bytes + c0b : kOutside;
  }
  i32x4_t xr[KH][KW];
#pragma unroll
  for (int ky = 0; ky < KH; ++ky) {
    row_ok[ky] = (unsigned)(iy0 + ky) < (unsigned)H;
    const unsigned row = row_ok[ky] ? (n * (unsigned)H + (unsigned)(iy0 + ky)) * (unsigned)W * pix_bytes : kOutside;
#pragma unroll
    for (int kx = 0; kx < KW; ++kx)
      xr[ky][kx] = __builtin_amdgcn_raw_buffer_load_b128(rin, (int)(row | col_off[kx]) < 0 ? (int)kOutside : (int)(row + col_off[kx]), 0, 0);
  }
  float acc[V];
  int best[V];  // with_index: largest window index whose (in-range) tap equals the pooled value; 0 if none
  const float ident = AGG == PML_HIP_AGG_MAX ? -INFINITY : (AGG == PML_HIP_AGG_MIN ? INFINITY : 0.f);
#pragma unroll
  for (int i = 0; i < V; ++i) {
    acc[i] = ident;
    best[i] = 0;
  }
#pragma unroll
  for (int ky = 0; ky < KH; ++ky)
#pragma unroll
    for (int kx = 0; kx < KW; ++kx) {
      const bool live = row_ok[ky] && col_ok[kx];
      const int k = ky * KW + kx;
      float x[V];
      if constexpr (ES == 2) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          x[2 * i] = __uint_as_float(((uint32_t)xr[ky][kx][i]) << 16);
          x[2 * i + 1] = __uint_as_float(((uint32_t)xr[ky][kx][i]) & 0xffff0000u);
        }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) x[i] = __int_as_float(xr[ky][kx][i]);
      }
#pragma unroll
      for (int i = 0; i < V; ++i) {
        if constexpr (AGG == PML_HIP_AGG_MAX) {
          // taps come in rising window index, so ">=" leaves the largest index among equal values
          if (WITH_INDEX) best[i] = (live & (x[i] >= acc[i])) ? k : best[i];
          acc[i] = (live & (x[i] > acc[i])) ? x[i] : acc[i];
        } else if constexpr (AGG == PML_HIP_AGG_MIN) {
          if (WITH_INDEX) best[i] = (live & (x[i] <= acc[i])) ? k : best[i];
          acc[i] = (live & (x[i] < acc[i])) ? x[i] : acc[i];
        } else {
          acc[i] += live ? x[i] : 0.f;
        }
      }
    }
  const unsigned o0 = pix * (unsigned)d.c + cv * V;  // in elements
  if constexpr (ES == 2) {
    store_streaming((i32x4_t*)((uint16_t*)a.out + o0), pack_bf16_rne(acc));
  } else {
    const f32x4_t o = {acc[0], acc[1], acc[2], acc[3]};
    store_streaming((f32x4_t*)((float*)a.out + o0), o);
  }
  if (WITH_INDEX) {
    int32_t* ip = (int32_t*)a.idx + o0;
#pragma unroll
    for (int i = 0; i < V; i += 4) {
      const i32x4_t w = {best[i], best[i + 1], best[i + 2], best[i + 3]};
      store_streaming((i32x4_t*)(ip + i), w);
    }
  }
}

inline unsigned grid_for(int64_t items) {
  int64_t blocks = (items + 255) / 256;
  if (blocks < 1) blocks = 1;
  const int64_t cap = 256 * 32;
  return (unsigned)(blocks < cap ? blocks : cap);
}


// Patch matrix of a convolution whose channel count does not fill 16-byte vectors (a 3-channel
// image stem): P[m][k] = I[n, oh*sh + kh*dh - ph, ow*sw + kw*dw - pw, ci] with k = (kh*KW + kw)*CI + ci,
// zero outside the image and for k >= KH*KW*CI.  One thread writes one 16-byte vector of a row.
template <typename T>
__global__ __launch_bounds__(256) void im2col_kernel(Im2colArgs a) {
  constexpr int V = 16 / (int)sizeof(T);
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int vecs = a.kpad / V;
  if (idx >= a.M * vecs) return;
  const int64_t m = idx / vecs;
  const int k0 = (int)(idx - m * vecs) * V;
  const int ow = (int)(m % a.OW);
  const int64_t t = m / a.OW;
  const int oh = (int)(t % a.OH);
  const int64_t nb = t / a.OH;
  const T* img = (const T*)a.in + nb * ((int64_t)a.H * a.W * a.CI);
  T vals[V];
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const int k = k0 + e;
    const int tap = k / a.CI, ci = k - tap * a.CI;
    const int kh = tap / a.KW, kw = tap - kh * a.KW;
    const int ih = oh * a.SH + kh * a.DH - a.PH, iw = ow * a.SW + kw * a.DW - a.PW;
    const bool ok = k < a.K && (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W;
    vals[e] = ok ? img[((int64_t)ih * a.W + iw) * a.CI + ci] : (T)0;
  }
  i32x4_t packed;
  __builtin_memcpy(&packed, vals, 16);
  *(i32x4_t*)((T*)a.out + m * a.kpad + k0) = packed;
}

// One thread writes one 16-byte vector of S (see S2dArgs).
template <typename T>
__global__ __launch_bounds__(256) void s2d_input_kernel(S2dArgs a) {
  constexpr int V = 16 / (int)sizeof(T);
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int vecs = a.CH / V;
  const int64_t total = (int64_t)a.N * a.HS * a.WS * vecs;
  if (idx >= total) return;
  const int v = (int)(idx % vecs);
  int64_t t = idx / vecs;
  const int c = (int)(t % a.WS);
  t /= a.WS;
  const int r = (int)(t % a.HS);
  const int64_t n = t / a.HS;
  const T* img = (const T*)a.in + n * ((int64_t)a.H * a.W * a.CI);
  T vals[V];
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const int ch = v * V + e;
    const int blk = ch / a.CI, ci = ch - blk * a.CI;  // blk = b*2 + bw
    const int ih = 2 * r + (blk >> 1), iw = 2 * c + (blk & 1);
    const bool ok = blk < 4 && ih < a.H && iw < a.W;
    vals[e] = ok ? img[((int64_t)ih * a.W + iw) * a.CI + ci] : (T)0;
  }
  i32x4_t packed;
  __builtin_memcpy(&packed, vals, 16);
  *(i32x4_t*)((T*)a.out + idx * V) = packed;
}

// One thread writes one element of G (see S2dArgs).
template <typename T>
__global__ __launch_bounds__(256) void s2d_filter_kernel(S2dArgs a) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t per_co = (int64_t)a.KA * a.KAW * a.CH;
  if (idx >= per_co * a.CO) return;
  const int co = (int)(idx / per_co);
  int rem = (int)(idx - co * per_co);
  const int ch = rem % a.CH;
  rem /= a.CH;
  const int aw = rem % a.KAW, ah = rem / a.KAW;
  const int blk = ch / a.CI, ci = ch - blk * a.CI;
  const int kh = 2 * ah + (blk >> 1) - a.EH, kw = 2 * aw + (blk & 1) - a.EW;
  const bool ok = blk < 4 && kh >= 0 && kh < a.KH && kw >= 0 && kw < a.KW;
  ((T*)a.gt)[idx] = ok ? ((const T*)a.filter)[(((int64_t)kh * a.KW + kw) * a.CI + ci) * a.CO + co] : (T)0;
}

}  // namespace

bool dwconv2d_takes_paired_filter(const pml_hip_dwconv2d_desc& d) {
  const int64_t opitch = d.out_pitch ? (int64_t)d.out_pitch : d.c;
  return d.kh == 3 && d.kw == 3 && d.stride_h == 1 && d.stride_w == 1 && d.dil_h == 1 && d.dil_w == 1 && d.tail.n_ops == 0 &&
         d.dtype == PML_HIP_BF16 && d.n * d.h * d.w * d.c * 2 < ((int64_t)1 << 30) && d.n * d.oh * d.ow * opitch * 2 < ((int64_t)1 << 31);
}

// The paired layout of a 3x3 bf16 filter [3][3][c] (host arrays: `filter` 9 * c bf16 values, `packed` 12 * c / 8 vectors
// of 16 bytes).  Returns false, leaving `packed` unfinished, when a weight is infinite or NaN.
bool dwconv2d_pair_filter(const uint16_t* filter, int64_t c, uint32_t* packed) {
  const int64_t cvecs = c / 8;
  for (int64_t i = 0; i < 9 * c; ++i)
    if ((filter[i] & 0x7f80u) == 0x7f80u) return false;
  for (int64_t cv = 0; cv < cvecs; ++cv)
    for (int kx = 0; kx < 3; ++kx)
      for (int h = 0; h < 2; ++h)
        for (int e = 0; e < 4; ++e) {
          const int64_t ch = cv * 8 + h * 4 + e;
          const uint32_t w0 = filter[(0 * 3 + kx) * c + ch], w1 = filter[(1 * 3 + kx) * c + ch], w2 = filter[(2 * 3 + kx) * c + ch];
          packed[((2 * kx + h) * cvecs + cv) * 4 + e] = w0 | (w1 << 16);
          packed[((6 + 2 * kx + h) * cvecs + cv) * 4 + e] = w2 << 16;  // the bf16 value as fp32
        }
  return true;
}

// Does the row-walking kernel (dwconv3x3_walk_kernel) take this convolution on a device of n_cus compute units, and with
// which cut of the image height?  Its threads take two pixels of a run of rows each; the height is cut into as many
// runs (of at least four rows) as keep every wavefront resident at once, two per SIMD, and the kernel is used where
// that gives every SIMD a wavefront at least -- smaller problems need the parallelism of a thread per four pixels.
// Measured against dwconv3x3_flat_kernel on one device, bf16: 64 x 19 x 19 x 728 15.1 -> 14.3 us, 32 x 56 x 56 x 256
// 19.9 -> 18.3, 128 x 28 x 28 x 512 36.6 -> 33.2, 32 x 112 x 112 x 64 19.4 -> 18.0.
bool dwconv2d_walks_rows(const pml_hip_dwconv2d_desc& d, int n_cus, int64_t* ysegs_out, int64_t* seg_rows_out) {
  if (!(d.kh == 3 && d.kw == 3 && d.stride_h == 1 && d.stride_w == 1 && d.dil_h == 1 && d.dil_w == 1 && d.tail.n_ops == 0 &&
        (d.dtype == PML_HIP_BF16 || d.dtype == PML_HIP_F32)))
    return false;
  const int es = dt_size(d.dtype), V = 16 / es;
  const int64_t opitch = d.out_pitch ? (int64_t)d.out_pitch : d.c;
  // offsets are 32-bit; the marks for taps outside the image need the input below 1 GiB
  if (d.n * d.h * d.w * d.c * es >= ((int64_t)1 << 30) || d.n * d.oh * d.ow * opitch * es >= ((int64_t)1 << 31)) return false;
  const int64_t per_seg = d.n * ((d.ow + 1) / 2) * (d.c / V);
  if (per_seg == 0) return false;
  const int64_t resident = (int64_t)n_cus * 4 * 2 * 64;
  int64_t ysegs = resident / per_seg;
  if (ysegs > (d.oh + 3) / 4) ysegs = (d.oh + 3) / 4;
  if (ysegs < 1) ysegs = 1;
  const int64_t seg_rows = (d.oh + ysegs - 1) / ysegs;
  ysegs = (d.oh + seg_rows - 1) / seg_rows;
  if (per_seg * ysegs < resident / 2 || per_seg * ysegs >= ((int64_t)1 << 31) - 256) return false;
  *ysegs_out = ysegs;
  *seg_rows_out = seg_rows;
  return true;
}

hipError_t dwconv2d_launch(const DwconvArgs& a, hipStream_t s) {
  const pml_hip_dwconv2d_desc& d = a.d;
  const int es = dt_size(d.dtype);
  const int V = 16 / es;
  const int64_t total = d.n * d.oh * d.ow * (d.c / V);
  if (total == 0) return hipSuccess;
  if (d.kh == 3 && d.kw == 3 && d.stride_h == 1 && d.stride_w == 1 && d.dil_h == 1 && d.dil_w == 1 && d.tail.n_ops == 0 &&
      (d.dtype == PML_HIP_BF16 || d.dtype == PML_HIP_F32)) {
    const int64_t total4 = d.n * d.oh * ((d.ow + kDwPx - 1) / kDwPx) * (d.c / V);
    // 32-bit index arithmetic where every element offset (and the rounded-up thread count) stays below 2^31
    const int64_t opitch = d.out_pitch ? (int64_t)d.out_pitch : d.c;
    const bool narrow = d.n * d.h * d.w * d.c < ((int64_t)1 << 31) - (1 << 24) && d.n * d.oh * d.ow * opitch < ((int64_t)1 << 31) - (1 << 24);
    const bool small = d.n * d.h * d.w * d.c * es < ((int64_t)1 << 31) && d.n * d.oh * d.ow * opitch * es < ((int64_t)1 << 31);
    if (small) {
      DwFlatArgs f;
      f.total = (unsigned)total4;
      f.cvecs = (unsigned)(d.c / V), f.xblocks = (unsigned)((d.ow + kDwPx - 1) / kDwPx), f.oh = (unsigned)d.oh;
      fast_div_magic(f.cvecs, &f.cv_magic, &f.cv_shift);
      fast_div_magic(f.xblocks, &f.xb_magic, &f.xb_shift);
      fast_div_magic(f.oh, &f.oh_magic, &f.oh_shift);
      f.in_bytes = (unsigned)(d.n * d.h * d.w * d.c * es);
      int64_t ysegs, seg_rows;
      if (dwconv2d_walks_rows(d, a.n_cus, &ysegs, &seg_rows)) {
        const int64_t cvecs = d.c / V, xblocks2 = (d.ow + 1) / 2, threads = d.n * xblocks2 * cvecs * ysegs;
        DwWalkArgs wk;
        wk.total = (unsigned)threads;
        wk.cvecs = (unsigned)cvecs, wk.xblocks = (unsigned)xblocks2, wk.ysegs = (unsigned)ysegs, wk.seg_rows = (unsigned)seg_rows;
        fast_div_magic(wk.cvecs, &wk.cv_magic, &wk.cv_shift);
        fast_div_magic(wk.xblocks, &wk.xb_magic, &wk.xb_shift);
        fast_div_magic(wk.ysegs, &wk.ys_magic, &wk.ys_shift);
        wk.in_bytes = (unsigned)(d.n * d.h * d.w * d.c * es);
        const unsigned wblocks = (unsigned)((threads + 255) / 256);
        if (es == 2)
          hipLaunchKernelGGL((dwconv3x3_walk_kernel<2>), dim3(wblocks), dim3(256), 0, s, a, wk);
        else
          hipLaunchKernelGGL((dwconv3x3_walk_kernel<4>), dim3(wblocks), dim3(256), 0, s, a, wk);
        return hipGetLastError();
      }
      const unsigned blocks = (unsigned)((total4 + 255) / 256);
      const size_t filter_lds = (size_t)12 * f.cvecs * 16;
      if (es == 2 && a.paired_filter != nullptr && filter_lds <= 48 * 1024) {
        // three workgroups per CU stay and share the blocks out among them (a multiple of 8, so that a workgroup's blocks
        // all belong to its XCD's range)
        const unsigned resident = (unsigned)(3 * a.n_cus + 7) / 8 * 8;
        const unsigned grid = blocks < resident ? blocks : resident;
        hipLaunchKernelGGL(dwconv3x3_flat_paired_kernel<true>, dim3(grid), dim3(256), filter_lds, s, a, f, (const i32x4_t*)a.paired_filter, blocks);
      } else if (es == 2 && a.paired_filter != nullptr)
        hipLaunchKernelGGL(dwconv3x3_flat_paired_kernel<false>, dim3(blocks), dim3(256), 0, s, a, f, (const i32x4_t*)a.paired_filter, blocks);
      else if (es == 2)
        hipLaunchKernelGGL((dwconv3x3_flat_kernel<2>), dim3(blocks), dim3(256), 0, s, a, f);
      else
        hipLaunchKernelGGL((dwconv3x3_flat_kernel<4>), dim3(blocks), dim3(256), 0, s, a, f);
    } else if (es == 2 && narrow)
      hipLaunchKernelGGL((dwconv3x3_kernel<2, uint32_t>), dim3(grid_for(total4)), dim3(256), 0, s, a, total4);
    else if (es == 2)
      hipLaunchKernelGGL((dwconv3x3_kernel<2, int64_t>), dim3(grid_for(total4)), dim3(256), 0, s, a, total4);
    else if (narrow)
      hipLaunchKernelGGL((dwconv3x3_kernel<4, uint32_t>), dim3(grid_for(total4)), dim3(256), 0, s, a, total4);
    else
      hipLaunchKernelGGL((dwconv3x3_kernel<4, int64_t>), dim3(grid_for(total4)), dim3(256), 0, s, a, total4);
    return hipGetLastError();
  }
  if (es == 2)
    hipLaunchKernelGGL((dwconv2d_kernel<2>), dim3(grid_for(total)), dim3(256), 0, s, a, total);
  else
    hipLaunchKernelGGL((dwconv2d_kernel<4>), dim3(grid_for(total)), dim3(256), 0, s, a, total);
  return hipGetLastError();
}

namespace {

// Whole-image pooling (one output pixel per image): the outputs alone are too few threads to keep HBM
// busy, so eight threads share the taps of one 16-byte channel vector -- thread g takes taps g, g + 8,
// ... with all of its loads in flight at once -- and the eight partial results are folded through LDS in a
// fixed order.  A workgroup covers 32 channel vectors of one image.
template <int ES>
__global__ __launch_bounds__(256) void pool_whole_kernel(PoolArgs a, int64_t chunks) {
  constexpr int V = VecIO<ES>::V;
  constexpr int kShare = 8, kMine = 8;  // up to kShare * kMine taps per pass
  const pml_hip_pool2d_desc& d = a.d;
  __shared__ float part[kShare][32][V + 1];
  const int64_t cvecs = d.c / V;
  const int64_t n = blockIdx.x / chunks;
  const int64_t cv = (blockIdx.x % chunks) * 32 + (threadIdx.x & 31);
  const int g = (int)(threadIdx.x >> 5);
  const bool live = cv < cvecs;
  const int64_t taps = d.h * d.w;
  const float ident = d.agg == PML_HIP_AGG_MAX ? -INFINITY : (d.agg == PML_HIP_AGG_MIN ? INFINITY : 0.f);
  float acc[V];
#pragma unroll
  for (int i = 0; i < V; ++i) acc[i] = ident;
  const int64_t base = n * taps * d.c + (live ? cv : 0) * V;
  for (int64_t t0 = g; t0 < taps; t0 += kShare * kMine) {
    float x[kMine][V];
#pragma unroll
    for (int u = 0; u < kMine; ++u) {
      const int64_t t = t0 + (int64_t)u * kShare;
      VecIO<ES>::load(a.in, base + (t < taps ? t : 0) * d.c, x[u]);
    }
#pragma unroll
    for (int u = 0; u < kMine; ++u) {
      if (t0 + (int64_t)u * kShare >= taps) break;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        if (d.agg == PML_HIP_AGG_MAX)
          acc[i] = (x[u][i] > acc[i]) ? x[u][i] : acc[i];
        else if (d.agg == PML_HIP_AGG_MIN)
          acc[i] = (x[u][i] < acc[i]) ? x[u][i] : acc[i];
        else
          acc[i] += x[u][i];
      }
    }
  }
#pragma unroll
  for (int i = 0; i < V; ++i) part[g][threadIdx.x & 31][i] = acc[i];
  __syncthreads();
  if (g != 0 || !live) return;
  for (int k = 1; k < kShare; ++k) {
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const float y = part[k][threadIdx.x][i];
      if (d.agg == PML_HIP_AGG_MAX)
        acc[i] = (y > acc[i]) ? y : acc[i];
      else if (d.agg == PML_HIP_AGG_MIN)
        acc[i] = (y < acc[i]) ? y : acc[i];
      else
        acc[i] += y;
    }
  }
  if (d.divisor != 0.f) {
    // a mean: the sum is rounded to the element type first, as the separate division would have found it
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = (ES == 2 ? __uint_as_float((uint32_t)f32_to_bf16_bits(acc[i]) << 16) : acc[i]) / d.divisor;
  }
  const int64_t o0 = n * d.c + cv * V;
  if constexpr (ES == 2) {
    i32x4_t o;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      o[i] = (int)((uint32_t)f32_to_bf16_bits(acc[2 * i]) | ((uint32_t)f32_to_bf16_bits(acc[2 * i + 1]) << 16));
    store_streaming((i32x4_t*)((uint16_t*)a.out + o0), o);
  } else {
    const f32x4_t o = {acc[0], acc[1], acc[2], acc[3]};
    store_streaming((f32x4_t*)((float*)a.out + o0), o);
  }
}

}  // namespace

hipError_t pool2d_launch(const PoolArgs& a, hipStream_t s) {
  const pml_hip_pool2d_desc& d = a.d;
  const int es = dt_size(d.dtype);
  const int V = 16 / es;
  const int64_t total = d.n * d.oh * d.ow * (d.c / V);
  if (total == 0) return hipSuccess;
  const bool whole = d.oh == 1 && d.ow == 1 && d.kh == d.h && d.kw == d.w && d.pad_h == 0 && d.pad_w == 0 && !d.with_index &&
                     (d.dtype == PML_HIP_BF16 || d.dtype == PML_HIP_F32) && d.h * d.w >= 16;
  if (whole) {
    const int64_t chunks = (d.c / V + 31) / 32;
    if (d.n * chunks <= 0x7fffffff) {
      if (es == 2)
        hipLaunchKernelGGL((pool_whole_kernel<2>), dim3((unsigned)(d.n * chunks)), dim3(256), 0, s, a, chunks);
      else
        hipLaunchKernelGGL((pool_whole_kernel<4>), dim3((unsigned)(d.n * chunks)), dim3(256), 0, s, a, chunks);
      return hipGetLastError();
    }
  }
  // windows of 3x3 or 2x2 taps over small tensors: the straight-line kernel
  const bool small = d.n * d.h * d.w * d.c * es < ((int64_t)1 << 31) && d.n * d.oh * d.ow * d.c * 4 < ((int64_t)1 << 31) &&
                     (d.dtype == PML_HIP_BF16 || d.dtype == PML_HIP_F32);
  if (small && d.kh == d.kw && (d.kh == 3 || d.kh == 2)) {
    PoolFlatArgs f;
    f.total = (unsigned)total;
    f.cvecs = (unsigned)(d.c / V), f.ow = (unsigned)d.ow, f.oh = (unsigned)d.oh;
    fast_div_magic(f.cvecs, &f.cv_magic, &f.cv_shift);
    fast_div_magic(f.ow, &f.ow_magic, &f.ow_shift);
    fast_div_magic(f.oh, &f.oh_magic, &f.oh_shift);
    f.in_bytes = (unsigned)(d.n * d.h * d.w * d.c * es);
    const unsigned blocks = (unsigned)((total + 255) / 256);
    auto go = [&](auto es_tag, auto idx_tag, auto agg_tag) {
      constexpr int kEs = decltype(es_tag)::value, kAgg = decltype(agg_tag)::value;
      constexpr bool kIdx = decltype(idx_tag)::value;
      if (d.kh == 3)
        hipLaunchKernelGGL((pool_flat_kernel<kEs, kIdx, kAgg, 3, 3>), dim3(blocks), dim3(256), 0, s, a, f);
      else
        hipLaunchKernelGGL((pool_flat_kernel<kEs, kIdx, kAgg, 2, 2>), dim3(blocks), dim3(256), 0, s, a, f);
    };
    auto with_agg = [&](auto es_tag, auto idx_tag) {
      switch (d.agg) {
        case PML_HIP_AGG_MAX: go(es_tag, idx_tag, std::integral_constant<int, PML_HIP_AGG_MAX>()); break;
        case PML_HIP_AGG_MIN: go(es_tag, idx_tag, std::integral_constant<int, PML_HIP_AGG_MIN>()); break;
        default: go(es_tag, idx_tag, std::integral_constant<int, PML_HIP_AGG_ADD>()); break;
      }
    };
    auto with_index = [&](auto es_tag) {
      if (d.with_index)
        with_agg(es_tag, std::true_type());
      else
        with_agg(es_tag, std::false_type());
    };
    if (es == 2)
      with_index(std::integral_constant<int, 2>());
    else
      with_index(std::integral_constant<int, 4>());
    return hipGetLastError();
  }
  // 32-bit index arithmetic where every element offset (and the rounded-up thread count) stays below 2^31
  const bool narrow = d.n * d.h * d.w * d.c < ((int64_t)1 << 31) - (1 << 24) && d.n * d.oh * d.ow * d.c < ((int64_t)1 << 31) - (1 << 24);
  auto launch = [&](auto kern) { hipLaunchKernelGGL(kern, dim3(grid_for(total)), dim3(256), 0, s, a, total); };
  auto pick_index = [&](auto es_tag, auto it_tag, auto agg_tag) {
    constexpr int kEs = decltype(es_tag)::value, kAgg = decltype(agg_tag)::value;
    typedef typename decltype(it_tag)::type it_t;
    if (d.with_index)
      launch(pool2d_kernel<kEs, true, it_t, kAgg>);
    else
      launch(pool2d_kernel<kEs, false, it_t, kAgg>);
  };
  auto pick_agg = [&](auto es_tag, auto it_tag) {
    switch (d.agg) {
      case PML_HIP_AGG_MAX: pick_index(es_tag, it_tag, std::integral_constant<int, PML_HIP_AGG_MAX>()); break;
      case PML_HIP_AGG_MIN: pick_index(es_tag, it_tag, std::integral_constant<int, PML_HIP_AGG_MIN>()); break;
      default: pick_index(es_tag, it_tag, std::integral_constant<int, PML_HIP_AGG_ADD>()); break;
    }
  };
  auto pick_it = [&](auto es_tag) {
    if (narrow)
      pick_agg(es_tag, std::common_type<uint32_t>());
    else
      pick_agg(es_tag, std::common_type<int64_t>());
  };
  if (es == 2)
    pick_it(std::integral_constant<int, 2>());
  else
    pick_it(std::integral_constant<int, 4>());
  return hipGetLastError();
}

hipError_t im2col_launch(int elem_size, const Im2colArgs& a, hipStream_t s) {
  const int v = 16 / elem_size;
  const int64_t total = a.M * (a.kpad / v);
  const unsigned blocks = (unsigned)((total + 255) / 256);
  switch (elem_size) {
    case 1: hipLaunchKernelGGL(im2col_kernel<uint8_t>, dim3(blocks), dim3(256), 0, s, a); break;
    case 2: hipLaunchKernelGGL(im2col_kernel<uint16_t>, dim3(blocks), dim3(256), 0, s, a); break;
    case 4: hipLaunchKernelGGL(im2col_kernel<uint32_t>, dim3(blocks), dim3(256), 0, s, a); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t s2d_input_launch(int elem_size, const S2dArgs& a, hipStream_t s) {
  const int64_t total = (int64_t)a.N * a.HS * a.WS * (a.CH * elem_size / 16);
  const unsigned blocks = (unsigned)((total + 255) / 256);
  switch (elem_size) {
    case 2: hipLaunchKernelGGL(s2d_input_kernel<uint16_t>, dim3(blocks), dim3(256), 0, s, a); break;
    case 4: hipLaunchKernelGGL(s2d_input_kernel<uint32_t>, dim3(blocks), dim3(256), 0, s, a); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t s2d_filter_launch(int elem_size, const S2dArgs& a, hipStream_t s) {
  const int64_t total = (int64_t)a.CO * a.KA * a.KAW * a.CH;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  switch (elem_size) {
    case 2: hipLaunchKernelGGL(s2d_filter_kernel<uint16_t>, dim3(blocks), dim3(256), 0, s, a); break;
    case 4: hipLaunchKernelGGL(s2d_filter_kernel<uint32_t>, dim3(blocks), dim3(256), 0, s, a); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace pml
