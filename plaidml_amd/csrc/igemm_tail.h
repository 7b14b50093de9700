// Internal: pieces shared by the MFMA kernels (igemm.hip, conv_halo.hip): the
// accumulator types, one 32-byte K-block of MFMA work per element kind, and the
// tail that walks an accumulator tile staged in LDS.
#pragma once

#include <hip/hip_runtime.h>

#include "device_common.h"
#include "plans.h"

#include <type_traits>

namespace pml {

// A loop whose counter is a compile-time constant in the body (accumulator registers can only be named, not indexed).
template <int I, int N, int STEP, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + STEP, N, STEP>(f);
  }
}

template <int KIND>
struct Acc;
template <>
struct Acc<KIND_BF16> {
  typedef f32x16_t type;
  typedef float scalar;
};
template <>
struct Acc<KIND_F32> {
  typedef f32x16_t type;
  typedef float scalar;
};
template <>
struct Acc<KIND_I8> {
  typedef i32x16_t type;
  typedef int scalar;
};
template <>
struct Acc<KIND_F32X3> {
  typedef f32x16_t type;
  typedef float scalar;
};
template <>
struct Acc<KIND_F32X3P> {
  typedef f32x16_t type;
  typedef float scalar;
};

template <int KIND>
__device__ inline void mma_block(typename Acc<KIND>::type& acc, const i32x4_t& a, const i32x4_t& b);

template <>
__device__ inline void mma_block<KIND_BF16>(f32x16_t& acc, const i32x4_t& a, const i32x4_t& b) {
  bf16x8_t av, bv;
  __builtin_memcpy(&av, &a, 16);
  __builtin_memcpy(&bv, &b, 16);
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, acc, 0, 0, 0);
}
template <>
__device__ inline void mma_block<KIND_I8>(i32x16_t& acc, const i32x4_t& a, const i32x4_t& b) {
  acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc, 0, 0, 0);
}
template <>
__device__ inline void mma_block<KIND_F32>(f32x16_t& acc, const i32x4_t& a, const i32x4_t& b) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__int_as_float(a[j]), __int_as_float(b[j]), acc, 0, 0, 0);
  }
}

// fp32 on the bf16 matrix pipe.  Eight fp32 values (two 16-byte fragments) become a bf16 "head" (round to nearest
// even) and a bf16 "remainder" (the rounded difference): x = head + remainder to about 2^-17 |x|.
__device__ __forceinline__ void split_f32x8(const i32x4_t& r0, const i32x4_t& r1, i32x4_t& head, i32x4_t& rem) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float x0 = __int_as_float(q < 2 ? r0[2 * q] : r1[2 * q - 4]);
    const float x1 = __int_as_float(q < 2 ? r0[2 * q + 1] : r1[2 * q - 3]);
    const bf16x2 h = __builtin_convertvector(f32x2{x0, x1}, bf16x2);
    uint32_t hb;
    __builtin_memcpy(&hb, &h, 4);
    head[q] = (int)hb;
    const float d0 = x0 - __uint_as_float(hb << 16), d1 = x1 - __uint_as_float(hb & 0xffff0000u);
    const bf16x2 l = __builtin_convertvector(f32x2{d0, d1}, bf16x2);
    uint32_t lb;
    __builtin_memcpy(&lb, &l, 4);
    rem[q] = (int)lb;
  }
}

// acc += a . b with a = a_head + a_rem, b = b_head + b_rem, the product of the two remainders dropped (2^-16 of the
// term).  The small products go first.
__device__ __forceinline__ void mma_split(f32x16_t& acc, const i32x4_t& a_head, const i32x4_t& a_rem, const i32x4_t& b_head,
                                          const i32x4_t& b_rem) {
  bf16x8_t ah, ar, bh, br;
  __builtin_memcpy(&ah, &a_head, 16);
  __builtin_memcpy(&ar, &a_rem, 16);
  __builtin_memcpy(&bh, &b_head, 16);
  __builtin_memcpy(&br, &b_rem, 16);
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ar, bh, acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, br, acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bh, acc, 0, 0, 0);
}

// Residual rows of a tile requested ahead of its K loop (tail_mode 2, at most 8 rows per thread):
// their latency then overlaps the operand loads and the MFMAs instead of following them.
template <int KIND, int BM, int BN, int NTHREADS>
struct TailPrefetch {
  static constexpr int TPR = BN / 4;
  static constexpr int RPP = NTHREADS / TPR;
  static constexpr int kIters = (BM + RPP - 1) / RPP;
  // (bf16 results take the direct tail, which prefetches in its own layout: the staged tail of the remaining
  // edge tiles loads its residual rows when it gets there)
  static constexpr bool kFits = kIters <= 8 && KIND != KIND_BF16;
  i32x4_t res[kFits ? kIters : 1];
  bool valid;
};

template <int KIND, int BM, int BN, int NTHREADS>
__device__ __forceinline__ void tail_prefetch(const IgemmArgs& p, int64_t m0, int64_t n0, int tid,
                                              TailPrefetch<KIND, BM, BN, NTHREADS>& pre) {
  typedef TailPrefetch<KIND, BM, BN, NTHREADS> P;
  pre.valid = false;
  if constexpr (P::kFits) {
    const int64_t n = n0 + (tid % P::TPR) * 4;
    if (p.tail_mode != 2 || n + 3 >= p.N || (p.ldc & 3) != 0) return;
    pre.valid = true;
    const int64_t res_rs = p.tail.operand_row_stride[0];
#pragma unroll
    for (int c = 0; c < P::kIters; ++c) {
      const int row = tid / P::TPR + c * P::RPP;
      const int64_t m = m0 + row;
      pre.res[c] = i32x4_t{0, 0, 0, 0};
      if (row < BM && m < p.M) {
        if (KIND != KIND_I8 && p.out_dtype == PML_HIP_BF16) {
          const uint2 x = *(const uint2*)((const uint16_t*)p.operands[0] + m * res_rs + n);
          pre.res[c][0] = (int)x.x;
          pre.res[c][1] = (int)x.y;
        } else {
          pre.res[c] = *(const i32x4_t*)((const int*)p.operands[0] + m * res_rs + n);
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------
// The common bf16 tails straight from the accumulators, without the trip through LDS: relu?(acc + bias),
// relu?(bf16(acc + bias) + residual) and the folded batch normalisation relu?(bf16(bf16(acc + bias) * scale) + shift),
// every step rounded to bf16 as the step-wise tail does.  A lane of a 32x32 block holds, for its row (lane & 31), the
// four columns 8g + 4 * (lane >> 5) ... of each group g; exchanging the upper half of group 2q with the
// lower half of group 2q + 1 (v_permlane32_swap) leaves every lane with eight neighbouring columns of its
// row -- columns 16q + 8 * (lane >> 5) ... -- which is one 16-byte store (8-byte stores measured a third
// slower).  The stores of a row's 64-byte run leave the wavefront within a few instructions of each other
// and meet again in L2.
// ---------------------------------------------------------------------------------------------------

// Whether the tile can take the direct tail (uniform over the workgroup).
template <int KIND>
__device__ __forceinline__ bool direct_tail_ok(const IgemmArgs& p, int64_t n0, int bn) {
  if constexpr (KIND != KIND_BF16) return false;
  const bool scale_shift = p.tail_mode == 3 && p.tail_ssr != 0 && p.init2 == nullptr;
  if (p.out_dtype != PML_HIP_BF16 || (p.tail_mode != 1 && p.tail_mode != 2 && !scale_shift)) return false;
  // (a tile that hangs over the last column is fine as long as N ends on a 16-byte piece: whole pieces are skipped)
  if ((n0 + bn > p.N && (p.N & 7) != 0) || (p.ldc & 7) != 0 || ((uintptr_t)p.C & 15) != 0) return false;
  if (p.init != nullptr && !(p.init_rs == 0 && p.init_cs == 1 && p.init_dtype == PML_HIP_BF16 && ((uintptr_t)p.init & 15) == 0)) return false;
  if (p.tail_mode == 2 && ((p.tail.operand_row_stride[0] & 7) != 0 || ((uintptr_t)p.operands[0] & 15) != 0)) return false;
  if (p.init2 != nullptr && ((uintptr_t)p.init2 & 15) != 0) return false;
  return true;
}

typedef unsigned int u32x4_tail_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void unpack_bf16x8(const i32x4_t& w, float* f) {
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    f[2 * q] = __uint_as_float((uint32_t)w[q] << 16);
    f[2 * q + 1] = __uint_as_float((uint32_t)w[q] & 0xffff0000u);
  }
}

__device__ __forceinline__ i32x4_t pack_bf16x8(const float* v) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  i32x4_t o;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const bf16x2 h = __builtin_convertvector(f32x2{v[2 * q], v[2 * q + 1]}, bf16x2);  // round to nearest even
    uint32_t w;
    __builtin_memcpy(&w, &h, 4);
    o[q] = (int)w;
  }
  return o;
}

// The value of a float after it has been rounded to bf16 (round to nearest even) -- two at a time.
__device__ __forceinline__ void round_pair_to_bf16(float& x, float& y) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  const bf16x2 h = __builtin_convertvector(f32x2{x, y}, bf16x2);
  uint32_t w;
  __builtin_memcpy(&w, &h, 4);
  x = __uint_as_float(w << 16);
  y = __uint_as_float(w & 0xffff0000u);
}

// mw, nw: first row / column of the wavefront's MI x NI blocks.
// What a result costs here is vector instructions (a 96 x 96 wavefront tile holds 144 results per lane), so: the
// per-column vectors (bias, scale, shift) are unpacked once per column block, not once per row block; a step whose
// operand is absent is not computed at all (uniform branches); relu is one NaN-keeping maximum; and the eight lane
// exchanges of a 32 x 32 block sit in one run with one pair of idle cycles around it instead of one pair each.
template <int MI, int NI>
__device__ __forceinline__ void direct_tail_bf16(const IgemmArgs& p, f32x16_t (&acc)[MI][NI], int64_t mw, int64_t nw, int lane) {
  const int hi = lane >> 5;
  const bool residual = p.tail_mode == 2;
  const bool scale_shift = p.tail_mode == 3;
  const int64_t rs = p.tail.operand_row_stride[0];
  const uint16_t* const scale = scale_shift ? (const uint16_t*)p.operands[p.tail.ops[0].operand] : nullptr;
  const uint16_t* const shift = scale_shift ? (const uint16_t*)p.operands[p.tail.ops[1].operand] : nullptr;
  const bool relu = scale_shift ? p.tail_ssr == 2 : p.tail_relu != 0;
  const float lo = relu ? 0.f : -__builtin_inff();  // relu as a lower clamp (the IEEE maximum keeps a NaN)
  const bool has_bias = p.init != nullptr || p.init2 != nullptr;
  // the last MFMAs must have written the accumulators before the lane exchange below reads them: the compiler
  // cannot see that read (it is assembler text), so the longest MFMA's passes are waited out here, once
  asm volatile("s_nop 15\n\ts_nop 3");
  // Order of the wavefront's 32x32 blocks.  With several block columns the blocks of a block row follow one another
  // (and the column vectors, hot in L1, are fetched again for every block): the 64-byte pieces that share a 128-byte
  // line of a result row are then stored within a few instructions of each other and leave L2 as one line.  With the
  // column blocks outermost a 192x384 tile wrote 1.86 x its result to memory (WRITE_SIZE 61.0 MB for 33.6 MB at
  // 23104 x 728 x 728: lines left L2 half-written and were written again), a 256x256 tile 1.50 x.
  constexpr bool kRowsOuter = NI > 1;
  bool col_ok[2];
  float bias[2][8], mul[2][8], add[2][8];
#pragma unroll
  for (int outer = 0; outer < (kRowsOuter ? MI : NI); ++outer) {
#pragma unroll
    for (int inner = 0; inner < (kRowsOuter ? NI : MI); ++inner) {
    const int i = kRowsOuter ? outer : inner, j = kRowsOuter ? inner : outer;
    if (kRowsOuter || inner == 0) {
    // the lane's two 8-column pieces of this block; one past the last column (a ragged last tile) is left out
#pragma unroll
    for (int q = 0; q < 2; ++q) col_ok[q] = nw + j * 32 + 16 * q + 8 * hi < p.N;
    auto column_vector = [&](const uint16_t* src, int q, float* out) {
      const i32x4_t bits = (src != nullptr && col_ok[q]) ? *(const i32x4_t*)(src + nw + j * 32 + 16 * q + 8 * hi) : i32x4_t{0, 0, 0, 0};
      unpack_bf16x8(bits, out);
    };
    if (has_bias) {
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        float second[8];
        column_vector((const uint16_t*)p.init, q, bias[q]);
        column_vector((const uint16_t*)p.init2, q, second);
#pragma unroll
        for (int e = 0; e < 8; ++e) bias[q][e] += second[e];
      }
    }
    if (scale_shift) {
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        column_vector(scale, q, mul[q]);
        column_vector(shift, q, add[q]);
      }
    }
    }
    {
      // Memory is touched 64 bytes of a row at a time: access t (0, 1) of the block covers rows 16 t .. 16 t + 15, lane l
      // the eight columns from mcol = 16 ((l / 16) % 2) + 8 (l / 32) of row 16 t + l % 16 -- four lanes per row.  The
      // values are worked on in the accumulators' arrangement (lane l: row l % 32, pieces q = 0, 1 at columns
      // 16 q + 8 hi), which as a memory access would touch 32 rows with 32 bytes each; v_permlane16_swap of the two
      // pieces' registers goes from one arrangement to the other, either way.  (Measured on 401408 x 256 x 64 with a
      // residual, the most memory-bound layer shape of ResNet-50 at batch 128: 137.6 -> 127.8 us.)
      const int mcol = 16 * ((lane >> 4) & 1) + 8 * hi;
      const bool mcol_ok = nw + j * 32 + mcol < p.N;
      i32x4_t res[2] = {i32x4_t{0, 0, 0, 0}, i32x4_t{0, 0, 0, 0}};
      if (residual) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const int64_t m = mw + i * 32 + 16 * t + (lane & 15);
          if (m < p.M && mcol_ok) res[t] = *(const i32x4_t*)((const uint16_t*)p.operands[0] + m * rs + nw + j * 32 + mcol);
        }
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const auto sw = __builtin_amdgcn_permlane16_swap((unsigned)res[0][d], (unsigned)res[1][d], false, false);
          res[0][d] = (int)sw[0];
          res[1][d] = (int)sw[1];
        }
      }
      // The lane holds columns 8 g + 4 hi + e (g = 0..3, e = 0..3) of its row.  Exchanging group 2 q + 1 of the lower
      // half wavefront with group 2 q of the upper one leaves lanes 0..31 with group 2 q whole (8 columns) and lanes
      // 32..63 with group 2 q + 1.  The exchange works on the accumulator registers themselves (the builtin made the
      // compiler copy all accumulators first), as one piece of assembler text: the compiler does not see through it,
      // so the idle cycles the instruction needs after a vector write of its operands and before a vector read of its
      // results are spelled out, once for the eight exchanges.
      f32x16_t& c = acc[i][j];
      asm volatile(
          "s_nop 1\n\t"
          "v_permlane32_swap_b32 %0, %4\n\tv_permlane32_swap_b32 %1, %5\n\tv_permlane32_swap_b32 %2, %6\n\tv_permlane32_swap_b32 %3, %7\n\t"
          "v_permlane32_swap_b32 %8, %12\n\tv_permlane32_swap_b32 %9, %13\n\tv_permlane32_swap_b32 %10, %14\n\tv_permlane32_swap_b32 %11, %15\n\t"
          "s_nop 1"
          : "+v"(c[0]), "+v"(c[1]), "+v"(c[2]), "+v"(c[3]), "+v"(c[4]), "+v"(c[5]), "+v"(c[6]), "+v"(c[7]), "+v"(c[8]), "+v"(c[9]),
            "+v"(c[10]), "+v"(c[11]), "+v"(c[12]), "+v"(c[13]), "+v"(c[14]), "+v"(c[15]));
      i32x4_t packed[2];
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = c[8 * q + e];
        if (has_bias) {
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] += bias[q][e];
        }
        if (residual) {
          // the contraction result is rounded first, then the bf16 addition rounds again
          float r[8];
          unpack_bf16x8(res[q], r);
#pragma unroll
          for (int e = 0; e < 8; e += 2) round_pair_to_bf16(v[e], v[e + 1]);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] += r[e];
        }
        if (scale_shift) {
          // three roundings: the contraction result, the product, the sum
#pragma unroll
          for (int e = 0; e < 8; e += 2) round_pair_to_bf16(v[e], v[e + 1]);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] *= mul[q][e];
#pragma unroll
          for (int e = 0; e < 8; e += 2) round_pair_to_bf16(v[e], v[e + 1]);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] += add[q][e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = __builtin_elementwise_maximum(v[e], lo);
        packed[q] = pack_bf16x8(v);
      }
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const auto sw = __builtin_amdgcn_permlane16_swap((unsigned)packed[0][d], (unsigned)packed[1][d], false, false);
        packed[0][d] = (int)sw[0];
        packed[1][d] = (int)sw[1];
      }
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int64_t m = mw + i * 32 + 16 * t + (lane & 15);
        if (m < p.M && mcol_ok) *(i32x4_t*)((uint16_t*)p.C + m * p.ldc + nw + j * 32 + mcol) = packed[t];
      }
    }
    }
  }
}

// Tail over an accumulator tile held in LDS as ctile[BM][BN + 4] (row-major):
// adds the initial value, runs the fused elementwise chain once per element and
// stores contiguous 8/16-byte pieces.  A thread owns 4 consecutive columns; rows
// advance by NTHREADS / (BN / 4) per pass.
template <int KIND, int BM, int BN, int NTHREADS>
__device__ __forceinline__ void tile_tail(const IgemmArgs& p, const typename Acc<KIND>::scalar* ctile, int64_t m0,
                                          int64_t n0, int tid,
                                          const TailPrefetch<KIND, BM, BN, NTHREADS>* pre = nullptr) {
  typedef typename Acc<KIND>::scalar accs_t;
  constexpr int CS = BN + 4;
  constexpr int kThreads = NTHREADS;
  constexpr int TPR = BN / 4;
  constexpr int RPP = kThreads / TPR;
  const int c4 = (tid % TPR) * 4;
  const int64_t n = n0 + c4;
  if (n >= p.N) return;
  const bool full4 = n + 3 < p.N;
  // tail_mode 1: relu? ; 2: + residual tensor of the result type (unit column stride), then relu?
  const bool fast = (p.tail_mode == 1 || p.tail_mode == 2) && full4 && (p.ldc & 3) == 0;
  const bool residual = p.tail_mode == 2;
  const int64_t res_rs = p.tail.operand_row_stride[0];
  // a per-column start value (bias) is the same for every row of this thread
  const bool col_init = p.init != nullptr && p.init_rs == 0;
  accs_t cinit[4] = {0, 0, 0, 0};
  if (col_init) {
    const int natural = KIND == KIND_I8 ? PML_HIP_I32 : p.out_dtype;
    const int ies = natural == PML_HIP_BF16 ? 2 : 4;
    if (full4 && p.init_cs == 1 && p.init_dtype == natural && (((uintptr_t)p.init + n * ies) & (4 * ies - 1)) == 0) {
      // contiguous bias of the result type: one 8- or 16-byte load
      if (natural == PML_HIP_BF16) {
        const uint2 w = *(const uint2*)((const uint16_t*)p.init + n);
        cinit[0] = (accs_t)__uint_as_float(w.x << 16);
        cinit[1] = (accs_t)__uint_as_float(w.x & 0xffff0000u);
        cinit[2] = (accs_t)__uint_as_float(w.y << 16);
        cinit[3] = (accs_t)__uint_as_float(w.y & 0xffff0000u);
      } else if (natural == PML_HIP_I32) {
        const i32x4_t w = *(const i32x4_t*)((const int*)p.init + n);
#pragma unroll
        for (int q = 0; q < 4; ++q) cinit[q] = (accs_t)w[q];
      } else {
        const f32x4_t w = *(const f32x4_t*)((const float*)p.init + n);
#pragma unroll
        for (int q = 0; q < 4; ++q) cinit[q] = (accs_t)w[q];
      }
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (n + q < p.N) {
          Scalar<float, int> b = load_scalar<float, int>(p.init, (n + q) * p.init_cs, p.init_dtype);
          cinit[q] = KIND == KIND_I8 ? (accs_t)b.i : (accs_t)b.f;
        }
      }
    }
  }
  // the per-column start value of a second product (a contiguous vector of the result type)
  if (p.init2 != nullptr) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (n + q < p.N) {
        Scalar<float, int> b = load_scalar<float, int>(p.init2, n + q, KIND == KIND_I8 ? PML_HIP_I32 : p.out_dtype);
        cinit[q] += KIND == KIND_I8 ? (accs_t)b.i : (accs_t)b.f;
      }
    }
  }
  const int row0 = tid / TPR;

  if (fast) {
    // Rows in batches of up to 8: all residual loads of a batch are issued before the first is used.
    constexpr int kIters = (BM + RPP - 1) / RPP;
    constexpr int kBatch = kIters < 8 ? kIters : 8;
#pragma unroll
    for (int it0 = 0; it0 < kIters; it0 += kBatch) {
      i32x4_t res[kBatch];
#pragma unroll
      for (int c = 0; c < kBatch; ++c) {
        const int row = row0 + (it0 + c) * RPP;
        const int64_t m = m0 + row;
        res[c] = i32x4_t{0, 0, 0, 0};
        if (TailPrefetch<KIND, BM, BN, NTHREADS>::kFits && pre != nullptr && pre->valid) {
          res[c] = pre->res[(it0 + c) % (TailPrefetch<KIND, BM, BN, NTHREADS>::kFits ? kIters : 1)];
        } else if (residual && row < BM && m < p.M) {
          if (KIND != KIND_I8 && p.out_dtype == PML_HIP_BF16) {
            const uint2 x = *(const uint2*)((const uint16_t*)p.operands[0] + m * res_rs + n);
            res[c][0] = (int)x.x;
            res[c][1] = (int)x.y;
          } else {
            res[c] = *(const i32x4_t*)((const int*)p.operands[0] + m * res_rs + n);
          }
        }
      }
#pragma unroll
      for (int c = 0; c < kBatch; ++c) {
        const int row = row0 + (it0 + c) * RPP;
        const int64_t m = m0 + row;
        if (row >= BM || m >= p.M) continue;
        accs_t v4[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) v4[q] = ctile[row * CS + c4 + q] + cinit[q];
        if (p.init && !col_init) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            Scalar<float, int> b = load_scalar<float, int>(p.init, m * p.init_rs + (n + q) * p.init_cs, p.init_dtype);
            v4[q] += KIND == KIND_I8 ? (accs_t)b.i : (accs_t)b.f;
          }
        }
        if (KIND == KIND_I8) {
          i32x4_t w;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int v = (int)((unsigned)(int)v4[q] + (unsigned)res[c][q]);
            w[q] = (p.tail_relu && v < 0) ? 0 : v;
          }
          *(i32x4_t*)((int*)p.C + m * p.ldc + n) = w;
        } else if (p.out_dtype == PML_HIP_BF16) {
          // v_cvt_pk_bf16_f32 rounds to nearest even.  relu is applied to the fp32 value just before
          // the last rounding (a result in (-2^-134, 0) stores +0 where the definition gives -0).
          typedef float f32x2 __attribute__((ext_vector_type(2)));
          typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
          float v[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] = (float)v4[q];
          if (residual) {
            // the contraction result is rounded first, then the bf16 addition rounds again
            const bf16x2 r01 = __builtin_convertvector(f32x2{v[0], v[1]}, bf16x2);
            const bf16x2 r23 = __builtin_convertvector(f32x2{v[2], v[3]}, bf16x2);
            uint32_t w01, w23;
            __builtin_memcpy(&w01, &r01, 4);
            __builtin_memcpy(&w23, &r23, 4);
            const uint32_t x01 = (uint32_t)res[c][0], x23 = (uint32_t)res[c][1];
            v[0] = __uint_as_float(w01 << 16) + __uint_as_float(x01 << 16);
            v[1] = __uint_as_float(w01 & 0xffff0000u) + __uint_as_float(x01 & 0xffff0000u);
            v[2] = __uint_as_float(w23 << 16) + __uint_as_float(x23 << 16);
            v[3] = __uint_as_float(w23 & 0xffff0000u) + __uint_as_float(x23 & 0xffff0000u);
          }
          if (p.tail_relu) {
#pragma unroll
            for (int q = 0; q < 4; ++q) v[q] = v[q] < 0.f ? 0.f : v[q];
          }
          const bf16x2 h01 = __builtin_convertvector(f32x2{v[0], v[1]}, bf16x2);
          const bf16x2 h23 = __builtin_convertvector(f32x2{v[2], v[3]}, bf16x2);
          uint32_t o01, o23;
          __builtin_memcpy(&o01, &h01, 4);
          __builtin_memcpy(&o23, &h23, 4);
          *(uint2*)((uint16_t*)p.C + m * p.ldc + n) = make_uint2(o01, o23);
        } else {
          f32x4_t w;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float v = residual ? (float)v4[q] + __int_as_float(res[c][q]) : (float)v4[q];
            w[q] = (p.tail_relu && v < 0.f) ? 0.f : v;
          }
          *(f32x4_t*)((float*)p.C + m * p.ldc + n) = w;
        }
      }
    }
    return;
  }

  // tail_mode 3: up to four float steps in the result type whose operands are immediates, scalars
  // or per-column vectors (scale / shift / clamp chains).  The operand values of this thread's four
  // columns are fetched once; every step rounds to the result type like the interpreter does.
  if (KIND != KIND_I8 && p.tail_mode == 3 && full4 && (p.ldc & 3) == 0) {
    const bool bf = p.out_dtype == PML_HIP_BF16;
    // rounding to the result type: the hardware conversion (round to nearest even, NaN quieted)
    auto rnd = [&](float x) {
      if (!bf) return x;
      typedef float f32x2 __attribute__((ext_vector_type(2)));
      typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
      const bf16x2 h = __builtin_convertvector(f32x2{x, 0.f}, bf16x2);
      uint32_t w;
      __builtin_memcpy(&w, &h, 4);
      return __uint_as_float(w << 16);
    };
    float xs[4][4];
#pragma unroll
    for (int st = 0; st < 4; ++st) {
#pragma unroll
      for (int q = 0; q < 4; ++q) xs[st][q] = 0.f;
      if (st < p.tail.n_ops) {
        const pml_hip_epi_op& op = p.tail.ops[st];
        if (op.operand_kind == PML_HIP_OPND_TENSOR) {
          const void* base = p.operands[op.operand];
          if (p.tail.operand_col_stride[op.operand] == 0) {
            const float x = bf ? __uint_as_float((uint32_t)((const uint16_t*)base)[0] << 16) : ((const float*)base)[0];
#pragma unroll
            for (int q = 0; q < 4; ++q) xs[st][q] = x;
          } else if (bf) {
            const uint2 w = *(const uint2*)((const uint16_t*)base + n);
            xs[st][0] = __uint_as_float(w.x << 16);
            xs[st][1] = __uint_as_float(w.x & 0xffff0000u);
            xs[st][2] = __uint_as_float(w.y << 16);
            xs[st][3] = __uint_as_float(w.y & 0xffff0000u);
          } else {
            const f32x4_t w = *(const f32x4_t*)((const float*)base + n);
#pragma unroll
            for (int q = 0; q < 4; ++q) xs[st][q] = w[q];
          }
        } else if (op.operand_kind == PML_HIP_OPND_IMM) {
#pragma unroll
          for (int q = 0; q < 4; ++q) xs[st][q] = rnd((float)op.imm);
        }
      }
    }
    // rows in batches of up to 8: all LDS reads of a batch are issued before the first value is used,
    // and a step's opcode is decoded once per batch instead of once per element
    constexpr int kRowsPerThread = (BM + RPP - 1) / RPP;
    constexpr int RB = kRowsPerThread < 8 ? kRowsPerThread : 8;
    for (int rowb = row0; rowb < BM; rowb += RB * RPP) {
      float v[RB][4];
#pragma unroll
      for (int r = 0; r < RB; ++r) {
        const int row = rowb + r * RPP;
        const int rr = row < BM ? row : BM - 1;
        if constexpr (sizeof(accs_t) == 4) {
          typedef accs_t acc4_t __attribute__((ext_vector_type(4)));
          const acc4_t c = *(const acc4_t*)&ctile[rr * CS + c4];
#pragma unroll
          for (int q = 0; q < 4; ++q) v[r][q] = (float)c[q] + (float)cinit[q];
        }
      }
      if (p.init && !col_init) {
#pragma unroll
        for (int r = 0; r < RB; ++r) {
          const int64_t m = m0 + rowb + r * RPP;
          if (rowb + r * RPP < BM && m < p.M) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              Scalar<float, int> b = load_scalar<float, int>(p.init, m * p.init_rs + (n + q) * p.init_cs, p.init_dtype);
              v[r][q] += b.f;
            }
          }
        }
      }
      auto each = [&](int st, auto fn) {
#pragma unroll
        for (int r = 0; r < RB; ++r)
#pragma unroll
          for (int q = 0; q < 4; ++q) v[r][q] = rnd(fn(v[r][q], xs[st][q]));
      };
      each(0, [](float a, float) { return a; });  // the contraction's own result, rounded to the result type
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        if (st < p.tail.n_ops) {
          switch (p.tail.ops[st].opcode) {
            case PML_HIP_EPI_ADD: each(st, [](float a, float b) { return a + b; }); break;
            case PML_HIP_EPI_SUB: each(st, [](float a, float b) { return a - b; }); break;
            case PML_HIP_EPI_RSUB: each(st, [](float a, float b) { return b - a; }); break;
            case PML_HIP_EPI_MUL: each(st, [](float a, float b) { return a * b; }); break;
            case PML_HIP_EPI_DIV: each(st, [](float a, float b) { return a / b; }); break;
            case PML_HIP_EPI_RDIV: each(st, [](float a, float b) { return b / a; }); break;
            case PML_HIP_EPI_MAX: each(st, [](float a, float b) { return (a < b) ? b : a; }); break;
            case PML_HIP_EPI_MIN: each(st, [](float a, float b) { return (a < b) ? a : b; }); break;
            case PML_HIP_EPI_RELU: each(st, [](float a, float) { return (a < 0.f) ? 0.f : a; }); break;
            case PML_HIP_EPI_NEG: each(st, [](float a, float) { return -a; }); break;
            case PML_HIP_EPI_MAX_GT: each(st, [](float a, float b) { return (a > b) ? a : b; }); break;
            default: break;
          }
        }
      }
#pragma unroll
      for (int r = 0; r < RB; ++r) {
        const int row = rowb + r * RPP;
        const int64_t m = m0 + row;
        if (row >= BM || m >= p.M) continue;
        if (bf) {
          const uint32_t h0 = __float_as_uint(v[r][0]) >> 16, h1 = __float_as_uint(v[r][1]) >> 16;
          const uint32_t h2 = __float_as_uint(v[r][2]) >> 16, h3 = __float_as_uint(v[r][3]) >> 16;
          *(uint2*)((uint16_t*)p.C + m * p.ldc + n) = make_uint2(h0 | (h1 << 16), h2 | (h3 << 16));
        } else {
          const f32x4_t w = {v[r][0], v[r][1], v[r][2], v[r][3]};
          *(f32x4_t*)((float*)p.C + m * p.ldc + n) = w;
        }
      }
    }
    return;
  }

  // tail_mode 4 (int32 accumulators): up to eight steps that store the running value to an extra
  // output, cast between si32 / f32 / si8, or are f32 arithmetic on immediates, scalars and per-column
  // vectors -- the requantisation chain  store, cast f32, * scale[col], clamp, round, cast si8.
  // Four columns at a time, 4 / 16-byte stores; the step semantics are the interpreter's.
  if constexpr (KIND == KIND_I8) {
    // (both outputs are addressed with 32-bit byte offsets into buffer descriptors of their exact size: a store past
    // the last row has an offset beyond the buffer and is dropped, so the row loop has no branches)
    if (p.tail_mode == 4 && p.tail_rq && full4 && (p.ldc & 3) == 0 && (p.init == nullptr || col_init) &&
        p.M * p.ldc * 4 < ((int64_t)1 << 31)) {
      // the requantisation chain as straight code: si32 sum (stored to the extra output as it is) -> f32 -> * scale
      // -> clamp -> round half away from zero -> si8.  Rounding and the cast are one step here: for x >= 0
      // floor(x + 0.5) and for x < 0 ceil(x - 0.5) both equal trunc(x + copysign(0.5, x)) -- the sum is the same
      // floating-point addition and floor / ceil of a value of that sign is truncation -- and the conversion to
      // an integer truncates by itself.  The clamps (v > lo ? v : lo, v < hi ? v : hi: a NaN goes to the bound) are
      // the hardware's max / min, which agree with them except in the sign of a zero, and a zero of either sign
      // becomes the same integer; the product they follow is never a signalling NaN.
      const float* const scale = (const float*)p.operands[p.rq_scale];
      f32x4_t sc;
      if (p.tail.operand_col_stride[p.rq_scale] == 0) {
        sc = f32x4_t{scale[0], scale[0], scale[0], scale[0]};
      } else {
        sc = *(const f32x4_t*)(scale + n);
      }
      auto pinned = [](int v) {
        v = __builtin_amdgcn_readfirstlane(v);
        asm volatile("" : "+s"(v));
        return v;
      };
      const float lo = __int_as_float(pinned(__float_as_int(p.rq_lo))), hi = __int_as_float(pinned(__float_as_int(p.rq_hi)));
      const int ldc = pinned((int)p.ldc);
      const unsigned bytes32 = (unsigned)pinned((int)(p.M * p.ldc * 4));
      constexpr unsigned kFlags = 0x00020000u;  // raw buffer, 32-bit data format
      const bool with_sums = p.rq_store >= 0;
      const __amdgpu_buffer_rsrc_t rsum = __builtin_amdgcn_make_buffer_rsrc(with_sums ? p.outs[with_sums ? p.rq_store : 0] : p.C, 0,
                                                                            with_sums ? (int)bytes32 : 0, kFlags);
      const __amdgpu_buffer_rsrc_t rq = __builtin_amdgcn_make_buffer_rsrc(p.C, 0, (int)(bytes32 >> 2), kFlags);
      // element offset of this thread's first row; rows past M are pushed beyond either buffer
      const unsigned first = (unsigned)((m0 + row0) * ldc + n);
      const int rows_left = (int)(p.M - m0) - row0;  // rows of this thread's column group that exist, counted from its first
      constexpr int kIters = (BM + RPP - 1) / RPP;
      constexpr int kRows = kIters < 8 ? kIters : 8;
#pragma unroll
      for (int it0 = 0; it0 < kIters; it0 += kRows) {
        i32x4_t acc4[kRows];
#pragma unroll
        for (int c = 0; c < kRows; ++c) {
          const int row = row0 + (it0 + c) * RPP;
          acc4[c] = *(const i32x4_t*)&ctile[(row < BM ? row : row0) * CS + c4];
        }
#pragma unroll
        for (int c = 0; c < kRows; ++c) {
          const int step = (it0 + c) * RPP;
          const bool live = row0 + step < BM && step < rows_left;
          const unsigned o = live ? first + (unsigned)(step * ldc) : 0x20000000u;  // past the si8 buffer; x 4 bytes = 2 GiB: past the si32 one
          i32x4_t a = acc4[c];
#pragma unroll
          for (int q = 0; q < 4; ++q) a[q] = (int)((unsigned)a[q] + (unsigned)(int)cinit[q]);  // (zeros when there is none)
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_tail_t, a), rsum, (int)(o << 2), 0, 0);
          uint32_t w = 0;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            float v = (float)a[q] * sc[q];
            v = __builtin_fmaxf(v, lo);
            v = __builtin_fminf(v, hi);
            const int t = (int)(v + __builtin_copysignf(0.5f, v));
            w |= (uint32_t)(t & 255) << (8 * q);
          }
          __builtin_amdgcn_raw_buffer_store_b32(w, rq, (int)o, 0, 0);
        }
      }
      return;
    }
  }
  if (KIND == KIND_I8 && p.tail_mode == 4 && full4 && (p.ldc & 3) == 0) {
    float xs[8][4];
#pragma unroll
    for (int st = 0; st < 8; ++st) {
#pragma unroll
      for (int q = 0; q < 4; ++q) xs[st][q] = 0.f;
      if (st < p.tail.n_ops) {
        const pml_hip_epi_op& op = p.tail.ops[st];
        if (op.opcode != PML_HIP_EPI_STORE && op.opcode != PML_HIP_EPI_CAST) {
          if (op.operand_kind == PML_HIP_OPND_TENSOR) {
            const float* base = (const float*)p.operands[op.operand];
            if (p.tail.operand_col_stride[op.operand] == 0) {
#pragma unroll
              for (int q = 0; q < 4; ++q) xs[st][q] = base[0];
            } else {
              const f32x4_t w = *(const f32x4_t*)(base + n);
#pragma unroll
              for (int q = 0; q < 4; ++q) xs[st][q] = w[q];
            }
          } else if (op.operand_kind == PML_HIP_OPND_IMM) {
#pragma unroll
            for (int q = 0; q < 4; ++q) xs[st][q] = (float)op.imm;
          }
        }
      }
    }
    // rows in batches of kRows, so that decoding a step is paid once per batch
    constexpr int kIters = (BM + RPP - 1) / RPP;
    constexpr int kRows = kIters < 4 ? kIters : 4;
    for (int it0 = 0; it0 < kIters; it0 += kRows) {
      int vi[kRows][4];
      float vf[kRows][4];
      bool live[kRows];
#pragma unroll
      for (int c = 0; c < kRows; ++c) {
        const int row = row0 + (it0 + c) * RPP;
        const int64_t m = m0 + row;
        live[c] = row < BM && m < p.M;
        const int rr = live[c] ? row : row0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          vi[c][q] = (int)ctile[rr * CS + c4 + q] + (int)cinit[q];
          vf[c][q] = 0.f;
        }
        if (live[c] && p.init && !col_init) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            Scalar<float, int> bb = load_scalar<float, int>(p.init, m * p.init_rs + (n + q) * p.init_cs, p.init_dtype);
            vi[c][q] = (int)((unsigned)vi[c][q] + (unsigned)bb.i);
          }
        }
      }
      int cur = PML_HIP_I32;
      auto store4 = [&](void* dst, int c) {
        const int64_t o = (m0 + row0 + (it0 + c) * RPP) * p.ldc + n;
        if (cur == PML_HIP_F32) {
          *(f32x4_t*)((float*)dst + o) = f32x4_t{vf[c][0], vf[c][1], vf[c][2], vf[c][3]};
        } else if (cur == PML_HIP_I32) {
          *(i32x4_t*)((int*)dst + o) = i32x4_t{vi[c][0], vi[c][1], vi[c][2], vi[c][3]};
        } else {
          *(uint32_t*)((uint8_t*)dst + o) = (uint32_t)(vi[c][0] & 255) | ((uint32_t)(vi[c][1] & 255) << 8) |
                                            ((uint32_t)(vi[c][2] & 255) << 16) | ((uint32_t)(vi[c][3] & 255) << 24);
        }
      };
#pragma unroll
      for (int st = 0; st < 8; ++st) {
        if (st < p.tail.n_ops) {
          const pml_hip_epi_op& op = p.tail.ops[st];
          if (op.opcode == PML_HIP_EPI_STORE) {
#pragma unroll
            for (int c = 0; c < kRows; ++c)
              if (live[c]) store4(p.outs[op.operand], c);
          } else if (op.opcode == PML_HIP_EPI_CAST) {
#pragma unroll
            for (int c = 0; c < kRows; ++c)
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                if (op.dtype == PML_HIP_F32) {
                  if (cur != PML_HIP_F32) vf[c][q] = (float)vi[c][q];
                } else {
                  int t = cur == PML_HIP_F32 ? (int)vf[c][q] : vi[c][q];
                  if (op.dtype == PML_HIP_I8) t = (int)(signed char)t;
                  vi[c][q] = t;
                }
              }
            cur = op.dtype;
          } else {
            auto each = [&](auto fn) {
#pragma unroll
              for (int c = 0; c < kRows; ++c)
#pragma unroll
                for (int q = 0; q < 4; ++q) vf[c][q] = fn(vf[c][q], xs[st][q]);
            };
            switch (op.opcode) {
              case PML_HIP_EPI_ADD: each([](float a, float b) { return a + b; }); break;
              case PML_HIP_EPI_SUB: each([](float a, float b) { return a - b; }); break;
              case PML_HIP_EPI_RSUB: each([](float a, float b) { return b - a; }); break;
              case PML_HIP_EPI_MUL: each([](float a, float b) { return a * b; }); break;
              case PML_HIP_EPI_DIV: each([](float a, float b) { return a / b; }); break;
              case PML_HIP_EPI_RDIV: each([](float a, float b) { return b / a; }); break;
              case PML_HIP_EPI_MAX: each([](float a, float b) { return (a < b) ? b : a; }); break;
              case PML_HIP_EPI_MIN: each([](float a, float b) { return (a < b) ? a : b; }); break;
              case PML_HIP_EPI_RELU: each([](float a, float) { return (a < 0.f) ? 0.f : a; }); break;
              case PML_HIP_EPI_NEG: each([](float a, float) { return -a; }); break;
              case PML_HIP_EPI_MAX_GT: each([](float a, float b) { return (a > b) ? a : b; }); break;
              case PML_HIP_EPI_ROUND: each([](float a, float) { return c_round<float>(a); }); break;
              case PML_HIP_EPI_FLOOR: each([](float a, float) { return floorf(a); }); break;
              case PML_HIP_EPI_CEIL: each([](float a, float) { return ceilf(a); }); break;
              default: break;
            }
          }
        }
      }
#pragma unroll
      for (int c = 0; c < kRows; ++c)
        if (live[c]) store4(p.C, c);
    }
    return;
  }

  for (int row = row0; row < BM; row += RPP) {
    const int64_t m = m0 + row;
    if (m >= p.M) break;
    accs_t v4[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) v4[q] = ctile[row * CS + c4 + q];
    if (col_init || p.init2 != nullptr) {
#pragma unroll
      for (int q = 0; q < 4; ++q) v4[q] += cinit[q];
    }
    if (p.init && !col_init) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (n + q < p.N) {
          Scalar<float, int> b = load_scalar<float, int>(p.init, m * p.init_rs + (n + q) * p.init_cs, p.init_dtype);
          v4[q] += KIND == KIND_I8 ? (accs_t)b.i : (accs_t)b.f;
        }
      }
    }
    for (int q = 0; q < 4; ++q) {
      if (n + q >= p.N) break;
      const int64_t nn = n + q;
      Scalar<float, int> v;
      v.f = 0;
      v.i = 0;
      int cur = p.out_dtype;
      if (KIND == KIND_I8)
        v.i = (int)v4[q];
      else
        v.f = round_float_to<float>(cur, (float)v4[q]);
      const int64_t o = m * p.ldc + nn;
      if (p.tail_mode == 1) {
        if (p.tail_relu) {
          if (KIND == KIND_I8)
            v.i = v.i < 0 ? 0 : v.i;
          else
            v.f = v.f < 0.f ? 0.f : v.f;
        }
      } else {
        int64_t off[PML_HIP_MAX_EPI_OPERANDS];
#pragma unroll
        for (int k = 0; k < PML_HIP_MAX_EPI_OPERANDS; ++k)
          off[k] = k < p.tail.n_operands ? m * p.tail.operand_row_stride[k] + nn * p.tail.operand_col_stride[k] : 0;
        v = run_tail<float, int>(p.tail, v, &cur, p.operands, off, p.outs, o);
      }
      store_scalar<float, int>(p.C, o, cur, v);
    }
  }
}

}  // namespace pml
