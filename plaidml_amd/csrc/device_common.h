// Shared device-side helpers of the gfx950 kernel library: element-type
// conversions with the reference cast rules and the interpreter for the fused
// elementwise tail.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "pml_hip.h"

namespace pml {
// A result vector that nothing in the kernel reads again, where a wavefront's store covers whole 128-byte lines
// (consecutive lanes, consecutive 16 bytes), stored as non-temporal: L2 passes such lines on instead of keeping them
// at the expense of input lines that neighbouring threads still share.  Used by the pooling kernels (3x3/2 max-pool
// with indices over 64 x 19 x 19 x 728 bf16: 11.2-11.7 -> 10.0-10.2 us on one device).  Measured and not used: the
// depthwise kernels (the kernel gains 0.5 us, the matrix product that reads its result next loses 2) and stores that
// fill a line piece by piece from several instructions (the accumulator-layout tails of the matrix and convolution
// kernels lose a quarter to a third with it).
template <typename T>
__device__ inline void store_streaming(T* p, const T& v) {
  __builtin_nontemporal_store(v, p);
}


typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) int i32x4_t;
typedef __attribute__((ext_vector_type(16))) int i32x16_t;

__host__ __device__ inline bool dt_is_float(int dt) {
  return dt == PML_HIP_F16 || dt == PML_HIP_F32 || dt == PML_HIP_F64 || dt == PML_HIP_BF16;
}
__host__ __device__ inline bool dt_is_unsigned(int dt) {
  return dt == PML_HIP_U8 || dt == PML_HIP_U16 || dt == PML_HIP_U32 || dt == PML_HIP_U64 || dt == PML_HIP_BOOL;
}
__host__ __device__ inline int dt_size(int dt) {
  switch (dt) {
    case PML_HIP_BOOL:
    case PML_HIP_I8:
    case PML_HIP_U8:
      return 1;
    case PML_HIP_I16:
    case PML_HIP_U16:
    case PML_HIP_F16:
    case PML_HIP_BF16:
      return 2;
    case PML_HIP_I32:
    case PML_HIP_U32:
    case PML_HIP_F32:
      return 4;
    case PML_HIP_I64:
    case PML_HIP_U64:
    case PML_HIP_F64:
      return 8;
  }
  return 0;
}

// Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.  A kernel whose neighbouring workgroups
// read overlapping data (window rows) takes its work in this order instead of blockIdx.x: XCD x then owns one
// contiguous range of work blocks (ranges differ by at most one when the count is no multiple of 8), and what two
// neighbours share is fetched into one L2 once instead of into up to eight.
__device__ inline unsigned xcd_contiguous_block(unsigned bid, unsigned nblocks) {
  const unsigned per = nblocks / 8, rem = nblocks % 8, x = bid % 8;
  return x * per + (x < rem ? x : rem) + bid / 8;
}

__device__ inline float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// round-to-nearest-even fp32 -> bf16 storage bits
__device__ inline uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);  // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
__device__ inline float round_to_bf16(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

__device__ inline float f16_bits_to_f32(uint16_t b) {
  _Float16 h;
  __builtin_memcpy(&h, &b, 2);
  return (float)h;
}
__device__ inline uint16_t f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;
  uint16_t b;
  __builtin_memcpy(&b, &h, 2);
  return b;
}

// A scalar travelling through an elementwise chain: floats in FT, integers in IT.
// (float,int32) serves the types up to 32 bits on the fast paths; (double,int64)
// serves every type on the general path.  A float operation done in double and
// rounded once to float equals the float operation for + - * / and sqrt.
template <typename FT, typename IT>
struct Scalar {
  FT f;
  IT i;
};

template <typename FT>
__device__ inline FT round_float_to(int dt, FT f) {
  switch (dt) {
    case PML_HIP_BF16:
      return (FT)round_to_bf16((float)f);
    case PML_HIP_F16:
      return (FT)f16_bits_to_f32(f32_to_f16_bits((float)f));
    case PML_HIP_F32:
      return (FT)(float)f;
    default:
      return f;
  }
}

template <typename IT>
__device__ inline IT wrap_int_to(int dt, IT i) {
  switch (dt) {
    case PML_HIP_BOOL:
      return (IT)(i & 1);
    case PML_HIP_I8:
      return (IT)(int8_t)i;
    case PML_HIP_U8:
      return (IT)(uint8_t)i;
    case PML_HIP_I16:
      return (IT)(int16_t)i;
    case PML_HIP_U16:
      return (IT)(uint16_t)i;
    case PML_HIP_I32:
      return (IT)(int32_t)i;
    case PML_HIP_U32:
      return sizeof(IT) == 8 ? (IT)(uint32_t)i : i;
    default:
      return i;
  }
}

template <typename FT, typename IT>
__device__ inline Scalar<FT, IT> load_scalar(const void* p, int64_t off, int dt) {
  Scalar<FT, IT> r;
  r.f = 0;
  r.i = 0;
  switch (dt) {
    case PML_HIP_BOOL:
    case PML_HIP_U8:
      r.i = (IT)((const uint8_t*)p)[off];
      break;
    case PML_HIP_I8:
      r.i = (IT)((const int8_t*)p)[off];
      break;
    case PML_HIP_I16:
      r.i = (IT)((const int16_t*)p)[off];
      break;
    case PML_HIP_U16:
      r.i = (IT)((const uint16_t*)p)[off];
      break;
    case PML_HIP_I32:
      r.i = (IT)((const int32_t*)p)[off];
      break;
    case PML_HIP_U32:
      r.i = (IT)((const uint32_t*)p)[off];
      break;
    case PML_HIP_I64:
    case PML_HIP_U64:
      r.i = (IT)((const int64_t*)p)[off];
      break;
    case PML_HIP_F16:
      r.f = (FT)f16_bits_to_f32(((const uint16_t*)p)[off]);
      break;
    case PML_HIP_BF16:
      r.f = (FT)bf16_bits_to_f32(((const uint16_t*)p)[off]);
      break;
    case PML_HIP_F32:
      r.f = (FT)((const float*)p)[off];
      break;
    case PML_HIP_F64:
      r.f = (FT)((const double*)p)[off];
      break;
  }
  return r;
}

template <typename FT, typename IT>
__device__ inline void store_scalar(void* p, int64_t off, int dt, Scalar<FT, IT> v) {
  switch (dt) {
    case PML_HIP_BOOL:
    case PML_HIP_U8:
    case PML_HIP_I8:
      ((uint8_t*)p)[off] = (uint8_t)v.i;
      break;
    case PML_HIP_I16:
    case PML_HIP_U16:
      ((uint16_t*)p)[off] = (uint16_t)v.i;
      break;
    case PML_HIP_I32:
    case PML_HIP_U32:
      ((uint32_t*)p)[off] = (uint32_t)v.i;
      break;
    case PML_HIP_I64:
    case PML_HIP_U64:
      ((int64_t*)p)[off] = (int64_t)v.i;
      break;
    case PML_HIP_F16:
      ((uint16_t*)p)[off] = f32_to_f16_bits((float)v.f);
      break;
    case PML_HIP_BF16:
      ((uint16_t*)p)[off] = f32_to_bf16_bits((float)v.f);
      break;
    case PML_HIP_F32:
      ((float*)p)[off] = (float)v.f;
      break;
    case PML_HIP_F64:
      ((double*)p)[off] = (double)v.f;
      break;
  }
}

// tile.cast: widen integers by the source's signedness, narrow by truncation,
// fp -> int truncates toward zero, int -> fp converts by the source's
// signedness, fp -> fp rounds to nearest even.
template <typename FT, typename IT>
__device__ inline Scalar<FT, IT> convert_scalar(Scalar<FT, IT> v, int from, int to) {
  if (from == to) return v;
  typedef typename std::conditional<sizeof(IT) == 8, uint64_t, uint32_t>::type UT;
  Scalar<FT, IT> r;
  r.f = 0;
  r.i = 0;
  const bool ff = dt_is_float(from), tf = dt_is_float(to);
  if (to == PML_HIP_BOOL) {
    r.i = ff ? (IT)(v.f != (FT)0) : (IT)(v.i != 0);
  } else if (ff && tf) {
    r.f = round_float_to<FT>(to, v.f);
  } else if (ff) {
    if (dt_is_unsigned(to))
      r.i = wrap_int_to<IT>(to, (IT)(UT)v.f);
    else
      r.i = wrap_int_to<IT>(to, (IT)v.f);
  } else if (tf) {
    FT x = (dt_is_unsigned(from) && sizeof(IT) == 8 && from == PML_HIP_U64) ? (FT)(UT)v.i : (FT)v.i;
    if (from == PML_HIP_U32 && sizeof(IT) == 4) x = (FT)(UT)v.i;
    r.f = round_float_to<FT>(to, x);
  } else {
    r.i = wrap_int_to<IT>(to, v.i);
  }
  return r;
}

template <typename FT>
__device__ inline FT c_round(FT x) {
  return x >= (FT)0 ? floor(x + (FT)0.5) : ceil(x - (FT)0.5);
}

// The tail of a contraction or a standalone elementwise chain.  `opnd_off[j]`
// is the element offset into operands[j] for the current output element and
// `out_off` the offset used by STORE steps.  Returns the final value; *cur_dt
// is updated to its element type.
template <typename FT, typename IT>
__device__ inline Scalar<FT, IT> run_tail(const pml_hip_epilogue& t, Scalar<FT, IT> v, int* cur_dt,
                                          const void* const* operands, const int64_t* opnd_off, void* const* outs,
                                          int64_t out_off) {
  typedef typename std::conditional<sizeof(IT) == 8, uint64_t, uint32_t>::type UT;
  int cur = *cur_dt;
  for (int s = 0; s < t.n_ops; ++s) {
    const pml_hip_epi_op& op = t.ops[s];
    const int dt = op.dtype;
    if (op.opcode == PML_HIP_EPI_STORE) {
      store_scalar<FT, IT>(outs[op.operand], out_off, cur, v);
      continue;
    }
    if (op.opcode == PML_HIP_EPI_CAST) {
      v = convert_scalar<FT, IT>(v, cur, dt);
      cur = dt;
      continue;
    }
    Scalar<FT, IT> x;
    x.f = 0;
    x.i = 0;
    if (op.operand_kind == PML_HIP_OPND_TENSOR) {
      const int od = t.operand_dtype[op.operand];
      x = convert_scalar<FT, IT>(load_scalar<FT, IT>(operands[op.operand], opnd_off[op.operand], od), od, dt);
    } else if (op.operand_kind == PML_HIP_OPND_IMM) {
      if (dt_is_float(dt))
        x.f = round_float_to<FT>(dt, (FT)op.imm);
      else
        x.i = wrap_int_to<IT>(dt, (IT)op.imm);
    }
    v = convert_scalar<FT, IT>(v, cur, dt);
    const bool isf = dt_is_float(dt);
    const bool uns = dt_is_unsigned(dt);
    bool is_cmp = false, cmp = false;
    if (isf) {
      FT a = v.f, b = x.f, r = a;
      switch (op.opcode) {
        case PML_HIP_EPI_ADD: r = a + b; break;
        case PML_HIP_EPI_SUB: r = a - b; break;
        case PML_HIP_EPI_RSUB: r = b - a; break;
        case PML_HIP_EPI_MUL: r = a * b; break;
        case PML_HIP_EPI_DIV: r = a / b; break;
        case PML_HIP_EPI_RDIV: r = b / a; break;
        case PML_HIP_EPI_MAX: r = (a < b) ? b : a; break;
        case PML_HIP_EPI_MIN: r = (a < b) ? a : b; break;
        case PML_HIP_EPI_RELU: r = (a < (FT)0) ? (FT)0 : a; break;
        case PML_HIP_EPI_NEG: r = -a; break;
        case PML_HIP_EPI_EXP: r = sizeof(FT) == 4 || dt != PML_HIP_F64 ? (FT)expf((float)a) : (FT)exp((double)a); break;
        case PML_HIP_EPI_LOG: r = sizeof(FT) == 4 || dt != PML_HIP_F64 ? (FT)logf((float)a) : (FT)log((double)a); break;
        case PML_HIP_EPI_SQRT: r = sizeof(FT) == 4 || dt != PML_HIP_F64 ? (FT)sqrtf((float)a) : (FT)sqrt((double)a); break;
        case PML_HIP_EPI_TANH: r = sizeof(FT) == 4 || dt != PML_HIP_F64 ? (FT)tanhf((float)a) : (FT)tanh((double)a); break;
        case PML_HIP_EPI_FLOOR: r = floor(a); break;
        case PML_HIP_EPI_CEIL: r = ceil(a); break;
        case PML_HIP_EPI_ROUND: r = c_round<FT>(a); break;
        case PML_HIP_EPI_CMP_LT: is_cmp = true; cmp = a < b; break;
        case PML_HIP_EPI_CMP_GT: is_cmp = true; cmp = a > b; break;
        case PML_HIP_EPI_CMP_LE: is_cmp = true; cmp = a <= b; break;
        case PML_HIP_EPI_CMP_GE: is_cmp = true; cmp = a >= b; break;
        case PML_HIP_EPI_CMP_EQ: is_cmp = true; cmp = a == b; break;
        case PML_HIP_EPI_CMP_NE: is_cmp = true; cmp = (a < b) || (a > b); break;  // ordered not-equal
        case PML_HIP_EPI_MAX_GT: r = (a > b) ? a : b; break;
#define PML_MATH1(OP, FN) \
  case OP: r = sizeof(FT) == 4 || dt != PML_HIP_F64 ? (FT)FN##f((float)a) : (FT)FN((double)a); break;
        PML_MATH1(PML_HIP_EPI_SIN, sin)
        PML_MATH1(PML_HIP_EPI_COS, cos)
        PML_MATH1(PML_HIP_EPI_TAN, tan)
        PML_MATH1(PML_HIP_EPI_SINH, sinh)
        PML_MATH1(PML_HIP_EPI_COSH, cosh)
        PML_MATH1(PML_HIP_EPI_ASIN, asin)
        PML_MATH1(PML_HIP_EPI_ACOS, acos)
        PML_MATH1(PML_HIP_EPI_ATAN, atan)
        PML_MATH1(PML_HIP_EPI_ASINH, asinh)
        PML_MATH1(PML_HIP_EPI_ACOSH, acosh)
        PML_MATH1(PML_HIP_EPI_ATANH, atanh)
        PML_MATH1(PML_HIP_EPI_ERF, erf)
#undef PML_MATH1
        case PML_HIP_EPI_POW:
          r = sizeof(FT) == 4 || dt != PML_HIP_F64 ? (FT)powf((float)a, (float)b) : (FT)pow((double)a, (double)b);
          break;
        case PML_HIP_EPI_RPOW:
          r = sizeof(FT) == 4 || dt != PML_HIP_F64 ? (FT)powf((float)b, (float)a) : (FT)pow((double)b, (double)a);
          break;
        case PML_HIP_EPI_MOD:
          r = sizeof(FT) == 4 || dt != PML_HIP_F64 ? (FT)fmodf((float)a, (float)b) : (FT)fmod((double)a, (double)b);
          break;
        case PML_HIP_EPI_RMOD:
          r = sizeof(FT) == 4 || dt != PML_HIP_F64 ? (FT)fmodf((float)b, (float)a) : (FT)fmod((double)b, (double)a);
          break;
        // truth values: ordered "not equal to zero", so a NaN is false
        case PML_HIP_EPI_LOGICAL_AND: is_cmp = true; cmp = (a < 0 || a > 0) && (b < 0 || b > 0); break;
        case PML_HIP_EPI_LOGICAL_OR: is_cmp = true; cmp = (a < 0 || a > 0) || (b < 0 || b > 0); break;
        case PML_HIP_EPI_LOGICAL_XOR: is_cmp = true; cmp = (a < 0 || a > 0) != (b < 0 || b > 0); break;
        case PML_HIP_EPI_LOGICAL_NOT: is_cmp = true; cmp = a == (FT)0; break;
        default: break;
      }
      v.f = round_float_to<FT>(dt, r);
    } else {
      IT a = v.i, b = x.i, r = a;
      UT ua = (UT)a, ub = (UT)b;
      switch (op.opcode) {
        case PML_HIP_EPI_ADD: r = (IT)(ua + ub); break;
        case PML_HIP_EPI_SUB: r = (IT)(ua - ub); break;
        case PML_HIP_EPI_RSUB: r = (IT)(ub - ua); break;
        case PML_HIP_EPI_MUL: r = (IT)(ua * ub); break;
        case PML_HIP_EPI_DIV: r = b == 0 ? 0 : (uns ? (IT)(ua / ub) : a / b); break;
        case PML_HIP_EPI_RDIV: r = a == 0 ? 0 : (uns ? (IT)(ub / ua) : b / a); break;
        case PML_HIP_EPI_MAX: r = (uns ? (ua < ub) : (a < b)) ? b : a; break;
        case PML_HIP_EPI_MIN: r = (uns ? (ua < ub) : (a < b)) ? a : b; break;
        case PML_HIP_EPI_RELU: r = (!uns && a < 0) ? 0 : a; break;
        case PML_HIP_EPI_NEG: r = (IT)((UT)0 - ua); break;
        case PML_HIP_EPI_CMP_LT: is_cmp = true; cmp = uns ? (ua < ub) : (a < b); break;
        case PML_HIP_EPI_CMP_GT: is_cmp = true; cmp = uns ? (ua > ub) : (a > b); break;
        case PML_HIP_EPI_CMP_LE: is_cmp = true; cmp = uns ? (ua <= ub) : (a <= b); break;
        case PML_HIP_EPI_CMP_GE: is_cmp = true; cmp = uns ? (ua >= ub) : (a >= b); break;
        case PML_HIP_EPI_CMP_EQ: is_cmp = true; cmp = a == b; break;
        case PML_HIP_EPI_CMP_NE: is_cmp = true; cmp = a != b; break;
        case PML_HIP_EPI_MAX_GT: r = (uns ? (ua > ub) : (a > b)) ? a : b; break;
        case PML_HIP_EPI_MOD: r = b == 0 ? 0 : (uns ? (IT)(ua % ub) : a % b); break;
        case PML_HIP_EPI_RMOD: r = a == 0 ? 0 : (uns ? (IT)(ub % ua) : b % a); break;
        case PML_HIP_EPI_BIT_AND: r = a & b; break;
        case PML_HIP_EPI_BIT_OR: r = a | b; break;
        case PML_HIP_EPI_BIT_XOR: r = a ^ b; break;
        case PML_HIP_EPI_BIT_NOT: r = (IT)((UT)-1 - ua); break;
        // shift counts at or beyond the type's width are undefined in the reference: 0 here (sign fill for
        // an arithmetic right shift)
        case PML_HIP_EPI_SHL: r = ub >= sizeof(IT) * 8 ? 0 : (IT)(ua << ub); break;
        case PML_HIP_EPI_RSHL: r = ua >= sizeof(IT) * 8 ? 0 : (IT)(ub << ua); break;
        case PML_HIP_EPI_SHR: {
          const UT n = ub >= sizeof(IT) * 8 ? (UT)(sizeof(IT) * 8 - 1) : ub;
          r = uns ? (ub >= sizeof(IT) * 8 ? 0 : (IT)(ua >> n)) : (a >> n);
          break;
        }
        case PML_HIP_EPI_RSHR: {
          const UT n = ua >= sizeof(IT) * 8 ? (UT)(sizeof(IT) * 8 - 1) : ua;
          r = uns ? (ua >= sizeof(IT) * 8 ? 0 : (IT)(ub >> n)) : (b >> n);
          break;
        }
        case PML_HIP_EPI_LOGICAL_AND: is_cmp = true; cmp = a != 0 && b != 0; break;
        case PML_HIP_EPI_LOGICAL_OR: is_cmp = true; cmp = a != 0 || b != 0; break;
        case PML_HIP_EPI_LOGICAL_XOR: is_cmp = true; cmp = (a != 0) != (b != 0); break;
        case PML_HIP_EPI_LOGICAL_NOT: is_cmp = true; cmp = a == 0; break;
        default: break;
      }
      v.i = wrap_int_to<IT>(dt, r);
    }
    if (is_cmp) {
      v.f = 0;
      v.i = cmp ? 1 : 0;
      cur = PML_HIP_BOOL;
    } else {
      cur = dt;
    }
  }
  *cur_dt = cur;
  return v;
}

}  // namespace pml
