// Kernels that accept any contraction / elementwise chain in scope: the
// safety net beneath the specialised MFMA and window kernels, plus the small
// utility kernels (fill, iota, select).
#include <hip/hip_runtime.h>

#include "device_common.h"
#include "plans.h"

namespace pml {

namespace {

// ---------------------------------------------------------------------------
// any contraction: one thread per output element, odometer over the reduction box
// ---------------------------------------------------------------------------

template <typename FT, typename IT>
__device__ inline Scalar<FT, IT> combine(int combo, int dt, int cmp_dt, const Scalar<FT, IT>* x) {
  typedef typename std::conditional<sizeof(IT) == 8, uint64_t, uint32_t>::type UT;
  Scalar<FT, IT> r;
  r.f = 0;
  r.i = 0;
  const bool isf = dt_is_float(dt);
  switch (combo) {
    case PML_HIP_COMBO_NONE:
      r = x[0];
      break;
    case PML_HIP_COMBO_ADD:
      if (isf)
        r.f = x[0].f + x[1].f;
      else
        r.i = wrap_int_to<IT>(dt, (IT)((UT)x[0].i + (UT)x[1].i));
      break;
    case PML_HIP_COMBO_MUL:
      if (isf)
        r.f = x[0].f * x[1].f;
      else
        r.i = wrap_int_to<IT>(dt, (IT)((UT)x[0].i * (UT)x[1].i));
      break;
    case PML_HIP_COMBO_COND: {
      const bool eq = dt_is_float(cmp_dt) ? (x[0].f == x[1].f) : (x[0].i == x[1].i);
      if (eq) r = x[2];
      break;
    }
    default:
      break;
  }
  return r;
}

template <typename FT, typename IT>
__device__ inline void aggregate(int agg, int dt, Scalar<FT, IT>& acc, const Scalar<FT, IT>& v) {
  typedef typename std::conditional<sizeof(IT) == 8, uint64_t, uint32_t>::type UT;
  const bool isf = dt_is_float(dt);
  const bool uns = dt_is_unsigned(dt);
  switch (agg) {
    case PML_HIP_AGG_ASSIGN:
      acc = v;
      break;
    case PML_HIP_AGG_ADD:
      if (isf)
        acc.f = acc.f + v.f;
      else
        acc.i = wrap_int_to<IT>(dt, (IT)((UT)acc.i + (UT)v.i));
      break;
    case PML_HIP_AGG_MUL:
      if (isf)
        acc.f = acc.f * v.f;
      else
        acc.i = wrap_int_to<IT>(dt, (IT)((UT)acc.i * (UT)v.i));
      break;
    case PML_HIP_AGG_MAX:
      if (isf)
        acc.f = (v.f > acc.f) ? v.f : acc.f;
      else
        acc.i = (uns ? ((UT)v.i > (UT)acc.i) : (v.i > acc.i)) ? v.i : acc.i;
      break;
    case PML_HIP_AGG_MIN:
      if (isf)
        acc.f = (v.f < acc.f) ? v.f : acc.f;
      else
        acc.i = (uns ? ((UT)v.i < (UT)acc.i) : (v.i < acc.i)) ? v.i : acc.i;
      break;
  }
}

// One point of the reduction box: checks every input access, loads, combines and aggregates into acc.
template <typename FT, typename IT>
__device__ inline void accumulate_point(const pml_hip_contract_desc& d, const ContractArgs& a, const int64_t* base,
                                        const int64_t* idx, int acc_dt, Scalar<FT, IT>& acc) {
  bool ok = true;
  int64_t off[4] = {0, 0, 0, 0};
  for (int f = 0; f < d.n_forms && ok; ++f) {
    const pml_hip_form& fm = d.forms[f];
    if (fm.operand == 0) continue;
    int64_t s = base[f];
    for (int v = d.n_out_idx; v < d.n_idx; ++v) s += (int64_t)fm.coef[v] * idx[v];
    if (fm.den != 1) {
      if (s % fm.den != 0) {
        ok = false;
        break;
      }
      s /= fm.den;
    }
    if (s < 0 || s >= fm.size) {
      ok = false;
      break;
    }
    if (fm.operand > 0) off[fm.operand] += s * fm.stride;
  }
  if (ok) {
    Scalar<FT, IT> x[3];
    for (int q = 0; q < d.n_src; ++q) {
      const int sd = d.src_dtype[q];
      Scalar<FT, IT> raw = load_scalar<FT, IT>(a.srcs[q], off[q + 1], sd);
      if (d.combo == PML_HIP_COMBO_COND && q < 2) {
        x[q] = convert_scalar<FT, IT>(raw, sd, d.cmp_dtype);
      } else if (!dt_is_float(sd) && !dt_is_float(acc_dt) && sd != PML_HIP_BOOL && dt_size(sd) < dt_size(acc_dt) &&
                 d.combo != PML_HIP_COMBO_COND) {
        // operands of a contraction body are signless: widening is zero-extension
        Scalar<FT, IT> z = raw;
        const int bits = dt_size(sd) * 8;
        z.i = raw.i & (IT)((((uint64_t)1) << bits) - 1);
        x[q] = z;
      } else {
        x[q] = convert_scalar<FT, IT>(raw, sd, acc_dt);
      }
    }
    Scalar<FT, IT> v = combine<FT, IT>(d.combo, acc_dt, d.cmp_dtype, x);
    aggregate<FT, IT>(d.agg, acc_dt, acc, v);
  }
}

template <typename FT, typename IT>
__global__ __launch_bounds__(256) void contract_kernel(ContractArgs a) {
  const pml_hip_contract_desc& d = a.d;
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= d.out_elems) return;

  int64_t idx[PML_HIP_MAX_IDX];
  {
    int64_t t = gid;
    for (int v = d.n_out_idx - 1; v >= 0; --v) {
      const int64_t range = d.hi[v] - d.lo[v] + 1;
      idx[v] = d.lo[v] + t % range;
      t /= range;
    }
  }
  // contribution of the output indices to every form
  int64_t base[PML_HIP_MAX_FORMS];
  for (int f = 0; f < d.n_forms; ++f) {
    int64_t s = d.forms[f].c0;
    for (int v = 0; v < d.n_out_idx; ++v) s += (int64_t)d.forms[f].coef[v] * idx[v];
    base[f] = s;
  }
  // the output element of this thread; skip if its access is not valid
  int64_t out_off = 0;
  for (int f = 0; f < d.n_forms; ++f) {
    if (d.forms[f].operand != 0) continue;
    int64_t q = base[f];
    const int den = d.forms[f].den;
    if (den != 1) {
      if (q % den != 0) return;
      q /= den;
    }
    if (q < 0 || q >= d.forms[f].size) return;
    out_off += q * d.forms[f].stride;
  }

  const int dt = d.dtype;
  // bf16 / f16 results accumulate in fp32 and are rounded once at the end
  const int acc_dt = (dt == PML_HIP_BF16 || dt == PML_HIP_F16) ? PML_HIP_F32 : dt;
  Scalar<FT, IT> acc;
  if (d.has_init) {
    acc = convert_scalar<FT, IT>(load_scalar<FT, IT>(a.out, out_off, dt), dt, acc_dt);
  } else {
    acc.f = dt_is_float(dt) ? (FT)d.identity_f : (FT)0;
    acc.i = dt_is_float(dt) ? (IT)0 : wrap_int_to<IT>(dt, (IT)d.identity_i);
  }

  bool empty = false;
  for (int v = d.n_out_idx; v < d.n_idx; ++v) {
    idx[v] = d.lo[v];
    if (d.lo[v] > d.hi[v]) empty = true;
  }
  while (!empty) {
    accumulate_point<FT, IT>(d, a, base, idx, acc_dt, acc);
    int v = d.n_idx - 1;
    for (; v >= d.n_out_idx; --v) {
      if (++idx[v] <= d.hi[v]) break;
      idx[v] = d.lo[v];
    }
    if (v < d.n_out_idx) break;
  }
  store_scalar<FT, IT>(a.out, out_off, dt, convert_scalar<FT, IT>(acc, acc_dt, dt));
}

// Few outputs, long reductions (row max / row sum of a softmax, global pooling): one workgroup per
// output point.  Thread t takes the points t, t + 256, ... of the linearised reduction box, starting
// from the aggregation's identity; the 256 partial results and the initial value (if any) are then
// aggregated once.  Only for add / mul / max / min, whose result does not depend on grouping (up to
// floating-point rounding).
template <typename FT, typename IT>
__global__ __launch_bounds__(256) void contract_coop_kernel(ContractArgs a, int64_t red_count) {
  const pml_hip_contract_desc& d = a.d;
  const int64_t gid = blockIdx.x;
  __shared__ FT part_f[256];
  __shared__ IT part_i[256];

  int64_t idx[PML_HIP_MAX_IDX];
  {
    int64_t t = gid;
    for (int v = d.n_out_idx - 1; v >= 0; --v) {
      const int64_t range = d.hi[v] - d.lo[v] + 1;
      idx[v] = d.lo[v] + t % range;
      t /= range;
    }
  }
  int64_t base[PML_HIP_MAX_FORMS];
  for (int f = 0; f < d.n_forms; ++f) {
    int64_t s = d.forms[f].c0;
    for (int v = 0; v < d.n_out_idx; ++v) s += (int64_t)d.forms[f].coef[v] * idx[v];
    base[f] = s;
  }
  int64_t out_off = 0;
  for (int f = 0; f < d.n_forms; ++f) {
    if (d.forms[f].operand != 0) continue;
    int64_t q = base[f];
    const int den = d.forms[f].den;
    if (den != 1) {
      if (q % den != 0) return;  // uniform over the workgroup
      q /= den;
    }
    if (q < 0 || q >= d.forms[f].size) return;
    out_off += q * d.forms[f].stride;
  }
  const int dt = d.dtype;
  const int acc_dt = (dt == PML_HIP_BF16 || dt == PML_HIP_F16) ? PML_HIP_F32 : dt;
  Scalar<FT, IT> ident;
  ident.f = dt_is_float(dt) ? (FT)d.identity_f : (FT)0;
  ident.i = dt_is_float(dt) ? (IT)0 : wrap_int_to<IT>(dt, (IT)d.identity_i);
  Scalar<FT, IT> acc = ident;
  for (int64_t r = threadIdx.x; r < red_count; r += 256) {
    int64_t t = r;
    for (int v = d.n_idx - 1; v >= d.n_out_idx; --v) {
      const int64_t range = d.hi[v] - d.lo[v] + 1;
      idx[v] = d.lo[v] + t % range;
      t /= range;
    }
    accumulate_point<FT, IT>(d, a, base, idx, acc_dt, acc);
  }
  part_f[threadIdx.x] = acc.f;
  part_i[threadIdx.x] = acc.i;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) {
      Scalar<FT, IT> x, y;
      x.f = part_f[threadIdx.x], x.i = part_i[threadIdx.x];
      y.f = part_f[threadIdx.x + w], y.i = part_i[threadIdx.x + w];
      aggregate<FT, IT>(d.agg, acc_dt, x, y);
      part_f[threadIdx.x] = x.f;
      part_i[threadIdx.x] = x.i;
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    Scalar<FT, IT> total;
    total.f = part_f[0], total.i = part_i[0];
    if (d.has_init) {
      Scalar<FT, IT> start = convert_scalar<FT, IT>(load_scalar<FT, IT>(a.out, out_off, dt), dt, acc_dt);
      aggregate<FT, IT>(d.agg, acc_dt, start, total);
      total = start;
    }
    store_scalar<FT, IT>(a.out, out_off, dt, convert_scalar<FT, IT>(total, acc_dt, dt));
  }
}

// ---------------------------------------------------------------------------
// elementwise chain with N-d broadcasting
// ---------------------------------------------------------------------------

template <typename FT, typename IT>
__global__ __launch_bounds__(256) void eltwise_kernel(EltwiseArgs a) {
  const pml_hip_eltwise_desc& d = a.d;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; gid < a.total; gid += stride) {
    int64_t t = gid;
    int64_t in_off = 0;
    int64_t off[PML_HIP_MAX_EPI_OPERANDS] = {0, 0, 0, 0, 0, 0};
    for (int r = d.rank - 1; r >= 0; --r) {
      const int64_t c = t % d.sizes[r];
      t /= d.sizes[r];
      in_off += c * d.in_strides[r];
      for (int q = 0; q < d.tail.n_operands; ++q) off[q] += c * d.operand_strides[q][r];
    }
    int cur = d.in_dtype;
    Scalar<FT, IT> v = load_scalar<FT, IT>(a.in, in_off, cur);
    v = run_tail<FT, IT>(d.tail, v, &cur, a.operands, off, a.outs, gid);
    store_scalar<FT, IT>(a.out, gid, cur, v);
  }
}

// Contiguous fast path: the first input has the output's shape, every operand is
// either output-shaped, a vector along the last dimension, or a single element,
// and all element types are 2 bytes wide or all 4 bytes wide.  Each thread
// moves 16 bytes per tensor.
template <int ES>
__global__ __launch_bounds__(256) void eltwise_vec_kernel(EltwiseArgs a, int64_t inner, unsigned opnd_full_mask,
                                                          unsigned opnd_vec_mask) {
  constexpr int V = 16 / ES;
  const pml_hip_eltwise_desc& d = a.d;
  const int64_t n_vec = a.total / V;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  constexpr int U = 4;  // independent 16-byte loads in flight per thread
  for (int64_t g0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g0 < n_vec; g0 += U * stride) {
    i32x4_t raw[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t g = g0 + u * stride;
      if (g < n_vec) raw[u] = *(const i32x4_t*)((const unsigned char*)a.in + g * V * ES);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t g = g0 + u * stride;
      if (g >= n_vec) break;
      const int64_t e0 = g * V;
      i32x4_t res;
      const int64_t c0 = e0 % inner;
#pragma unroll
      for (int e = 0; e < V; ++e) {
        int cur = d.in_dtype;
        Scalar<float, int> v = load_scalar<float, int>(&raw[u], e, cur);
        int64_t off[PML_HIP_MAX_EPI_OPERANDS];
#pragma unroll
        for (int q = 0; q < PML_HIP_MAX_EPI_OPERANDS; ++q)
          off[q] = ((opnd_full_mask >> q) & 1) ? e0 + e : (((opnd_vec_mask >> q) & 1) ? c0 + e : 0);
        v = run_tail<float, int>(d.tail, v, &cur, a.operands, off, a.outs, e0 + e);
        store_scalar<float, int>(&res, e, cur, v);
      }
      *(i32x4_t*)((unsigned char*)a.out + e0 * ES) = res;
    }
  }
}

template <typename FT, typename IT>
__global__ __launch_bounds__(256) void select_kernel(pml_hip_select_desc d, const void* c, const void* t, const void* f,
                                                     void* out, int64_t total) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; gid < total; gid += stride) {
    int64_t r = gid, co = 0, to = 0, fo = 0;
    for (int k = d.rank - 1; k >= 0; --k) {
      const int64_t x = r % d.sizes[k];
      r /= d.sizes[k];
      co += x * d.cond_strides[k];
      to += x * d.t_strides[k];
      fo += x * d.f_strides[k];
    }
    Scalar<FT, IT> cv = load_scalar<FT, IT>(c, co, d.cond_dtype);
    const bool pick = dt_is_float(d.cond_dtype) ? (cv.f != (FT)0) : (cv.i != 0);
    Scalar<FT, IT> v = pick ? convert_scalar<FT, IT>(load_scalar<FT, IT>(t, to, d.t_dtype), d.t_dtype, d.out_dtype)
                            : convert_scalar<FT, IT>(load_scalar<FT, IT>(f, fo, d.f_dtype), d.f_dtype, d.out_dtype);
    store_scalar<FT, IT>(out, gid, d.out_dtype, v);
  }
}

__global__ __launch_bounds__(256) void index_kernel(int32_t* out, int64_t total, int64_t inner, int64_t extent) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; gid < total; gid += stride)
    out[gid] = (int32_t)((gid / inner) % extent);
}

__global__ __launch_bounds__(256) void fill_kernel(uint32_t* p, uint32_t pattern, size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) p[i] = pattern;
}

inline unsigned grid_for(int64_t work_items) {
  int64_t blocks = (work_items + 255) / 256;
  if (blocks < 1) blocks = 1;
  const int64_t cap = 256 * 32;  // 256 CUs, deep enough to cover HBM latency
  return (unsigned)(blocks < cap ? blocks : cap);
}

bool is_wide(int dt) { return dt == PML_HIP_F64 || dt == PML_HIP_I64 || dt == PML_HIP_U64; }

}  // namespace

hipError_t contract_launch(const ContractArgs& a, hipStream_t s) {
  const pml_hip_contract_desc& d = a.d;
  bool wide = is_wide(d.dtype) || is_wide(d.cmp_dtype);
  for (int q = 0; q < d.n_src; ++q) wide = wide || is_wide(d.src_dtype[q]);
  const unsigned blocks = (unsigned)((d.out_elems + 255) / 256);
  if (blocks == 0) return hipSuccess;
  // too few outputs to fill the chip and a long reduction: one workgroup per output
  int64_t red_count = 1;
  for (int v = d.n_out_idx; v < d.n_idx; ++v) red_count *= d.hi[v] >= d.lo[v] ? d.hi[v] - d.lo[v] + 1 : 0;
  if (d.agg != PML_HIP_AGG_ASSIGN && d.out_elems <= 4096 && red_count >= 512) {
    if (wide)
      hipLaunchKernelGGL((contract_coop_kernel<double, int64_t>), dim3((unsigned)d.out_elems), dim3(256), 0, s, a, red_count);
    else
      hipLaunchKernelGGL((contract_coop_kernel<float, int>), dim3((unsigned)d.out_elems), dim3(256), 0, s, a, red_count);
    return hipGetLastError();
  }
  if (wide)
    hipLaunchKernelGGL((contract_kernel<double, int64_t>), dim3(blocks), dim3(256), 0, s, a);
  else
    hipLaunchKernelGGL((contract_kernel<float, int>), dim3(blocks), dim3(256), 0, s, a);
  return hipGetLastError();
}

hipError_t eltwise_launch(const EltwiseArgs& a, hipStream_t s) {
  if (a.total == 0) return hipSuccess;
  const pml_hip_eltwise_desc& d = a.d;
  if (a.wide) {
    hipLaunchKernelGGL((eltwise_kernel<double, int64_t>), dim3(grid_for(a.total)), dim3(256), 0, s, a);
    return hipGetLastError();
  }
  // try the 16-byte path
  const int es = dt_size(d.in_dtype);
  bool vec_ok = (es == 2 || es == 4) && dt_size(d.out_dtype) == es && d.rank >= 1;
  int64_t inner = d.rank >= 1 ? d.sizes[d.rank - 1] : 1;
  unsigned full_mask = 0, vec_mask = 0;
  if (vec_ok) {
    int64_t st = 1;
    for (int r = d.rank - 1; r >= 0; --r) {
      if (d.sizes[r] != 1 && d.in_strides[r] != st) vec_ok = false;
      st *= d.sizes[r];
    }
    for (int q = 0; q < d.tail.n_operands && vec_ok; ++q) {
      bool full = true, vec = true, scal = true;
      int64_t st2 = 1;
      for (int r = d.rank - 1; r >= 0; --r) {
        const int64_t os = d.operand_strides[q][r];
        if (d.sizes[r] != 1) {
          if (os != st2) full = false;
          if (os != ((r == d.rank - 1) ? 1 : 0)) vec = false;
          if (os != 0) scal = false;
        }
        st2 *= d.sizes[r];
      }
      if (full)
        full_mask |= 1u << q;
      else if (vec)
        vec_mask |= 1u << q;
      else if (!scal)
        vec_ok = false;
    }
    for (int k = 0; k < d.tail.n_ops; ++k) {
      const pml_hip_epi_op& op = d.tail.ops[k];
      if (op.opcode == PML_HIP_EPI_STORE) vec_ok = false;
      if (op.opcode == PML_HIP_EPI_CAST && dt_size(op.dtype) != es && k == d.tail.n_ops - 1) vec_ok = false;
    }
    const int V = 16 / es;
    if (a.total % V != 0 || inner % V != 0) vec_ok = false;
    if (((uintptr_t)a.in | (uintptr_t)a.out) & 15) vec_ok = false;
  }
  if (vec_ok) {
    const int V = 16 / es;
    const unsigned g = grid_for(a.total / V);
    if (es == 2)
      hipLaunchKernelGGL((eltwise_vec_kernel<2>), dim3(g), dim3(256), 0, s, a, inner, full_mask, vec_mask);
    else
      hipLaunchKernelGGL((eltwise_vec_kernel<4>), dim3(g), dim3(256), 0, s, a, inner, full_mask, vec_mask);
    return hipGetLastError();
  }
  hipLaunchKernelGGL((eltwise_kernel<float, int>), dim3(grid_for(a.total)), dim3(256), 0, s, a);
  return hipGetLastError();
}

hipError_t select_launch(const pml_hip_select_desc& d, const void* c, const void* t, const void* f, void* out,
                         hipStream_t s) {
  int64_t total = 1;
  for (int r = 0; r < d.rank; ++r) total *= d.sizes[r];
  if (total == 0) return hipSuccess;
  const bool wide = is_wide(d.cond_dtype) || is_wide(d.t_dtype) || is_wide(d.f_dtype) || is_wide(d.out_dtype);
  if (wide)
    hipLaunchKernelGGL((select_kernel<double, int64_t>), dim3(grid_for(total)), dim3(256), 0, s, d, c, t, f, out, total);
  else
    hipLaunchKernelGGL((select_kernel<float, int>), dim3(grid_for(total)), dim3(256), 0, s, d, c, t, f, out, total);
  return hipGetLastError();
}

hipError_t index_launch(void* out, int rank, const int64_t* sizes, int axis, hipStream_t s) {
  int64_t total = 1, inner = 1;
  for (int r = 0; r < rank; ++r) total *= sizes[r];
  for (int r = axis + 1; r < rank; ++r) inner *= sizes[r];
  if (total == 0) return hipSuccess;
  hipLaunchKernelGGL(index_kernel, dim3(grid_for(total)), dim3(256), 0, s, (int32_t*)out, total, inner, sizes[axis]);
  return hipGetLastError();
}

hipError_t fill_u32_launch(void* p, uint32_t pattern, size_t n_words, hipStream_t s) {
  if (n_words == 0) return hipSuccess;
  hipLaunchKernelGGL(fill_kernel, dim3(grid_for((int64_t)n_words)), dim3(256), 0, s, (uint32_t*)p, pattern, n_words);
  return hipGetLastError();
}

}  // namespace pml
