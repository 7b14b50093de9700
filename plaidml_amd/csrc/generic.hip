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
    case PML_HIP_COMBO_EQ:  // a one-bit result; its aggregation wraps to one bit as well
      r.i = (dt_is_float(cmp_dt) ? (x[0].f == x[1].f) : (x[0].i == x[1].i)) ? 1 : 0;
      break;
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
      if ((d.combo == PML_HIP_COMBO_COND || d.combo == PML_HIP_COMBO_EQ) && q < 2) {
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

// Reductions along memory: one source, no combination, every access always in range, and the reduced
// indices together walk a contiguous run of the source.  A group of `lanes` threads (one wavefront, or
// the whole workgroup for long runs) owns one output point, reads its run with consecutive lanes on
// consecutive elements, and folds the partial results with cross-lane shuffles.  What a softmax's row
// max / row sum, a mean or a norm over the innermost axes turn into.
struct RowsArgs {
  int64_t out_stride[PML_HIP_MAX_IDX];  // of each output index, in elements of the output
  int64_t src_stride[PML_HIP_MAX_IDX];  // of each output index, in elements of the source
  int64_t range[PML_HIP_MAX_IDX];
  int64_t out_base, src_base;           // offsets of the box's lowest corner
  int64_t cols;                         // length of the contiguous run
  int32_t lanes;                        // 64 or 256
};

// DT / AGG fix the element type (source and result alike) and the aggregation at compile time, which
// folds every type switch away: a reduction launched once per network pass finds its code nowhere in
// the caches, and what it costs is then the length of the code it has to fetch.  DT = 0: both from the
// descriptor.
template <typename FT, typename IT, int DT, int AGG>
__global__ __launch_bounds__(256) void contract_rows_kernel(ContractArgs a, RowsArgs ra) {
  const pml_hip_contract_desc& d = a.d;
  __shared__ FT part_f[4];
  __shared__ IT part_i[4];
  const int per_block = 256 / ra.lanes;
  const int64_t row = (int64_t)blockIdx.x * per_block + (ra.lanes == 64 ? (int)(threadIdx.x >> 6) : 0);
  const bool live = row < d.out_elems;  // uniform over a wavefront
  const int lane = ra.lanes == 64 ? (int)(threadIdx.x & 63) : (int)threadIdx.x;
  int64_t out_off = ra.out_base, src_off = ra.src_base;
  {
    int64_t t = live ? row : 0;
    for (int v = d.n_out_idx - 1; v >= 0; --v) {
      const int64_t c = t % ra.range[v];
      t /= ra.range[v];
      out_off += c * ra.out_stride[v];
      src_off += c * ra.src_stride[v];
    }
  }
  const int dt = DT ? DT : d.dtype, sd = DT ? DT : d.src_dtype[0], agg = DT ? AGG : d.agg;
  const int acc_dt = (dt == PML_HIP_BF16 || dt == PML_HIP_F16) ? PML_HIP_F32 : dt;
  const bool widen = !dt_is_float(sd) && !dt_is_float(acc_dt) && sd != PML_HIP_BOOL && dt_size(sd) < dt_size(acc_dt);
  Scalar<FT, IT> acc;
  acc.f = dt_is_float(dt) ? (FT)d.identity_f : (FT)0;
  acc.i = dt_is_float(dt) ? (IT)0 : wrap_int_to<IT>(dt, (IT)d.identity_i);
  if (live) {
    constexpr int U = 8;  // loads in flight per lane: a row is short, so its latency is what costs
    for (int64_t j0 = lane; j0 < ra.cols; j0 += (int64_t)U * ra.lanes) {
      Scalar<FT, IT> raw[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t j = j0 + (int64_t)u * ra.lanes;
        if (j < ra.cols) raw[u] = load_scalar<FT, IT>(a.srcs[0], src_off + j, sd);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (j0 + (int64_t)u * ra.lanes >= ra.cols) break;
        Scalar<FT, IT> x = raw[u];
        if (widen)
          x.i = raw[u].i & (IT)((((uint64_t)1) << (dt_size(sd) * 8)) - 1);
        else
          x = convert_scalar<FT, IT>(raw[u], sd, acc_dt);
        aggregate<FT, IT>(agg, acc_dt, acc, x);
      }
    }
  }
  for (int w = 32; w > 0; w >>= 1) {
    Scalar<FT, IT> y;
    y.f = __shfl_xor(acc.f, w, 64);
    y.i = __shfl_xor(acc.i, w, 64);
    aggregate<FT, IT>(agg, acc_dt, acc, y);
  }
  if (ra.lanes == 256) {
    if ((threadIdx.x & 63) == 0) {
      part_f[threadIdx.x >> 6] = acc.f;
      part_i[threadIdx.x >> 6] = acc.i;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      for (int w = 1; w < 4; ++w) {
        Scalar<FT, IT> y;
        y.f = part_f[w], y.i = part_i[w];
        aggregate<FT, IT>(agg, acc_dt, acc, y);
      }
    }
  }
  if (live && lane == 0) {
    if (d.has_init) {
      Scalar<FT, IT> start = convert_scalar<FT, IT>(load_scalar<FT, IT>(a.out, out_off, dt), dt, acc_dt);
      aggregate<FT, IT>(agg, acc_dt, start, acc);
      acc = start;
    }
    store_scalar<FT, IT>(a.out, out_off, dt, convert_scalar<FT, IT>(acc, acc_dt, dt));
  }
}

// Fills `ra` if the contraction is a reduction along memory in the sense above.
bool rows_form(const pml_hip_contract_desc& d, RowsArgs* ra) {
  if (d.combo != PML_HIP_COMBO_NONE || d.n_src != 1 || d.agg == PML_HIP_AGG_ASSIGN) return false;
  if (d.n_idx <= d.n_out_idx || d.out_elems <= 0) return false;
  int64_t os[PML_HIP_MAX_IDX] = {}, ss[PML_HIP_MAX_IDX] = {};
  ra->out_base = ra->src_base = 0;
  for (int v = 0; v < d.n_idx; ++v)
    if (d.hi[v] < d.lo[v]) return false;
  for (int f = 0; f < d.n_forms; ++f) {
    const pml_hip_form& fm = d.forms[f];
    if (fm.den != 1 || (fm.operand != 0 && fm.operand != 1)) return false;
    int64_t lo = fm.c0, hi = fm.c0;
    for (int v = 0; v < d.n_idx; ++v) {
      lo += (int64_t)fm.coef[v] * (fm.coef[v] >= 0 ? d.lo[v] : d.hi[v]);
      hi += (int64_t)fm.coef[v] * (fm.coef[v] >= 0 ? d.hi[v] : d.lo[v]);
    }
    if (lo < 0 || hi >= fm.size) return false;
    int64_t corner = fm.c0;
    for (int v = 0; v < d.n_idx; ++v) {
      corner += (int64_t)fm.coef[v] * d.lo[v];
      (fm.operand == 0 ? os : ss)[v] += (int64_t)fm.coef[v] * fm.stride;
    }
    (fm.operand == 0 ? ra->out_base : ra->src_base) += corner * fm.stride;
  }
  int64_t run = 1;
  for (int v = d.n_idx - 1; v >= d.n_out_idx; --v) {
    if (os[v] != 0 || ss[v] != run) return false;
    run *= d.hi[v] - d.lo[v] + 1;
  }
  for (int v = 0; v < d.n_out_idx; ++v) {
    ra->out_stride[v] = os[v];
    ra->src_stride[v] = ss[v];
    ra->range[v] = d.hi[v] - d.lo[v] + 1;
  }
  ra->cols = run;
  return true;
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
// and the input's and the output's elements are ES and OES bytes wide: both 2, both 4, or a narrower output
// (the int32 -> int8 end of a requantisation chain).  Each thread reads 16 bytes of the input at a time and
// writes the 16 / ES results (16, 8 or 4 bytes).
typedef int i32x2_t __attribute__((ext_vector_type(2)));

template <int ES, int OES = ES>
__global__ __launch_bounds__(256) void eltwise_vec_kernel(EltwiseArgs a, int64_t inner, unsigned opnd_full_mask,
                                                          unsigned opnd_vec_mask) {
  static_assert(OES <= ES && (16 / ES) * OES >= 4, "a thread stores at least one 32-bit word");
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
      if constexpr (OES == ES) {
        *(i32x4_t*)((unsigned char*)a.out + e0 * ES) = res;
      } else if constexpr (V * OES == 8) {
        *(i32x2_t*)((unsigned char*)a.out + e0 * OES) = i32x2_t{res[0], res[1]};
      } else {
        *(int*)((unsigned char*)a.out + e0 * OES) = res[0];
      }
    }
  }
}

// The same layout, for the chains most networks are made of: every step a plain arithmetic function
// in the chain's own floating element type (DT: fp32 or bf16), no extra outputs.  The step's opcode is
// decoded once per 16-byte vector, not once per element, and the kernel carries none of the rarely used
// functions, so its code stays small enough to run from the instruction cache.
__host__ __device__ inline bool short_chain_op(int opcode) {
  switch (opcode) {
    case PML_HIP_EPI_ADD: case PML_HIP_EPI_SUB: case PML_HIP_EPI_RSUB: case PML_HIP_EPI_MUL: case PML_HIP_EPI_DIV:
    case PML_HIP_EPI_RDIV: case PML_HIP_EPI_MAX: case PML_HIP_EPI_MIN: case PML_HIP_EPI_RELU: case PML_HIP_EPI_NEG:
    case PML_HIP_EPI_EXP: case PML_HIP_EPI_LOG: case PML_HIP_EPI_SQRT: case PML_HIP_EPI_TANH: case PML_HIP_EPI_MAX_GT:
      return true;
    default:
      return false;
  }
}

template <int DT>
__global__ __launch_bounds__(256) void eltwise_short_kernel(EltwiseArgs a, int64_t inner, unsigned opnd_full_mask,
                                                            unsigned opnd_vec_mask, unsigned opnd_row_mask) {
  constexpr int ES = DT == PML_HIP_F32 ? 4 : 2;
  constexpr int V = 16 / ES;
  const pml_hip_eltwise_desc& d = a.d;
  const int64_t n_vec = a.total / V;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < n_vec; g += stride) {
    const int64_t e0 = g * V;
    const int64_t c0 = e0 % inner;
    i32x4_t raw = *(const i32x4_t*)((const unsigned char*)a.in + e0 * ES);
    float x[V], y[V];
#pragma unroll
    for (int e = 0; e < V; ++e) x[e] = load_scalar<float, int>(&raw, e, DT).f;
    for (int s = 0; s < d.tail.n_ops; ++s) {
      const pml_hip_epi_op& op = d.tail.ops[s];
      if (op.operand_kind == PML_HIP_OPND_TENSOR) {
        const int q = op.operand;
        const unsigned char* base = (const unsigned char*)a.operands[q];
        if (((opnd_full_mask | opnd_vec_mask) >> q) & 1) {
          const int64_t at = ((opnd_full_mask >> q) & 1) ? e0 : c0;
          i32x4_t w = *(const i32x4_t*)(base + at * ES);
#pragma unroll
          for (int e = 0; e < V; ++e) y[e] = load_scalar<float, int>(&w, e, DT).f;
        } else {
          // one value for the whole tensor, or one per innermost line (a vector never crosses a line)
          const float b = load_scalar<float, int>(base, ((opnd_row_mask >> q) & 1) ? e0 / inner : 0, DT).f;
#pragma unroll
          for (int e = 0; e < V; ++e) y[e] = b;
        }
      } else {
        const float b = op.operand_kind == PML_HIP_OPND_IMM ? round_float_to<float>(DT, (float)op.imm) : 0.0f;
#pragma unroll
        for (int e = 0; e < V; ++e) y[e] = b;
      }
#define PML_EACH(EXPR)                   \
  _Pragma("unroll") for (int e = 0; e < V; ++e) { \
    const float p = x[e], q = y[e];      \
    x[e] = round_float_to<float>(DT, EXPR); \
  }                                      \
  break;
      switch (op.opcode) {
        case PML_HIP_EPI_ADD: PML_EACH(p + q)
        case PML_HIP_EPI_SUB: PML_EACH(p - q)
        case PML_HIP_EPI_RSUB: PML_EACH(q - p)
        case PML_HIP_EPI_MUL: PML_EACH(p * q)
        case PML_HIP_EPI_DIV: PML_EACH(p / q)
        case PML_HIP_EPI_RDIV: PML_EACH(q / p)
        case PML_HIP_EPI_MAX: PML_EACH((p < q) ? q : p)
        case PML_HIP_EPI_MIN: PML_EACH((p < q) ? p : q)
        case PML_HIP_EPI_RELU: PML_EACH((p < 0.0f) ? 0.0f : p)
        case PML_HIP_EPI_NEG: PML_EACH(-p)
        case PML_HIP_EPI_EXP: PML_EACH(expf(p))
        case PML_HIP_EPI_LOG: PML_EACH(logf(p))
        case PML_HIP_EPI_SQRT: PML_EACH(sqrtf(p))
        case PML_HIP_EPI_TANH: PML_EACH(tanhf(p))
        case PML_HIP_EPI_MAX_GT: PML_EACH((p > q) ? p : q)
        default: break;
      }
#undef PML_EACH
    }
    i32x4_t res;
#pragma unroll
    for (int e = 0; e < V; ++e) {
      Scalar<float, int> v;
      v.f = x[e];
      v.i = 0;
      store_scalar<float, int>(&res, e, DT, v);
    }
    *(i32x4_t*)((unsigned char*)a.out + e0 * ES) = res;
  }
}

// The end of a quantised layer as a launch of its own: int32 sums -> cast to fp32 -> a chain of plain fp32
// arithmetic (scale per column, clamps, rounding) -> cast to an 8- or 16-bit integer.  Like the short-chain
// kernel the steps are decoded once per thread and pass, not per element; a thread turns V = 16 / OES int32
// values (V / 4 loads of 16 bytes) into one 16-byte store.  Each step is the interpreter's expression for
// that step on the same fp32 values (steps stay separate loop iterations, so none is contracted with its
// neighbour), which keeps the two bit-identical.
__host__ __device__ inline bool requant_chain_op(int opcode) {
  return short_chain_op(opcode) || opcode == PML_HIP_EPI_ROUND || opcode == PML_HIP_EPI_FLOOR || opcode == PML_HIP_EPI_CEIL;
}

template <int OES>
__global__ __launch_bounds__(256) void eltwise_requant_kernel(EltwiseArgs a, int64_t inner, unsigned opnd_full_mask,
                                                              unsigned opnd_vec_mask) {
  constexpr int V = 16 / OES, L = V / 4;
  const pml_hip_eltwise_desc& d = a.d;
  const int64_t n_vec = a.total / V;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const bool to_unsigned = dt_is_unsigned(d.out_dtype);
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < n_vec; g += stride) {
    const int64_t e0 = g * V;
    const int64_t c0 = e0 % inner;
    float x[V], y[V];
#pragma unroll
    for (int l = 0; l < L; ++l) {
      const i32x4_t raw = *(const i32x4_t*)((const unsigned char*)a.in + (e0 + 4 * l) * 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) x[4 * l + e] = (float)raw[e];  // the chain's leading cast
    }
    for (int s = 1; s + 1 < d.tail.n_ops; ++s) {
      const pml_hip_epi_op& op = d.tail.ops[s];
      if (op.operand_kind == PML_HIP_OPND_TENSOR) {
        const int q = op.operand;
        const unsigned char* base = (const unsigned char*)a.operands[q];
        if (((opnd_full_mask | opnd_vec_mask) >> q) & 1) {
          const int64_t at = ((opnd_full_mask >> q) & 1) ? e0 : c0;
#pragma unroll
          for (int l = 0; l < L; ++l) {
            const f32x4_t w = *(const f32x4_t*)(base + (at + 4 * l) * 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) y[4 * l + e] = w[e];
          }
        } else {
          const float b = *(const float*)base;
#pragma unroll
          for (int e = 0; e < V; ++e) y[e] = b;
        }
      } else {
        const float b = op.operand_kind == PML_HIP_OPND_IMM ? (float)op.imm : 0.0f;
#pragma unroll
        for (int e = 0; e < V; ++e) y[e] = b;
      }
#define PML_EACH(EXPR)                            \
  _Pragma("unroll") for (int e = 0; e < V; ++e) { \
    const float p = x[e], q = y[e];               \
    x[e] = EXPR;                                  \
  }                                               \
  break;
      switch (op.opcode) {
        case PML_HIP_EPI_ADD: PML_EACH(p + q)
        case PML_HIP_EPI_SUB: PML_EACH(p - q)
        case PML_HIP_EPI_RSUB: PML_EACH(q - p)
        case PML_HIP_EPI_MUL: PML_EACH(p * q)
        case PML_HIP_EPI_DIV: PML_EACH(p / q)
        case PML_HIP_EPI_RDIV: PML_EACH(q / p)
        case PML_HIP_EPI_MAX: PML_EACH((p < q) ? q : p)
        case PML_HIP_EPI_MIN: PML_EACH((p < q) ? p : q)
        case PML_HIP_EPI_RELU: PML_EACH((p < 0.0f) ? 0.0f : p)
        case PML_HIP_EPI_NEG: PML_EACH(-p)
        case PML_HIP_EPI_EXP: PML_EACH(expf(p))
        case PML_HIP_EPI_LOG: PML_EACH(logf(p))
        case PML_HIP_EPI_SQRT: PML_EACH(sqrtf(p))
        case PML_HIP_EPI_TANH: PML_EACH(tanhf(p))
        case PML_HIP_EPI_MAX_GT: PML_EACH((p > q) ? p : q)
        case PML_HIP_EPI_ROUND: PML_EACH(c_round<float>(p))
        case PML_HIP_EPI_FLOOR: PML_EACH(floorf(p))
        case PML_HIP_EPI_CEIL: PML_EACH(ceilf(p))
        default: break;
      }
#undef PML_EACH
    }
    // the closing cast: toward zero into 32 bits (by the target's signedness), then the low OES bytes
    i32x4_t res = {0, 0, 0, 0};
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const unsigned v = to_unsigned ? (unsigned)x[e] : (unsigned)(int)x[e];
      if constexpr (OES == 1)
        res[e / 4] |= (int)((v & 0xffu) << (8 * (e % 4)));
      else
        res[e / 2] |= (int)((v & 0xffffu) << (16 * (e % 2)));
    }
    *(i32x4_t*)((unsigned char*)a.out + e0 * OES) = res;
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
  RowsArgs ra;
  if (!wide && red_count >= 64 && rows_form(d, &ra)) {
    // a wavefront per output point; the whole workgroup when the points alone would not fill the chip
    ra.lanes = (ra.cols >= 2048 && d.out_elems * 64 < (int64_t)256 * 1024) ? 256 : 64;
    const int per_block = 256 / ra.lanes;
    const int64_t nb = (d.out_elems + per_block - 1) / per_block;
    if (nb <= 0x7fffffff) {
      const dim3 grid((unsigned)nb), block(256);
      const bool same = d.src_dtype[0] == d.dtype;
#define PML_ROWS(DT, AGG)                                                                                   \
  if (same && d.dtype == DT && d.agg == AGG) {                                                              \
    hipLaunchKernelGGL((contract_rows_kernel<float, int, DT, AGG>), grid, block, 0, s, a, ra);              \
    return hipGetLastError();                                                                               \
  }
      PML_ROWS(PML_HIP_BF16, PML_HIP_AGG_ADD)
      PML_ROWS(PML_HIP_BF16, PML_HIP_AGG_MAX)
      PML_ROWS(PML_HIP_BF16, PML_HIP_AGG_MIN)
      PML_ROWS(PML_HIP_F32, PML_HIP_AGG_ADD)
      PML_ROWS(PML_HIP_F32, PML_HIP_AGG_MAX)
      PML_ROWS(PML_HIP_F32, PML_HIP_AGG_MIN)
#undef PML_ROWS
      hipLaunchKernelGGL((contract_rows_kernel<float, int, 0, 0>), grid, block, 0, s, a, ra);
      return hipGetLastError();
    }
  }
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
  // int32 -> fp32 chain -> narrow integer
  if (d.in_dtype == PML_HIP_I32 && d.tail.n_ops >= 2 && d.rank >= 1 && d.tail.ops[0].opcode == PML_HIP_EPI_CAST &&
      d.tail.ops[0].dtype == PML_HIP_F32 && d.tail.ops[d.tail.n_ops - 1].opcode == PML_HIP_EPI_CAST &&
      d.tail.ops[d.tail.n_ops - 1].dtype == d.out_dtype && !dt_is_float(d.out_dtype) && d.out_dtype != PML_HIP_BOOL &&
      (dt_size(d.out_dtype) == 1 || dt_size(d.out_dtype) == 2)) {
    const int V = 16 / dt_size(d.out_dtype);
    const int64_t inner = d.sizes[d.rank - 1];
    bool ok = a.total % V == 0 && inner % V == 0 && ((((uintptr_t)a.in | (uintptr_t)a.out) & 15) == 0);
    int64_t st = 1;
    for (int r = d.rank - 1; r >= 0; --r) {
      if (d.sizes[r] != 1 && d.in_strides[r] != st) ok = false;
      st *= d.sizes[r];
    }
    unsigned full_mask = 0, vec_mask = 0;
    for (int q = 0; q < d.tail.n_operands && ok; ++q) {
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
      if (d.tail.operand_dtype[q] != PML_HIP_F32 || !(full || vec || scal)) ok = false;
      if (full)
        full_mask |= 1u << q;
      else if (vec)
        vec_mask |= 1u << q;
      if ((full || vec) && ((uintptr_t)a.operands[q] & 15)) ok = false;
    }
    for (int k = 1; k + 1 < d.tail.n_ops && ok; ++k)
      ok = requant_chain_op(d.tail.ops[k].opcode) && d.tail.ops[k].dtype == PML_HIP_F32;
    if (ok) {
      const unsigned g = grid_for(a.total / V);
      if (dt_size(d.out_dtype) == 1)
        hipLaunchKernelGGL((eltwise_requant_kernel<1>), dim3(g), dim3(256), 0, s, a, inner, full_mask, vec_mask);
      else
        hipLaunchKernelGGL((eltwise_requant_kernel<2>), dim3(g), dim3(256), 0, s, a, inner, full_mask, vec_mask);
      return hipGetLastError();
    }
  }
  // try the 16-byte path
  const int es = dt_size(d.in_dtype);
  const int oes = dt_size(d.out_dtype);
  bool vec_ok = (es == 2 || es == 4) && (oes == es || (es == 4 && (oes == 1 || oes == 2))) && d.rank >= 1;
  int64_t inner = d.rank >= 1 ? d.sizes[d.rank - 1] : 1;
  unsigned full_mask = 0, vec_mask = 0, row_mask = 0;
  if (vec_ok) {
    int64_t st = 1;
    for (int r = d.rank - 1; r >= 0; --r) {
      if (d.sizes[r] != 1 && d.in_strides[r] != st) vec_ok = false;
      st *= d.sizes[r];
    }
    for (int q = 0; q < d.tail.n_operands && vec_ok; ++q) {
      bool full = true, vec = true, scal = true, row = true;
      int64_t st2 = 1;
      for (int r = d.rank - 1; r >= 0; --r) {
        const int64_t os = d.operand_strides[q][r];
        if (d.sizes[r] != 1) {
          if (os != st2) full = false;
          if (os != ((r == d.rank - 1) ? 1 : 0)) vec = false;
          if (os != 0) scal = false;
          if (os != ((r == d.rank - 1) ? 0 : st2 / inner)) row = false;
        }
        st2 *= d.sizes[r];
      }
      if (full)
        full_mask |= 1u << q;
      else if (vec)
        vec_mask |= 1u << q;
      else if (scal)
        ;
      else if (row)
        row_mask |= 1u << q;  // one value per innermost line: only the short-chain kernel takes these
      else
        vec_ok = false;
    }
    for (int k = 0; k < d.tail.n_ops; ++k) {
      const pml_hip_epi_op& op = d.tail.ops[k];
      if (op.opcode == PML_HIP_EPI_STORE) vec_ok = false;
      if (op.opcode == PML_HIP_EPI_CAST && dt_size(op.dtype) != oes && k == d.tail.n_ops - 1) vec_ok = false;
    }
    const int V = 16 / es;
    if (a.total % V != 0 || inner % V != 0) vec_ok = false;
    if (((uintptr_t)a.in | (uintptr_t)a.out) & 15) vec_ok = false;
  }
  if (vec_ok) {
    const int V = 16 / es;
    const unsigned g = grid_for(a.total / V);
    bool short_chain = (d.in_dtype == PML_HIP_F32 || d.in_dtype == PML_HIP_BF16) && d.out_dtype == d.in_dtype;
    for (int k = 0; k < d.tail.n_ops && short_chain; ++k) {
      const pml_hip_epi_op& op = d.tail.ops[k];
      short_chain = short_chain_op(op.opcode) && op.dtype == d.in_dtype &&
                    (op.operand_kind != PML_HIP_OPND_TENSOR || d.tail.operand_dtype[op.operand] == d.in_dtype);
    }
    for (int q = 0; q < d.tail.n_operands; ++q)  // it reads whole-tensor and per-column operands 16 bytes at a time
      if ((((full_mask | vec_mask) >> q) & 1) && ((uintptr_t)a.operands[q] & 15)) short_chain = false;
    if (short_chain) {
      if (d.in_dtype == PML_HIP_F32)
        hipLaunchKernelGGL((eltwise_short_kernel<PML_HIP_F32>), dim3(g), dim3(256), 0, s, a, inner, full_mask, vec_mask,
                           row_mask);
      else
        hipLaunchKernelGGL((eltwise_short_kernel<PML_HIP_BF16>), dim3(g), dim3(256), 0, s, a, inner, full_mask, vec_mask,
                           row_mask);
      return hipGetLastError();
    }
    if (row_mask == 0) {
      if (es == 2)
        hipLaunchKernelGGL((eltwise_vec_kernel<2>), dim3(g), dim3(256), 0, s, a, inner, full_mask, vec_mask);
      else if (oes == 2)
        hipLaunchKernelGGL((eltwise_vec_kernel<4, 2>), dim3(g), dim3(256), 0, s, a, inner, full_mask, vec_mask);
      else if (oes == 1)
        hipLaunchKernelGGL((eltwise_vec_kernel<4, 1>), dim3(g), dim3(256), 0, s, a, inner, full_mask, vec_mask);
      else
        hipLaunchKernelGGL((eltwise_vec_kernel<4>), dim3(g), dim3(256), 0, s, a, inner, full_mask, vec_mask);
      return hipGetLastError();
    }
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

// Softmax over the last axis: a workgroup per row, three walks over the row (maximum, sum of exponentials, quotients;
// rows are short and stay in the caches), each reduction folded through the wavefronts' lanes and then through LDS in
// a fixed order.  BF: every intermediate is rounded to bf16 where the separate operations would have stored it.
template <bool BF>
__global__ __launch_bounds__(256) void softmax_rows_kernel(const void* x_, void* y_, int64_t cols) {
  __shared__ float part[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t row = blockIdx.x;
  auto load = [&](int64_t c) {
    if constexpr (BF) return bf16_bits_to_f32(((const uint16_t*)x_)[row * cols + c]);
    return ((const float*)x_)[row * cols + c];
  };
  auto rounded = [](float v) { return BF ? round_to_bf16(v) : v; };
  auto across = [&](float v, auto fold) {
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) v = fold(v, __shfl_xor(v, d, 64));
    __syncthreads();  // (the previous reduction's readers are done with `part`)
    if (lane == 0) part[wave] = v;
    __syncthreads();
    return fold(fold(part[0], part[1]), fold(part[2], part[3]));
  };
  float m = -INFINITY;
  for (int64_t c = tid; c < cols; c += 256) {
    const float v = load(c);
    m = v > m ? v : m;
  }
  m = across(m, [](float a, float b) { return b > a ? b : a; });
  float sum = 0.f;
  for (int64_t c = tid; c < cols; c += 256) sum += rounded(expf(rounded(load(c) - m)));
  sum = rounded(across(sum, [](float a, float b) { return a + b; }));
  for (int64_t c = tid; c < cols; c += 256) {
    const float q = rounded(rounded(expf(rounded(load(c) - m))) / sum);
    if constexpr (BF)
      ((uint16_t*)y_)[row * cols + c] = f32_to_bf16_bits(q);
    else
      ((float*)y_)[row * cols + c] = q;
  }
}

hipError_t softmax_launch(const pml_hip_softmax_desc& d, const void* x, void* y, hipStream_t s) {
  if (d.rows == 0 || d.cols == 0) return hipSuccess;
  if (d.rows > 0x7fffffff) return hipErrorInvalidValue;
  if (d.dtype == PML_HIP_BF16)
    hipLaunchKernelGGL(softmax_rows_kernel<true>, dim3((unsigned)d.rows), dim3(256), 0, s, x, y, d.cols);
  else
    hipLaunchKernelGGL(softmax_rows_kernel<false>, dim3((unsigned)d.rows), dim3(256), 0, s, x, y, d.cols);
  return hipGetLastError();
}

hipError_t fill_u32_launch(void* p, uint32_t pattern, size_t n_words, hipStream_t s) {
  if (n_words == 0) return hipSuccess;
  hipLaunchKernelGGL(fill_kernel, dim3(grid_for((int64_t)n_words)), dim3(256), 0, s, (uint32_t*)p, pattern, n_words);
  return hipGetLastError();
}

}  // namespace pml
