// gather, scatter and argsort: the Tile operations that are neither contractions nor elementwise maps.
// Scalar semantics follow pmlc/conversion/linalg_to_pxa/tile_to_pxa_special_patterns.cc (ArgSortOpConversion
// :29-298, GatherOpConversion :300-760, ScatterOpConversion :762-896).  All three are index-driven,
// bandwidth / latency bound passes: one thread per result element (gather), per update element (scatter), one
// workgroup per sorted line (argsort).
#include <hip/hip_runtime.h>

#include <mutex>
#include <type_traits>

#include "device_common.h"
#include "plans.h"

namespace pml {
namespace {

constexpr int R = PML_HIP_MAX_SPECIAL_RANK;

inline unsigned blocks_for(int64_t items) {
  int64_t b = (items + 255) / 256;
  if (b < 1) b = 1;
  return (unsigned)(b < 256 * 32 ? b : 256 * 32);
}

__device__ inline void zero_elem(void* dst, int64_t d, int es) {
  switch (es) {
    case 1: ((uint8_t*)dst)[d] = 0; break;
    case 2: ((uint16_t*)dst)[d] = 0; break;
    case 4: ((uint32_t*)dst)[d] = 0; break;
    default: ((uint64_t*)dst)[d] = 0; break;
  }
}

// raw copy of one element of `es` bytes
__device__ inline void copy_elem(void* dst, int64_t d, const void* src, int64_t s, int es) {
  switch (es) {
    case 1: ((uint8_t*)dst)[d] = ((const uint8_t*)src)[s]; break;
    case 2: ((uint16_t*)dst)[d] = ((const uint16_t*)src)[s]; break;
    case 4: ((uint32_t*)dst)[d] = ((const uint32_t*)src)[s]; break;
    default: ((uint64_t*)dst)[d] = ((const uint64_t*)src)[s]; break;
  }
}

__device__ inline int64_t load_index(const void* p, int64_t off, int dt) {
  switch (dt) {
    case PML_HIP_I8: return ((const int8_t*)p)[off];
    case PML_HIP_U8:
    case PML_HIP_BOOL: return ((const uint8_t*)p)[off];
    case PML_HIP_I16: return ((const int16_t*)p)[off];
    case PML_HIP_U16: return ((const uint16_t*)p)[off];
    case PML_HIP_I32: return ((const int32_t*)p)[off];
    case PML_HIP_U32: return ((const uint32_t*)p)[off];
    default: return ((const int64_t*)p)[off];
  }
}

struct GatherGeom {
  int out_rank;
  int64_t out_sizes[R];
  int64_t strides[R];  // tensor
  int64_t idx_strides[R];
  int64_t total;
};

__device__ inline int clamp_tap(int v, int upper) {
  v = v < 0 ? 0 : v;
  return v < upper ? v : upper;
}

// One interpolated read along the axis for a floating tensor and a floating position, computed in FT
// (float for f16 / bf16 / f32 tensors, double for f64) and rounded to the element type after every
// arithmetic step, as the reference's per-operation element type does.
template <typename FT>
__device__ inline FT interpolate(const pml_hip_gather_desc& d, const void* tensor, int64_t base, int64_t axis_stride, FT pos) {
  const int upper = (int)d.sizes[d.axis] - 1;
  auto tap = [&](int i) {
    Scalar<FT, int64_t> v = load_scalar<FT, int64_t>(tensor, base + (int64_t)clamp_tap(i, upper) * axis_stride, d.dtype);
    return v.f;
  };
  auto rnd = [&](FT x) { return round_float_to<FT>(d.dtype, x); };
  const FT fl = floor(pos), ce = ceil(pos);
  FT result;
  if (d.interpolation == PML_HIP_INTERP_NEAREST) {
    int i;
    const bool halfway = pos == rnd(fl + (FT)0.5);
    switch (d.nearest) {
      case PML_HIP_NEAREST_ROUND_PREFER_FLOOR: i = halfway ? (int)fl : (int)floor(rnd(pos + (FT)0.5)); break;
      case PML_HIP_NEAREST_ROUND_PREFER_CEIL: i = halfway ? (int)ce : (int)floor(rnd(pos + (FT)0.5)); break;
      case PML_HIP_NEAREST_FLOOR: i = (int)fl; break;
      case PML_HIP_NEAREST_CEIL: i = (int)ce; break;
      default: i = (int)pos; break;  // SIMPLE: truncation
    }
    result = tap(i);
  } else if (d.interpolation == PML_HIP_INTERP_LINEAR) {
    const FT g0 = tap((int)ce), g1 = tap((int)fl);
    const FT c0 = rnd(pos - fl), c1 = rnd((FT)1 - c0);
    result = rnd(rnd(c0 * g0) + rnd(c1 * g1));
  } else {
    // cubic convolution with coefficient a over the taps floor-1, floor, ceil, ceil+1
    const FT a = rnd((FT)d.cube_coeff);
    const FT g[4] = {tap((int)fl - 1), tap((int)fl), tap((int)ce), tap((int)ce + 1)};
    const FT s1 = rnd(pos - fl), s2 = rnd(s1 * s1), s3 = rnd(s2 * s1);
    const FT s_a = rnd(a * s1), s2_a = rnd(a * s2), s3_a = rnd(a * s3);
    const FT s3_a2 = rnd(rnd(a + (FT)2) * s3), s2_a3 = rnd(rnd(a + (FT)3) * s2);
    const FT s2_2a3 = rnd(rnd(rnd(a + a) + (FT)3) * s2);
    FT p[4];
    p[0] = rnd(rnd(s3_a - rnd(s2_a * (FT)2)) + s_a);
    p[1] = rnd(rnd(s3_a2 - s2_a3) + (FT)1);
    p[2] = rnd(rnd(s2_2a3 - s3_a2) - s_a);
    p[3] = rnd(s2_a - s3_a);
    for (int i = 0; i < 4; ++i) p[i] = rnd(p[i] * g[i]);
    result = rnd(rnd(rnd(p[0] + p[1]) + p[2]) + p[3]);
  }
  if (d.oob == PML_HIP_OOB_RETURN_ZERO && (pos > (FT)upper || pos < (FT)0)) result = (FT)0;
  return result;
}

template <typename FT>
__global__ __launch_bounds__(256) void gather_kernel(pml_hip_gather_desc d, GatherGeom g, const void* tensor, const void* indices,
                                                     void* out) {
  const int es = dt_size(d.dtype);
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; gid < g.total; gid += step) {
    int64_t c[R];
    int64_t r = gid;
    for (int k = g.out_rank - 1; k >= 0; --k) {
      c[k] = r % g.out_sizes[k];
      r /= g.out_sizes[k];
    }
    if (d.mode == PML_HIP_GATHER_ND) {
      const int lead = d.idx_rank - 1;
      const int depth = (int)d.idx_sizes[lead];
      int64_t ioff = 0;
      for (int k = 0; k < lead; ++k) ioff += c[k] * g.idx_strides[k];
      int64_t src = 0;
      bool inside = true;
      for (int k = 0; k < d.batch_dims; ++k) src += c[k] * g.strides[k];
      for (int k = 0; k < depth; ++k) {
        const int64_t at = load_index(indices, ioff + k, d.idx_dtype);
        inside = inside && at >= 0 && at < d.sizes[d.batch_dims + k];
        src += at * g.strides[d.batch_dims + k];
      }
      for (int k = lead; k < g.out_rank; ++k) src += c[k] * g.strides[d.batch_dims + depth + (k - lead)];
      // an index outside the tensor is undefined in the reference; it reads as zero here
      if (inside)
        copy_elem(out, gid, tensor, src, es);
      else
        zero_elem(out, gid, es);
      continue;
    }
    // NORMAL: result coordinates are (tensor dims before the axis, the indices' dims, tensor dims after it)
    int64_t ioff = 0, base = 0;
    for (int k = 0; k < d.axis; ++k) base += c[k] * g.strides[k];
    for (int k = 0; k < d.idx_rank; ++k) ioff += c[d.axis + k] * g.idx_strides[k];
    for (int k = d.axis + 1; k < d.rank; ++k) base += c[d.axis + d.idx_rank + (k - d.axis - 1)] * g.strides[k];
    const int64_t axis_stride = g.strides[d.axis];
    auto plain_read = [&](int64_t at) {
      if (at >= 0 && at < d.sizes[d.axis])
        copy_elem(out, gid, tensor, base + at * axis_stride, es);
      else
        zero_elem(out, gid, es);
    };
    if (!dt_is_float(d.idx_dtype)) {
      plain_read(load_index(indices, ioff, d.idx_dtype));
    } else {
      Scalar<FT, int64_t> pos = load_scalar<FT, int64_t>(indices, ioff, d.idx_dtype);
      if (!dt_is_float(d.dtype)) {
        plain_read((int64_t)(int)pos.f);  // fptosi, then a plain read
      } else {
        Scalar<FT, int64_t> v;
        v.i = 0;
        v.f = interpolate<FT>(d, tensor, base, axis_stride, pos.f);
        store_scalar<FT, int64_t>(out, gid, d.dtype, v);
      }
    }
  }
}

struct ScatterGeom {
  int64_t strides[R];      // result
  int64_t idx_strides[R];
  int64_t total;           // update elements
};

__global__ __launch_bounds__(256) void scatter_kernel(pml_hip_scatter_desc d, ScatterGeom g, const void* indices, const void* updates,
                                                      void* out) {
  const int es = dt_size(d.dtype);
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; gid < g.total; gid += step) {
    int64_t c[R];
    int64_t r = gid;
    for (int k = d.upd_rank - 1; k >= 0; --k) {
      c[k] = r % d.upd_sizes[k];
      r /= d.upd_sizes[k];
    }
    int64_t dst = 0;
    bool inside = true;
    if (d.mode == PML_HIP_SCATTER_UPDATE_ND) {
      const int lead = d.idx_rank - 1;
      const int depth = (int)d.idx_sizes[lead];
      int64_t ioff = 0;
      for (int k = 0; k < lead; ++k) ioff += c[k] * g.idx_strides[k];
      for (int k = 0; k < depth; ++k) {
        const int64_t at = load_index(indices, ioff + k, d.idx_dtype);
        inside = inside && at >= 0 && at < d.sizes[k];
        dst += at * g.strides[k];
      }
      for (int k = lead; k < d.upd_rank; ++k) {
        inside = inside && c[k] < d.sizes[depth + (k - lead)];
        dst += c[k] * g.strides[depth + (k - lead)];
      }
    } else if (d.mode == PML_HIP_SCATTER_UPDATE_SLICE) {
      // update dims: (result dims before the axis, the indices' dims, result dims after the axis)
      int64_t ioff = 0;
      for (int k = 0; k < d.idx_rank; ++k) ioff += c[d.axis + k] * g.idx_strides[k];
      for (int k = 0; k < d.axis; ++k) {
        inside = inside && c[k] < d.sizes[k];
        dst += c[k] * g.strides[k];
      }
      const int64_t at = load_index(indices, ioff, d.idx_dtype);
      inside = inside && at >= 0 && at < d.sizes[d.axis];
      dst += at * g.strides[d.axis];
      for (int k = d.axis + d.idx_rank; k < d.upd_rank; ++k) {
        const int r = d.axis + 1 + (k - d.axis - d.idx_rank);
        inside = inside && c[k] < d.sizes[r];
        dst += c[k] * g.strides[r];
      }
    } else {
      // NORMAL / UPDATE_ELT: the index is read at the update's leading coordinates and replaces coordinate `axis`
      int64_t ioff = 0;
      for (int k = 0; k < d.idx_rank; ++k) ioff += c[k] * g.idx_strides[k];
      const int64_t at = load_index(indices, ioff, d.idx_dtype);
      inside = at >= 0 && at < d.sizes[d.axis];
      for (int k = 0; k < d.upd_rank; ++k) {
        // the other coordinates come from the update's own shape, which may exceed the result's
        inside = inside && (k == d.axis || c[k] < d.sizes[k]);
        dst += (k == d.axis ? at : c[k]) * g.strides[k];
      }
    }
    if (!inside) continue;  // undefined in the reference; the update is dropped here
    if (d.mode != PML_HIP_SCATTER_NORMAL) {
      copy_elem(out, dst, updates, gid, es);
      continue;
    }
    switch (d.dtype) {
      case PML_HIP_F32: atomicAdd((float*)out + dst, ((const float*)updates)[gid]); break;
      case PML_HIP_F64: atomicAdd((double*)out + dst, ((const double*)updates)[gid]); break;
      case PML_HIP_I32:
      case PML_HIP_U32: atomicAdd((unsigned*)out + dst, ((const unsigned*)updates)[gid]); break;
      case PML_HIP_I64:
      case PML_HIP_U64: atomicAdd((unsigned long long*)out + dst, ((const unsigned long long*)updates)[gid]); break;
      case PML_HIP_F16:
      case PML_HIP_BF16: {
        // 16-bit floats: compare-and-swap on the containing word, the sum rounded to the element type
        uint32_t* word = (uint32_t*)((char*)out + ((dst * 2) & ~(int64_t)3));
        const int shift = ((dst * 2) & 2) ? 16 : 0;
        const uint16_t ub = ((const uint16_t*)updates)[gid];
        const float u = d.dtype == PML_HIP_BF16 ? bf16_bits_to_f32(ub) : f16_bits_to_f32(ub);
        uint32_t old = *word, assumed;
        do {
          assumed = old;
          const uint16_t cur = (uint16_t)(assumed >> shift);
          const float sum = (d.dtype == PML_HIP_BF16 ? bf16_bits_to_f32(cur) : f16_bits_to_f32(cur)) + u;
          const uint16_t nb = d.dtype == PML_HIP_BF16 ? f32_to_bf16_bits(sum) : f32_to_f16_bits(sum);
          old = atomicCAS(word, assumed, (assumed & ~(0xffffu << shift)) | ((uint32_t)nb << shift));
        } while (old != assumed);
        break;
      }
      default: {
        // 8- and 16-bit integers: compare-and-swap on the containing word
        const int64_t byte = dst * es;
        uint32_t* word = (uint32_t*)((char*)out + (byte & ~(int64_t)3));
        const int shift = (int)(byte & 3) * 8;
        const uint32_t mask = (es == 1 ? 0xffu : 0xffffu) << shift;
        const uint32_t u = es == 1 ? ((const uint8_t*)updates)[gid] : ((const uint16_t*)updates)[gid];
        uint32_t old = *word, assumed;
        do {
          assumed = old;
          const uint32_t sum = (((assumed & mask) >> shift) + u) << shift;
          old = atomicCAS(word, assumed, (assumed & ~mask) | (sum & mask));
        } while (old != assumed);
        break;
      }
    }
  }
}

// Keys are compared as the element type compares: signed / unsigned integers widened to 64 bits, floats by value.
template <typename T>
__device__ inline bool before(T a, T b, int direction) {
  if constexpr (std::is_floating_point<T>::value) {
    // NaNs sort behind every number in both directions (the reference leaves their place to its selection
    // sort's visiting order); this keeps the result a permutation
    if (a != a) return false;
    if (b != b) return true;
  }
  return direction == 0 ? a < b : a > b;
}

template <typename T, typename LOAD>
__device__ inline void rank_line(LOAD load, int n, int direction, int32_t* out, int64_t out_base, int64_t out_stride, T* keys) {
  // position of element i in the sorted line = #{j : key_j strictly before key_i} + #{j < i : neither is before
  // the other}: exactly what a stable sort with this comparison yields
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const T ki = keys ? keys[i] : load(i);
    int pos = 0;
    for (int j = 0; j < n; ++j) {
      const T kj = keys ? keys[j] : load(j);
      pos += before<T>(kj, ki, direction) || (j < i && !before<T>(ki, kj, direction));
    }
    out[out_base + (int64_t)pos * out_stride] = i;
  }
}

constexpr int kArgsortLdsKeys = 8192;

template <typename T>
__global__ __launch_bounds__(256) void argsort_kernel(pml_hip_argsort_desc d, const void* tensor, int32_t* out, int64_t inner,
                                                      int64_t lines) {
  __shared__ T keys[kArgsortLdsKeys];
  const int n = (int)d.sizes[d.axis];
  for (int64_t line = blockIdx.x; line < lines; line += gridDim.x) {
    const int64_t base = (line / inner) * n * inner + line % inner;
    auto load = [&](int i) -> T {
      const int64_t off = base + (int64_t)i * inner;
      if constexpr (std::is_same<T, float>::value) {
        return load_scalar<float, int>(tensor, off, d.dtype).f;
      } else if constexpr (std::is_same<T, double>::value) {
        return ((const double*)tensor)[off];
      } else if constexpr (std::is_same<T, uint64_t>::value) {
        return (uint64_t)load_index(tensor, off, d.dtype);
      } else {
        return (int64_t)load_index(tensor, off, d.dtype);
      }
    };
    const bool staged = n <= kArgsortLdsKeys;
    if (staged) {
      __syncthreads();  // the previous line's readers are done
      for (int i = threadIdx.x; i < n; i += blockDim.x) keys[i] = load(i);
      __syncthreads();
    }
    rank_line<T>(load, n, d.direction, out, base, inner, staged ? keys : nullptr);
  }
}

// ---- prng -----------------------------------------------------------------------------------------------
// One step of the three recurrences (pmlc/rt/prng.cc:31-37).  Each is linear over GF(2): masks, shifts, XORs.
__host__ __device__ inline uint32_t taus_step(int c, uint32_t s) {
  switch (c) {
    case 0: return ((s & 4294967294u) << 12) ^ (((s << 13) ^ s) >> 19);
    case 1: return ((s & 4294967288u) << 4) ^ (((s << 2) ^ s) >> 25);
    default: return ((s & 4294967280u) << 17) ^ (((s << 3) ^ s) >> 11);
  }
}

// jump[c][j] is the matrix of 2^j steps of component c, stored by columns: column b = image of bit b
struct JumpTable {
  uint32_t col[3][40][32];
};
__device__ JumpTable g_jump;

__device__ inline uint32_t apply_jump(const uint32_t* cols, uint32_t x) {
  uint32_t r = 0;
  for (int b = 0; b < 32; ++b)
    if ((x >> b) & 1u) r ^= cols[b];
  return r;
}

// the state after `n` steps from `s`
__device__ inline uint32_t jump_ahead(int c, uint32_t s, uint64_t n) {
  for (int j = 0; j < 40 && n; ++j, n >>= 1)
    if (n & 1) s = apply_jump(g_jump.col[c][j], s);
  return s;
}

constexpr int kPrngRun = 64;  // consecutive values per thread

__global__ __launch_bounds__(256) void prng_kernel(const uint32_t* state, int64_t count, float* values, uint32_t* new_state) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t first = t * kPrngRun;
  if (values && first < count) {
    uint32_t s0 = jump_ahead(0, state[0], (uint64_t)first), s1 = jump_ahead(1, state[1], (uint64_t)first),
             s2 = jump_ahead(2, state[2], (uint64_t)first);
    const int64_t last = first + kPrngRun < count ? first + kPrngRun : count;
    for (int64_t i = first; i < last; ++i) {
      values[i] = (float)((double)(s0 ^ s1 ^ s2) / 4294967296.0);
      s0 = taus_step(0, s0);
      s1 = taus_step(1, s1);
      s2 = taus_step(2, s2);
    }
  }
  if (new_state && t == 0) {
    const uint32_t in0 = state[0], in1 = state[1], in2 = state[2];  // read before writing: the two may alias
    new_state[0] = jump_ahead(0, in0, (uint64_t)count);
    new_state[1] = jump_ahead(1, in1, (uint64_t)count);
    new_state[2] = jump_ahead(2, in2, (uint64_t)count);
  }
}

}  // namespace

hipError_t prng_launch(const void* state, int64_t count, void* values, void* new_state, hipStream_t s) {
  if (count >= (int64_t{1} << 40)) return hipErrorInvalidValue;
  // the table depends on nothing but the recurrences: built on the host once and uploaded to each device on first use
  static JumpTable table;
  static bool built = false;
  static bool uploaded[64] = {false};
  static std::mutex mu;
  {
    std::lock_guard<std::mutex> lock(mu);
    if (!built) {
      for (int c = 0; c < 3; ++c) {
        for (int b = 0; b < 32; ++b) table.col[c][0][b] = taus_step(c, 1u << b);
        for (int j = 1; j < 40; ++j)
          for (int b = 0; b < 32; ++b) {
            // (M^2) e_b = M (M e_b)
            uint32_t x = table.col[c][j - 1][b], r = 0;
            for (int k = 0; k < 32; ++k)
              if ((x >> k) & 1u) r ^= table.col[c][j - 1][k];
            table.col[c][j][b] = r;
          }
      }
      built = true;
    }
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
    if (!uploaded[dev]) {
      e = hipMemcpyToSymbol(HIP_SYMBOL(g_jump), &table, sizeof(table));
      if (e != hipSuccess) return e;
      uploaded[dev] = true;
    }
  }
  const int64_t threads = values ? (count + kPrngRun - 1) / kPrngRun : 1;
  const int64_t blocks = threads > 0 ? (threads + 255) / 256 : 1;
  hipLaunchKernelGGL(prng_kernel, dim3((unsigned)(blocks > 0 ? blocks : 1)), dim3(256), 0, s, (const uint32_t*)state, count,
                     (float*)values, (uint32_t*)new_state);
  return hipGetLastError();
}

hipError_t gather_launch(const pml_hip_gather_desc& d, const void* tensor, const void* indices, void* out, hipStream_t s) {
  GatherGeom g{};
  int64_t st = 1;
  for (int k = d.rank - 1; k >= 0; --k) {
    g.strides[k] = st;
    st *= d.sizes[k];
  }
  st = 1;
  for (int k = d.idx_rank - 1; k >= 0; --k) {
    g.idx_strides[k] = st;
    st *= d.idx_sizes[k];
  }
  int n = 0;
  if (d.mode == PML_HIP_GATHER_ND) {
    const int depth = (int)d.idx_sizes[d.idx_rank - 1];
    for (int k = 0; k + 1 < d.idx_rank; ++k) g.out_sizes[n++] = d.idx_sizes[k];
    for (int k = d.batch_dims + depth; k < d.rank; ++k) g.out_sizes[n++] = d.sizes[k];
  } else {
    for (int k = 0; k < d.axis; ++k) g.out_sizes[n++] = d.sizes[k];
    for (int k = 0; k < d.idx_rank; ++k) g.out_sizes[n++] = d.idx_sizes[k];
    for (int k = d.axis + 1; k < d.rank; ++k) g.out_sizes[n++] = d.sizes[k];
  }
  g.out_rank = n;
  g.total = 1;
  for (int k = 0; k < n; ++k) g.total *= g.out_sizes[k];
  if (g.total == 0) return hipSuccess;
  if (d.dtype == PML_HIP_F64 || d.idx_dtype == PML_HIP_F64)
    hipLaunchKernelGGL(gather_kernel<double>, dim3(blocks_for(g.total)), dim3(256), 0, s, d, g, tensor, indices, out);
  else
    hipLaunchKernelGGL(gather_kernel<float>, dim3(blocks_for(g.total)), dim3(256), 0, s, d, g, tensor, indices, out);
  return hipGetLastError();
}

hipError_t scatter_launch(const pml_hip_scatter_desc& d, const void* data, const void* indices, const void* updates, void* out,
                          hipStream_t s) {
  ScatterGeom g{};
  int64_t st = 1;
  for (int k = d.rank - 1; k >= 0; --k) {
    g.strides[k] = st;
    st *= d.sizes[k];
  }
  const int64_t bytes = st * dt_size(d.dtype);
  st = 1;
  for (int k = d.idx_rank - 1; k >= 0; --k) {
    g.idx_strides[k] = st;
    st *= d.idx_sizes[k];
  }
  g.total = 1;
  for (int k = 0; k < d.upd_rank; ++k) g.total *= d.upd_sizes[k];
  if (bytes > 0) {
    hipError_t e = hipMemcpyAsync(out, data, (size_t)bytes, hipMemcpyDeviceToDevice, s);
    if (e != hipSuccess) return e;
  }
  if (g.total == 0 || bytes == 0) return hipSuccess;
  hipLaunchKernelGGL(scatter_kernel, dim3(blocks_for(g.total)), dim3(256), 0, s, d, g, indices, updates, out);
  return hipGetLastError();
}

hipError_t argsort_launch(const pml_hip_argsort_desc& d, const void* tensor, void* out, hipStream_t s) {
  int64_t inner = 1, outer = 1;
  for (int k = d.axis + 1; k < d.rank; ++k) inner *= d.sizes[k];
  for (int k = 0; k < d.axis; ++k) outer *= d.sizes[k];
  const int64_t lines = inner * outer;
  if (lines == 0 || d.sizes[d.axis] == 0) return hipSuccess;
  const dim3 grid((unsigned)(lines < 256 * 16 ? lines : 256 * 16)), block(256);
  if (d.dtype == PML_HIP_F64)
    hipLaunchKernelGGL(argsort_kernel<double>, grid, block, 0, s, d, tensor, (int32_t*)out, inner, lines);
  else if (dt_is_float(d.dtype))
    hipLaunchKernelGGL(argsort_kernel<float>, grid, block, 0, s, d, tensor, (int32_t*)out, inner, lines);
  else if (d.dtype == PML_HIP_U64)
    hipLaunchKernelGGL(argsort_kernel<uint64_t>, grid, block, 0, s, d, tensor, (int32_t*)out, inner, lines);
  else
    hipLaunchKernelGGL(argsort_kernel<int64_t>, grid, block, 0, s, d, tensor, (int32_t*)out, inner, lines);
  return hipGetLastError();
}

}  // namespace pml
