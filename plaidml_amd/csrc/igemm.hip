// Dense contractions on the matrix cores: GEMM and implicit-GEMM 2-D convolution.
//
// One kernel template serves fp32, bf16 and int8.  Both MFMA operands are read
// K-contiguous: A is [M][K] (or gathered from an NHWC image for a convolution)
// and B is presented as Bt[N][K]; a [K][N] right-hand side is transposed once
// into that form by transpose_pack below.  In byte terms every variant is the
// same machine: a K-slab is 128 bytes per row, a lane fetches 16 bytes of an A row
// and 16 bytes of a Bt row from LDS per 32-byte K-block, and issues
//   bf16: one  v_mfma_f32_32x32x16_bf16
//   int8: one  v_mfma_i32_32x32x32_i8
//   fp32: four v_mfma_f32_32x32x2_f32   (the k order inside a block is permuted
//         identically for A and Bt, which leaves the sum unchanged)
// 256 threads = 4 wavefronts in a 2x2 grid; LDS is double-buffered and the next
// slab travels global -> registers while the current one feeds the MFMAs.
#include <hip/hip_runtime.h>

#include "device_common.h"
#include "plans.h"

namespace pml {

#define PML_CAT_(a, b) a##b
#define PML_CAT(a, b) PML_CAT_(a, b)
hipError_t igemm_launch_kind_0(int cfg, bool conv, const IgemmArgs& a, hipStream_t s);
hipError_t igemm_launch_kind_1(int cfg, bool conv, const IgemmArgs& a, hipStream_t s);
hipError_t igemm_launch_kind_2(int cfg, bool conv, const IgemmArgs& a, hipStream_t s);

namespace {

constexpr int kSlabBytes = 128;                // bytes of K per LDS row
constexpr int kRowStride = kSlabBytes + 16;    // padded LDS row (16B-slot skew: conflict-free b128 reads)
constexpr int kThreads = 256;

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

// XCD-aware tile order: hardware deals consecutive workgroup ids round-robin to
// the 8 XCDs, each with its own L2.  Re-number so that one XCD works on a
// contiguous run of tiles (neighbouring tiles share A rows / Bt rows in L2).
__device__ inline int xcd_remap(int bid, int nblocks) {
  constexpr int kXcds = 8;
  if (nblocks % kXcds != 0) return bid;
  const int per = nblocks / kXcds;
  return (bid % kXcds) * per + (bid / kXcds);
}

// Applies init + tail to one 32x32 accumulator block staged in LDS (row stride
// 33 words) and stores it.  Lane l handles rows l/8 + 8*it, columns 4*(l%8)..+3.
template <int KIND>
__device__ __attribute__((noinline)) void tail_block(const IgemmArgs& p, const typename Acc<KIND>::scalar* patch,
                                                     int64_t m_base, int64_t n_base, int lane) {
  const int c4 = (lane & 7) * 4;
  const int64_t n = n_base + c4;
  if (n >= p.N) return;
  const bool fast = p.tail_mode == 1 && n + 3 < p.N && (p.ldc & 3) == 0;
  for (int it = 0; it < 4; ++it) {
    const int row = it * 8 + (lane >> 3);
    const int64_t m = m_base + row;
    if (m >= p.M) continue;
    if (fast) {
      // (optional init) -> round to the result type -> (optional relu) -> one vector store
      if (KIND == KIND_I8) {
        i32x4_t v;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          int iv = (int)patch[row * 33 + c4 + q];
          if (p.init) iv += load_scalar<float, int>(p.init, m * p.init_rs + (n + q) * p.init_cs, p.init_dtype).i;
          if (p.tail_relu) iv = iv < 0 ? 0 : iv;
          v[q] = iv;
        }
        *(i32x4_t*)((int*)p.C + m * p.ldc + n) = v;
      } else {
        float f[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float fv = (float)patch[row * 33 + c4 + q];
          if (p.init) fv += load_scalar<float, int>(p.init, m * p.init_rs + (n + q) * p.init_cs, p.init_dtype).f;
          f[q] = fv;
        }
        if (p.out_dtype == PML_HIP_BF16) {
          uint16_t h[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            h[q] = f32_to_bf16_bits(f[q]);
            if (p.tail_relu && (h[q] & 0x8000u) && (h[q] & 0x7fffu) <= 0x7f80u && (h[q] & 0x7fffu) != 0) h[q] = 0;
          }
          uint2 w = make_uint2((uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16));
          *(uint2*)((uint16_t*)p.C + m * p.ldc + n) = w;
        } else {
          f32x4_t v;
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] = (p.tail_relu && f[q] < 0.f) ? 0.f : f[q];
          *(f32x4_t*)((float*)p.C + m * p.ldc + n) = v;
        }
      }
      continue;
    }
    for (int q = 0; q < 4; ++q) {
      if (n + q >= p.N) break;
      Scalar<float, int> v;
      v.f = 0;
      v.i = 0;
      int cur = p.out_dtype;
      const int64_t nn = n + q;
      if (KIND == KIND_I8) {
        int iv = (int)patch[row * 33 + c4 + q];
        if (p.init) iv += load_scalar<float, int>(p.init, m * p.init_rs + nn * p.init_cs, p.init_dtype).i;
        v.i = iv;
      } else {
        float fv = (float)patch[row * 33 + c4 + q];
        if (p.init) fv += load_scalar<float, int>(p.init, m * p.init_rs + nn * p.init_cs, p.init_dtype).f;
        v.f = round_float_to<float>(cur, fv);
      }
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
        for (int k = 0; k < PML_HIP_MAX_EPI_OPERANDS; ++k)
          off[k] = k < p.tail.n_operands ? m * p.tail.operand_row_stride[k] + nn * p.tail.operand_col_stride[k] : 0;
        v = run_tail<float, int>(p.tail, v, &cur, p.operands, off, p.outs, o);
      }
      store_scalar<float, int>(p.C, o, cur, v);
    }
  }
}

template <int KIND, int BM, int BN, bool CONV>
__global__ __launch_bounds__(kThreads) void igemm_kernel(IgemmArgs p) {
  constexpr int ES = KIND == KIND_BF16 ? 2 : (KIND == KIND_I8 ? 1 : 4);
  constexpr int WM = BM / 2, WN = BN / 2;
  constexpr int MI = WM / 32, NI = WN / 32;
  constexpr int A_VECS = BM * 8 / kThreads;  // 16-byte vectors per thread per slab
  constexpr int B_VECS = BN * 8 / kThreads;
  typedef typename Acc<KIND>::type acc_t;
  typedef typename Acc<KIND>::scalar accs_t;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int kStage = (BM + BN) * kRowStride;  // one buffer: A rows then Bt rows

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  const int tiles_n = (int)((p.N + BN - 1) / BN);
  const int tiles_m = (int)((p.M + BM - 1) / BM);
  const int tile = xcd_remap(blockIdx.x, tiles_m * tiles_n);
  const int64_t m0 = (int64_t)(tile / tiles_n) * BM;
  const int64_t n0 = (int64_t)(tile % tiles_n) * BN;

  // ---- per-thread load assignments (fixed across slabs) ----
  // vector v of row r:  r = tid/8 + 32*i,  v = tid%8
  const int lv = tid & 7;
  const int lr = tid >> 3;
  const int64_t kbytes_total = p.K * ES;  // GEMM: bytes per A row;  CONV: CI*ES bytes per tap

  // A rows
  const unsigned char* a_row[A_VECS];
  bool a_ok[A_VECS];
  int a_ih0[A_VECS], a_iw0[A_VECS];
#pragma unroll
  for (int i = 0; i < A_VECS; ++i) {
    const int64_t m = m0 + lr + 32 * i;
    a_ok[i] = m < p.M;
    if (CONV) {
      const int64_t mm = a_ok[i] ? m : 0;
      const int ow = (int)(mm % p.OW);
      const int64_t t = mm / p.OW;
      const int oh = (int)(t % p.OH);
      const int64_t nb = t / p.OH;
      a_ih0[i] = oh * p.SH - p.PH;
      a_iw0[i] = ow * p.SW - p.PW;
      a_row[i] = (const unsigned char*)p.A + nb * p.H * p.W * p.CI * ES;
    } else {
      a_ih0[i] = a_iw0[i] = 0;
      a_row[i] = (const unsigned char*)p.A + (a_ok[i] ? m : 0) * p.lda * ES;
    }
  }
  const unsigned char* b_row[B_VECS];
  bool b_ok[B_VECS];
#pragma unroll
  for (int i = 0; i < B_VECS; ++i) {
    const int64_t n = n0 + lr + 32 * i;
    b_ok[i] = n < p.N;
    b_row[i] = (const unsigned char*)p.Bt + (b_ok[i] ? n : 0) * p.ldbt * ES;
  }

  // number of slabs: GEMM ceil(K*ES/128); CONV taps * ceil(CI*ES/128)
  const int slabs_per_tap = CONV ? (int)((p.CI * ES + kSlabBytes - 1) / kSlabBytes) : 0;
  const int n_slabs = CONV ? p.KH * p.KW * slabs_per_tap : (int)((kbytes_total + kSlabBytes - 1) / kSlabBytes);

  i32x4_t ra[A_VECS], rb[B_VECS];

  auto load_slab = [&](int s) {
    if (CONV) {
      const int tap = s / slabs_per_tap;
      const int cs = s - tap * slabs_per_tap;
      const int kh = tap / p.KW, kw = tap - kh * p.KW;
      const int64_t cb = (int64_t)cs * kSlabBytes + lv * 16;  // byte offset inside the channel vector
      const bool c_ok = cb < p.CI * ES;
#pragma unroll
      for (int i = 0; i < A_VECS; ++i) {
        const int ih = a_ih0[i] + kh * p.DH, iw = a_iw0[i] + kw * p.DW;
        const bool ok = a_ok[i] && c_ok && ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
        i32x4_t v = {0, 0, 0, 0};
        if (ok) v = *(const i32x4_t*)(a_row[i] + ((int64_t)ih * p.W + iw) * p.CI * ES + cb);
        ra[i] = v;
      }
      // Bt row n holds K = taps*CI elements: tap-major, channel-minor
      const int64_t kb = ((int64_t)tap * p.CI) * ES + cb;
#pragma unroll
      for (int i = 0; i < B_VECS; ++i) {
        i32x4_t v = {0, 0, 0, 0};
        if (b_ok[i] && c_ok) v = *(const i32x4_t*)(b_row[i] + kb);
        rb[i] = v;
      }
    } else {
      const int64_t kb = (int64_t)s * kSlabBytes + lv * 16;
      const bool k_ok = kb < kbytes_total;
#pragma unroll
      for (int i = 0; i < A_VECS; ++i) {
        i32x4_t v = {0, 0, 0, 0};
        if (a_ok[i] && k_ok) v = *(const i32x4_t*)(a_row[i] + kb);
        ra[i] = v;
      }
#pragma unroll
      for (int i = 0; i < B_VECS; ++i) {
        i32x4_t v = {0, 0, 0, 0};
        if (b_ok[i] && k_ok) v = *(const i32x4_t*)(b_row[i] + kb);
        rb[i] = v;
      }
    }
  };
  auto store_slab = [&](int buf) {
#pragma unroll
    for (int i = 0; i < A_VECS; ++i) *(i32x4_t*)(smem + buf * kStage + (lr + 32 * i) * kRowStride + lv * 16) = ra[i];
#pragma unroll
    for (int i = 0; i < B_VECS; ++i)
      *(i32x4_t*)(smem + buf * kStage + (BM + lr + 32 * i) * kRowStride + lv * 16) = rb[i];
  };

  acc_t acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  load_slab(0);
  store_slab(0);
  __syncthreads();

  const int frow = lane & 31;   // row of the 32x32 block this lane feeds
  const int fk = (lane >> 5) * 16;  // its 16-byte half of a 32-byte K-block

  for (int s = 0; s < n_slabs; ++s) {
    const int buf = s & 1;
    if (s + 1 < n_slabs) load_slab(s + 1);
    const unsigned char* a_base = smem + buf * kStage + (wm * WM + frow) * kRowStride + fk;
    const unsigned char* b_base = smem + buf * kStage + (BM + wn * WN + frow) * kRowStride + fk;
#pragma unroll
    for (int kb = 0; kb < kSlabBytes / 32; ++kb) {
      i32x4_t fa[MI], fb[NI];
#pragma unroll
      for (int i = 0; i < MI; ++i) fa[i] = *(const i32x4_t*)(a_base + i * 32 * kRowStride + kb * 32);
#pragma unroll
      for (int j = 0; j < NI; ++j) fb[j] = *(const i32x4_t*)(b_base + j * 32 * kRowStride + kb * 32);
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) mma_block<KIND>(acc[i][j], fa[i], fb[j]);
    }
    if (s + 1 < n_slabs) store_slab(buf ^ 1);
    __syncthreads();
  }

  // ---- tail and store.  In a 32x32 block a lane owns column lane%32 and rows
  // 8*(r/4) + 4*(lane/32) + r%4 for r in [0,16).  Each block is staged through
  // this wavefront's private LDS patch so that a lane then owns four consecutive
  // columns of one row: stores are 8/16-byte pieces of contiguous row segments,
  // and the tail code exists once instead of once per accumulator register.
  accs_t* patch = (accs_t*)(smem + wave * (32 * 33 * 4));
  const int ccol = lane & 31;
  const int crow = (lane >> 5) * 4;
#pragma unroll
  for (int i = 0; i < MI; ++i) {
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      __syncthreads();
#pragma unroll
      for (int r = 0; r < 16; ++r) patch[(8 * (r >> 2) + crow + (r & 3)) * 33 + ccol] = acc[i][j][r];
      __syncthreads();
      tail_block<KIND>(p, patch, m0 + wm * WM + i * 32, n0 + wn * WN + j * 32, lane);
    }
  }
}

// Bt[n][k] = B[k][n]: LDS-tiled transpose, 64x64 elements per workgroup.
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T* __restrict__ B, T* __restrict__ Bt, int64_t K,
                                                        int64_t N, int64_t ldb, int64_t ldbt) {
  __shared__ T tile[64][65];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int64_t k0 = (int64_t)blockIdx.y * 64, n0 = (int64_t)blockIdx.x * 64;
  for (int r = ty; r < 64; r += 4) {
    const int64_t k = k0 + r, n = n0 + tx;
    tile[r][tx] = (k < K && n < N) ? B[k * ldb + n] : (T)0;
  }
  __syncthreads();
  for (int r = ty; r < 64; r += 4) {
    const int64_t n = n0 + r, k = k0 + tx;
    if (n < N && k < K) Bt[n * ldbt + k] = tile[tx][r];
  }
}

template <int KIND, int BM, int BN, bool CONV>
hipError_t launch_cfg(const IgemmArgs& a, hipStream_t s) {
  const int64_t tiles = ((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  const size_t lds = 2 * (size_t)(BM + BN) * kRowStride;
  auto kern = igemm_kernel<KIND, BM, BN, CONV>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(kThreads), lds, s, a);
  return hipGetLastError();
}

template <int KIND, bool CONV>
hipError_t launch_kind(int cfg, const IgemmArgs& a, hipStream_t s) {
  switch (cfg) {
    case TILE_128x128: return launch_cfg<KIND, 128, 128, CONV>(a, s);
    case TILE_128x64: return launch_cfg<KIND, 128, 64, CONV>(a, s);
    case TILE_256x64: return launch_cfg<KIND, 256, 64, CONV>(a, s);
    case TILE_64x64: return launch_cfg<KIND, 64, 64, CONV>(a, s);
  }
  return hipErrorInvalidValue;
}

}  // namespace

#ifndef PML_KIND
#error "compile with -DPML_KIND=0|1|2 (fp32 | bf16 | int8); -DPML_KIND=0 also emits the shared entry points"
#endif

// One translation unit per element kind keeps each compile short and lets make run them in parallel.
hipError_t PML_CAT(igemm_launch_kind_, PML_KIND)(int cfg, bool conv, const IgemmArgs& a, hipStream_t s) {
  return conv ? launch_kind<PML_KIND, true>(cfg, a, s) : launch_kind<PML_KIND, false>(cfg, a, s);
}

#if PML_KIND == 0
hipError_t igemm_launch(int kind, int cfg, bool conv, const IgemmArgs& a, hipStream_t s) {
  switch (kind) {
    case KIND_F32: return igemm_launch_kind_0(cfg, conv, a, s);
    case KIND_BF16: return igemm_launch_kind_1(cfg, conv, a, s);
    case KIND_I8: return igemm_launch_kind_2(cfg, conv, a, s);
  }
  return hipErrorInvalidValue;
}

hipError_t transpose_pack(int elem_size, const void* B, void* Bt, int64_t K, int64_t N, int64_t ldb, int64_t ldbt,
                          hipStream_t s) {
  dim3 grid((unsigned)((N + 63) / 64), (unsigned)((K + 63) / 64));
  switch (elem_size) {
    case 1:
      hipLaunchKernelGGL(transpose_kernel<uint8_t>, grid, dim3(256), 0, s, (const uint8_t*)B, (uint8_t*)Bt, K, N, ldb, ldbt);
      break;
    case 2:
      hipLaunchKernelGGL(transpose_kernel<uint16_t>, grid, dim3(256), 0, s, (const uint16_t*)B, (uint16_t*)Bt, K, N, ldb, ldbt);
      break;
    case 4:
      hipLaunchKernelGGL(transpose_kernel<uint32_t>, grid, dim3(256), 0, s, (const uint32_t*)B, (uint32_t*)Bt, K, N, ldb, ldbt);
      break;
    default:
      return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

#endif  // PML_KIND == 0

}  // namespace pml
