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
// 256 threads = 4 wavefronts; LDS is double-buffered and the next slab travels
// global -> registers while the current one feeds the MFMAs.  After the K loop
// the accumulator tile is staged through LDS so that the tail runs once per
// element in row-major order and stores are contiguous 8/16-byte pieces.
#include <hip/hip_runtime.h>

#include "device_common.h"
#include "igemm_tail.h"
#include "plans.h"

namespace pml {

#define PML_CAT_(a, b) a##b
#define PML_CAT(a, b) PML_CAT_(a, b)
hipError_t igemm_launch_kind_0(int cfg, bool conv, const IgemmArgs& a, hipStream_t s);
hipError_t igemm_launch_kind_1(int cfg, bool conv, const IgemmArgs& a, hipStream_t s);
hipError_t igemm_launch_kind_2(int cfg, bool conv, const IgemmArgs& a, hipStream_t s);

namespace {

constexpr int kSlabBytes = 128;              // bytes of K per LDS row
constexpr int kRowStride = kSlabBytes + 16;  // padded LDS row (16B-slot skew: conflict-free b128 reads)
constexpr int kThreads = 256;

// XCD-aware tile order: hardware deals consecutive workgroup ids round-robin to
// the 8 XCDs, each with its own L2.  Re-number so that one XCD works on a
// contiguous run of tiles (neighbouring tiles share A rows / Bt rows in L2).
__device__ inline int xcd_remap(int bid, int nblocks) {
  constexpr int kXcds = 8;
  if (nblocks % kXcds != 0) return bid;
  const int per = nblocks / kXcds;
  return (bid % kXcds) * per + (bid / kXcds);
}

// BM x BN output tile, WAVES_M x WAVES_N wavefront grid (WAVES_M * WAVES_N == 4).
template <int KIND, int BM, int BN, int WAVES_M, bool CONV>
__global__ __launch_bounds__(kThreads) void igemm_kernel(IgemmArgs p) {
  constexpr int ES = KIND == KIND_BF16 ? 2 : (KIND == KIND_I8 ? 1 : 4);
  constexpr int WAVES_N = 4 / WAVES_M;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int MI = WM / 32, NI = WN / 32;
  constexpr int A_VECS = BM * 8 / kThreads;  // 16-byte vectors per thread per slab
  constexpr int B_VECS = BN * 8 / kThreads;
  constexpr int kStage = (BM + BN) * kRowStride;  // one buffer: A rows then Bt rows
  typedef typename Acc<KIND>::type acc_t;
  typedef typename Acc<KIND>::scalar accs_t;
  typedef accs_t acc4_t __attribute__((ext_vector_type(4)));

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  const int tiles_n = (int)((p.N + BN - 1) / BN);
  const int tiles_m = (int)((p.M + BM - 1) / BM);
  const int tile = xcd_remap(blockIdx.x, tiles_m * tiles_n);
  const int64_t m0 = (int64_t)(tile / tiles_n) * BM;
  const int64_t n0 = (int64_t)(tile % tiles_n) * BN;

  // ---- per-thread load assignments (fixed across slabs): vector lv of rows lr + 32*i ----
  const int lv = tid & 7;
  const int lr = tid >> 3;
  const int kbytes_row = (int)(CONV ? p.CI * ES : p.K * ES);  // valid bytes per (tap) row

  const unsigned char* a_row[A_VECS];  // GEMM: row start; CONV: image start
  bool a_ok[A_VECS];
  int a_ih0[A_VECS], a_iw0[A_VECS];
#pragma unroll
  for (int i = 0; i < A_VECS; ++i) {
    const int64_t m = m0 + lr + 32 * i;
    a_ok[i] = m < p.M;
    const int64_t mm = a_ok[i] ? m : 0;
    if (CONV) {
      const int ow = (int)(mm % p.OW);
      const int64_t t = mm / p.OW;
      const int oh = (int)(t % p.OH);
      const int64_t nb = t / p.OH;
      a_ih0[i] = oh * p.SH - p.PH;
      a_iw0[i] = ow * p.SW - p.PW;
      a_row[i] = (const unsigned char*)p.A + nb * ((int64_t)p.H * p.W * p.CI * ES);
    } else {
      a_ih0[i] = a_iw0[i] = 0;
      a_row[i] = (const unsigned char*)p.A + mm * p.lda * ES;
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

  const int slabs_per_tap = (kbytes_row + kSlabBytes - 1) / kSlabBytes;
  const int n_slabs = CONV ? p.KH * p.KW * slabs_per_tap : slabs_per_tap;
  const int pix_bytes = p.CI * ES;

  i32x4_t ra[A_VECS], rb[B_VECS];
  const i32x4_t zero4 = {0, 0, 0, 0};

  // Loads are unconditional from a clamped (always valid) address; the value is
  // replaced by zero afterwards when the element is outside the problem.
  auto load_slab = [&](int s) {
    if (CONV) {
      const int tap = s / slabs_per_tap;
      const int cs = s - tap * slabs_per_tap;
      const int kh = tap / p.KW, kw = tap - kh * p.KW;
      const int cb = cs * kSlabBytes + lv * 16;  // byte offset inside the channel vector
      const bool c_ok = cb < kbytes_row;
      const int cbs = c_ok ? cb : 0;
      const int dh = kh * p.DH, dw = kw * p.DW;
#pragma unroll
      for (int i = 0; i < A_VECS; ++i) {
        const int ih = a_ih0[i] + dh, iw = a_iw0[i] + dw;
        const bool ok = a_ok[i] && c_ok && (unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W;
        const int off = ok ? (ih * p.W + iw) * pix_bytes + cbs : 0;
        const i32x4_t v = *(const i32x4_t*)(a_row[i] + off);
        ra[i] = ok ? v : zero4;
      }
      const int kb = tap * pix_bytes + cbs;  // Bt row: tap-major, channel-minor
#pragma unroll
      for (int i = 0; i < B_VECS; ++i) {
        const i32x4_t v = *(const i32x4_t*)(b_row[i] + kb);
        rb[i] = (b_ok[i] && c_ok) ? v : zero4;
      }
    } else {
      const int kb = s * kSlabBytes + lv * 16;
      const bool k_ok = kb < kbytes_row;
      const int kbs = k_ok ? kb : 0;
#pragma unroll
      for (int i = 0; i < A_VECS; ++i) {
        const i32x4_t v = *(const i32x4_t*)(a_row[i] + kbs);
        ra[i] = (a_ok[i] && k_ok) ? v : zero4;
      }
#pragma unroll
      for (int i = 0; i < B_VECS; ++i) {
        const i32x4_t v = *(const i32x4_t*)(b_row[i] + kbs);
        rb[i] = (b_ok[i] && k_ok) ? v : zero4;
      }
    }
  };
  auto store_slab = [&](int buf) {
    unsigned char* base = smem + buf * kStage + lr * kRowStride + lv * 16;
#pragma unroll
    for (int i = 0; i < A_VECS; ++i) *(i32x4_t*)(base + (32 * i) * kRowStride) = ra[i];
#pragma unroll
    for (int i = 0; i < B_VECS; ++i) *(i32x4_t*)(base + (BM + 32 * i) * kRowStride) = rb[i];
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

  const int frow = lane & 31;       // row of the 32x32 block this lane feeds
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
        for (int j = 0; j < NI; ++j) mma_block<KIND>(acc[i][j], fb[j], fa[i]);
    }
    if (s + 1 < n_slabs) store_slab(buf ^ 1);
    __syncthreads();
  }

  // ---- stage the accumulator tile in LDS as ctile[BM][BN + 4] ----
  // The MFMAs ran with the Bt fragment as the row operand, so in a 32x32 block a
  // lane owns tile row (m) lane%32 and the columns (n) 8*(r/4) + 4*(lane/32) + r%4:
  // four consecutive columns per register quad, one 16-byte LDS store each.
  constexpr int CS = BN + 4;
  static_assert((size_t)BM * CS * 4 <= 2 * (size_t)kStage, "accumulator tile must fit in the pipeline buffers");
  accs_t* ctile = (accs_t*)smem;
  {
    const int crow = lane & 31;
    const int ccol = (lane >> 5) * 4;
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NI; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          acc4_t q;
#pragma unroll
          for (int e = 0; e < 4; ++e) q[e] = acc[i][j][4 * g + e];
          *(acc4_t*)&ctile[(wm * WM + i * 32 + crow) * CS + wn * WN + j * 32 + 8 * g + ccol] = q;
        }
  }
  __syncthreads();

  tile_tail<KIND, BM, BN, kThreads>(p, ctile, m0, n0, tid);
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

template <int KIND, int BM, int BN, int WAVES_M, bool CONV>
hipError_t launch_cfg(const IgemmArgs& a, hipStream_t s) {
  const int64_t tiles = ((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  const size_t lds = 2 * (size_t)(BM + BN) * kRowStride;
  auto kern = igemm_kernel<KIND, BM, BN, WAVES_M, CONV>;
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
    case TILE_128x128: return launch_cfg<KIND, 128, 128, 2, CONV>(a, s);
    case TILE_128x64: return launch_cfg<KIND, 128, 64, 2, CONV>(a, s);
    case TILE_256x64: return launch_cfg<KIND, 256, 64, 4, CONV>(a, s);
    case TILE_64x64: return launch_cfg<KIND, 64, 64, 2, CONV>(a, s);
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
