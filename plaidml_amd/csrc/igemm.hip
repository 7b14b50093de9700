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
//
// Data movement.  256 threads = 4 wavefronts.  Slabs travel global -> LDS directly
// (buffer_load ... lds, 16 bytes per lane, no register staging) into a ring of
// three stages, two slabs ahead of the MFMAs, with one s_barrier per slab.  A
// load whose element lies outside the problem (M / N / K tails, convolution
// padding) carries an offset beyond the buffer and delivers zeros.  One such
// instruction of a wavefront fills 8 rows x 128 bytes contiguously, so LDS rows
// are not padded; instead the lane that fills 16-byte slot u of row r fetches
// chunk u ^ ((r >> 1) & 7) of that row, and readers apply the same XOR: 16
// consecutive rows then read 16 different slots (no bank conflicts).
// After the K loop the accumulators are staged through LDS so that the tail runs
// once per element in row-major order and stores are contiguous 8/16-byte pieces.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "device_common.h"
#include "igemm_tail.h"
#include "plans.h"

namespace pml {

#define PML_CAT_(a, b) a##b
#define PML_CAT(a, b) PML_CAT_(a, b)
hipError_t igemm_launch_kind_0(int cfg, bool conv, const IgemmArgs& a, hipStream_t s);
hipError_t igemm_launch_kind_1(int cfg, bool conv, const IgemmArgs& a, hipStream_t s);
hipError_t igemm_launch_kind_2(int cfg, bool conv, const IgemmArgs& a, hipStream_t s);
hipError_t igemm_launch_kind_3(int cfg, bool conv, const IgemmArgs& a, hipStream_t s);
hipError_t igemm_launch_kind_4(int cfg, bool conv, const IgemmArgs& a, hipStream_t s);

namespace {

constexpr int kSlabBytes = 128;  // bytes of K per LDS row
constexpr int kThreads = 256;
constexpr int kLdsBytes = 160 * 1024;
constexpr unsigned kRsrcFlags = 0x00020000u;   // raw buffer, 32-bit data format
constexpr unsigned kBufRange = 0x80000000u;    // every real offset is below 2 GiB (checked at launch) ...
constexpr unsigned kOutside = 0x80000000u;     // ... and this one reads as zeros, with any slab offset added

#define PML_LDS(p) ((__attribute__((address_space(3))) void*)(p))

// Sum of two byte offsets, each of which may be the "outside" mark.
__device__ inline unsigned join_offsets(unsigned x, unsigned y) { return ((x | y) & kOutside) ? kOutside : x + y; }

// STAGES = 0: as many as pay for the tile; 2: two, and LDS rounded up to what staging the whole result
// tile needs (a short-K, bandwidth-bound GEMM gains more from a second workgroup on the CU than from a
// third slab in flight)
template <int BM, int BN, int STAGES = 0, int SLAB = 128>
struct Ring {
  static constexpr int kStage = (BM + BN) * SLAB;                       // A rows then Bt rows
  // 64x64 tiles run two stages: 32 KB of LDS lets five workgroups share a CU, and for this tile
  // residency hides more latency than a third slab in flight does
  static constexpr int kStages = STAGES ? STAGES : ((BM * BN <= 64 * 64) ? 2 : (3 * kStage <= kLdsBytes ? 3 : 2));
  static constexpr int kTileBytes = BM * (BN + 4) * 4;
  static constexpr int kBytes = (STAGES && kTileBytes > kStages * kStage && kTileBytes <= kLdsBytes) ? kTileBytes : kStages * kStage;
  // 256 bytes behind the ring take what the "touch" loads of a residual tensor bring (their only purpose is to
  // pull the rows into the caches; a load that writes LDS needs no register to land in).  Not for 64x64 tiles:
  // five of their 32 KB rings fill a CU's LDS exactly.
  static constexpr int kDump = BM * BN > 64 * 64 ? 256 : 0;
  static constexpr int kAlloc = kBytes + kDump;
  static_assert(kAlloc <= kLdsBytes, "the ring must fit the CU's LDS");
};

// BM x BN output tile, WAVES_M x WAVES_N wavefront grid; NT threads = 4, 8 or 16 wavefronts (one, two or four
// per SIMD).  WAVES_K = 2: two such grids, each multiplying one half of the K-blocks of every slab; their
// partial results meet in LDS before the tail (more wavefronts for problems with few tiles and a long K).
// Wavefronts per SIMD the register allocation has to leave room for: those of as many workgroups as the LDS
// footprint lets a CU hold (at most two are counted on).
template <int BM, int BN, int STAGES, int SLAB, int NT>
constexpr int igemm_waves_per_simd() {
  return (NT / 256) * (2 * Ring<BM, BN, STAGES, SLAB>::kAlloc <= kLdsBytes ? 2 : 1);
}

// BKN: the right-hand side is the caller's row-major B[K][N] (p.Bt, p.ldbt its row length): a slab is then the
// rows of B as they lie in memory, [k][n] in LDS, and nothing is transposed by a launch of its own.
// fp32 kinds: a lane gathers the four K-values of its fragment with four 4-byte reads (32 consecutive columns per
// half wavefront: no bank conflicts); the fp32 MFMA takes one K-value per lane anyway.
// int8: the 16 K-values of a lane's fragment come from two transposing LDS reads (ds_read_b64_tr_b8: the 16 lanes
// of a group each name 8 bytes -- here 8 columns of one K-row -- and lane i receives byte i % 8 of the data named
// by lanes i / 8, i / 8 + 2, ..., i.e. 8 K-values of column i).  The 16-byte chunks of K-row k are stored at
// positions XORed with k % 8 so that the 8 rows of such a read fall into different banks.
// SPLITK: the K loop of a tile is shared out among p.sk_splits workgroups (workgroup id = split x tiles + tile), each
// of which multiplies p.sk_per consecutive slabs and leaves its partial tile, untouched by any tail, in the workspace
// p.ws[split][M][sk_pitch]; splitk_reduce_kernel below adds the parts up and runs the tail.  For problems with few
// tiles and a long K (the 3x3 convolutions of a network's last stages at batch 1: 8 tiles of 72 slabs), which would
// otherwise leave most of the chip idle for the length of one long serial loop.
template <int KIND, int BM, int BN, int WAVES_M, bool CONV, int NT = kThreads, int STAGES = 0, int WAVES_K = 1, int SLAB = 128,
          bool BKN = false, bool SPLITK = false>
__global__ __launch_bounds__(NT, (igemm_waves_per_simd<BM, BN, STAGES, SLAB, NT>())) void igemm_kernel(IgemmArgs p_by_value) {
  // The argument block is read where the dispatcher put it (the kernel-argument segment, scalar loads),
  // through a reference: taking the by-value parameter's address instead makes the compiler copy all of
  // it to scratch memory as soon as one field is indexed with a run-time value.
  const IgemmArgs& p = *(const IgemmArgs*)(const __attribute__((address_space(4))) void*)__builtin_amdgcn_kernarg_segment_ptr();
  typedef Ring<BM, BN, STAGES, SLAB> ring_t;
  // bytes of K per LDS row and ring stage: 128 (four 32-byte K-blocks), or 64 for the large tiles, whose
  // 160 KB of LDS then hold five stages instead of two -- what a CU has in flight is what hides memory latency
  constexpr int kSlabBytes = SLAB;
  constexpr int CPR = SLAB / 16;                      // 16-byte chunks per row
  constexpr int kSwzShift = SLAB == 128 ? 1 : 2;      // chunk u of row r sits in slot u ^ ((r >> shift) & (CPR - 1))
  static_assert(SLAB == 128 || SLAB == 64, "rows of 128 or 64 bytes");
  constexpr int ES = KIND == KIND_BF16 ? 2 : (KIND == KIND_I8 ? 1 : 4);
  constexpr bool kSplit = KIND == KIND_F32X3 || KIND == KIND_F32X3P;  // fp32 operands as three bf16 products
  constexpr bool kSplitB = KIND == KIND_F32X3P;                       // ... the right-hand side split when it was packed
  static_assert(!BKN || ((KIND == KIND_F32 || KIND == KIND_F32X3 || KIND == KIND_I8) && !CONV && SLAB == 128),
                "a [K][N] right-hand side: fp32 and int8 GEMMs only");
  constexpr int kRowChunks = BN * ES / 16;                       // BKN: 16-byte chunks of one K-row of the tile
  constexpr int kRowKey = kRowChunks >= 8 ? 7 : kRowChunks - 1;  // int8: chunk positions are XORed with (k & kRowKey) * kRowKeyMul
  constexpr int kRowKeyMul = kRowChunks >= 16 ? 2 : 1;
  constexpr int kWaves = NT / 64;
  constexpr int kRowsPerPass = NT / CPR;  // operand rows one load of all threads covers
  constexpr int WAVES_N = kWaves / WAVES_M / WAVES_K;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int MI = WM / 32, NI = WN / 32;
  constexpr int A_VECS = BM * CPR / NT;  // 16-byte vectors per thread per slab
  constexpr int B_VECS = BN * CPR / NT;
  static_assert(BM % kRowsPerPass == 0 && BN % kRowsPerPass == 0, "tile sides are whole load passes");
  constexpr int kStage = ring_t::kStage;
  constexpr int kStages = ring_t::kStages;
  constexpr int kLoads = A_VECS + B_VECS;          // loads a thread issues per slab
  static_assert((kStages - 1) * kLoads <= 63, "the vmcnt field counts at most 63 loads");
  static_assert((kSlabBytes / 32 / WAVES_K) % 2 == 0, "fragment buffers alternate per K-block and must line up across slabs");
  // (The vmcnt arithmetic below counts this kernel's own requests: a configuration whose registers spill
  // puts scratch loads and stores into the same counter and is wrong, not just slow -- 256x256 with 16
  // wavefronts needs 198 registers of the 128 it may have and failed its tests for that reason.)
  typedef typename Acc<KIND>::type acc_t;
  typedef typename Acc<KIND>::scalar accs_t;
  typedef accs_t acc4_t __attribute__((ext_vector_type(4)));

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wk = wave / (WAVES_M * WAVES_N);  // which part of every slab's K-blocks
  const int wm = (wave % (WAVES_M * WAVES_N)) / WAVES_N, wn = wave % WAVES_N;

  int tile_m, tile_n;
  unsigned tile_id = blockIdx.x;
  int split = 0;
  if constexpr (SPLITK) {
    static_assert(WAVES_K == 1 && !BKN, "the split over workgroups stands alone");
    split = (int)(tile_id / (unsigned)p.sk_tiles);
    tile_id -= (unsigned)split * (unsigned)p.sk_tiles;
  }
  tile_of(p.order, tile_id, &tile_m, &tile_n);
  const int64_t m0 = (int64_t)tile_m * BM;
  const int64_t n0 = (int64_t)tile_n * BN;

  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void*)p.A, 0, (int)kBufRange, kRsrcFlags);
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void*)p.Bt, 0, (int)kBufRange, kRsrcFlags);
  // the second product of a two-product GEMM (the first one's operands again when there is none)
  const bool two = !CONV && p.K2 > 0;
  const __amdgpu_buffer_rsrc_t ra2 = __builtin_amdgcn_make_buffer_rsrc((void*)(two ? p.A2 : p.A), 0, (int)kBufRange, kRsrcFlags);
  const __amdgpu_buffer_rsrc_t rb2 = __builtin_amdgcn_make_buffer_rsrc((void*)(two ? p.Bt2 : p.Bt), 0, (int)kBufRange, kRsrcFlags);

  // ---- per-thread load assignments (fixed across slabs): slot lv of rows lr + kRowsPerPass*i ----
  const int lv = tid % CPR;
  const int lr = tid / CPR;
  const int lc = lv ^ ((lr >> kSwzShift) & (CPR - 1));        // the chunk of its row this thread fetches
  int kbytes_row = __builtin_amdgcn_readfirstlane((int)(CONV ? p.CI * ES : p.K * ES));  // valid bytes per (tap) row
  asm volatile("" : "+s"(kbytes_row));

  // Loop-invariant scalars of the geometry, pinned to scalar registers: read through the argument block inside
  // the K loop they would be re-fetched there (a scalar load and a wait that also drains the LDS reads).
  auto pinned = [](int v) {
    v = __builtin_amdgcn_readfirstlane(v);
    asm volatile("" : "+s"(v));
    return v;
  };
  const int cH = pinned(CONV ? p.H : 0), cW = pinned(CONV ? p.W : 0);
  const int cKW = pinned(CONV ? p.KW : 1), cKH = pinned(CONV ? p.KH : 1);
  const int cDH = pinned(CONV ? p.DH : 0), cDW = pinned(CONV ? p.DW : 0);
  const int pix_bytes = pinned(p.CI * ES);                               // bytes of one tap's K-run
  const int pix_pitch = pinned(p.pix_pitch ? p.pix_pitch : p.CI * ES);   // bytes between neighbouring input pixels
  // a K-run that spans several pixels (pitch < run): chunk byte -> pixel as multiply-and-shift, exact for the
  // few thousand bytes a run can have; otherwise every chunk lies in the tap's own pixel
  const unsigned pitch_magic = (CONV && p.pix_pitch) ? (unsigned)pinned((int)(((1u << 20) + (unsigned)p.pix_pitch - 1) / (unsigned)p.pix_pitch)) : 0u;

  // GEMM: byte offset of the row, kOutside for rows past M.  CONV: byte offset of input pixel (ih0, iw0) of the
  // row's output pixel, the one its tap (0, 0) reads -- possibly before the image's first byte, which is why it
  // is only ever used together with the bounds check on (ih0 + dh, iw0 + dw); rows past M fail that check.
  unsigned a_off[A_VECS];
  int a_ih0[A_VECS], a_iw0[A_VECS];
#pragma unroll
  for (int i = 0; i < A_VECS; ++i) {
    const int64_t m = m0 + lr + kRowsPerPass * i;
    const bool ok = m < p.M;
    const int64_t mm = ok ? m : 0;
    if (CONV) {
      // pixel numbers stay below 2^31 (the launcher checks the operand sizes)
      const unsigned mu = (unsigned)mm;
      const unsigned nb = fast_div(mu, p.div_per_magic, p.div_per_shift);
      const unsigned rem = mu - nb * (unsigned)(p.OH * p.OW);
      const unsigned ohu = fast_div(rem, p.div_ow_magic, p.div_ow_shift);
      const int oh = (int)ohu, ow = (int)(rem - ohu * (unsigned)p.OW);
      a_ih0[i] = ok ? oh * p.SH - p.PH : -(1 << 28);
      a_iw0[i] = ow * p.SW - p.PW;
      a_off[i] = (unsigned)((int64_t)nb * ((int64_t)cH * cW * pix_pitch)) + (unsigned)((a_ih0[i] * cW + a_iw0[i]) * pix_pitch);
    } else {
      a_ih0[i] = a_iw0[i] = 0;
      a_off[i] = ok ? (unsigned)(mm * p.lda * ES) : kOutside;
    }
  }
  unsigned b_off[B_VECS];
  int b_krow[BKN ? B_VECS : 1];  // BKN: the row of the slab (0..31) this thread's chunk belongs to
#pragma unroll
  for (int i = 0; i < B_VECS; ++i) {
    if constexpr (BKN) {
      const int c = tid + i * NT;
      b_krow[i] = c / kRowChunks;
      const int chunk = KIND == KIND_I8 ? (c % kRowChunks) ^ ((b_krow[i] & kRowKey) * kRowKeyMul) : c % kRowChunks;  // what this LDS position holds
      const int64_t n = n0 + chunk * (16 / ES);
      b_off[i] = n < p.N ? (unsigned)(((int64_t)b_krow[i] * p.ldbt + n) * ES) : kOutside;
    } else {
      const int64_t n = n0 + lr + kRowsPerPass * i;
      b_off[i] = n < p.N ? (unsigned)(n * p.ldbt * ES) : kOutside;
    }
  }
  unsigned a2_off[CONV ? 1 : A_VECS], b2_off[CONV ? 1 : B_VECS];
  if constexpr (!CONV) {
#pragma unroll
    for (int i = 0; i < A_VECS; ++i) {
      const int64_t m = m0 + lr + kRowsPerPass * i;
      int64_t row = m;
      if (two && p.g2_stride > 0) {
        const unsigned mu = (unsigned)(m < p.M ? m : 0);
        const unsigned nb = fast_div(mu, p.g2_ohw_magic, p.g2_ohw_shift);
        const unsigned rem = mu - nb * (unsigned)p.g2_ohw;
        const unsigned oy = fast_div(rem, p.g2_ow_magic, p.g2_ow_shift);
        const unsigned ox = rem - oy * (unsigned)p.g2_ow;
        row = ((int64_t)nb * p.g2_h + (int64_t)oy * p.g2_stride) * p.g2_w + (int64_t)ox * p.g2_stride;
      }
      a2_off[i] = (two && m < p.M) ? (unsigned)(row * p.lda2 * ES) : kOutside;
    }
#pragma unroll
    for (int i = 0; i < B_VECS; ++i) {
      const int64_t n = n0 + lr + kRowsPerPass * i;
      b2_off[i] = (two && n < p.N) ? (unsigned)(n * p.ldbt2 * ES) : kOutside;
    }
  }

  const int slabs_per_tap = pinned((kbytes_row + kSlabBytes - 1) / kSlabBytes);
  const int k2_bytes = pinned(two ? (int)(p.K2 * ES) : 0);
  const int first_bytes = slabs_per_tap * kSlabBytes;  // where the second product's slabs begin on the slab axis
  const int n_slabs = CONV ? p.KH * p.KW * slabs_per_tap : slabs_per_tap + (k2_bytes + kSlabBytes - 1) / kSlabBytes;

  // Requests of the next slab into ring stage `stage`, one 16-byte-per-lane load at a time (index l: the A
  // rows first, then the Bt rows) so that they can be spread between the MFMAs.  Slabs are prepared in order,
  // one per call, so the filter tap and the position inside its channel run are counters, not quotients.
  // Past the last slab every offset is outside: the request count per slab stays constant, which is what
  // the vmcnt arithmetic below relies on.
  unsigned char* req_base = smem;
  unsigned req_a = 0, req_b = 0;  // slab-dependent part of the A / Bt offsets
  int req_k0 = 0;                 // BKN: first K-index of the slab
  int req_dh = 0, req_dw = 0;     // CONV: the tap's displacement in input rows / columns (columns: plus the chunk's pixel)
  bool req_ok = false;
  bool req_second = false;        // GEMM: the slab belongs to the second product
  int nx_kh = 0, nx_kw = 0, nx_cs = 0, nx_dh = 0, nx_dw = 0, nx_tap = 0;  // CONV: tap and slab-in-tap of the next slab
  int nx_kbo = 0;                                                          // GEMM: its first byte of K
  int slab_count = n_slabs;  // slabs this workgroup multiplies
  if constexpr (SPLITK) {
    // this workgroup's run of slabs: the counters start where slab `first` begins
    const int first = split * p.sk_per;
    slab_count = n_slabs - first < p.sk_per ? n_slabs - first : p.sk_per;
    if (CONV) {
      const int tap = first / slabs_per_tap;
      nx_cs = first - tap * slabs_per_tap;
      nx_kh = tap / cKW;
      nx_kw = tap - nx_kh * cKW;
      nx_tap = tap * pix_bytes;
      nx_dh = nx_kh * cDH;
      nx_dw = nx_kw * cDW;
    } else {
      nx_kbo = first * kSlabBytes;
    }
  }
  auto prepare_slab = [&](int stage) {
    req_base = smem + stage * kStage + wave * 1024;  // one request of a wavefront fills 1 KB
    if (CONV) {
      const int cb = nx_cs * kSlabBytes + lc * 16;  // byte offset inside the tap's K-run
      req_ok = (nx_kh < cKH) & (cb < kbytes_row);
      const int px = (int)(((unsigned)cb * pitch_magic) >> 20);
      req_dh = nx_dh;
      req_dw = nx_dw + px;
      req_a = (unsigned)((nx_dh * cW + nx_dw) * pix_pitch + cb);
      req_b = req_ok ? (unsigned)(nx_tap + cb) : kOutside;  // Bt row: tap-major, channel-minor
      if (++nx_cs == slabs_per_tap) {
        nx_cs = 0;
        nx_tap += pix_bytes;
        nx_dw += cDW;
        if (++nx_kw == cKW) {
          nx_kw = 0;
          nx_dw = 0;
          ++nx_kh;
          nx_dh += cDH;
        }
      }
    } else {
      req_second = nx_kbo >= first_bytes;
      const int kbo = (req_second ? nx_kbo - first_bytes : nx_kbo) + lc * 16;
      req_a = req_b = kbo < (req_second ? k2_bytes : kbytes_row) ? (unsigned)kbo : kOutside;
      if constexpr (BKN) {
        req_k0 = nx_kbo / ES;
        req_b = (unsigned)((int64_t)req_k0 * p.ldbt * ES);  // the slab's first row of B
      }
      nx_kbo += kSlabBytes;
    }
  };
  auto issue_load = [&](int l) {
    if (l < A_VECS) {
      unsigned off;
      if (CONV) {
        const bool ok = req_ok & ((unsigned)(a_ih0[l] + req_dh) < (unsigned)cH) & ((unsigned)(a_iw0[l] + req_dw) < (unsigned)cW);
        off = ok ? a_off[l] + req_a : kOutside;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, PML_LDS(req_base + l * kRowsPerPass * kSlabBytes), 16, (int)off, 0, 0, 0);
      } else {
        off = join_offsets(req_second ? a2_off[l] : a_off[l], req_a);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(req_second ? ra2 : ra, PML_LDS(req_base + l * kRowsPerPass * kSlabBytes), 16, (int)off, 0, 0, 0);
      }
    } else {
      const int i = l - A_VECS;
      if (CONV) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, PML_LDS(req_base + (BM + i * kRowsPerPass) * kSlabBytes), 16,
                                                 (int)join_offsets(b_off[i], req_b), 0, 0, 0);
      } else if constexpr (BKN) {
        const unsigned off = (b_off[i] != kOutside && req_k0 + b_krow[i] < (int)p.K) ? b_off[i] + req_b : kOutside;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, PML_LDS(req_base + (BM + i * kRowsPerPass) * kSlabBytes), 16, (int)off, 0, 0, 0);
      } else {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(req_second ? rb2 : rb, PML_LDS(req_base + (BM + i * kRowsPerPass) * kSlabBytes), 16,
                                                 (int)join_offsets(req_second ? b2_off[i] : b_off[i], req_b), 0, 0, 0);
      }
    }
  };

  // a residual tensor of the tail is requested now, so that it arrives under the K loop
  TailPrefetch<KIND, BM, BN, NT> pre;
  const bool direct = !SPLITK && WAVES_K == 1 && direct_tail_ok<KIND>(p, n0, BN);

  pre.valid = false;
  if (!direct && !SPLITK) tail_prefetch<KIND, BM, BN, NT>(p, m0, n0, tid, pre);
  // The direct tail reads its residual rows only after the K loop.  One 4-byte load per lane and 32x32 block,
  // issued here and landing in the dump area of LDS, brings the 64 bytes a row contributes to the block into the
  // caches: a short-K GEMM then waits for operands and residual together instead of one after the other.
  // (Holding the rows in registers from here on -- 8 per block -- made the 128-register configurations spill.)
  if constexpr (KIND == KIND_BF16 && WAVES_K == 1 && ring_t::kDump > 0 && MI * NI <= 4) {
    if (direct && p.tail_mode == 2) {
      const __amdgpu_buffer_rsrc_t rr = __builtin_amdgcn_make_buffer_rsrc((void*)p.operands[0], 0, (int)kBufRange, kRsrcFlags);
      const int64_t rs = p.tail.operand_row_stride[0];
      // (the lane number through an opaque move, so that nothing worked out here is kept for the tail)
      int lane_t = lane;
      asm volatile("" : "+v"(lane_t));
#pragma unroll
      for (int j = 0; j < NI; ++j)
#pragma unroll
        for (int i = 0; i < MI; ++i) {
          const int64_t m = m0 + wm * WM + i * 32 + (lane_t & 31);
          const int64_t col = n0 + wn * WN + j * 32 + 16 * (lane_t >> 5);
          const int64_t off = (m * rs + col) * 2;
          const unsigned voff = (m < p.M && col < p.N && off < (int64_t)kBufRange) ? (unsigned)off : kOutside;
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rr, PML_LDS(smem + ring_t::kBytes), 4, (int)voff, 0, 0, 0);
        }
    }
  }

  acc_t acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  // Every ring stage is requested before the first multiply: kStages slabs in flight.
#pragma unroll
  for (int s = 0; s < kStages; ++s) {
    prepare_slab(s);
#pragma unroll
    for (int l = 0; l < kLoads; ++l) issue_load(l);
  }

  const int frow = lane & 31;  // row of the 32x32 block this lane feeds
  // byte offset of its 16-byte half of each of the wavefront's 32-byte K-blocks, swizzled
  constexpr int kBlocks = kSlabBytes / 32 / WAVES_K;
  // (fslot_b: the Bt fragment's; different only for the split fp32 kind.  That kind takes a pair of K-blocks as one
  // bf16 MFMA step of 16 K-values, the lane's eight values being two neighbouring 16-byte chunks of the fp32 row;
  // a right-hand side that was split when it was packed keeps, per 128 bytes of a row, the 32 bf16 heads in the
  // first 64 bytes and the 32 remainders in the second, and the pair's two reads fetch one of each.)
  int fslot[kBlocks], fslot_b[kBlocks];
#pragma unroll
  for (int kb = 0; kb < kBlocks; ++kb) {
    const int gb = wk * kBlocks + kb, h = lane >> 5, key = (lane >> kSwzShift) & (CPR - 1);
    if constexpr (kSplit) {
      fslot[kb] = (((gb & ~1) * 2 + 2 * h + (gb & 1)) ^ key) * 16;
      fslot_b[kb] = kSplitB ? ((((gb & 1) * 4 + (gb >> 1) * 2 + h) ^ key) * 16) : fslot[kb];
    } else {
      fslot[kb] = ((gb * 2 + h) ^ key) * 16;
      fslot_b[kb] = fslot[kb];
    }
    // BKN: chunk c of a row holds K-values 4c .. 4c + 3 (int8: 16c .. 16c + 15), which in [k][n] order are that
    // many rows of BN elements
    if constexpr (BKN) fslot_b[kb] = (kSplit ? ((gb & ~1) * 2 + 2 * h + (gb & 1)) : (gb * 2 + h)) * (16 / ES) * (BN * ES);
  }
  // BKN, int8: what a lane names in a transposing read of 32-column block j -- K-row (lane % 16) / 2 of the 8, the
  // 8 columns (lane % 2) of the 16 its group of lanes covers -- as a byte offset into the stage's [k][n] part
  int bcol[(BKN && KIND == KIND_I8) ? NI : 1];
  if constexpr (BKN && KIND == KIND_I8) {
    const int jrow = (lane & 15) >> 1;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int chunk = (wn * WN + j * 32) / 16 + ((lane >> 4) & 1);
      bcol[j] = jrow * BN + ((chunk ^ ((jrow & kRowKey) * kRowKeyMul)) * 16) + (lane & 1) * 8;
    }
  }
  // the Bt fragment of 32-column block j for the K-block whose slot is `slot`, out of the stage whose Bt part `bb`
  // points into (at the wavefront's first column and the lane's row or column)
  auto read_b = [&](const unsigned char* bb, int j, int slot) {
    if constexpr (BKN && KIND == KIND_I8) {
      typedef int v2i_t __attribute__((ext_vector_type(2)));
      typedef __attribute__((address_space(3))) v2i_t* lds_v2i_ptr;
      const v2i_t lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_ptr)PML_LDS(bb + slot + bcol[j]));
      const v2i_t hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_ptr)PML_LDS(bb + slot + bcol[j] + 8 * BN));
      return i32x4_t{lo[0], lo[1], hi[0], hi[1]};
    } else if constexpr (BKN) {
      i32x4_t v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = *(const int*)(bb + slot + e * (BN * 4) + j * 32 * 4);
      return v;
    } else {
      return *(const i32x4_t*)(bb + j * 32 * kSlabBytes + slot);
    }
  };

  // The loop is rotated by one K-block: the one synchronisation point of a slab sits before its LAST
  // K-block, whose fragments are in registers by then.  Past it every wavefront is done reading this
  // slab's stage, and the next slab has landed (vmcnt leaves only the younger slabs outstanding); so the
  // last K-block's MFMAs cover the first fragment reads of the next slab and the requests that refill this
  // stage with slab s + kStages, and no MFMA ever waits behind a barrier for LDS or memory.
  constexpr int kOutstanding = (kStages - 2) * kLoads;  // requests that may still be in flight at the sync point
  constexpr int kSlots = MI * NI;
  i32x4_t fa[2][MI], fb[2][NI];
  // fp32 as three bf16 products: a pair of K-blocks (8 fp32 values per lane and fragment) is split into bf16 heads
  // and remainders at its second block and multiplied there; the first block of a pair only fetches
  i32x4_t xa_head[kSplit ? MI : 1], xa_rem[kSplit ? MI : 1];
  i32x4_t xb_head[kSplit && !kSplitB ? NI : 1], xb_rem[kSplit && !kSplitB ? NI : 1];
  const unsigned char* a_base = smem + (wm * WM + frow) * kSlabBytes;
  const unsigned char* b_base = !BKN ? smem + (BM + wn * WN + frow) * kSlabBytes
                                     : smem + BM * kSlabBytes + (KIND == KIND_I8 ? 0 : (wn * WN + frow) * 4);
  __builtin_amdgcn_s_waitcnt(0x0F70 | (((kStages - 1) * kLoads) & 15) | ((((kStages - 1) * kLoads) >> 4) << 14));
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int i = 0; i < MI; ++i) fa[0][i] = *(const i32x4_t*)(a_base + i * 32 * kSlabBytes + fslot[0]);
#pragma unroll
  for (int j = 0; j < NI; ++j) fb[0][j] = read_b(b_base, j, fslot_b[0]);

  int stage = 0;  // ring stage of slab s
  for (int s = 0; s < slab_count; ++s) {
    int next_stage = stage + 1;
    if (next_stage == kStages) next_stage = 0;
    const unsigned char* a_next = smem + next_stage * kStage + (wm * WM + frow) * kSlabBytes;
    const unsigned char* b_next = smem + next_stage * kStage +
                                  (!BKN ? (BM + wn * WN + frow) * kSlabBytes
                                        : BM * kSlabBytes + (KIND == KIND_I8 ? 0 : (wn * WN + frow) * 4));
#pragma unroll
    for (int kb = 0; kb < kBlocks; ++kb) {
      const int cur = kb & 1, nxt = cur ^ 1;
      const bool last = kb + 1 == kBlocks;
      if (last) {
        // fragments of this K-block are in registers (lgkmcnt 0), slab s + 1 has landed
        __builtin_amdgcn_s_waitcnt(0x0070 | (kOutstanding & 15) | ((kOutstanding >> 4) << 14));
        __builtin_amdgcn_s_barrier();
        prepare_slab(stage);
      }
      const unsigned char* ra_ = last ? a_next : a_base;
      const unsigned char* rb_ = last ? b_next : b_base;
      const int fs = fslot[last ? 0 : kb + 1];
      const int fs_b = fslot_b[last ? 0 : kb + 1];
      if constexpr (kSplit) {
        if (cur == 1) {
#pragma unroll
          for (int i = 0; i < MI; ++i) split_f32x8(fa[0][i], fa[1][i], xa_head[i], xa_rem[i]);
          if constexpr (!kSplitB) {
#pragma unroll
            for (int j = 0; j < NI; ++j) split_f32x8(fb[0][j], fb[1][j], xb_head[j], xb_rem[j]);
          }
        }
      }
#pragma unroll
      for (int m = 0; m < kSlots; ++m) {
        if constexpr (kSplit) {
          // (Bt's fragment is the row operand, as in mma_block; a packed right-hand side's two reads of the pair are
          // its heads and its remainders)
          if (cur == 1) {
            if constexpr (kSplitB) {
              mma_split(acc[m / NI][m % NI], fb[0][m % NI], fb[1][m % NI], xa_head[m / NI], xa_rem[m / NI]);
            } else {
              mma_split(acc[m / NI][m % NI], xb_head[m % NI], xb_rem[m % NI], xa_head[m / NI], xa_rem[m / NI]);
            }
          }
        } else {
          mma_block<KIND>(acc[m / NI][m % NI], fb[cur][m % NI], fa[cur][m / NI]);
        }
        if (last) {
#pragma unroll
          for (int l = m; l < kLoads; l += kSlots) issue_load(l);
        }
#pragma unroll
        for (int d = m; d < MI + NI; d += kSlots) {
          if (d < MI)
            fa[nxt][d] = *(const i32x4_t*)(ra_ + d * 32 * kSlabBytes + fs);
          else
            fb[nxt][d - MI] = read_b(rb_, d - MI, fs_b);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    stage = next_stage;
    a_base = a_next;
    b_base = b_next;
  }
  // drain the (all-outside) requests still in flight before LDS is reused
  __builtin_amdgcn_s_waitcnt(0x0F70);
  // the common bf16 tails go straight from the accumulators to memory
  if constexpr (KIND == KIND_BF16 && WAVES_K == 1) {
    if (direct) {
      // (the lane number through an opaque move: the tail's addresses are then worked out here, after the K loop,
      // instead of being carried through it in registers the loop needs)
      int lane_now = lane;
      asm volatile("" : "+v"(lane_now));
      direct_tail_bf16<MI, NI>(p, acc, m0 + wm * WM, n0 + wn * WN, lane_now);
      return;
    }
  }
  __syncthreads();

  // ---- stage accumulators in LDS and run the tail ----
  // The MFMAs ran with the Bt fragment as the row operand, so in a 32x32 block a
  // lane owns tile row (m) lane%32 and the columns (n) 8*(r/4) + 4*(lane/32) + r%4:
  // four consecutive columns per register quad, one 16-byte LDS store each.
  const int crow = lane & 31;
  const int ccol = (lane >> 5) * 4;
  static_assert(WAVES_K == 1 || (size_t)BM * (BN + 4) * 4 <= (size_t)ring_t::kBytes, "partial results meet in the whole-tile buffer");
  if constexpr ((size_t)BM * (BN + 4) * 4 <= (size_t)ring_t::kBytes) {
    // the whole tile fits in the pipeline buffers: ctile[BM][BN + 4], tail by all threads
    constexpr int CS = BN + 4;
    accs_t* ctile = (accs_t*)smem;
#pragma unroll
    for (int part = 0; part < WAVES_K; ++part) {
      if (part == wk) {
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              acc4_t* dst = (acc4_t*)&ctile[(wm * WM + i * 32 + crow) * CS + wn * WN + j * 32 + 8 * g + ccol];
              acc4_t q;
#pragma unroll
              for (int e = 0; e < 4; ++e) q[e] = acc[i][j][4 * g + e];
              if (part > 0) q += *dst;  // the parts before this one are already there
              *dst = q;
            }
      }
      __syncthreads();
    }
    if constexpr (SPLITK) {
      // the partial tile as it is: four columns per thread, rows of the workspace are whole 16-byte vectors
      constexpr int TPR = BN / 4, RPP = NT / TPR;
      const int c4 = (tid % TPR) * 4;
      if (n0 + c4 < p.sk_pitch) {
        accs_t* const mine = (accs_t*)p.ws + (int64_t)split * p.M * p.sk_pitch;
#pragma unroll
        for (int row = tid / TPR; row < BM; row += RPP)
          if (m0 + row < p.M) *(acc4_t*)&mine[(m0 + row) * p.sk_pitch + n0 + c4] = *(const acc4_t*)&ctile[row * CS + c4];
      }
      return;
    }
    tile_tail<KIND, BM, BN, NT>(p, ctile, m0, n0, tid, &pre);
  } else {
    // large tiles: every wavefront stages RB of its 32-row blocks at a time in a private
    // region, wtile[RB * 32][WN + 4], and runs the tail over them with its 64 lanes
    constexpr int CS = WN + 4;
    constexpr int kBudget = ring_t::kBytes / kWaves / 16 * 16;  // bytes per wavefront
    constexpr int kFit = kBudget / (32 * CS * 4);
    constexpr int RB = kFit >= MI ? MI : (kFit >= 4 ? 4 : (kFit >= 2 ? 2 : 1));  // MI is a power of two
    static_assert(kFit >= 1, "one 32-row block of a wavefront's columns must fit its share of LDS");
    static_assert(RB >= 1 && MI % RB == 0, "row blocks must stage evenly");
    accs_t* wtile = (accs_t*)(smem + wave * kBudget);
    // (a compile-time loop: with a run-time row-block number the accumulators would be indexed
    // dynamically and live in scratch memory)
    static_for<0, MI, RB>([&](auto i0c) {
      constexpr int i0 = decltype(i0c)::value;
#pragma unroll
      for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            acc4_t q;
#pragma unroll
            for (int e = 0; e < 4; ++e) q[e] = acc[i0 + i][j][4 * g + e];
            *(acc4_t*)&wtile[(i * 32 + crow) * CS + j * 32 + 8 * g + ccol] = q;
          }
      // the staging region is private to the wavefront: its own LDS counter orders stores and reads
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      tile_tail<KIND, RB * 32, WN, 64>(p, wtile, m0 + wm * WM + i0 * 32, n0 + wn * WN, lane);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    });
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

// The same for one-byte elements without LDS: a thread takes 16 K-rows x 4 N-columns as 16 dwords,
// turns the four 4x4 byte blocks in registers (v_perm_b32) and writes 16 bytes of K to each of its four
// Bt rows.  A wavefront covers 64 x 64 elements: 64-byte runs on both sides.
// K % 16 == 0, N % 4 == 0, ldb % 4 == 0, ldbt % 16 == 0, B 4-byte and Bt 16-byte aligned.
__global__ __launch_bounds__(256) void transpose_bytes_kernel(const uint8_t* __restrict__ B, uint8_t* __restrict__ Bt,
                                                              int64_t K, int64_t N, int64_t ldb, int64_t ldbt) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t n = ((int64_t)blockIdx.x * 4 + wave) * 64 + 4 * (lane & 15);
  const int64_t k = (int64_t)blockIdx.y * 64 + 16 * (lane >> 4);
  if (n >= N || k >= K) return;
  unsigned r[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) r[i] = *(const unsigned*)(B + (k + i) * ldb + n);
  i32x4_t out[4];
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    // rows 4b .. 4b+3: t0 = {r0.0 r1.0 r0.1 r1.1}, t1 = {r0.2 r1.2 r0.3 r1.3}, t2 / t3 the same of rows 2, 3
    const unsigned t0 = __builtin_amdgcn_perm(r[4 * b + 1], r[4 * b], 0x05010400u);
    const unsigned t1 = __builtin_amdgcn_perm(r[4 * b + 1], r[4 * b], 0x07030602u);
    const unsigned t2 = __builtin_amdgcn_perm(r[4 * b + 3], r[4 * b + 2], 0x05010400u);
    const unsigned t3 = __builtin_amdgcn_perm(r[4 * b + 3], r[4 * b + 2], 0x07030602u);
    out[0][b] = (int)__builtin_amdgcn_perm(t2, t0, 0x05040100u);
    out[1][b] = (int)__builtin_amdgcn_perm(t2, t0, 0x07060302u);
    out[2][b] = (int)__builtin_amdgcn_perm(t3, t1, 0x05040100u);
    out[3][b] = (int)__builtin_amdgcn_perm(t3, t1, 0x07060302u);
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) *(i32x4_t*)(Bt + (n + j) * ldbt + k) = out[j];
}

// The same for 4-byte elements with 16-byte global accesses on both sides: a workgroup turns a 64 x 64
// tile through LDS (row stride 65 words: the transposed reads touch every bank once).
// K % 4 == 0, N % 4 == 0, ldb % 4 == 0, ldbt % 4 == 0, both pointers 16-byte aligned.
__global__ __launch_bounds__(256) void transpose_words_kernel(const uint32_t* __restrict__ B, uint32_t* __restrict__ Bt,
                                                              int64_t K, int64_t N, int64_t ldb, int64_t ldbt) {
  __shared__ uint32_t tile[64][65];
  const int c4 = (threadIdx.x & 15) * 4, r0 = threadIdx.x >> 4;
  const int64_t k0 = (int64_t)blockIdx.y * 64, n0 = (int64_t)blockIdx.x * 64;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + 16 * i;
    i32x4_t v = {0, 0, 0, 0};
    if (k0 + r < K && n0 + c4 < N) v = *(const i32x4_t*)(B + (k0 + r) * ldb + n0 + c4);
#pragma unroll
    for (int j = 0; j < 4; ++j) tile[r][c4 + j] = (uint32_t)v[j];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = r0 + 16 * i;
    if (n0 + n < N && k0 + c4 < K) {
      i32x4_t v;
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = (int)tile[c4 + j][n];
      *(i32x4_t*)(Bt + (n0 + n) * ldbt + k0 + c4) = v;
    }
  }
}

// Second pass of a K split over workgroups: a workgroup per 16 rows x 64 columns of the result, a thread per four
// columns, adds the partial tiles in split order (int32: exact whatever the order; eight loads in flight per thread)
// into the LDS layout the one-pass kernel stages its accumulators in, and runs the same tail code over it.  (The two
// passes are two launches on purpose: the partial tiles then pass from one to the other across a kernel boundary.
// Handing them over inside one launch -- an arrival count per tile, the last workgroup adds up -- was measured both
// ways it can be made coherent between the chip's L2 caches: a device-wide release and acquire around the count
// in every wavefront, 25-40 us a layer of ResNet-50 at batch 1; parts written and read as device-scope atomic
// accesses of 8 bytes, about 20 us; against 12-13 us for the two launches.)
template <int KIND>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(IgemmArgs p_by_value, int strips_n) {
  const IgemmArgs& p = *(const IgemmArgs*)(const __attribute__((address_space(4))) void*)__builtin_amdgcn_kernarg_segment_ptr();
  typedef typename Acc<KIND>::scalar accs_t;
  typedef accs_t acc4_t __attribute__((ext_vector_type(4)));
  constexpr int CS = 64 + 4;
  __shared__ __attribute__((aligned(16))) accs_t ctile[16 * CS];
  const int tid = threadIdx.x;
  const int strip_m = (int)(blockIdx.x / (unsigned)strips_n), strip_n = (int)(blockIdx.x % (unsigned)strips_n);
  const int64_t m0 = (int64_t)strip_m * 16, n0 = (int64_t)strip_n * 64;
  const int row = tid >> 4, c4 = (tid & 15) * 4;
  acc4_t sum = {0, 0, 0, 0};
  if (m0 + row < p.M && n0 + c4 < p.sk_pitch) {
    const int64_t part = (int64_t)p.M * p.sk_pitch;
    const accs_t* const at = (const accs_t*)p.ws + (m0 + row) * p.sk_pitch + n0 + c4;
    for (int sp = 0; sp < p.sk_splits; sp += 8) {
      acc4_t got[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) got[u] = sp + u < p.sk_splits ? *(const acc4_t*)(at + (sp + u) * part) : acc4_t{0, 0, 0, 0};
#pragma unroll
      for (int u = 0; u < 8; ++u) sum += got[u];
    }
  }
  *(acc4_t*)&ctile[row * CS + c4] = sum;
  __syncthreads();
  tile_tail<KIND, 16, 64, 256>(p, ctile, m0, n0, tid);
}

// The two launches of a 64 x 64 tiling whose K loop is split over workgroups (a.ws, a.sk_* prepared by the caller).
template <int KIND, bool CONV>
hipError_t launch_splitk(const IgemmArgs& a, hipStream_t s) {
  if constexpr (KIND == KIND_F32X3P) {
    return hipErrorInvalidValue;
  } else {
    const int64_t tiles_m = (a.M + 63) / 64, tiles_n = (a.N + 63) / 64;
    const int64_t tiles = tiles_m * tiles_n;
    if (tiles <= 0 || tiles * a.sk_splits >= ((int64_t)1 << 31) || a.b_kn || !a.ws || a.sk_splits < 2) return hipErrorInvalidValue;
    const size_t lds = Ring<64, 64, 0, 128>::kAlloc;
    auto kern = igemm_kernel<KIND, 64, 64, 2, CONV, kThreads, 0, 1, 128, false, true>;
    static DynamicLdsLimit limit;
    if (hipError_t e = limit.ensure((const void*)kern, lds); e != hipSuccess) return e;
    IgemmArgs b = a;
    b.order = make_tile_order((int)tiles_m, (int)tiles_n);
    b.sk_tiles = (int)tiles;
    hipLaunchKernelGGL(kern, dim3((unsigned)(tiles * a.sk_splits)), dim3(kThreads), lds, s, b);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    const int64_t strips = ((a.M + 15) / 16) * tiles_n;
    if (strips >= ((int64_t)1 << 31)) return hipErrorInvalidValue;
    hipLaunchKernelGGL(splitk_reduce_kernel<KIND>, dim3((unsigned)strips), dim3(256), 0, s, b, (int)tiles_n);
    return hipGetLastError();
  }
}

template <int KIND, int BM, int BN, int WAVES_M, bool CONV, int NT = kThreads, int STAGES = 0, int WAVES_K = 1, int SLAB = 128>
hipError_t launch_cfg(const IgemmArgs& a, hipStream_t s) {
  if constexpr ((KIND == KIND_F32 || KIND == KIND_F32X3 || KIND == KIND_I8) && !CONV && SLAB == 128 && (BN & (BN - 1)) == 0) {
    if (a.b_kn) {
      const int64_t tiles_m = (a.M + BM - 1) / BM, tiles_n = (a.N + BN - 1) / BN;
      const int64_t tiles = tiles_m * tiles_n;
      if (tiles <= 0 || tiles >= ((int64_t)1 << 31) || a.K2 > 0) return hipErrorInvalidValue;
      const size_t lds = Ring<BM, BN, STAGES, SLAB>::kAlloc;
      auto kern = igemm_kernel<KIND, BM, BN, WAVES_M, CONV, NT, STAGES, WAVES_K, SLAB, true>;
      static DynamicLdsLimit limit;
      if (hipError_t e = limit.ensure((const void*)kern, lds); e != hipSuccess) return e;
      IgemmArgs b = a;
      b.order = make_tile_order((int)tiles_m, (int)tiles_n);
      hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(NT), lds, s, b);
      return hipGetLastError();
    }
  } else {
    if (a.b_kn) return hipErrorInvalidValue;
  }
  const int64_t tiles_m = (a.M + BM - 1) / BM, tiles_n = (a.N + BN - 1) / BN;
  const int64_t tiles = tiles_m * tiles_n;
  if (tiles <= 0 || tiles >= ((int64_t)1 << 31)) return hipErrorInvalidValue;
  const size_t lds = Ring<BM, BN, STAGES, SLAB>::kAlloc;
  auto kern = igemm_kernel<KIND, BM, BN, WAVES_M, CONV, NT, STAGES, WAVES_K, SLAB>;
  static DynamicLdsLimit limit;
  if (hipError_t e = limit.ensure((const void*)kern, lds); e != hipSuccess) return e;
  IgemmArgs b = a;
  b.order = make_tile_order((int)tiles_m, (int)tiles_n);
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(NT), lds, s, b);
  return hipGetLastError();
}

template <int KIND, bool CONV>
hipError_t launch_kind(int cfg, const IgemmArgs& a, hipStream_t s) {
  switch (cfg) {
    case TILE_64x64_KSPLIT:
      if (a.ws && a.sk_splits >= 2) return launch_splitk<KIND, CONV>(a, s);
      return launch_cfg<KIND, 64, 64, 2, CONV>(a, s);  // (nothing to split, or no workspace: the plain tile)
    case TILE_64x64: return launch_cfg<KIND, 64, 64, 2, CONV>(a, s);
    case TILE_128x64: return launch_cfg<KIND, 128, 64, 2, CONV>(a, s);
    case TILE_128x128: return launch_cfg<KIND, 128, 128, 2, CONV>(a, s);
    case TILE_128x64_W8: return launch_cfg<KIND, 128, 64, 4, CONV, 512>(a, s);
    case TILE_128x128_W8: return launch_cfg<KIND, 128, 128, 2, CONV, 512>(a, s);
    case TILE_128x128_W8_S2:
      // (128 registers do not hold the split kind's fragments: it takes the one-workgroup-per-CU form)
      if constexpr (KIND == KIND_F32X3 || KIND == KIND_F32X3P) {
        return launch_cfg<KIND, 128, 128, 2, CONV, 512>(a, s);
      } else {
        return launch_cfg<KIND, 128, 128, 2, CONV, 512, 2>(a, s);
      }
    case TILE_64x64_W8_K2: return launch_cfg<KIND, 64, 64, 2, CONV, 512, 0, 2>(a, s);
    case TILE_128x64_N2:
      // four wavefronts side by side in M, each 32 rows x 64 columns: one left-hand fragment (the one that is split
      // in registers) feeds six MFMAs.  Built for the split fp32 kind only.
      if constexpr (KIND == KIND_F32X3 || KIND == KIND_F32X3P) {
        return launch_cfg<KIND, 128, 64, 4, CONV>(a, s);
      } else {
        return launch_cfg<KIND, 128, 64, 2, CONV>(a, s);
      }
    case TILE_192x384_W8:
      // eight wavefronts of 96 x 96 (2 x 4): per MFMA half the global -> LDS bytes of a 128 x 128 tile and 0.67 KB of
      // fragment reads; 144 accumulation registers per lane, so 16- and 8-bit elements only
      if constexpr (KIND == KIND_BF16 || KIND == KIND_I8) {
        return launch_cfg<KIND, 192, 384, 2, CONV, 512, 2>(a, s);
      } else {
        return launch_cfg<KIND, 128, 128, 2, CONV, 512>(a, s);
      }
    case TILE_256x128_W16:
    case TILE_256x256_W8:
      // (the split fp32 kind keeps heads and remainders of every fragment in registers beside the raw values:
      // the largest tiles are not built for it)
      if constexpr (KIND == KIND_F32X3 || KIND == KIND_F32X3P) {
        return launch_cfg<KIND, 128, 128, 2, CONV, 512>(a, s);
      } else {
        if (cfg == TILE_256x128_W16) return launch_cfg<KIND, 256, 128, 4, CONV, 1024>(a, s);
        return launch_cfg<KIND, 256, 256, 2, CONV, 512>(a, s);
      }
  }
  return hipErrorInvalidValue;
}

}  // namespace

#ifndef PML_KIND
#error "compile with -DPML_KIND=0|1|2|3|4 (fp32 | bf16 | int8 | fp32 as three bf16 products | the same, right-hand side split when packed); -DPML_KIND=0 also emits the shared entry points"
#endif

// One translation unit per element kind keeps each compile short and lets make run them in parallel.
hipError_t PML_CAT(igemm_launch_kind_, PML_KIND)(int cfg, bool conv, const IgemmArgs& a, hipStream_t s) {
  return conv ? launch_kind<PML_KIND, true>(cfg, a, s) : launch_kind<PML_KIND, false>(cfg, a, s);
}

#if PML_KIND == 1
// Measurement aid, not part of any contraction: what the matrix cores sustain on operands that never leave LDS
// (no global traffic, no barriers), 8 wavefronts per CU with 128x64 tiles' instruction mix -- 8 MFMAs and 6
// fragment reads per K-block.  With `random` the LDS holds random bf16 values of magnitude about 1, otherwise a
// constant: the difference is what the switching activity of real data costs in clock frequency, i.e. the ceiling
// a GEMM on N(0,1) data can reach on this device.  clk[0]: core clock ticks, clk[1]: 100 MHz ticks.
__global__ __launch_bounds__(512) void mfma_probe_kernel(int iters, int random, float* sink, unsigned long long* clk) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  for (int o = tid * 4; o < 128 * 1024; o += 512 * 4) {
    unsigned h = (o + blockIdx.x * 7919u) * 2654435761u;
    h ^= h >> 15;
    h *= 2246822519u;
    h ^= h >> 13;
    const unsigned lo = (h & 0x807f) | (0x3f00 + ((h >> 8) & 0x0180)), hi = ((h >> 16) & 0x807f) | (0x3f00 + ((h >> 24) & 0x0180));
    *(unsigned*)(smem + o) = random ? (lo | (hi << 16)) : 0x3f803f80u;
  }
  __syncthreads();
  unsigned long long t0 = 0, r0 = 0;
  if (tid == 0 && blockIdx.x == 0) {
    t0 = __builtin_amdgcn_s_memtime();
    r0 = __builtin_amdgcn_s_memrealtime();
  }
  f32x16_t acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  i32x4_t fa[2][4], fb[2][2];
  const unsigned char* base = smem + (wave & 3) * 16384 + ((lane & 31) * 128) + (((lane >> 5) ^ ((lane >> 1) & 7)) * 16);
#pragma unroll
  for (int i = 0; i < 4; ++i) fa[0][i] = *(const i32x4_t*)(base + i * 4096);
#pragma unroll
  for (int j = 0; j < 2; ++j) fb[0][j] = *(const i32x4_t*)(base + 65536 + j * 4096);
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      const int cur = kb & 1, nxt = cur ^ 1;
#pragma unroll
      for (int m = 0; m < 8; ++m) {
        mma_block<KIND_BF16>(acc[m / 2][m % 2], fb[cur][m % 2], fa[cur][m / 2]);
        if (m < 4) fa[nxt][m] = *(const i32x4_t*)(base + m * 4096 + (it & 1) * 64);
        else if (m < 6) fb[nxt][m - 4] = *(const i32x4_t*)(base + 65536 + (m - 4) * 4096 + (it & 1) * 64);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  if (tid == 0 && blockIdx.x == 0) {
    clk[0] = __builtin_amdgcn_s_memtime() - t0;
    clk[1] = __builtin_amdgcn_s_memrealtime() - r0;
  }
  float total = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) total += acc[i][j][e];
  if (total == 123.456f) sink[0] = total;  // keeps the accumulators alive
}

// MFMAs (32x32x16 bf16) issued by one launch of `iters` rounds on `blocks` workgroups.
hipError_t mfma_probe_launch(int blocks, int iters, int random, float* sink, unsigned long long* clk, hipStream_t s) {
  static DynamicLdsLimit limit;
  if (hipError_t e = limit.ensure((const void*)mfma_probe_kernel, 128 * 1024); e != hipSuccess) return e;
  hipLaunchKernelGGL(mfma_probe_kernel, dim3((unsigned)blocks), dim3(512), 128 * 1024, s, iters, random, sink, clk);
  return hipGetLastError();
}
#endif

#if PML_KIND == 0
hipError_t igemm_launch(int kind, int cfg, bool conv, const IgemmArgs& a, hipStream_t s) {
  // the kernel addresses both operands with 32-bit byte offsets below 2 GiB
  const int64_t es = kind == KIND_BF16 ? 2 : (kind == KIND_I8 ? 1 : 4);
  const int64_t a_bytes = conv ? (int64_t)a.NB * a.H * a.W * (a.pix_pitch ? a.pix_pitch : a.CI * es) + 256 : a.M * a.lda * es;
  const int64_t b_bytes = a.N * a.ldbt * es;
  if (a_bytes >= ((int64_t)1 << 31) || b_bytes >= ((int64_t)1 << 31) || (conv && a.M >= ((int64_t)1 << 31))) return hipErrorInvalidValue;
  switch (kind) {
    case KIND_F32: return igemm_launch_kind_0(cfg, conv, a, s);
    case KIND_BF16: return igemm_launch_kind_1(cfg, conv, a, s);
    case KIND_I8: return igemm_launch_kind_2(cfg, conv, a, s);
    case KIND_F32X3: return igemm_launch_kind_3(cfg, conv, a, s);
    case KIND_F32X3P: return igemm_launch_kind_4(cfg, conv, a, s);
  }
  return hipErrorInvalidValue;
}

// In place, per 32 fp32 values (128 bytes) of a row: their 32 bf16 heads (round to nearest even), then the 32 bf16
// remainders (the rounded differences) -- the form the split fp32 kind reads a packed right-hand side in.
__global__ __launch_bounds__(256) void split_rows_kernel(float* bt, int64_t rows, int64_t ld, int64_t chunks_per_row) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= rows * chunks_per_row) return;
  i32x4_t* at = (i32x4_t*)(bt + (t / chunks_per_row) * ld + (t % chunks_per_row) * 32);
  i32x4_t raw[8], head[4], rem[4];
#pragma unroll
  for (int u = 0; u < 8; ++u) raw[u] = at[u];
#pragma unroll
  for (int u = 0; u < 4; ++u) split_f32x8(raw[2 * u], raw[2 * u + 1], head[u], rem[u]);
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    at[u] = head[u];
    at[4 + u] = rem[u];
  }
}

hipError_t split_rows_launch(void* bt, int64_t rows, int64_t ld, int64_t k, hipStream_t s) {
  if (k % 32 != 0 || ld % 4 != 0 || ((uintptr_t)bt & 15) != 0) return hipErrorInvalidValue;
  const int64_t chunks = k / 32, total = rows * chunks;
  hipLaunchKernelGGL(split_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, (float*)bt, rows, ld, chunks);
  return hipGetLastError();
}

hipError_t transpose_pack(int elem_size, const void* B, void* Bt, int64_t K, int64_t N, int64_t ldb, int64_t ldbt,
                          hipStream_t s) {
  dim3 grid((unsigned)((N + 63) / 64), (unsigned)((K + 63) / 64));
  switch (elem_size) {
    case 1:
      if (K % 16 == 0 && N % 4 == 0 && ldb % 4 == 0 && ldbt % 16 == 0 && ((uintptr_t)B & 3) == 0 && ((uintptr_t)Bt & 15) == 0) {
        dim3 grid_b((unsigned)((N + 255) / 256), (unsigned)((K + 63) / 64));
        hipLaunchKernelGGL(transpose_bytes_kernel, grid_b, dim3(256), 0, s, (const uint8_t*)B, (uint8_t*)Bt, K, N, ldb, ldbt);
        break;
      }
      hipLaunchKernelGGL(transpose_kernel<uint8_t>, grid, dim3(256), 0, s, (const uint8_t*)B, (uint8_t*)Bt, K, N, ldb, ldbt);
      break;
    case 2:
      hipLaunchKernelGGL(transpose_kernel<uint16_t>, grid, dim3(256), 0, s, (const uint16_t*)B, (uint16_t*)Bt, K, N, ldb, ldbt);
      break;
    case 4:
      if (K % 4 == 0 && N % 4 == 0 && ldb % 4 == 0 && ldbt % 4 == 0 && (((uintptr_t)B | (uintptr_t)Bt) & 15) == 0) {
        hipLaunchKernelGGL(transpose_words_kernel, grid, dim3(256), 0, s, (const uint32_t*)B, (uint32_t*)Bt, K, N, ldb, ldbt);
        break;
      }
      hipLaunchKernelGGL(transpose_kernel<uint32_t>, grid, dim3(256), 0, s, (const uint32_t*)B, (uint32_t*)Bt, K, N, ldb, ldbt);
      break;
    default:
      return hipErrorInvalidValue;
  }
  return hipGetLastError();
}
#endif  // PML_KIND == 0

}  // namespace pml
