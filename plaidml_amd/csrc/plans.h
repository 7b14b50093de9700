// Internal: kernel argument blocks, plan records and launcher prototypes shared
// by the C ABI (pml_hip.hip) and the kernel translation units.
#pragma once

#include <hip/hip_runtime.h>

#include <mutex>
#include <stdint.h>

#include <string>

#include "pml_hip.h"

namespace pml {

// The dynamic-LDS ceiling of a kernel (hipFuncAttributeMaxDynamicSharedMemorySize) belongs to the kernel on one
// device.  One of these per kernel instantiation remembers, per device, the largest size already set.
struct DynamicLdsLimit {
  std::mutex lock;
  size_t set[32] = {};
  hipError_t ensure(const void* kernel, size_t bytes) {
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
    std::lock_guard<std::mutex> hold(lock);
    size_t& have = set[dev & 31];
    if (bytes <= have) return hipSuccess;
    if (hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes); e != hipSuccess) return e;
    have = bytes;
    return hipSuccess;
  }
};


// KIND_F32X3: fp32 operands in memory and in LDS, each split in registers into a bf16 head and a bf16 remainder and
// multiplied as three bf16 products (head x head + remainder x head + head x remainder), fp32 accumulation
// KIND_F32X3P: the same with a right-hand side that was split when it was packed (per 32 K-values of a row of Bt:
// their 32 bf16 heads, then their 32 bf16 remainders), so that only the left-hand fragments are split in registers
enum { KIND_F32 = 0, KIND_BF16 = 1, KIND_I8 = 2, KIND_F32X3 = 3, KIND_F32X3P = 4 };
// _W8 / _W16: eight / sixteen wavefronts per workgroup (two / four per SIMD) instead of four; _S2: two ring stages; _K2: two wavefront grids share the K-blocks of every slab
enum { TILE_64x64 = PML_HIP_TILE_64x64, TILE_128x64 = PML_HIP_TILE_128x64, TILE_128x128 = PML_HIP_TILE_128x128, TILE_128x64_W8 = PML_HIP_TILE_128x64_W8,
       TILE_128x128_W8 = PML_HIP_TILE_128x128_W8, TILE_256x128_W16 = PML_HIP_TILE_256x128_W16, TILE_128x128_W8_S2 = PML_HIP_TILE_128x128_W8_S2,
       TILE_64x64_W8_K2 = PML_HIP_TILE_64x64_W8_K2, TILE_256x256_W8 = PML_HIP_TILE_256x256_W8, TILE_128x64_N2 = PML_HIP_TILE_128x64_N2,
       TILE_192x384_W8 = PML_HIP_TILE_192x384_W8, TILE_64x64_KSPLIT = PML_HIP_TILE_64x64_KSPLIT };

struct TailPtrs {
  const void* operands[PML_HIP_MAX_EPI_OPERANDS];
  void* outs[PML_HIP_MAX_EPI_OPERANDS];
};

// Arguments of the MFMA GEMM / implicit-GEMM kernel (passed by value).
// n / d for n < 2^31 as one 32x32 -> 64 multiply and a shift, with a pair (magic, shift) made on the host
inline void fast_div_magic(unsigned d, unsigned* magic, int* shift) {
  int l = 0;
  while ((1ull << l) < d) ++l;
  *shift = 31 + l;
  *magic = (unsigned)(((1ull << (31 + l)) + d - 1) / d);
}
#if defined(__HIPCC__)
__device__ inline unsigned fast_div(unsigned n, unsigned magic, int shift) {
  return (unsigned)(((unsigned long long)n * magic) >> shift);
}
#endif

// XCD-aware tile order of the GEMM grid, prepared on the host so that a workgroup finds its tile with a few
// scalar multiplies (the divisions by run-time grid sizes took about 150 vector instructions per wavefront).
// Hardware deals consecutive workgroup ids round-robin to the 8 XCDs, each with its own L2, and a CU takes the next
// id of its XCD when it falls free: the workgroups resident on an XCD at any time are a run of about 32 consecutive
// "local" numbers bid / 8.  What such a run costs the L2 is the number of distinct A rows plus Bt rows under its
// tiles, so a run should be a compact block, not a strip, and above all the tiles that share an A row block must
// not be dealt to eight different L2s (a 181 x 6 grid in workgroup-id order fetched A 6.5 times from memory).
// XCD x therefore owns a contiguous range of tile numbers t (the ranges differ by at most one tile when the count
// is no multiple of 8), and t walks the grid in blocks of th x tw tiles (32 tiles, as square as the grid allows).
// When the grid divides into whole blocks, blocks are numbered row-major and walked row-major; otherwise t walks
// groups of th tile rows column by column, the last group being as short as the grid leaves it.  (4096^2 with
// 256x256 tiles: 2 x 16 strips fetch 576 KB per K-slab and XCD, 4 x 8 blocks 384 KB; what misses L2 comes over the
// fabric from the last-level cache, whose bandwidth is the scarce one.)
struct TileOrder {
  int per, rem;                    // tiles per XCD; the first `rem` XCDs take one more
  int blocked;                     // 1: whole th x tw blocks (tw a power of two), 0: groups of th tile rows
  int th, tw_shift, blocks_n;      // blocked
  int group, last_rows, tiles_m;   // grouped: tiles in a full group, tile rows of the last group
  unsigned bn_magic, group_magic, th_magic, last_magic;
  int bn_shift, group_shift, th_shift, last_shift;
};
inline TileOrder make_tile_order(int tiles_m, int tiles_n) {
  constexpr int kXcds = 8, kRun = 32;
  TileOrder o{};
  const int nblocks = tiles_m * tiles_n;
  o.per = nblocks / kXcds;
  o.rem = nblocks % kXcds;
  o.tiles_m = tiles_m;
  int th = 0, tw = 0;
  if (o.rem == 0 && o.per % kRun == 0) {
    if (tiles_m % 4 == 0 && tiles_n % 8 == 0) { th = 4; tw = 8; }
    else if (tiles_m % 8 == 0 && tiles_n % 4 == 0) { th = 8; tw = 4; }
    else if (tiles_m % 16 == 0 && tiles_n % 2 == 0) { th = 16; tw = 2; }
    else if (tiles_m % 2 == 0 && tiles_n % 16 == 0) { th = 2; tw = 16; }
  }
  if (th) {
    o.blocked = 1;
    o.th = th;
    while ((1 << o.tw_shift) < tw) ++o.tw_shift;
    o.blocks_n = tiles_n / tw;
    fast_div_magic((unsigned)o.blocks_n, &o.bn_magic, &o.bn_shift);
    return o;
  }
  tw = tiles_n < 8 ? tiles_n : 8;
  o.th = kRun / tw;
  o.group = o.th * tiles_n;
  o.last_rows = tiles_m % o.th ? tiles_m % o.th : o.th;
  fast_div_magic((unsigned)o.group, &o.group_magic, &o.group_shift);
  fast_div_magic((unsigned)o.th, &o.th_magic, &o.th_shift);
  fast_div_magic((unsigned)o.last_rows, &o.last_magic, &o.last_shift);
  return o;
}
#if defined(__HIPCC__)
__host__ __device__
#endif
inline void tile_of(const TileOrder& o, unsigned bid, int* tm, int* tn) {
  const unsigned x = bid & 7u;
  const unsigned t = x * (unsigned)o.per + (x < (unsigned)o.rem ? x : (unsigned)o.rem) + (bid >> 3);
  auto div = [](unsigned n, unsigned magic, int shift) { return (unsigned)(((unsigned long long)n * magic) >> shift); };
  if (o.blocked) {
    const unsigned blk = t >> 5, in = t & 31u;
    const unsigned q = div(blk, o.bn_magic, o.bn_shift), r = blk - q * (unsigned)o.blocks_n;
    *tm = (int)(q * (unsigned)o.th + (in >> o.tw_shift));
    *tn = (int)((r << o.tw_shift) + (in & ((1u << o.tw_shift) - 1u)));
    return;
  }
  const unsigned gi = div(t, o.group_magic, o.group_shift), in = t - gi * (unsigned)o.group;
  const unsigned first_m = gi * (unsigned)o.th;
  const bool last = (unsigned)o.tiles_m - first_m < (unsigned)o.th;
  const unsigned rows = last ? (unsigned)o.last_rows : (unsigned)o.th;
  const unsigned q = last ? div(in, o.last_magic, o.last_shift) : div(in, o.th_magic, o.th_shift);
  *tm = (int)(first_m + in - q * rows);
  *tn = (int)q;
}

struct IgemmArgs {
  TileOrder order;  // filled in by the launcher for the tile grid of the configuration it launches
  int b_kn;         // 1: Bt / ldbt are the caller's row-major B[K][N] and its row length (fp32 and int8 GEMMs)
  // conv_blocks4x4_kernel only: the caller's NHWC image of 3 bf16 channels (raw_h x raw_w pixels, raw_w even), from
  // which the kernel builds the rows of 2x2 pixel blocks itself; null: A already holds the re-blocked image
  const void* raw_in;
  int raw_h, raw_w;
  int64_t M, N, K;
  const void* A;
  int64_t lda;
  const void* Bt;  // [N][K], K contiguous
  int64_t ldbt;
  void* C;
  int64_t ldc;
  // convolution geometry (CONV instantiations only)
  int H, W, CI, OH, OW, KH, KW, SH, SW, PH, PW, DH, DW;
  // bytes between consecutive input pixels; 0 = CI * element size.  Smaller than that when the "channel
  // vector" of a tap spans several pixels (igemm_kernel only)
  int pix_pitch;
  // resident-filter convolution only: image count, LDS rows of the input window, number of 256-pixel tiles
  // halo_variant: 0 = general resident kernel, 1 / 2 = pipelined 3x3 kernel with that many 32-pixel chunks per row
  // b_raw: 1 = Bt points at the caller's [K][N] matrix instead of the packed [N][K] one (pipelined kernels only);
  //        2 = Bt points at the filter in register order (the register-filter kernel only; regfilter_image_launch)
  int NB, halo_rows, n_tiles, halo_variant, b_raw;
  int n_cus;  // compute units of the device (persistent grids)
  // n / (OH*OW) and n / OW as multiply-and-shift (see fast_div); set for every convolution
  unsigned div_per_magic, div_ow_magic;
  int div_per_shift, div_ow_shift;
  // result type of the contraction, optional initial value
  int out_dtype;
  const void* init;
  int init_dtype;
  int64_t init_rs, init_cs;
  // fast tail: 0 = interpret `tail`; 1 = (optional relu) then store as c_dtype
  int tail_mode;
  int tail_relu;
  int tail_ssr;  // tail_mode 3 only: 1 = result * column vector + column vector, 2 = the same and relu (all in the bf16 result type)
  // tail_mode 4 only: 1 = the chain is exactly a requantisation -- (store the si32 sum to outs[rq_store])? cast f32,
  // * operands[rq_scale] (one f32 per column, or a single one), lower clamp rq_lo (v > lo ? v : lo), upper clamp rq_hi
  // (v < hi ? v : hi), round half away from zero, cast si8 -- which the tail then runs as straight code
  int tail_rq, rq_store, rq_scale;
  float rq_lo, rq_hi;
  // K split over workgroups (TILE_64x64_KSPLIT): the workspace of partial tiles [sk_splits][M][sk_pitch] (accumulator
  // type), slabs per split, and -- filled in by the launcher -- the number of result tiles
  void* ws;
  int sk_splits, sk_per, sk_pitch, sk_tiles;
  int c_dtype;
  pml_hip_epilogue tail;
  const void* operands[PML_HIP_MAX_EPI_OPERANDS];
  void* outs[PML_HIP_MAX_EPI_OPERANDS];
  // A second product summed into the same result, C = A . Bt^T + A2 . Bt2^T (GEMM instantiations only; K2 = 0: none).
  // Row m of A2 starts at element lda2 * m, or, with g2_stride > 0, at the pixel the output pixel m reads in an
  // NHWC image walked with that stride (a 1x1 convolution): ((n * g2_h + oy * stride) * g2_w + ox * stride) * lda2
  // with n, oy, ox from m by g2_ohw / g2_ow.  init2: a second per-column initial value of the result type or null.
  const void* A2;
  const void* Bt2;
  const void* init2;
  int64_t K2, lda2, ldbt2;
  int g2_stride, g2_h, g2_w, g2_ohw, g2_ow;
  unsigned g2_ohw_magic, g2_ow_magic;
  int g2_ohw_shift, g2_ow_shift;
  // conv_blocks4x4_w8_kernel only: pool = 1 applies a 3x3 stride-2 max-pool to the convolution's rows before they leave the
  // chip -- C is then the pooled tensor [NB][pool_oh][pool_ow][N], pooled pixel (y, x) covering result rows 2y - pool_pt ..
  // + 2 and columns 2x - pool_pl .. + 2 as far as they exist
  int pool, pool_oh, pool_ow, pool_pt, pool_pl;
};

hipError_t igemm_launch(int kind, int cfg, bool conv, const IgemmArgs& a, hipStream_t s);
// How TILE_64x64_KSPLIT shares the K loop out: slabs of 128 bytes of K in all, and for a device of n_cus compute units
// the number of splits (1: not worth splitting) with the slabs each takes -- about one workgroup per CU, at least two
// slabs per split, at most 16 splits.
inline int64_t igemm_slabs(const IgemmArgs& a, bool conv, int es) {
  return conv ? (int64_t)a.KH * a.KW * (((int64_t)a.CI * es + 127) / 128) : (a.K * es + 127) / 128;
}
inline void igemm_split_plan(int64_t m, int64_t n, int64_t slabs, int n_cus, int* splits, int* per) {
  const int64_t tiles = ((m + 63) / 64) * ((n + 63) / 64);
  int64_t want = tiles > 0 ? ((int64_t)n_cus + tiles - 1) / tiles : 1;
  if (want > 16) want = 16;
  if (want > slabs / 2) want = slabs / 2;
  if (want < 2) {
    *splits = 1;
    *per = (int)slabs;
    return;
  }
  *per = (int)((slabs + want - 1) / want);
  *splits = (int)((slabs + *per - 1) / *per);  // every split has work
}
// Resident-filter convolution (conv_halo.hip): LDS bytes a shape needs, or 0 when the
// shape does not qualify; `a.halo_rows` and `a.n_tiles` are filled in by conv_halo_prepare.
size_t conv_halo_prepare(int kind, IgemmArgs* a, bool filter_in_lds = false);
hipError_t conv_halo_launch(int kind, const IgemmArgs& a, size_t lds_bytes, int n_cus, hipStream_t s);
// The packed 3x3 filter Bt[64][ldbt] of the register-filter kernel (halo_variant 3) re-laid into the order that kernel
// keeps it in registers: kRegfilterImageBytes bytes at `image`.
constexpr size_t kRegfilterImageBytes = 2 * 36 * 64 * 16;
hipError_t regfilter_image_launch(const void* bt, int64_t ldbt_bytes, void* image, hipStream_t s);
bool regfilter_takes_image(int ow);  // rows of `ow` output pixels leave the image room in LDS (otherwise the packed Bt is used)
// The re-blocked few-channel convolution with 4x4 block taps of 16 channels and 64 output channels: LDS bytes of the
// row-walking kernel, or 0 when `a` (already pointing at the re-blocked input) does not qualify.
size_t conv_blocks4x4_prepare(int kind, const IgemmArgs& a);
hipError_t conv_blocks4x4_launch(const IgemmArgs& a, size_t lds_bytes, int n_cus, hipStream_t s);
hipError_t mfma_probe_launch(int blocks, int iters, int random, float* sink, unsigned long long* clk, hipStream_t s);
// splits a packed fp32 Bt[rows][ld] in place (k values per row, a multiple of 32) into the heads / remainders form
hipError_t split_rows_launch(void* bt, int64_t rows, int64_t ld, int64_t k, hipStream_t s);
hipError_t transpose_pack(int elem_size, const void* B, void* Bt, int64_t K, int64_t N, int64_t ldb, int64_t ldbt,
                          hipStream_t s);

// generic kernels (generic.hip)
struct ContractArgs {
  pml_hip_contract_desc d;
  const void* srcs[3];
  void* out;
};
hipError_t contract_launch(const ContractArgs& a, hipStream_t s);

struct EltwiseArgs {
  pml_hip_eltwise_desc d;
  const void* in;
  void* out;
  const void* operands[PML_HIP_MAX_EPI_OPERANDS];
  void* outs[PML_HIP_MAX_EPI_OPERANDS];
  int64_t total;
  int wide;  // 1: some element type needs the (double, int64) interpreter
};
hipError_t eltwise_launch(const EltwiseArgs& a, hipStream_t s);
hipError_t select_launch(const pml_hip_select_desc& d, const void* c, const void* t, const void* f, void* out,
                         hipStream_t s);
hipError_t index_launch(void* out, int rank, const int64_t* sizes, int axis, hipStream_t s);
hipError_t fill_u32_launch(void* p, uint32_t pattern, size_t n_words, hipStream_t s);
hipError_t softmax_launch(const pml_hip_softmax_desc& d, const void* x, void* y, hipStream_t s);

// special operations (special.hip)
hipError_t gather_launch(const pml_hip_gather_desc& d, const void* tensor, const void* indices, void* out, hipStream_t s);
hipError_t scatter_launch(const pml_hip_scatter_desc& d, const void* data, const void* indices, const void* updates, void* out,
                          hipStream_t s);
hipError_t argsort_launch(const pml_hip_argsort_desc& d, const void* tensor, void* out, hipStream_t s);
hipError_t prng_launch(const void* state, int64_t count, void* values, void* new_state, hipStream_t s);

// window kernels (window.hip)
struct DwconvArgs {
  pml_hip_dwconv2d_desc d;
  const void* in;
  const void* filter;
  void* out;
  const void* operands[PML_HIP_MAX_EPI_OPERANDS];
  void* outs[PML_HIP_MAX_EPI_OPERANDS];
  // a 3x3 bf16 filter of finite weights packed once with the taps of rows 0 and 1 paired (dwconv2d_pair_filter), or null
  const void* paired_filter;
  int n_cus;  // compute units of the device (the paired kernel sizes its grid by it)
};
hipError_t dwconv2d_launch(const DwconvArgs& a, hipStream_t s);
bool dwconv2d_takes_paired_filter(const pml_hip_dwconv2d_desc& d);
bool dwconv2d_walks_rows(const pml_hip_dwconv2d_desc& d, int n_cus, int64_t* ysegs, int64_t* seg_rows);
bool dwconv2d_pair_filter(const uint16_t* filter, int64_t c, uint32_t* packed);
struct Im2colArgs {
  const void* in;
  void* out;
  int64_t M;  // N * OH * OW rows
  int K, kpad;  // KH*KW*CI real columns, row length (a multiple of the 16-byte vector)
  int H, W, CI, OH, OW, KH, KW, SH, SW, PH, PW, DH, DW;
};
hipError_t im2col_launch(int elem_size, const Im2colArgs& a, hipStream_t s);
// Stride-2 convolution over few channels as a unit-stride one over 2x2 pixel blocks ("space to depth").
//   ih = 2*oh + kh - PH  with  kh + eh = 2*a + b  (eh = PH & 1)   ->   ih = 2*(oh + a - (PH + eh)/2) + b
// and likewise in w.  S[n][r][c][(b*2 + bw)*CI + ci] = I[n][2r + b][2c + bw][ci] (zero past the image,
// channels padded to CH); the filter becomes G[co][a][aw][(b*2 + bw)*CI + ci] = F[2a + b - eh][2aw + bw - ew][ci][co].
struct S2dArgs {
  const void* in;      // [N][H][W][CI]
  void* out;           // [N][HS][WS][CH]
  const void* filter;  // [KH][KW][CI][CO]  (filter kernel only)
  void* gt;            // [CO][KA][KAW][CH] (filter kernel only)
  int N, H, W, CI, HS, WS, CH, KH, KW, CO, KA, KAW, EH, EW;
};
hipError_t s2d_input_launch(int elem_size, const S2dArgs& a, hipStream_t s);
hipError_t s2d_filter_launch(int elem_size, const S2dArgs& a, hipStream_t s);
struct PoolArgs {
  pml_hip_pool2d_desc d;
  const void* in;
  void* out;
  void* idx;
};
hipError_t pool2d_launch(const PoolArgs& a, hipStream_t s);

}  // namespace pml
