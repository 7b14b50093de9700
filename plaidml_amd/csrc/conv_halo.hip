// 2-D convolution with the whole filter resident in LDS (unit stride, unit dilation).
//
// A persistent workgroup (one per CU, 256 threads = 4 wavefronts) keeps the packed
// filter Bt[CO][KH*KW*CI] in LDS for its whole life and walks over tiles of 256
// consecutive output pixels.  For each tile the input window that the tile's
// pixels touch is brought into LDS once, zero padding included, so that every one
// of the KH*KW taps reads its operand from LDS at a fixed offset from the pixel's
// own position: no per-tap address checks, and each input byte crosses the
// vector L1 once per tile instead of once per tap.  The window of the next tile
// travels global -> registers while the MFMAs of the current one run.
//
// LDS window addressing.  Images are stacked with their padding rows materialised:
// virtual row v = image * (H + pad_top + pad_bottom) + (ih + pad_top), virtual
// column = iw + pad_left, so output pixel (image, oh, ow) and tap (kh, kw) read
// virtual pixel (image * Hv + oh + kh, ow + kw).  A tile that runs across the end
// of an image simply holds the padding rows between the two.
//
// Every pixel is 128 bytes of channels (CI * element size), stored with a 144-byte
// stride; filter rows use an odd number of 16-byte slots too.  Both strides make
// the 16-byte-per-lane operand reads free of bank conflicts.
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <string>
#include <type_traits>

#include "device_common.h"
#include "igemm_tail.h"
#include "plans.h"

namespace pml {
namespace {

constexpr int kThreads = 256;
constexpr int kBM = 256;          // output pixels per tile (64 per wavefront)
constexpr int kBN = 64;           // output channels covered (CO <= 64)
constexpr int kPixBytes = 128;    // channel bytes per pixel
constexpr int kPixStride = 144;   // LDS stride of a pixel
constexpr int kMaxLoads = 24;     // 16-byte window vectors a thread may carry for the next tile

// Workgroup ids are dealt round-robin to the 8 XCDs (one L2 each).  Give every XCD a contiguous run
// of the tiles worked on at the same time, so the window rows two neighbouring tiles share are
// fetched from HBM once and found in that L2 by the other.
__device__ inline int first_tile(int bid, int nblocks) {
  constexpr int kXcds = 8;
  if (nblocks % kXcds != 0) return bid;
  return (bid % kXcds) * (nblocks / kXcds) + bid / kXcds;
}

struct TileGeom {
  int64_t m0;   // first output pixel
  int v0;       // virtual row of that pixel
  int nb0;      // its image
  int ihv0;     // its row inside the padded image (= oh)
  int nrows;    // window rows of the tile
};


__device__ inline TileGeom tile_geom(const IgemmArgs& p, int t, int Hv) {
  TileGeom g;
  // pixel numbers stay below 2^31 (checked on the host)
  const unsigned m0 = (unsigned)t * kBM;
  const unsigned per = (unsigned)(p.OH * p.OW);
  const unsigned nb = fast_div(m0, p.div_per_magic, p.div_per_shift);
  const unsigned oh = fast_div(m0 - nb * per, p.div_ow_magic, p.div_ow_shift);
  g.m0 = m0;
  g.nb0 = (int)nb;
  g.ihv0 = (int)oh;
  g.v0 = (int)(nb * Hv + oh);
  unsigned ml = m0 + kBM - 1;
  if (ml > (unsigned)p.M - 1) ml = (unsigned)p.M - 1;
  const unsigned nbl = fast_div(ml, p.div_per_magic, p.div_per_shift);
  const unsigned ohl = fast_div(ml - nbl * per, p.div_ow_magic, p.div_ow_shift);
  g.nrows = (int)(nbl * Hv + ohl) - g.v0 + p.KH;
  return g;
}

template <int KIND>
__global__ __launch_bounds__(kThreads) void conv_halo_kernel(IgemmArgs p) {
  constexpr int ES = KIND == KIND_BF16 ? 2 : (KIND == KIND_I8 ? 1 : 4);
  constexpr int MI = 2, NI = 2;  // 64 pixels x 64 channels per wavefront
  typedef typename Acc<KIND>::type acc_t;
  typedef typename Acc<KIND>::scalar accs_t;
  typedef accs_t acc4_t __attribute__((ext_vector_type(4)));

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int Hv = p.OH + p.KH - 1, Wv = p.OW + p.KW - 1;
  const int krow = p.KH * p.KW * kPixBytes;  // filter bytes per output channel
  const int brow = krow + 16;                // its LDS stride
  unsigned char* const sB = smem;
  unsigned char* const sH = smem + kBN * brow;

  // ---- filter -> LDS, once ----
  {
    const int vecs_per_row = krow / 16;
    const int total = kBN * vecs_per_row;
    const i32x4_t zero4 = {0, 0, 0, 0};
    for (int q = tid; q < total; q += kThreads) {
      const int row = q / vecs_per_row, vec = q - row * vecs_per_row;
      i32x4_t v = zero4;
      if (row < p.N) v = *(const i32x4_t*)((const unsigned char*)p.Bt + (int64_t)row * p.ldbt * ES + vec * 16);
      *(i32x4_t*)(sB + row * brow + vec * 16) = v;
    }
  }

  // ---- a thread's share of a window: vector lv of pixels lp, lp + 32, ... of every row ----
  const int lv = tid & 7, lp = tid >> 3;
  const int nchunks = (Wv + 31) >> 5;
  i32x4_t pf[kMaxLoads];
  unsigned pf_ok = 0;  // bit j: pf[j] is real data (otherwise the window gets zeros: padding)
  const i32x4_t zero4 = {0, 0, 0, 0};

  auto load_window = [&](const TileGeom& g) {
    int r = 0, c = 0, nb = g.nb0, ihv = g.ihv0;
    pf_ok = 0;
#pragma unroll
    for (int j = 0; j < kMaxLoads; ++j) {
      const int ih = ihv - p.PH;
      const int px = c * 32 + lp;
      const int iw = px - p.PW;
      const bool ok = r < g.nrows && nb < p.NB && (unsigned)ih < (unsigned)p.H && px < Wv && (unsigned)iw < (unsigned)p.W;
      const int64_t off = ok ? ((int64_t)(nb * p.H + ih) * p.W + iw) * kPixBytes + lv * 16 : 0;
      pf[j] = *(const i32x4_t*)((const unsigned char*)p.A + off);
      pf_ok |= (ok ? 1u : 0u) << j;
      if (++c == nchunks) {
        c = 0;
        ++r;
        if (++ihv == Hv) {
          ihv = 0;
          ++nb;
        }
      }
    }
  };
  auto store_window = [&](const TileGeom& g) {
    int r = 0, c = 0;
#pragma unroll
    for (int j = 0; j < kMaxLoads; ++j) {
      const int px = c * 32 + lp;
      if (r < g.nrows && px < Wv)
        *(i32x4_t*)(sH + (r * Wv + px) * kPixStride + lv * 16) = ((pf_ok >> j) & 1u) ? pf[j] : zero4;
      if (++c == nchunks) {
        c = 0;
        ++r;
      }
    }
  };

  // bias: the values of the output channels this lane owns (direct store path)
  const bool direct = p.tail_mode == 1 && (p.init == nullptr || p.init_rs == 0);
  accs_t cinit[NI][4][4];
#pragma unroll
  for (int j = 0; j < NI; ++j)
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        cinit[j][g][e] = 0;
        const int co = j * 32 + 8 * g + 4 * (lane >> 5) + e;
        if (direct && p.init != nullptr && co < p.N) {
          Scalar<float, int> b = load_scalar<float, int>(p.init, (int64_t)co * p.init_cs, p.init_dtype);
          cinit[j][g][e] = KIND == KIND_I8 ? (accs_t)b.i : (accs_t)b.f;
        }
      }

  int t = first_tile(blockIdx.x, gridDim.x);
  TileGeom g = tile_geom(p, t, Hv);
  load_window(g);
  store_window(g);
  __syncthreads();

  const unsigned per = (unsigned)(p.OH * p.OW);
  const int n_taps = p.KH * p.KW;

  for (; t < p.n_tiles; t += gridDim.x) {
    // ---- where this lane's pixels sit in the window ----
    int a_base[MI];
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      unsigned m = (unsigned)g.m0 + wave * 64 + i * 32 + (lane & 31);
      if (m > (unsigned)p.M - 1) m = (unsigned)p.M - 1;
      const unsigned nb = fast_div(m, p.div_per_magic, p.div_per_shift);
      const unsigned rem = m - nb * per;
      const unsigned oh = fast_div(rem, p.div_ow_magic, p.div_ow_shift), ow = rem - oh * (unsigned)p.OW;
      a_base[i] = (((int)(nb * Hv + oh) - g.v0) * Wv + (int)ow) * kPixStride + (lane >> 5) * 16;
    }
    const int b_base = (lane & 31) * brow + (lane >> 5) * 16;

    // ---- next tile's window: global -> registers ----
    const int t2 = t + gridDim.x;
    TileGeom g2 = g;
    if (t2 < p.n_tiles) {
      g2 = tile_geom(p, t2, Hv);
      load_window(g2);
    }

    acc_t acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NI; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    // ---- taps x four 32-byte K-blocks; fragments are fetched one K-block ahead ----
    i32x4_t fa[2][MI], fb[2][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i) fa[0][i] = *(const i32x4_t*)(sH + a_base[i]);
#pragma unroll
    for (int j = 0; j < NI; ++j) fb[0][j] = *(const i32x4_t*)(sB + b_base + j * 32 * brow);
    int kh = 0, kw = 0;
    for (int tap = 0; tap < n_taps; ++tap) {
      const int a_tap = (kh * Wv + kw) * kPixStride;
      if (++kw == p.KW) {
        kw = 0;
        ++kh;
      }
      const bool last = tap + 1 == n_taps;
      const int a_next = last ? a_tap : (kh * Wv + kw) * kPixStride;
      const int b_tap = tap * kPixBytes;
      const int b_next = last ? b_tap : b_tap + kPixBytes;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const int cur = ks & 1, nxt = cur ^ 1;
        const int ao = ks < 3 ? a_tap + (ks + 1) * 32 : a_next;
        const int bo = ks < 3 ? b_tap + (ks + 1) * 32 : b_next;
#pragma unroll
        for (int i = 0; i < MI; ++i) fa[nxt][i] = *(const i32x4_t*)(sH + a_base[i] + ao);
#pragma unroll
        for (int j = 0; j < NI; ++j) fb[nxt][j] = *(const i32x4_t*)(sB + b_base + j * 32 * brow + bo);
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int j = 0; j < NI; ++j) mma_block<KIND>(acc[i][j], fb[cur][j], fa[cur][i]);
      }
    }

    // In a 32x32 block a lane owns pixel lane%32 and the output channels
    // 8*(r/4) + 4*(lane/32) + r%4: four consecutive channels per register quad.
    if (direct) {
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        const int64_t m = g.m0 + wave * 64 + i * 32 + (lane & 31);
        if (m < p.M) {
#pragma unroll
          for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int co = j * 32 + 8 * q + 4 * (lane >> 5);
              if (co < p.N) {
                accs_t v4[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v4[e] = acc[i][j][4 * q + e] + cinit[j][q][e];
                if (KIND == KIND_I8) {
                  i32x4_t w;
#pragma unroll
                  for (int e = 0; e < 4; ++e) w[e] = (p.tail_relu && (int)v4[e] < 0) ? 0 : (int)v4[e];
                  *(i32x4_t*)((int*)p.C + m * p.ldc + co) = w;
                } else if (p.out_dtype == PML_HIP_BF16) {
                  uint32_t h[4];
#pragma unroll
                  for (int e = 0; e < 4; ++e) {
                    h[e] = f32_to_bf16_bits((float)v4[e]);
                    if (p.tail_relu && (h[e] & 0x8000u) && (h[e] & 0x7fffu) <= 0x7f80u && (h[e] & 0x7fffu) != 0) h[e] = 0;
                  }
                  *(uint2*)((uint16_t*)p.C + m * p.ldc + co) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
                } else {
                  f32x4_t w;
#pragma unroll
                  for (int e = 0; e < 4; ++e) w[e] = (p.tail_relu && (float)v4[e] < 0.f) ? 0.f : (float)v4[e];
                  *(f32x4_t*)((float*)p.C + m * p.ldc + co) = w;
                }
              }
            }
        }
      }
      __syncthreads();  // every wavefront is done reading the window
    } else {
      __syncthreads();
      constexpr int CS = kBN + 4;
      accs_t* ctile = (accs_t*)sH;
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            acc4_t w;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = acc[i][j][4 * q + e];
            *(acc4_t*)&ctile[(wave * 64 + i * 32 + (lane & 31)) * CS + j * 32 + 8 * q + 4 * (lane >> 5)] = w;
          }
      __syncthreads();
      tile_tail<KIND, kBM, kBN, kThreads>(p, ctile, g.m0, 0, tid);
      __syncthreads();
    }
    if (t2 < p.n_tiles) store_window(g2);
    g = g2;
    __syncthreads();
  }
}

// The 3x3 filter of 64 output channels on its way into LDS, held in registers between the two
// steps so that a kernel can put other work between requesting it and storing it.
// LDS row j*32 + 8q + 4h + e holds output channel 32h + 16j + 4q + e: after the MFMAs a lane
// (pixel, h) then owns the 16 consecutive channels 32h + 16j .. + 15 of block j in register order.
// The filter comes either packed as Bt[CO][K] or, with b_raw, as the caller's [K][CO] matrix
// (HWCK, 2- or 4-byte elements).  The raw form is transposed on the way in: a task is a square of
// kEpv K-indices x kEpv channels, read as kEpv 16-byte vectors along CO, turned in registers and
// written as kEpv 16-byte vectors along K.
template <int KIND, int NT = kThreads>
struct FilterStager {
  static constexpr int ES = KIND == KIND_BF16 ? 2 : (KIND == KIND_I8 ? 1 : 4);
  static constexpr int krow = 9 * kPixBytes;
  static constexpr int vecs_per_row = krow / 16;
  static constexpr int kFilterVecs = kBN * vecs_per_row / NT;
  static_assert(kBN * vecs_per_row % NT == 0, "filter vectors divide evenly over the threads");
  static constexpr int kEpv = 16 / ES;  // elements per 16-byte vector
  static constexpr int kCoGroups = kBN / kEpv;
  static constexpr int kTasks = (krow / 16) * kCoGroups;
  static constexpr int kTaskIters = (kTasks + NT - 1) / NT;
  static constexpr int kRawRegs = ES == 1 ? 1 : kTaskIters * kEpv;
  static constexpr int kFlRegs = kRawRegs > kFilterVecs ? kRawRegs : kFilterVecs;
  i32x4_t fl[kFlRegs];

  __device__ __forceinline__ void load(const IgemmArgs& p, int tid) {
    if (ES != 1 && p.b_raw) {
#pragma unroll
      for (int it = 0; it < kTaskIters; ++it) {
        const int task = tid + it * NT;
        if (task < kTasks) {
          const int kg = task / kCoGroups, cg = task - kg * kCoGroups;
#pragma unroll
          for (int kk = 0; kk < kEpv; ++kk)
            fl[(it * kEpv + kk) % kFlRegs] =
                *(const i32x4_t*)((const unsigned char*)p.Bt + ((int64_t)(kg * kEpv + kk) * kBN + cg * kEpv) * ES);
        }
      }
    } else {
#pragma unroll
      for (int k = 0; k < kFilterVecs; ++k) {
        const int q = tid + k * NT;
        const int row = q / vecs_per_row, vec = q - row * vecs_per_row;
        const int co = 32 * ((row >> 2) & 1) + 16 * (row >> 5) + 4 * ((row >> 3) & 3) + (row & 3);
        fl[k] = *(const i32x4_t*)((const unsigned char*)p.Bt + (int64_t)co * p.ldbt * ES + vec * 16);
      }
    }
  }

  // row_ptr(row): LDS address of filter row `row`
  template <typename F>
  __device__ __forceinline__ void store(const IgemmArgs& p, int tid, F row_ptr) {
    if (ES != 1 && p.b_raw) {
#pragma unroll
      for (int it = 0; it < kTaskIters; ++it) {
        const int task = tid + it * NT;
        if (task >= kTasks) break;
        const int kg = task / kCoGroups, cg = task - kg * kCoGroups;
        i32x4_t out[kEpv];
        if (ES == 4) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) out[e % kEpv][kk] = fl[(it * kEpv + kk) % kFlRegs][e];
        } else {
          // 16-bit elements: word w of vector kk holds channels 2w, 2w+1 at K index kk
#pragma unroll
          for (int w = 0; w < 4; ++w)
#pragma unroll
            for (int pr = 0; pr < 4; ++pr) {
              const unsigned a = (unsigned)fl[(it * kEpv + 2 * pr) % kFlRegs][w];
              const unsigned b2 = (unsigned)fl[(it * kEpv + 2 * pr + 1) % kFlRegs][w];
              out[(2 * w) % kEpv][pr] = (int)((a & 0xffffu) | (b2 << 16));
              out[(2 * w + 1) % kEpv][pr] = (int)((a >> 16) | (b2 & 0xffff0000u));
            }
        }
#pragma unroll
        for (int e = 0; e < kEpv; ++e) {
          const int co = cg * kEpv + e;
          const int row = ((co >> 4) & 1) * 32 + ((co >> 2) & 3) * 8 + (co >> 5) * 4 + (co & 3);
          *(i32x4_t*)(row_ptr(row) + kg * 16) = out[e];
        }
      }
    } else {
#pragma unroll
      for (int k = 0; k < kFilterVecs; ++k) {
        const int q = tid + k * NT;
        const int row = q / vecs_per_row, vec = q - row * vecs_per_row;
        *(i32x4_t*)(row_ptr(row) + vec * 16) = fl[k];
      }
    }
  }
};

// ---------------------------------------------------------------------------
// 3x3 filters, exactly 64 output channels, tail = bias? relu? store: the hot case.
//
// Same data movement as above, with the instruction streams arranged so that a
// wavefront's matrix pipe stays fed while it does everything else:
//  * the nine taps are unrolled, so the whole K loop of a tile is one basic block;
//  * the result of tile t stays in registers and its bias / relu / convert / store
//    work is cut into 16 pieces that sit between the MFMAs of tile t+1
//    (two accumulator sets alternate roles);
//  * window loads and output stores are buffer instructions: an offset beyond the
//    buffer reads zeros / drops the store, which is how padding, image ends and the
//    ragged last tile are handled without any branch in the stream.
// NCH = 32-pixel chunks per window row (1 or 2).
// ---------------------------------------------------------------------------
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

// relu as a lower clamp in one instruction (v_maximum3_f32: the IEEE 754-2019 maximum, which keeps a NaN like
// "x < lo ? lo : x" does; it orders -0 below +0, so a result of exactly -0 under relu is stored as +0).
// lo = 0 with relu, -infinity without.
__device__ __forceinline__ float relu_clamp(float x, float lo) { return __builtin_elementwise_maximum(x, lo); }

constexpr unsigned kRsrcFlags = 0x00020000u;  // raw buffer, 32-bit data format
#define PML_LDS(p) ((__attribute__((address_space(3))) void*)(p))
constexpr int kConvAhead = 2;                 // K-blocks (pairs of them in the register-filter kernel) operand fragments are fetched ahead
constexpr int kFar = 0x40000000;              // beyond any input this kernel accepts (<= 2^30 bytes); two of them still are

template <int KIND, int NCH>
__global__ __launch_bounds__(kThreads) void conv_halo3x3_kernel(IgemmArgs p) {
  constexpr int ES = KIND == KIND_BF16 ? 2 : (KIND == KIND_I8 ? 1 : 4);
  constexpr int MI = 2, NI = 2;
  constexpr int OES = KIND == KIND_BF16 ? 2 : 4;  // bytes per output element (bf16 -> bf16, fp32 -> fp32, int8 -> int32)
  constexpr int kTaps = 9;
  constexpr int krow = kTaps * kPixBytes, brow = krow + 16;
  constexpr int kRows = kMaxLoads / NCH;
  typedef typename Acc<KIND>::type acc_t;
  typedef typename Acc<KIND>::scalar accs_t;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned char* const sB = smem;
  unsigned char* const sH = smem + kBN * brow;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int Hv = p.OH + 2, Wv = p.OW + 2;

  // ---- filter -> LDS, once: all of a thread's 18 vectors are requested before the first is stored ----
  FilterStager<KIND> filter;
  filter.load(p, tid);
  auto store_filter = [&]() { filter.store(p, tid, [&](int row) { return sB + row * brow; }); };

  const __amdgpu_buffer_rsrc_t rin =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.A, 0, (int)((int64_t)p.NB * p.H * p.W * kPixBytes), kRsrcFlags);
  const __amdgpu_buffer_rsrc_t rout =
      __builtin_amdgcn_make_buffer_rsrc(p.C, 0, (int)(p.M * p.ldc * OES), kRsrcFlags);

  // ---- a thread's share of a window: vector lv of pixels lp (+32) of every row ----
  // Eight lanes carry one pixel (128 contiguous bytes).  Neighbouring lane groups take pixels 8 apart:
  // with the 144-byte pixel stride their 16-byte LDS slots then differ by 8 (mod 16) and a 16-lane
  // write touches every bank once.
  const int lv = tid & 7, lg = tid >> 3;
  const int lp = ((lg >> 1) & 7) + 8 * (lg & 1) + 16 * (lg >> 4);
  int g_off[NCH], l_off[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int px = c * 32 + lp, iw = px - p.PW;
    g_off[c] = (px < Wv && (unsigned)iw < (unsigned)p.W) ? iw * kPixBytes + lv * 16 : kFar;
    l_off[c] = px * kPixStride + lv * 16;
  }
  const bool chunk0 = lp < Wv, chunk1 = lp + 32 < Wv;  // does this thread's pixel of the chunk exist?

  u32x4_t pf[kMaxLoads];
  // byte offset of every window row in the input (uniform), or kFar for padding rows and rows past the tile
  int row_base[kRows];
  auto window_rows = [&](const TileGeom& g) {
    int nb = g.nb0, ihv = g.ihv0;
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const int ih = ihv - p.PH;
      const bool row_ok = r < g.nrows && nb < p.NB && (unsigned)ih < (unsigned)p.H;
      row_base[r] = row_ok ? (nb * p.H + ih) * p.W * kPixBytes : kFar;
      if (++ihv == Hv) {
        ihv = 0;
        ++nb;
      }
    }
  };
  auto load_vec = [&](int j) { pf[j] = __builtin_amdgcn_raw_buffer_load_b128(rin, row_base[j / NCH] + g_off[j % NCH], 0, 0); };
  auto load_window = [&](const TileGeom& g) {
    window_rows(g);
#pragma unroll
    for (int j = 0; j < kMaxLoads; ++j) load_vec(j);
  };
  auto store_window = [&](int nrows) {
    const int row_pitch = Wv * kPixStride;
    if (chunk0) {
#pragma unroll
      for (int r = 0; r < kRows; ++r)
        if (r < nrows) *(u32x4_t*)(sH + r * row_pitch + l_off[0]) = pf[r * NCH];
    }
    if (NCH == 2 && chunk1) {
#pragma unroll
      for (int r = 0; r < kRows; ++r)
        if (r < nrows) *(u32x4_t*)(sH + r * row_pitch + l_off[NCH - 1]) = pf[r * NCH + NCH - 1];
    }
  };

  // bias of the output channels this lane owns; relu as a lower clamp (x < lo ? lo : x keeps NaN)
  accs_t cinit[NI][4][4];
#pragma unroll
  for (int j = 0; j < NI; ++j)
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        cinit[j][q][e] = 0;
      }
  if (p.init != nullptr) {
    const int natural = KIND == KIND_BF16 ? PML_HIP_BF16 : (KIND == KIND_I8 ? PML_HIP_I32 : PML_HIP_F32);
    if (p.init_cs == 1 && p.init_dtype == natural && ((uintptr_t)p.init & 15) == 0) {
      // a contiguous bias of the result type: a lane's 16 channels of block j are 32 (bf16) or 64 bytes
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        const unsigned char* src = (const unsigned char*)p.init + (32 * (lane >> 5) + 16 * j) * OES;
        u32x4_t raw[OES];
#pragma unroll
        for (int v = 0; v < OES; ++v) raw[v] = *(const u32x4_t*)(src + v * 16);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          if (KIND == KIND_BF16) {
            const unsigned w = raw[r >> 3][(r >> 1) & 3];
            cinit[j][r >> 2][r & 3] = (accs_t)__uint_as_float((r & 1) ? (w & 0xffff0000u) : (w << 16));
          } else if (KIND == KIND_I8) {
            cinit[j][r >> 2][r & 3] = (accs_t)(int)raw[r >> 2][r & 3];
          } else {
            cinit[j][r >> 2][r & 3] = (accs_t)__uint_as_float(raw[r >> 2][r & 3]);
          }
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < NI; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            Scalar<float, int> b = load_scalar<float, int>(p.init, (int64_t)(32 * (lane >> 5) + 16 * j + 4 * q + e) * p.init_cs, p.init_dtype);
            cinit[j][q][e] = KIND == KIND_I8 ? (accs_t)b.i : (accs_t)b.f;
          }
    }
  }
  const float lo_f = p.tail_relu ? 0.f : -__builtin_inff();
  const int lo_i = p.tail_relu ? 0 : (int)0x80000000;

  const unsigned per = (unsigned)(p.OH * p.OW);
  const int b_base = (lane & 31) * brow + (lane >> 5) * 16;

  // where a tile's pixels of this lane sit: in the window (LDS) and in the output (bytes)
  auto place = [&](const TileGeom& g, int (&a_base)[MI], int (&m_off)[MI]) {
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      const unsigned m = (unsigned)g.m0 + wave * 64 + i * 32 + (lane & 31);
      const bool ok = m < (unsigned)p.M;
      const unsigned mc = ok ? m : (unsigned)p.M - 1;
      const unsigned nb = fast_div(mc, p.div_per_magic, p.div_per_shift);
      const unsigned rem = mc - nb * per;
      const unsigned oh = fast_div(rem, p.div_ow_magic, p.div_ow_shift), ow = rem - oh * (unsigned)p.OW;
      a_base[i] = (((int)(nb * Hv + oh) - g.v0) * Wv + (int)ow) * kPixStride + (lane >> 5) * 16;
      m_off[i] = ok ? (int)((m * (unsigned)p.ldc + 32 * (lane >> 5)) * OES) : (int)0x80000000;
    }
  };

  // one of the 16 pieces of a finished tile: 4 consecutive channels of one pixel
  // (bf16 output: two pieces share one 16-byte store)
  unsigned held[2] = {0, 0};
  auto finish_piece = [&](const acc_t (&acc)[MI][NI], const int (&m_off)[MI], int pc) {
    const int i = pc >> 3, j = (pc >> 2) & 1, q = pc & 3;
    const int off = m_off[i] + (j * 16 + 4 * q) * OES;
    if (KIND == KIND_I8) {
      u32x4_t w;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int v = (int)acc[i][j][4 * q + e] + (int)cinit[j][q][e];
        w[e] = (unsigned)(v < lo_i ? lo_i : v);
      }
      __builtin_amdgcn_raw_buffer_store_b128(w, rout, off, 0, 0);
    } else {
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[e] = (float)acc[i][j][4 * q + e] + (float)cinit[j][q][e];
        v[e] = relu_clamp(v[e], lo_f);
      }
      if (KIND == KIND_BF16) {
        const f32x2_t a01 = {v[0], v[1]}, a23 = {v[2], v[3]};
        const bf16x2_t h01 = __builtin_convertvector(a01, bf16x2_t), h23 = __builtin_convertvector(a23, bf16x2_t);
        unsigned w0, w1;
        __builtin_memcpy(&w0, &h01, 4);
        __builtin_memcpy(&w1, &h23, 4);
        if ((q & 1) == 0) {
          held[0] = w0;
          held[1] = w1;
        } else {
          const u32x4_t w = {held[0], held[1], w0, w1};
          __builtin_amdgcn_raw_buffer_store_b128(w, rout, off - 4 * OES, 0, 0);
        }
      } else {
        u32x4_t w;
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = __float_as_uint(v[e]);
        __builtin_amdgcn_raw_buffer_store_b128(w, rout, off, 0, 0);
      }
    }
  };

  // K loop of one tile (36 K-blocks of 32 bytes); with EPI the 16 pieces of the previous tile ride along
  int a_next[MI], m_next[MI];  // placement of the tile after the current one
  // The next tile (geometry g2) is prepared on the way: the offset of window row r is worked out right
  // before that row's loads are issued, one 16-byte vector per K-block, and its placement near the end.
  auto k_loop = [&](acc_t (&acc)[MI][NI], const int (&a_base)[MI], auto epi, const acc_t (&pacc)[MI][NI],
                    const int (&pm_off)[MI], const TileGeom& g2) {
    constexpr bool EPI = decltype(epi)::value;
    constexpr int kMfmaPerBlock = KIND == KIND_F32 ? 4 : 1;
    int w_nb = g2.nb0, w_ihv = g2.ihv0;
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NI; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
    // operand fragments are fetched kAhead K-blocks ahead (kAhead + 1 register sets)
    constexpr int kAhead = kConvAhead;
    i32x4_t fa[kAhead + 1][MI], fb[kAhead + 1][NI];
    auto frag_offsets = [&](int s1, int& ao, int& bo) {
      const int tap = s1 >> 2, ks = s1 & 3;
      ao = ((tap / 3) * Wv + tap % 3) * kPixStride + ks * 32;
      bo = tap * kPixBytes + ks * 32;
    };
#pragma unroll
    for (int s0 = 0; s0 < kAhead; ++s0) {
      int ao, bo;
      frag_offsets(s0, ao, bo);
#pragma unroll
      for (int i = 0; i < MI; ++i) fa[s0][i] = *(const i32x4_t*)(sH + a_base[i] + ao);
#pragma unroll
      for (int j = 0; j < NI; ++j) fb[s0][j] = *(const i32x4_t*)(sB + b_base + j * 32 * brow + bo);
    }
#pragma unroll
    for (int s = 0; s < kTaps * 4; ++s) {
      const int cur = s % (kAhead + 1), nxt = (s + kAhead) % (kAhead + 1);
      if (s + kAhead < kTaps * 4) {
        int ao, bo;
        frag_offsets(s + kAhead, ao, bo);
#pragma unroll
        for (int i = 0; i < MI; ++i) fa[nxt][i] = *(const i32x4_t*)(sH + a_base[i] + ao);
#pragma unroll
        for (int j = 0; j < NI; ++j) fb[nxt][j] = *(const i32x4_t*)(sB + b_base + j * 32 * brow + bo);
      }
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) mma_block<KIND>(acc[i][j], fb[cur][j], fa[cur][i]);
      if (s < kMaxLoads) {  // the next tile's window, one vector per K-block
        if (s % NCH == 0) {
          const int r = s / NCH, ih = w_ihv - p.PH;
          // (mask arithmetic instead of a conditional: a branch here would split the K-block)
          const int row_ok = (int)(r < g2.nrows) & (int)(w_nb < p.NB) & (int)((unsigned)ih < (unsigned)p.H);
          const int real = (w_nb * p.H + ih) * p.W * kPixBytes;
          row_base[r] = kFar ^ ((kFar ^ real) & -row_ok);
          const int wrap = (int)(w_ihv + 1 == Hv);
          w_ihv = (w_ihv + 1) & (wrap - 1);
          w_nb += wrap;
        }
        load_vec(s);
      }
      if (EPI && (s & 1) == 0 && (s >> 1) < 16) finish_piece(pacc, pm_off, s >> 1);
      if (s == 33) place(g2, a_next, m_next);
      // order inside the K-block: LDS reads and the window load first, then VALU work between the MFMAs
      __builtin_amdgcn_sched_group_barrier(0x100, MI + NI, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
#pragma unroll
      for (int q = 0; q < MI * NI; ++q) {
        __builtin_amdgcn_sched_group_barrier(0x008, kMfmaPerBlock, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
      }
      __builtin_amdgcn_sched_barrier(0);  // keep loads and pieces in the K-block they were put in
    }
  };

  acc_t accA[MI][NI], accB[MI][NI];
  int a_base[MI], m_offA[MI], m_offB[MI];

  int t = first_tile(blockIdx.x, gridDim.x);
  TileGeom g = tile_geom(p, t, Hv);
  load_window(g);
  store_filter();
  store_window(g.nrows);
  place(g, a_base, m_offA);
  __syncthreads();

  // Preparing tile t2 = t + gridDim.x (geometry, window loads, placement) is branch-free -- past the
  // last tile every row is out of range and every load returns zeros -- so it shares one basic block
  // with the K loop and is scheduled among the MFMAs.
  auto advance = [&](int t2, const TileGeom& g2) {
    __syncthreads();  // every wavefront is done reading the window
    if (t2 < p.n_tiles) store_window(g2.nrows);
    __syncthreads();
    t = t2;
    g = g2;
#pragma unroll
    for (int i = 0; i < MI; ++i) a_base[i] = a_next[i];
  };

  {
    const int t2 = t + gridDim.x;
    const TileGeom g2 = tile_geom(p, t2, Hv);
    k_loop(accA, a_base, std::false_type(), accA, m_offA, g2);
    advance(t2, g2);
  }
  for (;;) {
    if (t >= p.n_tiles) {
#pragma unroll
      for (int pc = 0; pc < 16; ++pc) finish_piece(accA, m_offA, pc);
      break;
    }
    {
#pragma unroll
      for (int i = 0; i < MI; ++i) m_offB[i] = m_next[i];
      const int t2 = t + gridDim.x;
      const TileGeom g2 = tile_geom(p, t2, Hv);
      k_loop(accB, a_base, std::true_type(), accA, m_offA, g2);
      advance(t2, g2);
    }
    if (t >= p.n_tiles) {
#pragma unroll
      for (int pc = 0; pc < 16; ++pc) finish_piece(accB, m_offB, pc);
      break;
    }
    {
#pragma unroll
      for (int i = 0; i < MI; ++i) m_offA[i] = m_next[i];
      const int t2 = t + gridDim.x;
      const TileGeom g2 = tile_geom(p, t2, Hv);
      k_loop(accA, a_base, std::true_type(), accB, m_offB, g2);
      advance(t2, g2);
    }
  }
}

// ---------------------------------------------------------------------------
// The same hot case with the filter in registers (16-bit and 8-bit elements).
//
// With the filter in LDS every MFMA needs one 16-byte LDS read per lane, and four wavefronts
// cannot pull that much out of LDS: the matrix pipe waits.  A wavefront owns 64 pixels x 64 channels,
// so it needs the whole 3x3x(128 bytes)x64 filter: 72 16-byte fragments per lane, 288 of the 512
// registers a lane has at one wavefront per SIMD.  They are loaded once; LDS traffic halves and LDS
// itself is free for two window buffers, filled by loads that write LDS directly (no register
// staging, no store phase): the window of tile t+1 arrives while tile t is computed.
//
// Window layout: pixel slot q = row * Wv + column (Wv = padded image width), 128 bytes each, rows
// packed without gaps.  A slot keeps its eight 16-byte channel vectors permuted: vector u sits at
// position u ^ ((column >> 1) & 7), which spreads the 32 pixels of an operand read over all banks
// and, depending on the column only, is the same for the three taps of a filter column.
// A wavefront-wide request (64 lanes x 16 bytes) fills 8 consecutive slots; requests are issued per
// row in 8 groups of 8 columns, and a lane whose column is past the row's end fetches what belongs
// into the slot it really writes, a pixel of the next row (written twice then, with the same bytes).
// ---------------------------------------------------------------------------
constexpr int kRegRows = 10;                   // window rows per buffer
constexpr int kRegBrow = 9 * kPixBytes + 16;   // stride of a staged filter row
// one window buffer: the last row's requests reach 64 columns
__host__ __device__ constexpr int reg_win_bytes(int Wv) { return ((kRegRows - 1) * Wv + 64) * kPixBytes; }
// staged filter rows that fit below the second window buffer (the first window is loaded into that one)
__host__ __device__ constexpr int reg_rows_low(int Wv) {
  return reg_win_bytes(Wv) / kRegBrow < kBN ? reg_win_bytes(Wv) / kRegBrow : kBN;
}
// 64 accumulator-typed initial values sit behind the window buffers and the staged filter rows beyond them
__host__ __device__ constexpr int reg_bias_off(int Wv) { return 2 * reg_win_bytes(Wv) + (kBN - reg_rows_low(Wv)) * kRegBrow; }
__host__ __device__ constexpr int reg_lds_bytes(int Wv) { return reg_bias_off(Wv) + kBN * 4; }

// WV: the padded image width if known at compile time (the row offsets of the taps then are
// immediates of the LDS reads), 0 = taken from the arguments.
// NI: 32-channel blocks per wavefront.  1: eight wavefronts (two per SIMD, 256 registers each), a
// wavefront holds the filter of its 32 channels.  2: four wavefronts with 512 registers, each
// holding the whole filter; one LDS read then feeds two MFMAs, but half of the filter sits in
// accumulation registers and is copied out before use, which costs more than the reads saved.
template <int KIND, int WV, int NI>
__global__ __launch_bounds__(512 / NI) void conv_regfilter3x3_kernel(IgemmArgs p) {
  static_assert(KIND != KIND_F32, "16-bit and 8-bit elements only");
  constexpr int kNT = 512 / NI;
  constexpr int MI = 2;
  constexpr int OES = KIND == KIND_BF16 ? 2 : 4;
  constexpr int kTaps = 9, kBlocks = kTaps * 4;  // K-blocks of 32 bytes
  typedef typename Acc<KIND>::type acc_t;
  typedef typename Acc<KIND>::scalar accs_t;
  typedef accs_t acc4_t __attribute__((ext_vector_type(4)));

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pg = wave & 3;                   // the wavefront's 64 pixels of a tile
  const int cb0 = NI == 1 ? wave >> 2 : 0;   // its first 32-channel block
  const int half = lane >> 5;
  const int Hv = p.OH + 2, Wv = WV ? WV : p.OW + 2;
  const int win_bytes = reg_win_bytes(Wv);

  const __amdgpu_buffer_rsrc_t rin =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.A, 0, (int)((int64_t)p.NB * p.H * p.W * kPixBytes), kRsrcFlags);
  const __amdgpu_buffer_rsrc_t rout =
      __builtin_amdgcn_make_buffer_rsrc(p.C, 0, (int)(p.M * p.ldc * OES), kRsrcFlags);

  // ---- window requests: a row is covered by 8 requests of 8 columns; wavefront w issues number w (+ 4) ----
  // Fixed for the kernel's life: a lane's column, whether that column is really one of the next row,
  // and its byte offset inside the input row (kFar where the slot is padding).
  int req_next[NI], req_col[NI];
#pragma unroll
  for (int c = 0; c < NI; ++c) {
    const int px = (wave + 4 * c) * 8 + (lane >> 3);
    req_next[c] = px >= Wv ? -1 : 0;  // all ones: the lane's slot belongs to the next row
    const int col = px - (Wv & req_next[c]), iw = col - p.PW;
    const int vec = (lane & 7) ^ ((col >> 1) & 7);  // the input vector that belongs into this lane's 16 bytes of the slot
    req_col[c] = (unsigned)iw < (unsigned)p.W ? iw * kPixBytes + vec * 16 : kFar;
  }
  // Lane r works out the input byte offset of window row r of a tile (kFar for rows of padding, rows
  // past the tile's window and rows past the last image); the requests pick the rows up from there.
  auto row_offsets = [&](const TileGeom& tg) {
    int nb = tg.nb0, ihv = tg.ihv0 + lane;
#pragma unroll
    for (int k = 0; k < 3; ++k) {  // a window of kRegRows rows ends at most 3 images further on
      const bool wrap = ihv >= Hv;
      ihv -= wrap ? Hv : 0;
      nb += wrap ? 1 : 0;
    }
    const int ih = ihv - p.PH;
    const bool ok = lane < tg.nrows && nb < p.NB && (unsigned)ih < (unsigned)p.H;
    return ok ? (nb * p.H + ih) * p.W * kPixBytes : kFar;
  };
  // rows: what row_offsets returned for the window's tile
  auto request = [&](unsigned char* win, int r, int c, int rows) {
    const int rb_cur = __builtin_amdgcn_readlane(rows, r), rb_next = __builtin_amdgcn_readlane(rows, r + 1);
    const int voff = rb_cur + ((rb_next - rb_cur) & req_next[c]) + req_col[c];  // two kFar still are outside
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rin, PML_LDS(win + (r * Wv + (wave + 4 * c) * 8) * kPixBytes), 16, voff, 0, 0,
                                             0);
  };

  // b_raw == 2: the filter was packed once into the order this kernel keeps it in registers (regfilter_image_kernel
  // below): fragment (channel block cb, K-block s) of lane l is the 16 bytes at ((cb * 36 + s) * 64 + l) * 16.  The
  // 72 KB go to LDS as they lie (requests that write LDS directly, no registers, nothing turned) and every fragment
  // read of a wavefront is 1 KB of consecutive bytes.  (Loading the fragments from memory straight into registers was
  // measured: 36 KB per wavefront through the vector memory path take longer than the whole trip through LDS.)
  const bool image = p.b_raw == 2;
  i32x4_t breg[kBlocks][NI];
  if (image) {
    // 72 requests of 1 KB into the first window buffer, nine per wavefront
    const __amdgpu_buffer_rsrc_t rimg = __builtin_amdgcn_make_buffer_rsrc((void*)p.Bt, 0, 2 * kBlocks * 1024, kRsrcFlags);
#pragma unroll
    for (int r = 0; r < 2 * kBlocks / (kNT / 64); ++r) {
      const int req = wave + (kNT / 64) * r;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rimg, PML_LDS(smem + req * 1024), 16, req * 1024 + lane * 16, 0, 0, 0);
    }
  }
  FilterStager<KIND, kNT> filter;
  if (!image) filter.load(p, tid);
  int t = first_tile(blockIdx.x, gridDim.x);
  TileGeom g = tile_geom(p, t, Hv);
  unsigned char* const win0 = smem;
  unsigned char* const win1 = smem + win_bytes;
  {
    // the first window goes into the second buffer: the filter is staged around it
    const int rows = row_offsets(g);
#pragma unroll
    for (int r = 0; r < kRegRows; ++r)
#pragma unroll
      for (int c = 0; c < NI; ++c) request(win1, r, c, rows);
  }

  // ---- filter -> LDS (transposed if raw) -> registers; initial values -> LDS ----
  const int rows_low = reg_rows_low(Wv), bias_off = reg_bias_off(Wv);
  auto filter_row = [&](int row) {
    return smem + (row < rows_low ? row * kRegBrow : 2 * win_bytes + (row - rows_low) * kRegBrow);
  };
  if (!image) filter.store(p, tid, filter_row);
  if (tid < kBN) {
    accs_t b = 0;
    if (p.init != nullptr) {
      Scalar<float, int> v = load_scalar<float, int>(p.init, (int64_t)tid * p.init_cs, p.init_dtype);
      b = KIND == KIND_I8 ? (accs_t)v.i : (accs_t)v.f;
    }
    *(accs_t*)(smem + bias_off + tid * 4) = b;
  }
  __syncthreads();
  // MFMA row 8q + 4h + e of channel block cb is given output channel 32cb + 16h + 4q + e, so that
  // a lane (pixel, h) ends up owning the 16 consecutive channels 32cb + 16h .. + 15 in register order;
  // the staged filter keeps that channel in row 32h + 8q + 4cb + e
  if (image) {
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int s = 0; s < kBlocks; ++s) breg[s][j] = *(const i32x4_t*)(smem + (((cb0 + j) * kBlocks + s) * 64 + lane) * 16);
  }
  if (!image) {
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int row = lane & 31;
      const unsigned char* src = filter_row(((row >> 2) & 1) * 32 + (row >> 3) * 8 + 4 * (cb0 + j) + (row & 3)) + half * 16;
#pragma unroll
      for (int s = 0; s < kBlocks; ++s) breg[s][j] = *(const i32x4_t*)(src + s * 32);
    }
  }
  const int co0 = 32 * cb0 + 16 * half;  // first of the lane's 16 output channels in its first block
  const unsigned char* const bias_src = smem + bias_off + co0 * 4;

  const float lo_f = p.tail_relu ? 0.f : -__builtin_inff();
  const int lo_i = p.tail_relu ? 0 : (int)0x80000000;
  const unsigned per = (unsigned)(p.OH * p.OW);

  // where the pixel of this lane in half `i` of a tile sits: byte offset of its window slot, its column
  // and its output byte offset
  auto place = [&](const TileGeom& tg, int i, int& a_q, int& a_ow, int& m_off) {
    const unsigned m = (unsigned)tg.m0 + pg * 64 + i * 32 + (lane & 31);
    const bool ok = m < (unsigned)p.M;
    const unsigned mc = ok ? m : (unsigned)p.M - 1;
    const unsigned nb = fast_div(mc, p.div_per_magic, p.div_per_shift);
    const unsigned rem = mc - nb * per;
    const unsigned oh = fast_div(rem, p.div_ow_magic, p.div_ow_shift), ow = rem - oh * (unsigned)p.OW;
    a_q = (((int)(nb * Hv + oh) - tg.v0) * Wv + (int)ow) * kPixBytes;
    a_ow = (int)ow;
    m_off = ok ? (int)((m * (unsigned)p.ldc + co0) * OES) : (int)0x80000000;
  };

  // one of the 4 NI pieces of a finished half tile: 4 consecutive channels of the lane's pixel
  // (bf16 output: two pieces share one 16-byte store)
  unsigned held[2] = {0, 0};
  auto finish_piece = [&](const acc_t (&acc)[NI], int m_off, int pc) {
    const int j = pc >> 2, q = pc & 3;
    const int off = m_off + (32 * j + 4 * q) * OES;
    if (KIND == KIND_I8) {
      u32x4_t w;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int v = (int)acc[j][4 * q + e];
        w[e] = (unsigned)(v < lo_i ? lo_i : v);
      }
      __builtin_amdgcn_raw_buffer_store_b128(w, rout, off, 0, 0);
    } else {
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[e] = (float)acc[j][4 * q + e];
        v[e] = relu_clamp(v[e], lo_f);
      }
      const f32x2_t a01 = {v[0], v[1]}, a23 = {v[2], v[3]};
      const bf16x2_t h01 = __builtin_convertvector(a01, bf16x2_t), h23 = __builtin_convertvector(a23, bf16x2_t);
      unsigned w0, w1;
      __builtin_memcpy(&w0, &h01, 4);
      __builtin_memcpy(&w1, &h23, 4);
      if ((q & 1) == 0) {
        held[0] = w0;
        held[1] = w1;
      } else {
        const u32x4_t w = {held[0], held[1], w0, w1};
        __builtin_amdgcn_raw_buffer_store_b128(w, rout, off - 4 * OES, 0, 0);
      }
    }
  };

  // placement of the two halves of the current tile and of the tile after it
  int a_q[MI], a_ow[MI], m_off[MI];
  int a_next[MI], ow_next[MI], m_next[MI];

  // K loop of half I of a tile (32 pixels x 32 NI channels per wavefront) out of window `cur`.  Two
  // accumulator sets alternate between the halves, so the finished half rides along: its pieces
  // (pacc, pm_off) sit between the MFMAs of this one.  Half 0 also carries the requests for the next
  // tile's window (geometry g2, into `nxt`), half 1 the placement of the next tile.  Past the last
  // tile every row is out of range and every request reads zeros, so none of this needs a branch.
  auto k_loop = [&](auto half_tag, acc_t (&acc)[NI], const unsigned char* cur, unsigned char* nxt,
                    const acc_t (&pacc)[NI], int pm_off, const TileGeom& g2) {
    constexpr int I = decltype(half_tag)::value;
    const int rows2 = I == 0 ? row_offsets(g2) : 0;
    // the accumulators start from the initial values of the lane's channels
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const acc4_t v = *(const acc4_t*)(bias_src + (32 * j + 4 * q) * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[j][4 * q + e] = v[e];
      }
    // Operand fragments are fetched kAhead K-blocks ahead.
    constexpr int kAhead = 2 * kConvAhead;
    i32x4_t fa[kAhead + 1];
    // K-blocks run filter column by filter column (kw outermost): the four permuted vector offsets of
    // a column serve its three taps, which differ by a uniform row offset only
    int col_off[4] = {0, 0, 0, 0};
    auto fetch = [&](int s1) {
      const int ks = s1 & 3, kh = (s1 >> 2) % 3, kw = s1 / 12;
      if (ks == 0 && kh == 0) {
        const int key = ((((a_ow[I] + kw) >> 1) & 7) ^ half) << 4;
#pragma unroll
        for (int k = 0; k < 4; ++k) col_off[k] = a_q[I] + kw * kPixBytes + (key ^ (k << 5));  // vector 2k + half
      }
      fa[s1 % (kAhead + 1)] = *(const i32x4_t*)(cur + col_off[ks] + kh * Wv * kPixBytes);
    };
#pragma unroll
    for (int s0 = 0; s0 < kAhead; ++s0) fetch(s0);
#pragma unroll
    for (int s = 0; s < kBlocks; ++s) {
      asm volatile("" ::: "memory");  // LDS reads stay in the K-block they were put in
      if (s + kAhead < kBlocks) fetch(s + kAhead);
      const int sb = (((s >> 2) % 3) * 3 + s / 12) * 4 + (s & 3);  // the K-block in the filter's own tap order
      // the MFMAs are kept from sinking past the end of their K-block (the compiler's first instruction
      // order otherwise gathers the pure MFMAs of a half behind all of its LDS reads)
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        mma_block<KIND>(acc[j], breg[sb][j], fa[s % (kAhead + 1)]);
        asm volatile("" ::"v"(acc[j][0]));
      }
      // the next tile's window, one request per K-block
      if (I == 0 && s < NI * kRegRows) request(nxt, s / NI, s % NI, rows2);
      if ((s % (8 / NI)) == 4 / NI && s / (8 / NI) < 4 * NI) finish_piece(pacc, pm_off, s / (8 / NI));
      if (I == 1 && s == 32) place(g2, 0, a_next[0], ow_next[0], m_next[0]);
      if (I == 1 && s == 34) place(g2, 1, a_next[1], ow_next[1], m_next[1]);
      // order inside the K-block: the LDS read and the window request first, then the MFMAs with VALU work behind them
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 12 / NI, 0);
      }
      __builtin_amdgcn_sched_barrier(0);  // keep requests and pieces in the K-block they were put in
    }
  };

  acc_t accX[NI], accY[NI];
  place(g, 0, a_q[0], a_ow[0], m_off[0]);
  place(g, 1, a_q[1], a_ow[1], m_off[1]);
  int m_last = (int)0x80000000;  // second half of the tile before: none precedes the first, its pieces are dropped
#pragma unroll
  for (int j = 0; j < NI; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) accY[j][r] = 0;
  __syncthreads();  // the filter is out of LDS, the first window is in

  // Tiles that do not fill a last round of all workgroups are dealt out in halves: with 1568 tiles on
  // 256 workgroups the 32 left after six rounds keep 64 workgroups busy for half a tile instead of 32
  // for a whole one.  t_half: the tile this workgroup takes one half of at the end (n_tiles: none).
  const int grid = (int)gridDim.x, pos = t;
  const int rem = p.n_tiles % grid, n_full = p.n_tiles - rem;
  const bool split = rem != 0 && 2 * rem <= grid;
  const int t_half = split && pos < 2 * rem ? n_full + (pos >> 1) : p.n_tiles;
  const int t_end = split ? n_full : p.n_tiles;

  unsigned char* cur = win1;
  unsigned char* nxt = win0;
  for (;;) {
    int t2 = t + grid;
    if (split && t2 >= n_full) t2 = t_half;
    const TileGeom g2 = tile_geom(p, t2, Hv);
    k_loop(std::integral_constant<int, 0>(), accX, cur, nxt, accY, m_last, g2);
    k_loop(std::integral_constant<int, 1>(), accY, cur, nxt, accX, m_off[0], g2);
    __syncthreads();  // every wavefront is done with the current window; the next one has arrived
    m_last = m_off[1];
    t = t2;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      a_q[i] = a_next[i];
      a_ow[i] = ow_next[i];
      m_off[i] = m_next[i];
    }
    unsigned char* const w = cur;
    cur = nxt;
    nxt = w;
    if (t >= t_end) break;
  }
  auto flush = [&](const acc_t (&acc)[NI], int off) {
#pragma unroll
    for (int pc = 0; pc < 4 * NI; ++pc) finish_piece(acc, off, pc);
  };
  if (t < p.n_tiles) {
    // one half of tile t_half: its window is in `cur`, its placement is made; nothing comes after it
    const TileGeom none = tile_geom(p, p.n_tiles, Hv);
    if ((pos & 1) == 0) {
      k_loop(std::integral_constant<int, 0>(), accX, cur, nxt, accY, m_last, none);
      flush(accX, m_off[0]);
    } else {
      flush(accY, m_last);
      k_loop(std::integral_constant<int, 1>(), accY, cur, nxt, accX, (int)0x80000000, none);
      flush(accY, m_off[1]);
    }
  } else {
    flush(accY, m_last);
  }
}

// The packed filter Bt[64][9 * 128 bytes] in the order conv_regfilter3x3_kernel holds it in registers: for channel
// block cb (32 channels), K-block s (32 bytes of a row) and lane l, the 16 bytes l >> 5 of that K-block in the row of
// channel 32 cb + 16 ((l >> 2) & 1) + 4 ((l & 31) >> 3) + (l & 3) -- the channel MFMA row l & 31 is given.
__global__ __launch_bounds__(256) void regfilter_image_kernel(const unsigned char* __restrict__ bt, int64_t ldbt_bytes,
                                                              i32x4_t* __restrict__ image) {
  const int q = blockIdx.x * 256 + threadIdx.x;  // (cb * 36 + s) * 64 + lane
  if (q >= 2 * 36 * 64) return;
  const int lane = q & 63, s = (q >> 6) % 36, cb = q / (64 * 36);
  const int row = lane & 31;
  const int co = 32 * cb + 16 * ((row >> 2) & 1) + 4 * (row >> 3) + (row & 3);
  image[q] = *(const i32x4_t*)(bt + co * ldbt_bytes + s * 32 + (lane >> 5) * 16);
}

template <int KIND, int WV>
hipError_t launch_regfilter(const IgemmArgs& a, size_t lds, int n_cus, hipStream_t s) {
  constexpr int NI = 1;  // measured on the 128 x 56 x 56 x 64 case: 33.7 us against 42.7 us with NI = 2
  auto kern = conv_regfilter3x3_kernel<KIND, WV, NI>;
  static DynamicLdsLimit limit;
  if (hipError_t e = limit.ensure((const void*)kern, lds); e != hipSuccess) return e;
  const int grid = a.n_tiles < n_cus ? a.n_tiles : n_cus;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512 / NI), lds, s, a);
  return hipGetLastError();
}

template <int KIND, int NCH>
hipError_t launch3x3(const IgemmArgs& a, size_t lds, int n_cus, hipStream_t s) {
  auto kern = conv_halo3x3_kernel<KIND, NCH>;
  static DynamicLdsLimit limit;
  if (hipError_t e = limit.ensure((const void*)kern, lds); e != hipSuccess) return e;
  const int grid = a.n_tiles < n_cus ? a.n_tiles : n_cus;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(kThreads), lds, s, a);
  return hipGetLastError();
}

template <int KIND>
hipError_t launch(const IgemmArgs& a, size_t lds, int n_cus, hipStream_t s) {
  auto kern = conv_halo_kernel<KIND>;
  static DynamicLdsLimit limit;
  if (hipError_t e = limit.ensure((const void*)kern, lds); e != hipSuccess) return e;
  const int grid = a.n_tiles < n_cus ? a.n_tiles : n_cus;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(kThreads), lds, s, a);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// The few-channel, stride-2 convolution at the head of an image network (7x7x3 -> 64), after its input has been
// re-blocked into 2x2 pixel blocks of 16 channels (32 bytes): a unit-stride convolution with 4x4 block taps, K = 256.
// As an implicit GEMM it has 4 slabs per tile and 25 thousand tiles, each of which fetches the same 32 KB filter
// and pays its own start-up and tail.  Here a workgroup walks down the output rows of one image:
//   - the filter lives in registers for the kernel's life (a wavefront holds all 64 channels: 16 taps x 2 blocks
//     of 32 channels x 16 bytes per lane);
//   - LDS holds a ring of five re-blocked input rows (one row of padding slots included); each output row needs
//     four of them, so every step fetches ONE new row (a 16-byte chunk per thread), which arrives in registers
//     while the current row is multiplied and is written into the slot the oldest row has left;
//   - a wavefront takes 32 neighbouring pixels: a tap's operand is one 16-byte LDS read per lane at consecutive
//     32-byte pixels (the two half-wavefronts read the two channel halves: 1 KB contiguous, no bank conflicts);
//   - MFMA row 8q + 4h + e is given output channel 32j + 16h + 4q + e, so a lane ends up with 16 consecutive
//     channels of its pixel and stores 32 bytes.
// One barrier per output row.  bf16, 64 output channels, plain tail (bias, optional ReLU).
// ---------------------------------------------------------------------------
constexpr int kBlkPixBytes = 32;
constexpr int kBlkRing = 5;

__global__ __launch_bounds__(256, 2) void conv_blocks4x4_kernel(IgemmArgs p, int rows_per_wg, int wgs_per_image) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), h = lane >> 5;
  const int n = (int)blockIdx.x / wgs_per_image, blk = (int)blockIdx.x % wgs_per_image;
  const int oy0 = blk * rows_per_wg;
  const int oy1 = oy0 + rows_per_wg < p.OH ? oy0 + rows_per_wg : p.OH;
  if (oy0 >= oy1) return;
  const int Wp = p.OW + 3;                      // pixel slots of an LDS row: source columns -PW .. OW + 2 - PW
  const int row_bytes = Wp * kBlkPixBytes;
  const int n_chunks = Wp * 2;                  // 16-byte chunks of a row (at most 2 per thread: OW <= 128)
  float* const bias = (float*)(smem + kBlkRing * row_bytes);
  unsigned char* const staging = smem + kBlkRing * row_bytes + 256;  // 4 KB per wavefront

  // the filter: MFMA row i of block j holds output channel 32j + 16 ((i >> 2) & 1) + 4 (i >> 3) + (i & 3)
  i32x4_t breg[16][2];
  {
    const int i = lane & 31;
    const int c = 16 * ((i >> 2) & 1) + 4 * (i >> 3) + (i & 3);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const unsigned char* src = (const unsigned char*)p.Bt + (int64_t)(32 * j + c) * p.ldbt * 2 + h * 16;
#pragma unroll
      for (int t = 0; t < 16; ++t) breg[t][j] = *(const i32x4_t*)(src + t * kBlkPixBytes);
    }
  }
  if (tid < 64) bias[tid] = p.init != nullptr ? load_scalar<float, int>(p.init, (int64_t)tid * p.init_cs, p.init_dtype).f : 0.f;

  // one re-blocked input row (or zeros where it lies outside the image) -> registers -> its ring slot
  auto fetch_row = [&](int sy, i32x4_t (&regs)[2]) {
    const bool row_ok = (unsigned)sy < (unsigned)p.H;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int c = tid + 256 * k, col = (c >> 1) - p.PW;
      regs[k] = i32x4_t{0, 0, 0, 0};
      if (!(c < n_chunks && row_ok && (unsigned)col < (unsigned)p.W)) continue;
      if (p.raw_in == nullptr) {
        regs[k] = *(const i32x4_t*)((const unsigned char*)p.A + (((int64_t)n * p.H + sy) * p.W + col) * kBlkPixBytes + (c & 1) * 16);
      } else {
        // block (sy, col) of a 3-channel image: pixels (2 sy, 2 col), (2 sy, 2 col + 1) -- 12 contiguous bytes --
        // then the same two of row 2 sy + 1, then 8 bytes of zeros; the width is even, so both runs start on
        // 4-byte boundaries
        const int* top = (const int*)((const unsigned char*)p.raw_in + (((int64_t)n * p.raw_h + 2 * sy) * p.raw_w + 2 * col) * 6);
        const int* bot = top + p.raw_w * 6 / 4;
        const bool bot_ok = 2 * sy + 1 < p.raw_h;
        if ((c & 1) == 0)
          regs[k] = i32x4_t{top[0], top[1], top[2], bot_ok ? bot[0] : 0};
        else if (bot_ok)
          regs[k] = i32x4_t{bot[1], bot[2], 0, 0};
      }
    }
  };
  auto put_row = [&](int ring_slot, const i32x4_t (&regs)[2]) {
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int c = tid + 256 * k;
      if (c < n_chunks) *(i32x4_t*)(smem + ring_slot * row_bytes + c * 16) = regs[k];
    }
  };
  // output row oy reads source rows oy - PH .. oy - PH + 3, kept in ring slots oy % 5 .. (oy + 3) % 5
  {
    i32x4_t regs[2];
    for (int t = 0; t < 4; ++t) {
      fetch_row(oy0 - p.PH + t, regs);
      put_row((oy0 + t) % kBlkRing, regs);
    }
  }
  __syncthreads();

  const float lo = p.tail_relu ? 0.f : -__builtin_inff();
  // Two fetches are in flight: the row the next step needs (`due`, requested one step ago and written to its slot at
  // the end of this step) and the row the step after that needs (`later`, requested now).  One step's arithmetic is
  // shorter than a trip to memory; two steps' worth of it covers more of one.
  auto step = [&](int oy, i32x4_t (&due)[2], i32x4_t (&later)[2]) {
    const bool more = oy + 1 < oy1;
    if (oy + 2 < oy1) fetch_row(oy + 5 - p.PH, later);
    for (int b = wave; b * 32 < p.OW; b += 4) {
      const int ox = b * 32 + (lane & 31);
      const int oxc = ox < p.OW ? ox : p.OW - 1;  // lanes past the row's end multiply its last pixel and store nothing
      f32x16_t acc[2];
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const f32x4_t v = *(const f32x4_t*)(bias + 32 * j + 16 * h + 4 * q);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[j][4 * q + e] = v[e];
        }
#pragma unroll
      for (int ty = 0; ty < 4; ++ty) {
        const unsigned char* base = smem + ((oy + ty) % kBlkRing) * row_bytes + oxc * kBlkPixBytes + h * 16;
#pragma unroll
        for (int tx = 0; tx < 4; ++tx) {
          const i32x4_t fa = *(const i32x4_t*)(base + tx * kBlkPixBytes);
#pragma unroll
          for (int j = 0; j < 2; ++j) mma_block<KIND_BF16>(acc[j], breg[ty * 4 + tx][j], fa);
        }
      }
      // The wavefront's 32 pixels x 128 bytes go through its own 4 KB of LDS, so that a store instruction writes
      // whole 128-byte lines (8 lanes per pixel) instead of 16 bytes in each of 64 lines.  The 16-byte chunks of a
      // pixel sit at positions XORed with the pixel number (bank conflicts of the writes: 4-way instead of 32-way).
      unsigned char* const stage = staging + wave * 4096;
      {
        const int px = lane & 31;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            unsigned w[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              float v0 = acc[j][8 * half + 2 * k], v1 = acc[j][8 * half + 2 * k + 1];
              v0 = relu_clamp(v0, lo);
              v1 = relu_clamp(v1, lo);
              const f32x2_t pair = {v0, v1};
              const bf16x2_t hh = __builtin_convertvector(pair, bf16x2_t);
              __builtin_memcpy(&w[k], &hh, 4);
            }
            const int chunk = 4 * j + 2 * h + half;  // channels 32 j + 16 h + 8 half .. + 7
            *(u32x4_t*)(stage + px * 128 + ((chunk ^ (px & 7)) << 4)) = u32x4_t{w[0], w[1], w[2], w[3]};
          }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      {
        const int chunk = lane & 7;
        unsigned char* const out_row = (unsigned char*)p.C + (((int64_t)n * p.OH + oy) * p.OW + b * 32) * p.ldc * 2 + chunk * 16;
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const int px = it * 8 + (lane >> 3);
          const u32x4_t v = *(const u32x4_t*)(stage + px * 128 + ((chunk ^ (px & 7)) << 4));
          if (b * 32 + px < p.OW) *(u32x4_t*)(out_row + (int64_t)px * p.ldc * 2) = v;
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
    if (more) put_row((oy + 4) % kBlkRing, due);  // the slot of row oy - 1, which nothing reads any more
    __syncthreads();
  };
  i32x4_t ra[2], rb[2];
  if (oy0 + 1 < oy1) fetch_row(oy0 + 4 - p.PH, ra);
  for (int oy = oy0; oy < oy1; oy += 2) {
    step(oy, ra, rb);
    if (oy + 1 < oy1) step(oy + 1, rb, ra);
  }
}


// The same walk with eight wavefronts per workgroup: wavefront w takes pixel block w % 4 (32 pixels) and the 32 output
// channels w / 4, so it holds half of the filter (64 registers) and four wavefronts share a SIMD (two workgroups per
// CU) instead of two -- twice the wavefronts to cover the chain LDS read -> MFMAs -> conversion -> store of a row step.
// A pixel's 128 bytes now come from two wavefronts: a finished row is staged in LDS (one 4 KB area per pixel block,
// two sets taking turns by row parity) and goes to memory at the start of the next step, after the step's barrier,
// every wavefront storing 16 pixels of its pixel block as whole 128-byte lines.
// POOL: the rows are not stored; the last four stay in LDS (the staging areas, taking turns by row number) and a 3x3
// stride-2 max-pool over them leaves instead (p.pool_*): rows_per_wg then counts pooled rows, and a workgroup computes
// the convolution rows its pooled rows cover (one more than twice as many: neighbouring workgroups both compute the row
// between them).  The values pooled are the stored bf16 values and the comparisons those of pool_flat_kernel, so the
// result is, bit for bit, that of the two launches.
template <bool POOL>
__global__ __launch_bounds__(512, 4) void conv_blocks4x4_w8_kernel(IgemmArgs p, int rows_per_wg, int wgs_per_image) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), h = lane >> 5;
  const int pb = wave & 3, j = wave >> 2;
  const int n = (int)blockIdx.x / wgs_per_image, blk = (int)blockIdx.x % wgs_per_image;
  int oy0 = blk * rows_per_wg;
  int oy1 = oy0 + rows_per_wg < p.OH ? oy0 + rows_per_wg : p.OH;
  int py0 = 0, py1 = 0;  // POOL: the workgroup's pooled rows
  if (POOL) {
    py0 = blk * rows_per_wg;
    py1 = py0 + rows_per_wg < p.pool_oh ? py0 + rows_per_wg : p.pool_oh;
    oy0 = 2 * py0 - p.pool_pt < 0 ? 0 : 2 * py0 - p.pool_pt;
    oy1 = 2 * (py1 - 1) - p.pool_pt + 3 < p.OH ? 2 * (py1 - 1) - p.pool_pt + 3 : p.OH;
    if (py0 >= py1) return;
  }
  if (oy0 >= oy1) return;
  const int Wp = p.OW + 3;                      // pixel slots of an LDS row: source columns -PW .. OW + 2 - PW
  const int row_bytes = Wp * kBlkPixBytes;
  const int n_chunks = Wp * 2;                  // 16-byte chunks of a row (at most one per thread: OW <= 128)
  float* const bias = (float*)(smem + kBlkRing * row_bytes);
  // staged result rows: two sets of four pixel blocks of 4 KB; POOL: four sets of OW pixels of 128 bytes (a row being
  // staged then never takes the place of one of the three a pooled row may still be reading)
  unsigned char* const staging = smem + kBlkRing * row_bytes + 256;
  constexpr int kSets = POOL ? 4 : 2;
  const int set_bytes = POOL ? p.OW * 128 : 4 * 4096;

  // the filter of the wavefront's 32 channels: MFMA row i holds output channel 32j + 16 ((i >> 2) & 1) + 4 (i >> 3) + (i & 3)
  i32x4_t breg[16];
  {
    const int i = lane & 31;
    const int c = 16 * ((i >> 2) & 1) + 4 * (i >> 3) + (i & 3);
    const unsigned char* src = (const unsigned char*)p.Bt + (int64_t)(32 * j + c) * p.ldbt * 2 + h * 16;
#pragma unroll
    for (int t = 0; t < 16; ++t) breg[t] = *(const i32x4_t*)(src + t * kBlkPixBytes);
  }
  if (tid < 64) bias[tid] = p.init != nullptr ? load_scalar<float, int>(p.init, (int64_t)tid * p.init_cs, p.init_dtype).f : 0.f;

  // one re-blocked input row (or zeros where it lies outside the image) -> a register -> its ring slot
  auto fetch_row = [&](int sy) {
    i32x4_t v = {0, 0, 0, 0};
    const int c = tid, col = (c >> 1) - p.PW;
    if (!(c < n_chunks && (unsigned)sy < (unsigned)p.H && (unsigned)col < (unsigned)p.W)) return v;
    if (p.raw_in == nullptr) return *(const i32x4_t*)((const unsigned char*)p.A + (((int64_t)n * p.H + sy) * p.W + col) * kBlkPixBytes + (c & 1) * 16);
    // block (sy, col) of a 3-channel image: pixels (2 sy, 2 col), (2 sy, 2 col + 1) -- 12 contiguous bytes -- then the
    // same two of row 2 sy + 1, then 8 bytes of zeros; the width is even, so both runs start on 4-byte boundaries
    const int* top = (const int*)((const unsigned char*)p.raw_in + (((int64_t)n * p.raw_h + 2 * sy) * p.raw_w + 2 * col) * 6);
    const int* bot = top + p.raw_w * 6 / 4;
    const bool bot_ok = 2 * sy + 1 < p.raw_h;
    if ((c & 1) == 0) return i32x4_t{top[0], top[1], top[2], bot_ok ? bot[0] : 0};
    if (bot_ok) v = i32x4_t{bot[1], bot[2], 0, 0};
    return v;
  };
  auto put_row = [&](int ring_slot, const i32x4_t& v) {
    if (tid < n_chunks) *(i32x4_t*)(smem + ring_slot * row_bytes + tid * 16) = v;
  };
  // output row oy reads source rows oy - PH .. oy - PH + 3, kept in ring slots oy % 5 .. (oy + 3) % 5
  for (int t = 0; t < 4; ++t) put_row((oy0 + t) % kBlkRing, fetch_row(oy0 - p.PH + t));
  __syncthreads();

  const float lo = p.tail_relu ? 0.f : -__builtin_inff();
  // the staged row oy leaves for memory: the wavefront's 16 pixels of its pixel block, eight lanes per pixel
  auto store_row = [&](int oy) {
    const unsigned char* const stage = staging + (oy % kSets) * set_bytes + pb * 4096;
    const int chunk = lane & 7;
    unsigned char* const out_row = (unsigned char*)p.C + (((int64_t)n * p.OH + oy) * p.OW + pb * 32) * p.ldc * 2 + chunk * 16;
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int px = 16 * j + it * 8 + (lane >> 3);
      const u32x4_t v = *(const u32x4_t*)(stage + px * 128 + ((chunk ^ (px & 7)) << 4));
      if (pb * 32 + px < p.OW) *(u32x4_t*)(out_row + (int64_t)px * p.ldc * 2) = v;
    }
  };
  // POOL: pooled row py out of the staged rows 2 py - pool_pt .. + 2 (those that exist): a thread per pooled pixel and
  // 16-byte chunk of channels, taps in rising window index, a tap replacing the running value when it is greater (a NaN
  // never is).  Behind a ReLU the staged values are +0 and above, or -infinity where the convolution gave NaN (see the
  // staging below): bf16 values of that kind compare like the 16-bit integers they are, two per instruction.
  // (a thread's three window columns are the same for every pooled row: their offsets inside a staged row, once)
  int pool_col[3] = {0, 0, 0};
  if (POOL) {
    const int ppx = tid >> 3, chunk = tid & 7;
#pragma unroll
    for (int kx = 0; kx < 3; ++kx) {
      int c = 2 * ppx - p.pool_pl + kx;
      c = c < 0 ? 0 : (c > p.OW - 1 ? p.OW - 1 : c);
      const int px = c & 31;
      pool_col[kx] = c * 128 + ((chunk ^ (px & 7)) << 4);
    }
  }
  auto pool_row = [&](int py) {
    const int ppx = tid >> 3, chunk = tid & 7;
    if (ppx >= p.pool_ow) return;
    typedef short i16x2_t __attribute__((ext_vector_type(2)));
    auto max_i16x2 = [](unsigned a, unsigned b) {
      return __builtin_bit_cast(unsigned, __builtin_elementwise_max(__builtin_bit_cast(i16x2_t, a), __builtin_bit_cast(i16x2_t, b)));
    };
    float best[8];
    unsigned best2[4];
#pragma unroll
    for (int e = 0; e < 8; ++e) best[e] = -__builtin_inff();
#pragma unroll
    for (int q = 0; q < 4; ++q) best2[q] = 0xff80ff80u;  // -infinity twice
    // A tap outside the image is replaced by the nearest one inside, which belongs to the same window: the maximum is
    // the same and no lane branches.  A window row's three reads are under way together (all nine would not fit the
    // registers beside the filter).
#pragma unroll
    for (int ky = 0; ky < 3; ++ky) {
      int r = 2 * py - p.pool_pt + ky;
      r = r < 0 ? 0 : (r > p.OH - 1 ? p.OH - 1 : r);
      u32x4_t v[3];
      const unsigned char* const row = staging + (r % kSets) * set_bytes;
#pragma unroll
      for (int kx = 0; kx < 3; ++kx) v[kx] = *(const u32x4_t*)(row + pool_col[kx]);
      if (p.tail_relu) {
#pragma unroll
        for (int k = 0; k < 3; ++k)
#pragma unroll
          for (int q = 0; q < 4; ++q) best2[q] = max_i16x2(best2[q], v[k][q]);
      } else {
#pragma unroll
        for (int k = 0; k < 3; ++k)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float lo_half = __uint_as_float(v[k][q] << 16), hi_half = __uint_as_float(v[k][q] & 0xffff0000u);
            best[2 * q] = lo_half > best[2 * q] ? lo_half : best[2 * q];
            best[2 * q + 1] = hi_half > best[2 * q + 1] ? hi_half : best[2 * q + 1];
          }
      }
    }
    u32x4_t o;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      o[q] = p.tail_relu ? best2[q] : (__float_as_uint(best[2 * q]) >> 16) | (__float_as_uint(best[2 * q + 1]) & 0xffff0000u);
    *(u32x4_t*)((unsigned char*)p.C + ((((int64_t)n * p.pool_oh + py) * p.pool_ow + ppx) * p.ldc + chunk * 8) * 2) = o;
  };
  // the pooled rows whose last existing window row is `oy` (at most two: a whole window, and one cut off by the image's
  // end); true if there was one
  auto pool_after = [&](int oy) {
    bool any = false;
    for (int py = py0; py < py1; ++py) {
      const int last = 2 * py - p.pool_pt + 2 < p.OH - 1 ? 2 * py - p.pool_pt + 2 : p.OH - 1;
      if (last != oy) continue;
      pool_row(py);
      any = true;
    }
    return any;
  };
  // Two fetches are in flight: the row the next step needs (`due`) and the row the step after that needs (`later`).
  auto step = [&](int oy, i32x4_t& due, i32x4_t& later) {
    const bool more = oy + 1 < oy1;
    if (oy + 2 < oy1) later = fetch_row(oy + 5 - p.PH);
    if (!POOL && oy > oy0) store_row(oy - 1);
    // POOL: the pooled rows that row oy - 1 completed go first, at every wavefront's own pace beside the others' MFMAs
    if (POOL && oy > oy0) pool_after(oy - 1);
    const bool active = pb * 32 < p.OW;  // (a row of at most 96 pixels leaves pixel blocks, and their wavefronts, without work)
    f32x16_t acc;
    if (active) {
      const int ox = pb * 32 + (lane & 31);
      const int oxc = ox < p.OW ? ox : p.OW - 1;  // lanes past the row's end multiply its last pixel; their values are staged and never stored
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const f32x4_t v = *(const f32x4_t*)(bias + 32 * j + 16 * h + 4 * q);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[4 * q + e] = v[e];
      }
#pragma unroll
      for (int ty = 0; ty < 4; ++ty) {
        const unsigned char* base = smem + ((oy + ty) % kBlkRing) * row_bytes + oxc * kBlkPixBytes + h * 16;
#pragma unroll
        for (int tx = 0; tx < 4; ++tx) mma_block<KIND_BF16>(acc, breg[ty * 4 + tx], *(const i32x4_t*)(base + tx * kBlkPixBytes));
      }
    }
    if (active) {
      // the lane's 16 channels 32 j + 16 h .. of pixel lane % 32: two 16-byte chunks of the pixel's 128 bytes, at positions
      // XORed with the pixel number
      unsigned char* const stage = staging + (oy % kSets) * set_bytes + pb * 4096;
      const int px = lane & 31;
      const bool staged = !POOL || pb * 32 + px < p.OW;  // (POOL: a set ends with the row's last pixel)
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        unsigned w[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          float v0 = acc[8 * half + 2 * k], v1 = acc[8 * half + 2 * k + 1];
          v0 = relu_clamp(v0, lo);
          v1 = relu_clamp(v1, lo);
          if (POOL && p.tail_relu) {  // a NaN is never the maximum of a window: it is staged as the value every other one beats
            v0 = v0 != v0 ? -__builtin_inff() : v0;
            v1 = v1 != v1 ? -__builtin_inff() : v1;
          }
          const f32x2_t pair = {v0, v1};
          const bf16x2_t hh = __builtin_convertvector(pair, bf16x2_t);
          __builtin_memcpy(&w[k], &hh, 4);
        }
        const int chunk = 4 * j + 2 * h + half;  // channels 32 j + 16 h + 8 half .. + 7
        if (staged) *(u32x4_t*)(stage + px * 128 + ((chunk ^ (px & 7)) << 4)) = u32x4_t{w[0], w[1], w[2], w[3]};
      }
    }
    if (more) put_row((oy + 4) % kBlkRing, due);  // the slot of row oy - 1, which nothing reads any more
    __syncthreads();
  };
  i32x4_t ra = {0, 0, 0, 0}, rb = {0, 0, 0, 0};
  if (oy0 + 1 < oy1) ra = fetch_row(oy0 + 4 - p.PH);
  for (int oy = oy0; oy < oy1; oy += 2) {
    step(oy, ra, rb);
    if (oy + 1 < oy1) step(oy + 1, rb, ra);
  }
  if (!POOL) store_row(oy1 - 1);
  if (POOL) pool_after(oy1 - 1);
}

}  // namespace

// Does the re-blocked convolution `a` (as conv_args describes it: H x W blocks of pix_pitch bytes, KH block rows of
// CI = 4 blocks x 16 channels) fit conv_blocks4x4_kernel?  Returns the LDS bytes it needs, or 0.
size_t conv_blocks4x4_prepare(int kind, const IgemmArgs& a) {
  if (kind != KIND_BF16 || a.KH != 4 || a.KW != 1 || a.CI != 64 || a.pix_pitch != kBlkPixBytes || a.K != 256) return 0;
  if (a.N != 64 || a.ldbt != 256 || a.OW > 128 || a.OW < 1 || a.SH != 1 || a.SW != 1 || a.DH != 1 || a.DW != 1) return 0;
  if (a.PH < 0 || a.PH > 3 || a.PW < 0 || a.PW > 3) return 0;
  if (a.tail_mode != 1 || a.out_dtype != PML_HIP_BF16 || a.c_dtype != PML_HIP_BF16 || a.init_rs != 0) return 0;
  if ((a.ldc * 2) % 16 != 0 || (((uintptr_t)a.C | (uintptr_t)a.Bt) & 15) != 0) return 0;
  return (size_t)kBlkRing * (a.OW + 3) * kBlkPixBytes + 64 * 4 + 4 * 4096;
}

hipError_t conv_blocks4x4_launch(const IgemmArgs& a, size_t lds, int n_cus, hipStream_t s) {
  // two workgroups per CU, each a run of consecutive output rows (with a fused pool: pooled rows) of one image
  const int out_rows = a.pool ? a.pool_oh : a.OH;
  int per_image = (2 * n_cus + a.NB - 1) / a.NB;
  per_image = per_image < 1 ? 1 : (per_image > out_rows ? out_rows : per_image);
  const int rows = (out_rows + per_image - 1) / per_image;
  per_image = (out_rows + rows - 1) / rows;
  // Runs of two rows and more take the eight-wavefront form (128 x 224 x 224 x 3: 76 us against 98-104 on one device; 8 and
  // 12 images, runs of two and three rows: 14.4 against 15.2 and 16.6 against 17.5).  One row per workgroup -- up to four
  // images -- is all prologue; there the two forms are within a microsecond of each other, the smaller one ahead as the
  // first kernel of a network (12.4 against 13.6 us), the larger one in a loop of its own (7.4 against 8.0).  The fused
  // pool exists in the eight-wavefront form only.
  if (rows >= 2 || a.pool) {
    const size_t lds8 = (size_t)kBlkRing * (a.OW + 3) * kBlkPixBytes + 64 * 4 + (a.pool ? (size_t)4 * a.OW * 128 : (size_t)8 * 4096);
    auto kern = a.pool ? conv_blocks4x4_w8_kernel<true> : conv_blocks4x4_w8_kernel<false>;
    static DynamicLdsLimit limit8[2];
    if (hipError_t e = limit8[a.pool ? 1 : 0].ensure((const void*)kern, lds8); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)(a.NB * per_image)), dim3(512), lds8, s, a, rows, per_image);
    return hipGetLastError();
  }
  static DynamicLdsLimit limit;
  if (hipError_t e = limit.ensure((const void*)conv_blocks4x4_kernel, lds); e != hipSuccess) return e;
  hipLaunchKernelGGL(conv_blocks4x4_kernel, dim3((unsigned)(a.NB * per_image)), dim3(256), lds, s, a, rows, per_image);
  return hipGetLastError();
}

size_t conv_halo_prepare(int kind, IgemmArgs* a, bool filter_in_lds) {
  const int es = kind == KIND_BF16 ? 2 : (kind == KIND_I8 ? 1 : 4);
  if (a->SH != 1 || a->SW != 1 || a->DH != 1 || a->DW != 1) return 0;
  if ((int64_t)a->CI * es != kPixBytes) return 0;
  if (a->N > kBN || (a->N & 7) != 0 || (a->ldc & 3) != 0) return 0;
  if (a->PH >= a->KH || a->PW >= a->KW) return 0;
  // the padded image must be exactly what the output geometry implies
  const int Hv = a->OH + a->KH - 1, Wv = a->OW + a->KW - 1;
  if (Hv < a->H + a->PH || Wv < a->W + a->PW) return 0;
  if (a->M >= ((int64_t)1 << 31) - ((int64_t)1 << 20)) return 0;  // tile numbers past the end must not wrap
  const int64_t per = (int64_t)a->OH * a->OW;
  const int64_t n_tiles = (a->M + kBM - 1) / kBM;
  int max_rows = 0;
  for (int64_t t = 0; t < n_tiles; ++t) {
    const int64_t m0 = t * kBM;
    int64_t ml = m0 + kBM - 1;
    if (ml > a->M - 1) ml = a->M - 1;
    const int64_t v0 = (m0 / per) * Hv + (m0 % per) / a->OW;
    const int64_t vl = (ml / per) * Hv + (ml % per) / a->OW;
    const int rows = (int)(vl - v0) + a->KH;
    if (rows > max_rows) max_rows = rows;
  }
  const int nchunks = (Wv + 31) / 32;
  if ((int64_t)max_rows * nchunks > kMaxLoads) return 0;
  const size_t filter = (size_t)kBN * ((size_t)a->KH * a->KW * kPixBytes + 16);
  size_t window = (size_t)max_rows * Wv * kPixStride;
  const size_t ctile = (size_t)kBM * (kBN + 4) * 4;
  if (window < ctile) window = ctile;
  const size_t total = filter + window;
  if (total > 160 * 1024) return 0;
  a->halo_rows = max_rows;
  a->n_tiles = (int)n_tiles;
  fast_div_magic((unsigned)per, &a->div_per_magic, &a->div_per_shift);
  fast_div_magic((unsigned)a->OW, &a->div_ow_magic, &a->div_ow_shift);
  // the pipelined 3x3 kernel: fast tail only, 64 channels out, buffer-addressable operands
  const int out_es = kind == KIND_BF16 ? 2 : 4;
  const bool out_fits = kind == KIND_BF16 ? a->out_dtype == PML_HIP_BF16 : true;
  a->halo_variant = (a->KH == 3 && a->KW == 3 && a->N == kBN && a->tail_mode == 1 && a->init_rs == 0 && out_fits &&
                     (int64_t)a->NB * a->H * a->W * kPixBytes <= ((int64_t)1 << 30) &&
                     a->M * a->ldc * out_es < ((int64_t)1 << 31) && nchunks <= 2)
                        ? nchunks
                        : 0;
  // filter in registers: 16- and 8-bit elements, two windows of at most kRegRows rows of 32 .. 64 pixels in LDS
  // (filter_in_lds: the caller's schedule keeps the filter in LDS)
  if (a->halo_variant && kind != KIND_F32 && max_rows <= kRegRows && Wv >= 32 && Wv <= 64 &&
      reg_lds_bytes(Wv) <= 160 * 1024 && !filter_in_lds) {
    a->halo_variant = 3;
    return (size_t)reg_lds_bytes(Wv);
  }
  return total;
}

// The image passes through the first window buffer while the first window arrives in the second: it must fit there.
bool regfilter_takes_image(int ow) { return (size_t)reg_win_bytes(ow + 2) >= kRegfilterImageBytes; }

hipError_t regfilter_image_launch(const void* bt, int64_t ldbt_bytes, void* image, hipStream_t s) {
  if ((((uintptr_t)bt | (uintptr_t)image) & 15) != 0 || ldbt_bytes % 16 != 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(regfilter_image_kernel, dim3(2 * 36 * 64 / 256), dim3(256), 0, s, (const unsigned char*)bt, ldbt_bytes, (i32x4_t*)image);
  return hipGetLastError();
}

hipError_t conv_halo_launch(int kind, const IgemmArgs& a, size_t lds_bytes, int n_cus, hipStream_t s) {
  if (a.halo_variant == 1) {
    switch (kind) {
      case KIND_F32: return launch3x3<KIND_F32, 1>(a, lds_bytes, n_cus, s);
      case KIND_BF16: return launch3x3<KIND_BF16, 1>(a, lds_bytes, n_cus, s);
      case KIND_I8: return launch3x3<KIND_I8, 1>(a, lds_bytes, n_cus, s);
    }
  } else if (a.halo_variant == 3) {
    switch (kind) {
      // 56-pixel rows (58 with padding) are compiled in
      case KIND_BF16:
        return a.OW + 2 == 58 ? launch_regfilter<KIND_BF16, 58>(a, lds_bytes, n_cus, s)
                              : launch_regfilter<KIND_BF16, 0>(a, lds_bytes, n_cus, s);
      case KIND_I8:
        return a.OW + 2 == 58 ? launch_regfilter<KIND_I8, 58>(a, lds_bytes, n_cus, s)
                              : launch_regfilter<KIND_I8, 0>(a, lds_bytes, n_cus, s);
    }
    return hipErrorInvalidValue;
  } else if (a.halo_variant == 2) {
    switch (kind) {
      case KIND_F32: return launch3x3<KIND_F32, 2>(a, lds_bytes, n_cus, s);
      case KIND_BF16: return launch3x3<KIND_BF16, 2>(a, lds_bytes, n_cus, s);
      case KIND_I8: return launch3x3<KIND_I8, 2>(a, lds_bytes, n_cus, s);
    }
  }
  switch (kind) {
    case KIND_F32: return launch<KIND_F32>(a, lds_bytes, n_cus, s);
    case KIND_BF16: return launch<KIND_BF16>(a, lds_bytes, n_cus, s);
    case KIND_I8: return launch<KIND_I8>(a, lds_bytes, n_cus, s);
  }
  return hipErrorInvalidValue;
}

}  // namespace pml
