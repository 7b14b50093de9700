// The C ABI of the kernel library (include/pml_hip.h): device set-up, memory,
// streams and the dispatch / invoke pairs that select a tiling once and launch
// it many times.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "device_common.h"
#include "plans.h"

namespace pml {
namespace {

thread_local std::string g_err;

int fail(const std::string& msg) {
  g_err = msg;
  return 1;
}
int check(hipError_t e, const char* what) {
  if (e == hipSuccess) return 0;
  g_err = std::string(what) + ": " + hipGetErrorString(e);
  return 1;
}

enum PlanKind { PLAN_GEMM = 1, PLAN_CONV, PLAN_DWCONV, PLAN_POOL, PLAN_ELTWISE, PLAN_CONTRACT };

struct Plan {
  int kind = 0;
  int mfma_kind = 0;
  int tile = 0;
  pml_hip_gemm_desc gemm;
  pml_hip_conv2d_desc conv;
  pml_hip_dwconv2d_desc dw;
  pml_hip_pool2d_desc pool;
  pml_hip_eltwise_desc elt;
  pml_hip_contract_desc con;
  // packed right-hand side Bt[N][K]
  void* bt = nullptr;
  int64_t bt_ld = 0;
  size_t bt_bytes = 0;
  bool packed = false;
  bool b_split = false;  // split fp32 kind: a right-hand side packed once is kept as bf16 heads + remainders
  std::atomic<bool> bt_is_split{false};  // ... and `bt` holds that form now (invokes that bring their own right-hand side clear it)
  // second product of a GEMM: its packed right-hand side Bt2[N][K2]
  void* bt2 = nullptr;
  bool packed2 = false;
  // convolution whose channels do not fill 16-byte vectors: patch matrix [M][kpad] + GEMM
  void* patches = nullptr;
  int64_t kpad = 0;
  // stride-2 convolution over few channels, run as a unit-stride one over 2x2 pixel blocks: the
  // re-blocked input [N][s2d_h][s2d_w][s2d_ch]; filter taps s2d_ka x s2d_kaw blocks
  // (allocated by the first invoke that needs it: the row-walking stem kernel builds its blocks from the image)
  bool via_s2d = false;
  void* s2d = nullptr;
  std::mutex s2d_mutex;
  int s2d_h = 0, s2d_w = 0, s2d_ch = 0, s2d_ka = 0, s2d_kaw = 0;
  // depthwise convolution: a constant filter kept by the plan ([kh][kw][c] as the caller holds it), and its paired
  // form for the 3x3 bf16 kernel when every weight is finite
  void* dw_filter = nullptr;
  void* dw_paired = nullptr;
  // K split over workgroups: workspace of partial tiles and how the slabs are shared out (splits < 2: no split)
  void* ws = nullptr;
  int sk_splits = 0, sk_per = 0, sk_pitch = 0;
  // register-filter convolution: a filter packed once, in the order the kernel holds it in registers
  void* reg_image = nullptr;
  // resident-filter convolution: LDS bytes (0 = not used), window rows, tile count, CUs of the device
  size_t halo_lds = 0;
  int halo_rows = 0, halo_tiles = 0, halo_variant = 0, n_cus = 0;
  std::string text;
  ~Plan() {
    if (bt) (void)hipFree(bt);
    if (bt2) (void)hipFree(bt2);
    if (patches) (void)hipFree(patches);
    if (s2d) (void)hipFree(s2d);
    if (reg_image) (void)hipFree(reg_image);
    if (ws) (void)hipFree(ws);
    if (dw_filter) (void)hipFree(dw_filter);
    if (dw_paired) (void)hipFree(dw_paired);
  }
};

int mfma_kind_of(int in_dtype, int flags = 0) {
  switch (in_dtype) {
    case PML_HIP_F32: return (flags & PML_HIP_FP32_AS_BF16X3) ? KIND_F32X3 : KIND_F32;
    case PML_HIP_BF16: return KIND_BF16;
    case PML_HIP_I8: return KIND_I8;
  }
  return -1;
}

const char* tile_name(int t) {
  switch (t) {
    case TILE_64x64: return "64x64";
    case TILE_128x64: return "128x64";
    case TILE_128x128: return "128x128";
    case TILE_128x64_W8: return "128x64 (8 wavefronts)";
    case TILE_128x128_W8: return "128x128 (8 wavefronts)";
    case TILE_256x128_W16: return "256x128 (16 wavefronts)";
    case TILE_64x64_W8_K2: return "64x64 (8 wavefronts, K split in two)";
    case TILE_256x256_W8: return "256x256 (8 wavefronts of 128x64)";
    case TILE_128x64_N2: return "128x64 (4 wavefronts of 32x64)";
    case TILE_128x128_W8_S2: return "128x128 (8 wavefronts, 2 stages)";
    case TILE_192x384_W8: return "192x384 (8 wavefronts of 96x96)";
    case TILE_64x64_KSPLIT: return "64x64, K split over workgroups";
  }
  return "?";
}

constexpr int kScheduleBits = 0xff << 8 | 0xf << 16;
constexpr int kMaxpoolBits = 0x1f << 20;
bool schedule_bits_ok(int flags) {
  return PML_HIP_FLAG_TILE_OF(flags) < PML_HIP_TILE_COUNT_ && PML_HIP_FLAG_CONV_OF(flags) <= PML_HIP_CONV_BLOCKS;
}
const char* const kTileShort[PML_HIP_TILE_COUNT_] = {"64x64", "128x64", "128x128", "128x64w8", "128x128w8", "256x128w16", "128x128w8s2", "64x64w8k2", "256x256w8", "128x64n2", "192x384w8", "64x64ks"};

// Stated tiling choice per shape class.  Measured on MI355X, bf16 unless said otherwise (us; w8 / w16 =
// 8 / 16 wavefronts per workgroup; s2 = two ring stages and LDS cut to what the result tile needs, so that two
// workgroups share a CU; the 4-wavefront 256x128 and 256x256 tiles that were tried as well are slower than
// 256x128w16 everywhere and are no longer built):
//                                    64x64  128x64  128x128  128x128w8  128x128w8s2  256x128w16
//   4096^3 (int8)                      137       -      119        112          121          83
//   4096^3                             198       -      173        163          115         108
//   conv 128x28x28x128 (*) 3x3x128      66      76       89         71           49          52
//   conv 128x14x14x256 (*) 3x3x256      64      72       73         61           45          45
//   conv 128x7x7x512   (*) 3x3x512      72      67       64         57           65          77
//   conv 128x56x56x256 (*) 1x1x512 /2   83     101        -         99           62          74
//   gemm 401408x256x64                  82     127      177        123           76          84
//   gemm 100352x512x128                 52      71      100         70           44          51
//   gemm 25088x256x1024                 27      27       30         24           20          22
//   gemm 6272x512x2048                  25      23       25         21           30          28
//   gemm 23104x728x728                  72      67       78         65           57          58
//   gemm 128x1000x2048                  14       -        -         19           19          25
//   gemm 1024^3 (fp32)                  33      45       77         71            -         127
// A descriptor may name its tile (PML_HIP_FLAG_TILE); every tile is tested on a ragged problem that way.
// One tile per workgroup and a serial load / multiply / store life per tile: latency is hidden by the
// other wavefronts of a SIMD -- 8 or 16 per workgroup instead of 4 -- and, for the bandwidth-bound shapes
// with a short K, by a second workgroup on the CU whose loads run under the first one's tail.  So: long K
// and at least two rounds of 256x128 tiles take that tile with 16 wavefronts; otherwise 128x128 with 8
// wavefronts, two to a CU if that still gives every CU a workgroup, one to a CU (three stages) below
// that; and for small problems the smaller of 64x64 and 128x64 by (rounds of resident workgroups) x
// (tile area), the larger tile on a tie.
// forced: a tile named by the descriptor's schedule bits (PML_HIP_FLAG_TILE), -1 = none
int choose_tile(int64_t m, int64_t n, int64_t k_bytes, int kind = KIND_BF16, bool plain_tail = true, int forced = -1, bool allow_split = true) {
  if (forced >= 0 && forced < PML_HIP_TILE_COUNT_ && (forced != TILE_128x64_N2 || kind == KIND_F32X3) &&
      (forced != TILE_192x384_W8 || kind == KIND_BF16 || kind == KIND_I8))
    return forced;
  auto tiles = [&](int64_t bm, int64_t bn) { return ((m + bm - 1) / bm) * ((n + bn - 1) / bn); };
  // Few tiles and a long K (a network's last stages at batch 1: 49 x 512 x 4608 is 8 tiles of 72 slabs): the K loop is
  // shared out among workgroups and a second launch adds the partial tiles up.  Measured inside ResNet-50 at batch 1.
  if (allow_split && tiles(64, 64) <= 64 && k_bytes >= 2048) return TILE_64x64_KSPLIT;
  if (kind == KIND_F32X3) {
    // A fragment that is split in registers costs 24 vector instructions whatever it is multiplied with, so the
    // tile a wavefront holds decides how many MFMAs share that cost -- but the problems this kind meets here are
    // short of tiles first.  Measured: configs[1] fp32 (n = 64) 137 us with 64x64, 146 with 128x64 as 32x64 per
    // wavefront, 155 with 128x64 as 64x32; 1024^3 25-27 us with 64x64 (either form), 34-47 with larger tiles.
    if (n > 64 && tiles(128, 128) >= 512) return TILE_128x128;
    if (tiles(64, 64) <= 512 && k_bytes >= 2048) return TILE_64x64_W8_K2;
    return TILE_64x64;
  }
  if (n <= 64) return TILE_64x64;  // (the 7x7 stem of ResNet-50 over 2x2 pixel blocks: 191 us against 207 us with 128x64w8)
  // Long K, at least three quarters of a round of 256x256 tiles and little of them hanging over the edges:
  // eight wavefronts of 128x64 (0.75 KB of LDS fragment reads per MFMA instead of 1.5).  Measured with N(0,1) /
  // uniform int8 data, 4096^3: bf16 121 us against 139 (256x128, 16 wavefronts), int8 73 against 84.
  // (Not under a tail that runs in steps -- requantisation chains: a wavefront stages its 128x64 part through a
  // 16 KB share of LDS in four rounds, 4096^3 int8 with that tail 132 us against 106 with 256x128.)
  if (kind != KIND_F32 && plain_tail && k_bytes >= 2048 && tiles(256, 256) >= 192 && tiles(256, 256) * 65536 * 10 <= m * n * 11)
    return TILE_256x256_W8;
  // Eight wavefronts of 96 x 96 on a 192 x 384 tile: per MFMA half the global -> LDS bytes of a 128 x 128 tile (the vector
  // memory path moves 64 bytes per clock and CU, which 128 x 128 tiles use up entirely) and 0.67 KB of fragment reads.
  // One workgroup per CU, so its tail is not hidden by a neighbour: it pays where the K loop is most of the work, the
  // columns fill whole tiles and the tiles fill a round of the chip -- 23104 x 728 x 728 (242 tiles) 39 us against 48.
  if (kind != KIND_F32 && kind != KIND_F32X3 && k_bytes >= 1024) {
    const int64_t tn = (n + 383) / 384, t = tiles(192, 384);
    if (tn * 384 * 100 <= n * 108 && ((t >= 200 && t <= 256) || t >= 640)) return TILE_192x384_W8;
  }
  if (k_bytes >= 4096 && tiles(256, 128) >= 512) return TILE_256x128_W16;
  // One round of 256x128 tiles that fills at least three quarters of the chip, K of 2 KB and more per row, bf16: the
  // 16-wavefront tile instead of 1.53 rounds of 128x128 tiles -- 25088 x 256 results, ResNet-50's 14x14x256 layers at
  // batch 128: the 3x3 convolutions 38.9 -> 37.3 us, the 1x1 layers with K = 1024 26.7 -> 25.3, the network 2.59 -> 2.57 ms
  // (measured with a schedule file before the rule was written down).
  if (kind == KIND_BF16 && k_bytes >= 2048 && tiles(256, 128) >= 192 && tiles(256, 128) <= 256) return TILE_256x128_W16;
  if (tiles(128, 128) >= 256) return TILE_128x128_W8_S2;
  if (tiles(128, 128) >= 128) return TILE_128x128_W8;
  // at most two 64x64 tiles per CU and a long K: a second wavefront grid takes half of every slab
  // (fp32 1024^3: 32.5 -> 28.8 us; bf16 128x1000x2048: 13.4 -> 11.6 us; bf16 2048^3, 1024 tiles: 26.7 -> 40.5 us)
  if (tiles(64, 64) <= 512 && k_bytes >= 2048) return TILE_64x64_W8_K2;
  const int64_t rounds_small = (tiles(64, 64) + 5 * 256 - 1) / (5 * 256);
  const int64_t rounds_wide = (tiles(128, 64) + 2 * 256 - 1) / (2 * 256);
  return rounds_small < 2 * rounds_wide ? TILE_64x64 : TILE_128x64;
}

// A tail that is only "relu?" can use the fast store path.
void classify_tail(const pml_hip_epilogue& t, int out_dtype, int c_dtype, int* mode, int* relu) {
  *mode = 0;
  *relu = 0;
  // int32 accumulators followed by stores / casts between si32, f32, si8 / f32 arithmetic on immediates,
  // scalars and per-column vectors (requantisation): checked by walking the element type through the chain
  if (out_dtype == PML_HIP_I32 && t.n_ops >= 1 && t.n_ops <= 8) {
    int cur = PML_HIP_I32;
    bool ok = true;
    for (int i = 0; i < t.n_ops && ok; ++i) {
      const pml_hip_epi_op& op = t.ops[i];
      if (op.opcode == PML_HIP_EPI_STORE) continue;
      if (op.opcode == PML_HIP_EPI_CAST) {
        if (op.dtype != PML_HIP_F32 && op.dtype != PML_HIP_I32 && op.dtype != PML_HIP_I8) ok = false;
        if (cur == PML_HIP_I8 && op.dtype != PML_HIP_I8) ok = false;  // si8 is only ever the last type
        cur = op.dtype;
        continue;
      }
      switch (op.opcode) {
        case PML_HIP_EPI_ADD: case PML_HIP_EPI_SUB: case PML_HIP_EPI_RSUB: case PML_HIP_EPI_MUL: case PML_HIP_EPI_DIV:
        case PML_HIP_EPI_RDIV: case PML_HIP_EPI_MAX: case PML_HIP_EPI_MIN: case PML_HIP_EPI_RELU: case PML_HIP_EPI_NEG:
        case PML_HIP_EPI_MAX_GT: case PML_HIP_EPI_ROUND: case PML_HIP_EPI_FLOOR: case PML_HIP_EPI_CEIL:
          break;
        default:
          ok = false;
      }
      if (cur != PML_HIP_F32 || op.dtype != PML_HIP_F32) ok = false;
      if (op.operand_kind == PML_HIP_OPND_TENSOR) {
        const int q = op.operand;
        if (t.operand_dtype[q] != PML_HIP_F32 || t.operand_row_stride[q] != 0 ||
            (t.operand_col_stride[q] != 0 && t.operand_col_stride[q] != 1))
          ok = false;
      }
    }
    bool plain = true;  // a chain of nothing but "relu" on si32 stays with mode 1 below
    for (int i = 0; i < t.n_ops; ++i)
      if (t.ops[i].opcode != PML_HIP_EPI_RELU) plain = false;
    if (ok && !plain && cur == c_dtype) {
      *mode = 4;
      return;
    }
  }
  if (c_dtype != out_dtype) return;
  if (t.n_ops == 0) {
    *mode = 1;
    return;
  }
  if (t.n_ops == 1 && t.ops[0].opcode == PML_HIP_EPI_RELU && t.ops[0].dtype == out_dtype) {
    *mode = 1;
    *relu = 1;
    return;
  }
  // + residual (a full tensor of the result type, unit column stride, rows on 4-element boundaries), relu?
  if ((t.n_ops == 1 || t.n_ops == 2) && t.ops[0].opcode == PML_HIP_EPI_ADD && t.ops[0].operand_kind == PML_HIP_OPND_TENSOR &&
      t.ops[0].operand == 0 && t.ops[0].dtype == out_dtype && t.operand_dtype[0] == out_dtype &&
      t.operand_col_stride[0] == 1 && (t.operand_row_stride[0] & 3) == 0 &&
      (t.n_ops == 1 || (t.ops[1].opcode == PML_HIP_EPI_RELU && t.ops[1].dtype == out_dtype))) {
    *mode = 2;
    *relu = t.n_ops == 2;
    return;
  }
  // up to four float steps in the result type on immediates, scalars and per-column vectors
  if ((out_dtype == PML_HIP_F32 || out_dtype == PML_HIP_BF16) && t.n_ops >= 1 && t.n_ops <= 4) {
    bool ok = true;
    for (int i = 0; i < t.n_ops && ok; ++i) {
      const pml_hip_epi_op& op = t.ops[i];
      switch (op.opcode) {
        case PML_HIP_EPI_ADD: case PML_HIP_EPI_SUB: case PML_HIP_EPI_RSUB: case PML_HIP_EPI_MUL: case PML_HIP_EPI_DIV:
        case PML_HIP_EPI_RDIV: case PML_HIP_EPI_MAX: case PML_HIP_EPI_MIN: case PML_HIP_EPI_RELU: case PML_HIP_EPI_NEG:
        case PML_HIP_EPI_MAX_GT:
          break;
        default:
          ok = false;
      }
      if (op.dtype != out_dtype) ok = false;
      if (op.operand_kind == PML_HIP_OPND_TENSOR) {
        const int q = op.operand;
        if (t.operand_dtype[q] != out_dtype || t.operand_row_stride[q] != 0 ||
            (t.operand_col_stride[q] != 0 && t.operand_col_stride[q] != 1))
          ok = false;
      }
    }
    if (ok) *mode = 3;
  }
}

// The scale / shift (/ relu) chain of a folded batch normalisation, bf16 throughout: result * v0[col] + v1[col].
// 0: the chain is something else; 1: without relu; 2: with relu.
int tail_scale_shift(const pml_hip_epilogue& t, int out_dtype, int mode) {
  if (mode != 3 || out_dtype != PML_HIP_BF16 || (t.n_ops != 2 && t.n_ops != 3)) return 0;
  const int want[3] = {PML_HIP_EPI_MUL, PML_HIP_EPI_ADD, PML_HIP_EPI_RELU};
  for (int i = 0; i < t.n_ops; ++i) {
    const pml_hip_epi_op& op = t.ops[i];
    if (op.opcode != want[i] || op.dtype != PML_HIP_BF16) return 0;
    if (i < 2 && (op.operand_kind != PML_HIP_OPND_TENSOR || t.operand_col_stride[op.operand] != 1 || t.operand_row_stride[op.operand] != 0 ||
                  t.operand_dtype[op.operand] != PML_HIP_BF16))
      return 0;
  }
  return t.n_ops - 1;
}

// The requantisation chain of an int8 contraction: store? cast f32, mul by a per-column (or single) f32 tensor operand,
// maxgt immediate, min immediate, round, cast si8.  Fills the kernel arguments that describe it; false: something else.
bool tail_requant(const pml_hip_epilogue& t, int out_dtype, int c_dtype, int mode, IgemmArgs* g) {
  if (g) g->tail_rq = 0;
  if (mode != 4 || out_dtype != PML_HIP_I32 || c_dtype != PML_HIP_I8) return false;
  const int first = (t.n_ops > 0 && t.ops[0].opcode == PML_HIP_EPI_STORE) ? 1 : 0;
  if (t.n_ops != first + 6) return false;
  const pml_hip_epi_op* o = t.ops + first;
  const bool shape = o[0].opcode == PML_HIP_EPI_CAST && o[0].dtype == PML_HIP_F32 && o[1].opcode == PML_HIP_EPI_MUL &&
                     o[1].dtype == PML_HIP_F32 && o[1].operand_kind == PML_HIP_OPND_TENSOR && o[2].opcode == PML_HIP_EPI_MAX_GT &&
                     o[2].dtype == PML_HIP_F32 && o[2].operand_kind == PML_HIP_OPND_IMM && o[3].opcode == PML_HIP_EPI_MIN &&
                     o[3].dtype == PML_HIP_F32 && o[3].operand_kind == PML_HIP_OPND_IMM && o[4].opcode == PML_HIP_EPI_ROUND &&
                     o[4].dtype == PML_HIP_F32 && o[5].opcode == PML_HIP_EPI_CAST && o[5].dtype == PML_HIP_I8;
  if (!shape) return false;
  if (g) {
    g->tail_rq = 1;
    g->rq_store = first ? t.ops[0].operand : -1;
    g->rq_scale = o[1].operand;
    g->rq_lo = (float)o[2].imm;
    g->rq_hi = (float)o[3].imm;
  }
  return true;
}

// allow64: the standalone elementwise kernel also runs 64-bit steps; the tails of the contraction kernels do not
bool valid_tail(const pml_hip_epilogue& t, bool allow64 = false) {
  if (t.n_ops < 0 || t.n_ops > PML_HIP_MAX_EPI_OPS) return false;
  if (t.n_operands < 0 || t.n_operands > PML_HIP_MAX_EPI_OPERANDS) return false;
  for (int i = 0; i < t.n_ops; ++i) {
    const pml_hip_epi_op& op = t.ops[i];
    if (op.opcode < PML_HIP_EPI_ADD || op.opcode > PML_HIP_EPI_LAST_) return false;
    if (op.operand_kind == PML_HIP_OPND_TENSOR && (op.operand < 0 || op.operand >= t.n_operands)) return false;
    if (op.opcode == PML_HIP_EPI_STORE && (op.operand < 0 || op.operand >= PML_HIP_MAX_EPI_OPERANDS)) return false;
    if (!allow64 && dt_size(op.dtype) == 8 && op.opcode != PML_HIP_EPI_STORE) return false;  // 64-bit steps: general path only
  }
  return true;
}

// Compute units of the current device (persistent kernels size their grids by it).
int device_cus() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    hipDeviceProp_t prop;
    cached[dev] = hipGetDeviceProperties(&prop, dev) == hipSuccess ? prop.multiProcessorCount : 256;
  }
  return cached[dev];
}

// Device memory of the entry point that allocates nothing (pml_hip_gemm_run_static): the transposed
// right-hand side Bt[N][K].  Every GPU the library runs on holds its own copy of the array until the process
// ends.  In host code the array's name is only a handle: the address kernels and copies use is looked up once
// per device, with that device current, and kept here.
static __device__ __align__(256) unsigned char scratch[PML_HIP_STATIC_SCRATCH_BYTES];
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {nullptr};
std::mutex g_scratch_mutex;

// Address of `scratch` on the current device; null (and the error text set) on failure.
void* scratch_of_current_device() {
  int dev = 0;
  if (check(hipGetDevice(&dev), "hipGetDevice")) return nullptr;
  if (dev < 0 || dev >= kMaxDevices) {
    fail("device ordinal beyond the per-device table");
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    if (check(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return nullptr;
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}

// A plan whose tile is TILE_64x64_KSPLIT: decides the split for m x n results over `slabs` slabs of K and allocates the
// workspace.  Leaves the plan unsplit (the plain 64 x 64 tile runs) when a split is not worth it or memory is short.
void prepare_split(Plan* p, int64_t m, int64_t n, int64_t slabs) {
  if (p->tile != TILE_64x64_KSPLIT) return;
  int splits = 1, per = 0;
  igemm_split_plan(m, n, slabs, device_cus(), &splits, &per);
  if (splits < 2) return;
  const int64_t pitch = (n + 3) / 4 * 4;
  if (pitch >= ((int64_t)1 << 31) || hipMalloc(&p->ws, (size_t)splits * m * pitch * 4) != hipSuccess) {
    p->ws = nullptr;
    return;
  }
  p->sk_splits = splits;
  p->sk_per = per;
  p->sk_pitch = (int)pitch;
}
void split_args(const Plan* p, IgemmArgs& g) {
  g.ws = p->ws;
  g.sk_splits = p->ws ? p->sk_splits : 0;
  g.sk_per = p->sk_per;
  g.sk_pitch = p->sk_pitch;
}

// Everything of the kernel arguments that the descriptor fixes (no operand pointers).
void conv_args(const Plan* p, IgemmArgs& g) {
  const pml_hip_conv2d_desc& d = p->conv;
  const int64_t K = d.kh * d.kw * d.ci;
  std::memset(&g, 0, sizeof g);
  g.M = d.n * d.oh * d.ow;
  g.N = d.co;
  g.K = K;
  g.A = nullptr;
  g.Bt = p->bt;
  g.ldbt = p->bt_ld;
  g.C = nullptr;
  g.ldc = d.co;
  g.H = (int)d.h;
  g.W = (int)d.w;
  g.CI = (int)d.ci;
  g.OH = (int)d.oh;
  g.OW = (int)d.ow;
  g.KH = (int)d.kh;
  g.KW = (int)d.kw;
  g.SH = (int)d.stride_h;
  g.SW = (int)d.stride_w;
  g.PH = (int)d.pad_h;
  g.PW = (int)d.pad_w;
  g.DH = (int)d.dil_h;
  g.DW = (int)d.dil_w;
  g.out_dtype = d.out_dtype;
  g.init = nullptr;
  g.init_dtype = d.init_dtype;
  g.init_rs = d.init_row_stride;
  g.init_cs = d.init_col_stride;
  g.c_dtype = d.c_dtype;
  classify_tail(d.tail, d.out_dtype, d.c_dtype, &g.tail_mode, &g.tail_relu);
  g.tail_ssr = tail_scale_shift(d.tail, d.out_dtype, g.tail_mode);
  tail_requant(d.tail, d.out_dtype, d.c_dtype, g.tail_mode, &g);
  g.tail = d.tail;
  g.NB = (int)d.n;
  g.n_cus = device_cus();
  g.halo_rows = p->halo_rows;
  g.n_tiles = p->halo_tiles;
  g.halo_variant = p->halo_variant;
  fast_div_magic((unsigned)(d.oh * d.ow), &g.div_per_magic, &g.div_per_shift);
  fast_div_magic((unsigned)d.ow, &g.div_ow_magic, &g.div_ow_shift);
  if (const int mp = PML_HIP_FLAG_MAXPOOL_OF(d.flags)) {
    g.pool = 1;
    g.pool_pt = (mp >> 1) & 1;
    g.pool_pl = (mp >> 3) & 1;
    g.pool_oh = (int)((d.oh + ((mp >> 1) & 1) + ((mp >> 2) & 1) - 3) / 2 + 1);
    g.pool_ow = (int)((d.ow + ((mp >> 3) & 1) + ((mp >> 4) & 1) - 3) / 2 + 1);
  }
  if (p->via_s2d) {
    // unit-stride convolution over the re-blocked input: one "tap" per block row, whose K-run covers
    // s2d_kaw neighbouring blocks of s2d_ch channels
    const int es = dt_size(d.in_dtype);
    g.K = (int64_t)p->s2d_ka * p->s2d_kaw * p->s2d_ch;
    g.H = p->s2d_h;
    g.W = p->s2d_w;
    g.CI = p->s2d_kaw * p->s2d_ch;
    g.pix_pitch = p->s2d_ch * es;
    g.KH = p->s2d_ka;
    g.KW = 1;
    g.SH = g.SW = 1;
    g.PH = ((int)d.pad_h + ((int)d.pad_h & 1)) / 2;
    g.PW = ((int)d.pad_w + ((int)d.pad_w & 1)) / 2;
  }
}

void s2d_args(const Plan* p, S2dArgs& a) {
  const pml_hip_conv2d_desc& d = p->conv;
  std::memset(&a, 0, sizeof a);
  a.N = (int)d.n, a.H = (int)d.h, a.W = (int)d.w, a.CI = (int)d.ci;
  a.HS = p->s2d_h, a.WS = p->s2d_w, a.CH = p->s2d_ch;
  a.KH = (int)d.kh, a.KW = (int)d.kw, a.CO = (int)d.co;
  a.KA = p->s2d_ka, a.KAW = p->s2d_kaw;
  a.EH = (int)d.pad_h & 1, a.EW = (int)d.pad_w & 1;
}

// Packs the caller's HWCK filter into the plan's Bt.
hipError_t pack_conv_filter(Plan* p, const void* filter, hipStream_t s) {
  const pml_hip_conv2d_desc& d = p->conv;
  const int es = dt_size(d.in_dtype);
  if (p->via_s2d) {
    S2dArgs a;
    s2d_args(p, a);
    a.filter = filter;
    a.gt = p->bt;
    return s2d_filter_launch(es, a, s);
  }
  if (hipError_t e = transpose_pack(es, filter, p->bt, d.kh * d.kw * d.ci, d.co, d.co, p->bt_ld, s); e != hipSuccess) return e;
  if (p->b_split) return split_rows_launch(p->bt, d.co, p->bt_ld, d.kh * d.kw * d.ci, s);
  return hipSuccess;
}

}  // namespace
}  // namespace pml

using namespace pml;

extern "C" {

const char* pml_hip_last_error(void) { return g_err.c_str(); }

int pml_hip_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) return 0;
  return n;
}

int pml_hip_init(int device_ordinal) {
  int n = pml_hip_device_count();
  if (n <= 0) return fail("no HIP device is visible");
  if (device_ordinal < 0 || device_ordinal >= n) return fail("device ordinal out of range");
  if (check(hipSetDevice(device_ordinal), "hipSetDevice")) return 1;
  return scratch_of_current_device() ? 0 : 1;
}

int pml_hip_device_name(char* buf, size_t buf_len) {
  if (!buf || buf_len == 0) return fail("null buffer");
  int dev = 0;
  if (check(hipGetDevice(&dev), "hipGetDevice")) return 1;
  hipDeviceProp_t prop;
  if (check(hipGetDeviceProperties(&prop, dev), "hipGetDeviceProperties")) return 1;
  std::snprintf(buf, buf_len, "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
  return 0;
}

int pml_hip_malloc(void** dptr, size_t nbytes) {
  if (!dptr) return fail("null out pointer");
  *dptr = nullptr;
  if (nbytes == 0) nbytes = 16;
  return check(hipMalloc(dptr, nbytes), "hipMalloc");
}
int pml_hip_free(void* dptr) { return dptr ? check(hipFree(dptr), "hipFree") : 0; }
int pml_hip_host_alloc(void** hptr, size_t nbytes) {
  if (!hptr) return fail("null out pointer");
  return check(hipHostMalloc(hptr, nbytes ? nbytes : 16, hipHostMallocDefault), "hipHostMalloc");
}
int pml_hip_host_free(void* hptr) { return hptr ? check(hipHostFree(hptr), "hipHostFree") : 0; }

int pml_hip_memcpy_h2d(void* dst, const void* src, size_t nbytes, pml_hip_stream s) {
  if (nbytes == 0) return 0;
  if (check(hipMemcpyAsync(dst, src, nbytes, hipMemcpyHostToDevice, (hipStream_t)s), "hipMemcpyAsync(h2d)")) return 1;
  return check(hipStreamSynchronize((hipStream_t)s), "hipStreamSynchronize");
}
int pml_hip_memcpy_d2h(void* dst, const void* src, size_t nbytes, pml_hip_stream s) {
  if (nbytes == 0) return 0;
  if (check(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToHost, (hipStream_t)s), "hipMemcpyAsync(d2h)")) return 1;
  return check(hipStreamSynchronize((hipStream_t)s), "hipStreamSynchronize");
}
int pml_hip_memcpy_d2d(void* dst, const void* src, size_t nbytes, pml_hip_stream s) {
  if (nbytes == 0) return 0;
  return check(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToDevice, (hipStream_t)s), "hipMemcpyAsync(d2d)");
}
int pml_hip_fill_u32(void* dptr, uint32_t pattern, size_t n_words, pml_hip_stream s) {
  return check(fill_u32_launch(dptr, pattern, n_words, (hipStream_t)s), "fill");
}

int pml_hip_stream_create(pml_hip_stream* s) {
  hipStream_t st;
  if (check(hipStreamCreate(&st), "hipStreamCreate")) return 1;
  *s = (pml_hip_stream)st;
  return 0;
}
int pml_hip_stream_destroy(pml_hip_stream s) { return check(hipStreamDestroy((hipStream_t)s), "hipStreamDestroy"); }
int pml_hip_stream_sync(pml_hip_stream s) { return check(hipStreamSynchronize((hipStream_t)s), "hipStreamSynchronize"); }
int pml_hip_event_create(pml_hip_event* e) {
  hipEvent_t ev;
  if (check(hipEventCreate(&ev), "hipEventCreate")) return 1;
  *e = (pml_hip_event)ev;
  return 0;
}
int pml_hip_capture_begin(pml_hip_stream s) {
  if (!s) return fail("pml_hip_capture_begin: the default stream cannot be captured");
  // (thread-local mode: other threads of the process may go on allocating while this one records)
  return check(hipStreamBeginCapture((hipStream_t)s, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
}
int pml_hip_capture_end(pml_hip_stream s, pml_hip_graph* graph) {
  if (!s || !graph) return fail("pml_hip_capture_end: null argument");
  *graph = nullptr;
  hipGraph_t g = nullptr;
  // (always called, also after a failed recording: it is what takes the stream out of capture mode)
  const hipError_t e = hipStreamEndCapture((hipStream_t)s, &g);
  if (e != hipSuccess || !g) {
    (void)hipGetLastError();
    return fail(std::string("hipStreamEndCapture: ") + hipGetErrorString(e));
  }
  hipGraphExec_t exec = nullptr;
  const hipError_t ei = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
  (void)hipGraphDestroy(g);
  if (check(ei, "hipGraphInstantiate")) return 1;
  *graph = (pml_hip_graph)exec;
  return 0;
}
int pml_hip_graph_launch(pml_hip_graph graph, pml_hip_stream s) {
  if (!graph) return fail("pml_hip_graph_launch: null graph");
  return check(hipGraphLaunch((hipGraphExec_t)graph, (hipStream_t)s), "hipGraphLaunch");
}
int pml_hip_graph_destroy(pml_hip_graph graph) {
  return graph ? check(hipGraphExecDestroy((hipGraphExec_t)graph), "hipGraphExecDestroy") : 0;
}
int pml_hip_event_destroy(pml_hip_event e) { return check(hipEventDestroy((hipEvent_t)e), "hipEventDestroy"); }
int pml_hip_event_record(pml_hip_event e, pml_hip_stream s) {
  return check(hipEventRecord((hipEvent_t)e, (hipStream_t)s), "hipEventRecord");
}
int pml_hip_event_sync(pml_hip_event e) { return check(hipEventSynchronize((hipEvent_t)e), "hipEventSynchronize"); }
int pml_hip_event_elapsed_ms(pml_hip_event start, pml_hip_event stop, float* ms) {
  return check(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop), "hipEventElapsedTime");
}

// ---------------------------------------------------------------------------
// GEMM
// ---------------------------------------------------------------------------

// Checks a GEMM descriptor; the MFMA kind (>= 0) or -1 with the error text set.
static int gemm_desc_kind(const pml_hip_gemm_desc* d) {
  if (!d) {
    fail("null descriptor");
    return -1;
  }
  const int kind = mfma_kind_of(d->in_dtype, d->flags);
  if (kind < 0) {
    fail("gemm: in_dtype must be F32, BF16 or I8");
    return -1;
  }
  const bool out_ok = (kind == KIND_I8) ? d->out_dtype == PML_HIP_I32
                                        : (d->out_dtype == PML_HIP_F32 || (kind == KIND_BF16 && d->out_dtype == PML_HIP_BF16));
  if (!out_ok) {
    fail("gemm: out_dtype does not fit in_dtype");
    return -1;
  }
  if ((d->flags & ~(PML_HIP_FP32_AS_BF16X3 | kScheduleBits)) != 0 || ((d->flags & PML_HIP_FP32_AS_BF16X3) && d->in_dtype != PML_HIP_F32) ||
      !schedule_bits_ok(d->flags)) {
    fail("gemm: flags may only hold PML_HIP_FP32_AS_BF16X3 (with in_dtype F32) and schedule overrides that name an existing tile");
    return -1;
  }
  if (d->m <= 0 || d->n <= 0 || d->k <= 0 || d->lda < d->k || d->ldb < (d->b_layout ? d->k : d->n) || d->ldc < d->n ||
      (d->b_layout != 0 && d->b_layout != 1)) {
    fail("gemm: bad sizes or leading dimensions");
    return -1;
  }
  const int es = dt_size(d->in_dtype);
  if ((d->k * es) % 16 != 0 || (d->lda * es) % 16 != 0 || (d->b_layout && (d->ldb * es) % 16 != 0)) {
    fail("gemm: K and the K-contiguous leading dimensions must cover whole 16-byte vectors");
    return -1;
  }
  if (!valid_tail(d->tail)) {
    fail("gemm: malformed tail");
    return -1;
  }
  if (d->k2 != 0) {
    if (kind != KIND_BF16 || d->k2 < 0 || (d->k2 * es) % 16 != 0 || (d->lda2 * es) % 16 != 0 || d->lda2 < d->k2 ||
        d->ldb2 < (d->b_layout ? d->k2 : d->n) || (d->b_layout && (d->ldb2 * es) % 16 != 0) || d->a2_stride < 0 ||
        (d->init2_kind != 0 && d->init2_kind != 1)) {
      fail("gemm: malformed second product (bf16 only; k2 and lda2 must cover whole 16-byte vectors)");
      return -1;
    }
    if (d->a2_stride > 0) {
      // rows of a strided 1x1 convolution: the result rows are the pixels of whole images
      if (d->a2_oh <= 0 || d->a2_ow <= 0 || d->m % (d->a2_oh * d->a2_ow) != 0 || (d->a2_oh - 1) * d->a2_stride >= d->a2_h ||
          (d->a2_ow - 1) * d->a2_stride >= d->a2_w || d->a2_oh * d->a2_ow > INT32_MAX || d->a2_h > INT32_MAX || d->a2_w > INT32_MAX) {
        fail("gemm: the second product's pixel rows do not fit its image");
        return -1;
      }
    }
  } else if (d->init2_kind != 0) {
    fail("gemm: a second initial value needs a second product");
    return -1;
  }
  return kind;
}

int pml_hip_gemm_tail_cheaper_apart(const pml_hip_gemm_desc* d) {
  if (!d || d->tail.n_ops == 0 || d->k2 != 0) return 0;
  const int kind = gemm_desc_kind(d);
  if (kind != KIND_I8) return 0;
  int mode = 0, relu = 0;
  classify_tail(d->tail, d->out_dtype, d->c_dtype, &mode, &relu);
  if (mode == 1 || mode == 2 || tail_requant(d->tail, d->out_dtype, d->c_dtype, mode, nullptr)) return 0;
  const int64_t k_bytes = d->k * dt_size(d->in_dtype);
  if (PML_HIP_FLAG_TILE_OF(d->flags) >= 0) return 0;  // a named tile is taken whatever the tail
  return choose_tile(d->m, d->n, k_bytes, kind, true) == TILE_256x256_W8 && choose_tile(d->m, d->n, k_bytes, kind, false) != TILE_256x256_W8;
}

int64_t pml_hip_gemm_dispatch(const pml_hip_gemm_desc* d) {
  const int kind = gemm_desc_kind(d);
  if (kind < 0) return 0;
  const int es = dt_size(d->in_dtype);
  Plan* p = new Plan();
  p->kind = PLAN_GEMM;
  p->mfma_kind = kind;
  p->gemm = *d;
  {
    int mode = 0, relu = 0;
    classify_tail(d->tail, d->out_dtype, d->c_dtype, &mode, &relu);
    const bool plain = mode == 1 || mode == 2 || tail_requant(d->tail, d->out_dtype, d->c_dtype, mode, nullptr);
    p->tile = choose_tile(d->m, d->n, (d->k + d->k2) * dt_size(d->in_dtype), kind, plain, PML_HIP_FLAG_TILE_OF(d->flags));
    // (a second product's slabs follow the first one's on the slab axis the splits share out)
    prepare_split(p, d->m, d->n, (d->k * dt_size(d->in_dtype) + 127) / 128 + (d->k2 * dt_size(d->in_dtype) + 127) / 128);
  }
  p->bt_ld = d->k;
  p->bt_bytes = (size_t)d->n * d->k * es;
  if (p->tile == TILE_64x64_KSPLIT && !p->ws) p->tile = TILE_64x64;  // (not worth splitting, or no memory for the workspace)
  p->b_split = kind == KIND_F32X3 && !d->b_layout && d->k % 32 == 0 && !p->ws;
  if (!d->b_layout && hipMalloc(&p->bt, p->bt_bytes) != hipSuccess) {
    delete p;
    fail("gemm: cannot allocate the packed right-hand side");
    return 0;
  }
  if (d->k2 > 0 && !d->b_layout && hipMalloc(&p->bt2, (size_t)d->n * d->k2 * es) != hipSuccess) {
    delete p;
    fail("gemm: cannot allocate the second packed right-hand side");
    return 0;
  }
  char buf[256];
  std::snprintf(buf, sizeof buf, "gemm %s m=%lld n=%lld k=%lld tile=%s mfma=%s", d->in_dtype == PML_HIP_F32 ? "f32" : d->in_dtype == PML_HIP_BF16 ? "bf16" : "i8",
                (long long)d->m, (long long)d->n, (long long)d->k, tile_name(p->tile),
                kind == KIND_F32 ? "f32_32x32x2" : kind == KIND_BF16 ? "f32_32x32x16_bf16" : kind == KIND_I8 ? "i32_32x32x32_i8" : "3 x f32_32x32x16_bf16 (fp32 split into bf16 head + remainder)");
  p->text = buf;
  if (d->k2 > 0) p->text += " + second product k2=" + std::to_string(d->k2) + (d->a2_stride > 0 ? " over pixel rows of stride " + std::to_string(d->a2_stride) : "");
  return (int64_t)(intptr_t)p;
}

// One GEMM launch sequence: the per-run transposition of a [K][N] right-hand side into `bt` (device memory of
// n x bt_ld elements; skipped when b is null, i.e. packed earlier, or already [N][K]), then the MFMA kernel.
// Shared by the plan-based entry point and by the one that allocates nothing.
struct SecondProduct {
  const void* a2 = nullptr;
  const void* b2 = nullptr;
  const void* init2 = nullptr;
  void* bt2 = nullptr;
  bool packed2 = false;
};

// An fp32 or int8 right-hand side that arrives with the call in its row-major [K][N] form is read as it is (the
// fp32 kinds gather their K-values from [k][n] slabs, int8 reads them with transposing LDS reads); everything else
// is transposed into Bt[N][K] first.  Rows must be whole 16-byte vectors.
static bool reads_b_as_given(const pml_hip_gemm_desc& d, int mfma_kind, const void* b, int tile) {
  if (mfma_kind != KIND_F32 && mfma_kind != KIND_F32X3 && mfma_kind != KIND_I8) return false;
  if (tile == TILE_64x64_KSPLIT) return false;  // (the split kernel reads Bt)
  if (tile == TILE_192x384_W8) return false;  // (24 chunks per row: the position swizzle of the [k][n] form needs a power of two)
  const int64_t es = mfma_kind == KIND_I8 ? 1 : 4, v = 16 / es;
  if (!(b && !d.b_layout && d.k2 == 0 && d.n % v == 0 && d.ldb % v == 0 && ((uintptr_t)b & 15) == 0 &&
        d.k * d.ldb * es < ((int64_t)1 << 31)))
    return false;
  if (mfma_kind == KIND_I8) {
    // The transposing reads make the int8 kernel about 15 % slower (4096^3: 86 us against 74 + 10 for the copy), so
    // they pay while the transposed copy -- a launch of at least 5 us, 3.2 TB/s beyond that -- costs more than
    // that share of the multiplication (priced at the 1.8 POP/s the kernel reaches): up to about 3500 rows at
    // K = N = 4096, always for small problems.
    const double t_gemm = 2.0 * (double)d.m * (double)d.n * (double)d.k / 1.8e15;
    const double t_copy = std::max(5e-6, 2.0 * (double)d.k * (double)d.n / 3.2e12);
    return 0.15 * t_gemm < t_copy;
  }
  return true;
}

static int gemm_run(const pml_hip_gemm_desc& d, int mfma_kind, int tile, void* bt, int64_t bt_ld, bool packed,
                    const void* a, const void* b, void* c, const void* init, const void* const* operands,
                    void* const* outs, pml_hip_stream s, const SecondProduct* second = nullptr, bool bt_is_split = false,
                    const Plan* split_plan = nullptr) {
  // (a right-hand side that arrives with the call is transposed per run and split in the kernel's registers: a
  // second small launch costs more than it saves; one packed once is kept split)
  const bool b_split = bt_is_split && !b;
  if (!a || !c) return fail("gemm_invoke: null operand");
  if (!b && (!packed || d.b_layout)) return fail("gemm_invoke: b is null and no packed right-hand side exists");
  if (d.b_layout && ((uintptr_t)b & 15) != 0) return fail("gemm_invoke: an [N][K] right-hand side must be 16-byte aligned");
  if (((uintptr_t)a & 15) != 0) return fail("gemm_invoke: A must be 16-byte aligned");
  if (d.init_kind && !init) return fail("gemm_invoke: the plan expects an initial value");
  const int es = dt_size(d.in_dtype);
  const bool b_as_given = reads_b_as_given(d, mfma_kind, b, tile);
  if (b && !d.b_layout && !b_as_given && check(transpose_pack(es, b, bt, d.k, d.n, d.ldb, bt_ld, (hipStream_t)s), "transpose_pack"))
    return 1;
  if (d.k2 > 0) {
    if (!second || !second->a2) return fail("gemm_invoke: the plan has a second product: use pml_hip_gemm_invoke2");
    if (!second->b2 && (!second->packed2 || d.b_layout)) return fail("gemm_invoke2: b2 is null and no packed right-hand side exists");
    if (((uintptr_t)second->a2 & 15) != 0 || (d.b_layout && ((uintptr_t)second->b2 & 15) != 0)) return fail("gemm_invoke2: the second product's operands must be 16-byte aligned");
    if (d.init2_kind && !second->init2) return fail("gemm_invoke2: the plan expects a second initial value");
    if (second->b2 && !d.b_layout &&
        check(transpose_pack(es, second->b2, second->bt2, d.k2, d.n, d.ldb2, d.k2, (hipStream_t)s), "transpose_pack"))
      return 1;
  }
  IgemmArgs g;
  std::memset(&g, 0, sizeof g);
  if (d.k2 > 0) {
    g.K2 = d.k2;
    g.A2 = second->a2;
    g.lda2 = d.lda2;
    g.Bt2 = d.b_layout ? second->b2 : second->bt2;
    g.ldbt2 = d.b_layout ? d.ldb2 : d.k2;
    g.init2 = d.init2_kind ? second->init2 : nullptr;
    g.g2_stride = d.a2_stride;
    if (d.a2_stride > 0) {
      g.g2_h = (int)d.a2_h;
      g.g2_w = (int)d.a2_w;
      g.g2_ohw = (int)(d.a2_oh * d.a2_ow);
      g.g2_ow = (int)d.a2_ow;
      fast_div_magic((unsigned)g.g2_ohw, &g.g2_ohw_magic, &g.g2_ohw_shift);
      fast_div_magic((unsigned)g.g2_ow, &g.g2_ow_magic, &g.g2_ow_shift);
    }
  }
  g.M = d.m;
  g.N = d.n;
  g.K = d.k;
  g.A = a;
  g.lda = d.lda;
  g.Bt = (d.b_layout || b_as_given) ? b : bt;
  g.ldbt = (d.b_layout || b_as_given) ? d.ldb : bt_ld;
  g.b_kn = b_as_given ? 1 : 0;
  g.C = c;
  g.ldc = d.ldc;
  g.out_dtype = d.out_dtype;
  g.init = d.init_kind ? init : nullptr;
  g.init_dtype = d.init_dtype;
  g.init_rs = d.init_row_stride;
  g.init_cs = d.init_col_stride;
  g.c_dtype = d.c_dtype;
  g.n_cus = device_cus();
  classify_tail(d.tail, d.out_dtype, d.c_dtype, &g.tail_mode, &g.tail_relu);
  g.tail_ssr = tail_scale_shift(d.tail, d.out_dtype, g.tail_mode);
  tail_requant(d.tail, d.out_dtype, d.c_dtype, g.tail_mode, &g);
  g.tail = d.tail;
  for (int i = 0; i < d.tail.n_operands; ++i) {
    if (!operands || !operands[i]) return fail("gemm_invoke: missing tail operand");
    g.operands[i] = operands[i];
  }
  for (int i = 0; i < PML_HIP_MAX_EPI_OPERANDS; ++i) g.outs[i] = outs ? outs[i] : nullptr;
  // the vector tails need 16-byte aligned operands and extra outputs; otherwise the interpreter runs
  if (g.tail_mode == 2 && ((uintptr_t)g.operands[0] & 15) != 0) g.tail_mode = 0;
  if (g.tail_mode == 3 || g.tail_mode == 4) {
    for (int i = 0; i < d.tail.n_operands; ++i)
      if (((uintptr_t)g.operands[i] & 15) != 0) g.tail_mode = 0;
    for (int i = 0; i < PML_HIP_MAX_EPI_OPERANDS; ++i)
      if (((uintptr_t)g.outs[i] & 15) != 0) g.tail_mode = 0;
  }
  for (int i = 0; i < d.tail.n_ops; ++i)
    if (d.tail.ops[i].opcode == PML_HIP_EPI_STORE && !g.outs[d.tail.ops[i].operand])
      return fail("gemm_invoke: missing extra output");
  if (split_plan && !b_split) split_args(split_plan, g);  // (the K split over workgroups is not built for a right-hand side packed split)
  return check(igemm_launch(b_split ? KIND_F32X3P : mfma_kind, tile, false, g, (hipStream_t)s), "igemm_launch");
}

int pml_hip_gemm_invoke(int64_t plan, const void* a, const void* b, void* c, const void* init,
                        const void* const* operands, void* const* outs, pml_hip_stream s) {
  Plan* p = (Plan*)(intptr_t)plan;
  if (!p || p->kind != PLAN_GEMM) return fail("gemm_invoke: not a gemm plan");
  const bool split = p->bt_is_split;
  // a right-hand side that this run transposes overwrites the packed copy
  if (b && !p->gemm.b_layout && !reads_b_as_given(p->gemm, p->mfma_kind, b, p->tile)) p->bt_is_split = false;
  return gemm_run(p->gemm, p->mfma_kind, p->tile, p->bt, p->bt_ld, p->packed, a, b, c, init, operands, outs, s, nullptr, split, p);
}

int pml_hip_gemm_invoke2(int64_t plan, const void* a, const void* b, void* c, const void* init, const void* a2, const void* b2,
                         const void* init2, const void* const* operands, void* const* outs, pml_hip_stream s) {
  Plan* p = (Plan*)(intptr_t)plan;
  if (!p || p->kind != PLAN_GEMM) return fail("gemm_invoke2: not a gemm plan");
  if (p->gemm.k2 <= 0) return fail("gemm_invoke2: the plan has no second product");
  SecondProduct sp;
  sp.a2 = a2;
  sp.b2 = b2;
  sp.init2 = init2;
  sp.bt2 = p->bt2;
  sp.packed2 = p->packed2;
  return gemm_run(p->gemm, p->mfma_kind, p->tile, p->bt, p->bt_ld, p->packed, a, b, c, init, operands, outs, s, &sp);
}

int pml_hip_gemm_run_static(const pml_hip_gemm_desc* d, const void* a, const void* b, void* c, const void* init,
                            const void* const* operands, void* const* outs, pml_hip_stream s) {
  const int kind = gemm_desc_kind(d);
  if (kind < 0) return 1;
  if (d->k2 != 0) return fail("gemm_run_static: a second product is not supported by this entry point");
  if (!b) return fail("gemm_run_static: b is null");
  void* bt = nullptr;
  if (!d->b_layout) {
    // n and k are positive and each below 2^31 by the check below, so the product cannot overflow
    if (d->n > PML_HIP_STATIC_SCRATCH_BYTES || d->k > PML_HIP_STATIC_SCRATCH_BYTES ||
        (uint64_t)d->n * (uint64_t)d->k * (uint64_t)dt_size(d->in_dtype) > (uint64_t)PML_HIP_STATIC_SCRATCH_BYTES)
      return fail("gemm_run_static: the transposed right-hand side (n x k elements) exceeds PML_HIP_STATIC_SCRATCH_BYTES (32 MiB)");
    bt = scratch_of_current_device();
    if (!bt) return 1;
  }
  int mode = 0, relu = 0;
  classify_tail(d->tail, d->out_dtype, d->c_dtype, &mode, &relu);
  const bool plain = mode == 1 || mode == 2 || tail_requant(d->tail, d->out_dtype, d->c_dtype, mode, nullptr);
  // (no workspace may be allocated here: the K loop is never split over workgroups)
  const int tile = choose_tile(d->m, d->n, d->k * dt_size(d->in_dtype), kind, plain, PML_HIP_FLAG_TILE_OF(d->flags), /*allow_split=*/false);
  return gemm_run(*d, kind, tile, bt, d->k, false, a, b, c, init, operands, outs, s);
}

// ---------------------------------------------------------------------------
// conv2d
// ---------------------------------------------------------------------------

// A plan (its descriptor, element kind and 2x2-block geometry filled in) whose convolution the row-walking kernel takes,
// with a result the fused 3x3 stride-2 max-pool can walk: a pooled row per thread group of 512 threads, eight per pixel.
static bool conv2d_takes_maxpool(const Plan* p) {
  const pml_hip_conv2d_desc& d = p->conv;
  const int path = PML_HIP_FLAG_CONV_OF(d.flags);
  if (!p->via_s2d || path == PML_HIP_CONV_IGEMM || path == PML_HIP_CONV_PATCHES) return false;
  IgemmArgs g;
  conv_args(p, g);
  // (the filter pointer's alignment is the allocator's: not part of the question)
  g.Bt = nullptr;
  if (!conv_blocks4x4_prepare(p->mfma_kind, g)) return false;
  return d.oh >= 3 && d.ow >= 3 && g.pool_oh >= 1 && g.pool_ow >= 1 && g.pool_ow <= 64 && d.tail.n_operands == 0;
}

int64_t pml_hip_conv2d_dispatch(const pml_hip_conv2d_desc* d) {
  if (!d) {
    fail("null descriptor");
    return 0;
  }
  const int kind = mfma_kind_of(d->in_dtype, d->flags);
  if (kind < 0) {
    fail("conv2d: in_dtype must be F32, BF16 or I8");
    return 0;
  }
  const bool out_ok = (kind == KIND_I8) ? d->out_dtype == PML_HIP_I32
                                        : (d->out_dtype == PML_HIP_F32 || (kind == KIND_BF16 && d->out_dtype == PML_HIP_BF16));
  if (!out_ok) {
    fail("conv2d: out_dtype does not fit in_dtype");
    return 0;
  }
  if ((d->flags & ~(PML_HIP_FP32_AS_BF16X3 | kScheduleBits | kMaxpoolBits)) != 0 || ((d->flags & PML_HIP_FP32_AS_BF16X3) && d->in_dtype != PML_HIP_F32) ||
      !schedule_bits_ok(d->flags) || (PML_HIP_FLAG_MAXPOOL_OF(d->flags) != 0 && (PML_HIP_FLAG_MAXPOOL_OF(d->flags) & 1) == 0)) {
    fail("conv2d: flags may only hold PML_HIP_FP32_AS_BF16X3 (with in_dtype F32) and schedule overrides that name an existing tile and path");
    return 0;
  }
  if (d->n <= 0 || d->h <= 0 || d->w <= 0 || d->ci <= 0 || d->co <= 0 || d->kh <= 0 || d->kw <= 0 || d->oh <= 0 ||
      d->ow <= 0 || d->stride_h <= 0 || d->stride_w <= 0 || d->dil_h <= 0 || d->dil_w <= 0) {
    fail("conv2d: bad geometry");
    return 0;
  }
  const int es = dt_size(d->in_dtype);
  // channels that do not fill 16-byte vectors: stride 2 runs over 2x2 pixel blocks, anything else over a patch matrix
  const bool odd_channels = (d->ci * es) % 16 != 0;
  const int path = PML_HIP_FLAG_CONV_OF(d->flags);
  const bool via_s2d = odd_channels && d->stride_h == 2 && d->stride_w == 2 && d->dil_h == 1 && d->dil_w == 1 &&
                       es >= 2 && d->ci <= 16 && path != PML_HIP_CONV_PATCHES;
  const bool via_patches = odd_channels && !via_s2d;
  if (d->n * d->h * d->w * d->ci >= ((int64_t)1 << 40) || d->h * d->w * d->ci * es >= ((int64_t)1 << 31) ||
      d->kh * d->kw * d->ci * es >= ((int64_t)1 << 31)) {
    fail("conv2d: tensor too large");
    return 0;
  }
  if (!valid_tail(d->tail)) {
    fail("conv2d: malformed tail");
    return 0;
  }
  Plan* p = new Plan();
  p->kind = PLAN_CONV;
  p->mfma_kind = kind;
  p->conv = *d;
  const int64_t M = d->n * d->oh * d->ow;
  const int64_t K = d->kh * d->kw * d->ci;
  p->tile = choose_tile(M, d->co, K * es, kind, false, PML_HIP_FLAG_TILE_OF(d->flags));
  p->bt_ld = K;
  if (via_s2d) {
    const int v = 16 / es;
    p->s2d_h = (int)(d->h + 1) / 2;
    p->s2d_w = (int)(d->w + 1) / 2;
    p->s2d_ch = (int)(4 * d->ci + v - 1) / v * v;
    p->s2d_ka = (int)(d->kh + (d->pad_h & 1) + 1) / 2;
    p->s2d_kaw = (int)(d->kw + (d->pad_w & 1) + 1) / 2;
    const int64_t k2 = (int64_t)p->s2d_ka * p->s2d_kaw * p->s2d_ch;
    p->tile = choose_tile(M, d->co, k2 * es, kind, false, PML_HIP_FLAG_TILE_OF(d->flags), /*allow_split=*/false);
    p->bt_ld = k2;
    p->via_s2d = true;
  }
  if (via_patches) {
    // rows padded with zeros to whole 16-byte vectors on both GEMM operands
    const int64_t v = 16 / es;
    p->kpad = (K + v - 1) / v * v;
    p->bt_ld = p->kpad;
    if (hipMalloc(&p->patches, (size_t)M * p->kpad * es) != hipSuccess) {
      delete p;
      fail("conv2d: cannot allocate the patch matrix");
      return 0;
    }
  }
  if (!via_s2d && !via_patches) prepare_split(p, M, d->co, d->kh * d->kw * ((d->ci * es + 127) / 128));
  if (p->tile == TILE_64x64_KSPLIT && !p->ws) p->tile = TILE_64x64;
  // (whole 128-byte chunks per filter tap, so that no chunk of heads + remainders straddles two taps)
  p->b_split = kind == KIND_F32X3 && !via_s2d && !via_patches && d->ci % 32 == 0 && !p->ws;
  p->bt_bytes = (size_t)d->co * p->bt_ld * es;
  if (hipMalloc(&p->bt, p->bt_bytes) != hipSuccess || hipMemset(p->bt, 0, p->bt_bytes) != hipSuccess) {
    delete p;
    fail("conv2d: cannot allocate the packed filter");
    return 0;
  }
  {
    // Filter small enough to stay in LDS: persistent resident-filter kernel (PML_HIP_CONV_IGEMM keeps the generic one).
    int dev = 0;
    hipDeviceProp_t prop;
    if (!odd_channels && kind != KIND_F32X3 && path != PML_HIP_CONV_IGEMM && hipGetDevice(&dev) == hipSuccess &&
        hipGetDeviceProperties(&prop, dev) == hipSuccess) {
      IgemmArgs g;
      conv_args(p, g);
      const size_t lds = conv_halo_prepare(kind, &g, path == PML_HIP_CONV_LDSFILTER);
      if (lds && lds <= prop.sharedMemPerBlock) {
        p->halo_lds = lds;
        p->halo_rows = g.halo_rows;
        p->halo_tiles = g.n_tiles;
        p->halo_variant = g.halo_variant;
        p->n_cus = prop.multiProcessorCount;
      }
    }
  }
  char buf[256];
  std::snprintf(buf, sizeof buf, "conv2d %s n=%lld %lldx%lldx%lld k=%lldx%lld co=%lld -> %lldx%lld (implicit gemm m=%lld n=%lld k=%lld) tile=%s",
                d->in_dtype == PML_HIP_F32 ? "f32" : d->in_dtype == PML_HIP_BF16 ? "bf16" : "i8", (long long)d->n,
                (long long)d->h, (long long)d->w, (long long)d->ci, (long long)d->kh, (long long)d->kw, (long long)d->co,
                (long long)d->oh, (long long)d->ow, (long long)M, (long long)d->co, (long long)K, p->halo_lds ? (p->halo_variant == 3 ? "256x64 resident filter, in registers" : p->halo_variant ? "256x64 resident filter, pipelined 3x3" : "256x64 resident filter") : tile_name(p->tile));
  p->text = buf;
  if (kind == KIND_F32X3) p->text += " mfma=3 x f32_32x32x16_bf16 (fp32 split into bf16 head + remainder)";
  if (via_patches) p->text += " via patch matrix (k padded to " + std::to_string(p->kpad) + ")";
  if (via_s2d) {
    p->text += " over 2x2 pixel blocks (" + std::to_string(p->s2d_ka) + "x" + std::to_string(p->s2d_kaw) + " block taps of " +
               std::to_string(p->s2d_ch) + " channels, k=" + std::to_string(p->bt_ld) + ")";
    IgemmArgs g;
    conv_args(p, g);
    if (path != PML_HIP_CONV_IGEMM && conv_blocks4x4_prepare(kind, g)) p->text += ", row by row with the filter in registers";
  }
  if (PML_HIP_FLAG_MAXPOOL_OF(d->flags)) {
    if (!conv2d_takes_maxpool(p)) {
      delete p;
      fail("conv2d: the fused max-pool needs the row-walking kernel (see pml_hip_conv2d_takes_maxpool) and a convolution result of at least 3 x 3 and at most 128 pixels a row");
      return 0;
    }
    IgemmArgs g;
    conv_args(p, g);
    p->text += " + max-pool 3x3 stride 2 -> " + std::to_string(g.pool_oh) + "x" + std::to_string(g.pool_ow);
  }
  return (int64_t)(intptr_t)p;
}

int pml_hip_conv2d_takes_maxpool(const pml_hip_conv2d_desc* d) {
  if (!d || !PML_HIP_FLAG_MAXPOOL_OF(d->flags)) return 0;
  const int kind = mfma_kind_of(d->in_dtype, d->flags);
  if (kind != KIND_BF16 || d->n <= 0 || d->h <= 0 || d->w <= 0 || d->ci <= 0 || d->co <= 0 || d->kh <= 0 || d->kw <= 0 || d->oh <= 0 ||
      d->ow <= 0 || !valid_tail(d->tail))
    return 0;
  // the plan's fields that conv_args reads, without any of its allocations
  Plan p;
  p.kind = PLAN_CONV;
  p.mfma_kind = kind;
  p.conv = *d;
  const int es = 2, v = 8;
  const bool via_s2d = (d->ci * es) % 16 != 0 && d->stride_h == 2 && d->stride_w == 2 && d->dil_h == 1 && d->dil_w == 1 && d->ci <= 16 &&
                       PML_HIP_FLAG_CONV_OF(d->flags) != PML_HIP_CONV_PATCHES;
  if (!via_s2d) return 0;
  p.s2d_h = (int)(d->h + 1) / 2;
  p.s2d_w = (int)(d->w + 1) / 2;
  p.s2d_ch = (int)(4 * d->ci + v - 1) / v * v;
  p.s2d_ka = (int)(d->kh + (d->pad_h & 1) + 1) / 2;
  p.s2d_kaw = (int)(d->kw + (d->pad_w & 1) + 1) / 2;
  p.bt_ld = (int64_t)p.s2d_ka * p.s2d_kaw * p.s2d_ch;
  p.via_s2d = true;
  return conv2d_takes_maxpool(&p) ? 1 : 0;
}

int pml_hip_conv2d_invoke(int64_t plan, const void* input, const void* filter, void* output, const void* init,
                          const void* const* operands, void* const* outs, pml_hip_stream s) {
  Plan* p = (Plan*)(intptr_t)plan;
  if (!p || p->kind != PLAN_CONV) return fail("conv2d_invoke: not a conv2d plan");
  const pml_hip_conv2d_desc& d = p->conv;
  if (!input || !output) return fail("conv2d_invoke: null operand");
  if (!filter && !p->packed) return fail("conv2d_invoke: filter is null and no packed filter exists");
  if (!p->patches && !p->via_s2d && ((uintptr_t)input & 15) != 0) return fail("conv2d_invoke: input must be 16-byte aligned");
  if (d.init_kind && !init) return fail("conv2d_invoke: the plan expects an initial value");
  const int es = dt_size(d.in_dtype);
  const int64_t K = d.kh * d.kw * d.ci;
  // the HWCK filter is a row-major [K][CO] matrix; the pipelined resident-filter kernel transposes it itself
  const bool raw_filter = filter && p->halo_lds && p->halo_variant && p->mfma_kind != KIND_I8;
  if (filter && !raw_filter && check(pack_conv_filter(p, filter, (hipStream_t)s), "pack_conv_filter")) return 1;
  // (a filter that arrives with the call replaces the packed one; its register-order copy follows it)
  if (filter && !raw_filter && p->reg_image &&
      check(regfilter_image_launch(p->bt, p->bt_ld * es, p->reg_image, (hipStream_t)s), "regfilter_image_launch"))
    return 1;
  IgemmArgs g;
  conv_args(p, g);
  if (raw_filter) {
    if (((uintptr_t)filter & 15) != 0) return fail("conv2d_invoke: filter must be 16-byte aligned");
    g.Bt = filter;
    g.ldbt = d.co;
    g.b_raw = 1;
  } else if (!filter && p->reg_image && p->halo_lds && p->halo_variant == 3) {
    g.Bt = p->reg_image;
    g.b_raw = 2;
  }
  g.A = input;
  g.C = output;
  g.init = d.init_kind ? init : nullptr;
  for (int i = 0; i < d.tail.n_operands; ++i) {
    if (!operands || !operands[i]) return fail("conv2d_invoke: missing tail operand");
    g.operands[i] = operands[i];
  }
  for (int i = 0; i < PML_HIP_MAX_EPI_OPERANDS; ++i) g.outs[i] = outs ? outs[i] : nullptr;
  // the vector tails need 16-byte aligned operands and extra outputs; otherwise the interpreter runs
  if (g.tail_mode == 2 && ((uintptr_t)g.operands[0] & 15) != 0) g.tail_mode = 0;
  if (g.tail_mode == 3 || g.tail_mode == 4) {
    for (int i = 0; i < d.tail.n_operands; ++i)
      if (((uintptr_t)g.operands[i] & 15) != 0) g.tail_mode = 0;
    for (int i = 0; i < PML_HIP_MAX_EPI_OPERANDS; ++i)
      if (((uintptr_t)g.outs[i] & 15) != 0) g.tail_mode = 0;
  }
  for (int i = 0; i < d.tail.n_ops; ++i)
    if (d.tail.ops[i].opcode == PML_HIP_EPI_STORE && !g.outs[d.tail.ops[i].operand])
      return fail("conv2d_invoke: missing extra output");
  if (p->patches) {
    Im2colArgs ic;
    ic.in = input;
    ic.out = p->patches;
    ic.M = g.M;
    ic.K = (int)K;
    ic.kpad = (int)p->kpad;
    ic.H = g.H, ic.W = g.W, ic.CI = g.CI, ic.OH = g.OH, ic.OW = g.OW, ic.KH = g.KH, ic.KW = g.KW;
    ic.SH = g.SH, ic.SW = g.SW, ic.PH = g.PH, ic.PW = g.PW, ic.DH = g.DH, ic.DW = g.DW;
    if (check(im2col_launch(es, ic, (hipStream_t)s), "im2col_launch")) return 1;
    g.A = p->patches;
    g.lda = p->kpad;
    g.K = p->kpad;
    return check(igemm_launch(p->mfma_kind, p->tile, false, g, (hipStream_t)s), "igemm_launch");
  }
  if (p->via_s2d) {
    // 4x4 block taps onto 64 channels (the 7x7x3 stride-2 head of an image network): the kernel that walks down
    // the rows with the filter in registers (PML_HIP_CONV_IGEMM keeps the implicit GEMM).  From a 3-channel bf16
    // image of even width it builds the 2x2 pixel blocks itself, row by row, and the re-blocking launch is skipped.
    const int path = PML_HIP_FLAG_CONV_OF(d.flags);
    const size_t lds = path == PML_HIP_CONV_IGEMM ? 0 : conv_blocks4x4_prepare(p->mfma_kind, g);
    const bool from_image = lds && d.ci == 3 && d.w % 2 == 0 && ((uintptr_t)input & 3) == 0 && path != PML_HIP_CONV_BLOCKS;
    if (!from_image) {
      {
        std::lock_guard<std::mutex> lock(p->s2d_mutex);
        // 256 spare bytes: a K-run that starts left of the image is addressed (never read) below the buffer's end only
        if (!p->s2d && hipMalloc(&p->s2d, (size_t)d.n * p->s2d_h * p->s2d_w * p->s2d_ch * es + 256) != hipSuccess) {
          p->s2d = nullptr;
          return fail("conv2d_invoke: cannot allocate the re-blocked input");
        }
      }
      g.A = p->s2d;
      S2dArgs sa;
      s2d_args(p, sa);
      sa.in = input;
      sa.out = p->s2d;
      if (check(s2d_input_launch(es, sa, (hipStream_t)s), "s2d_input_launch")) return 1;
    } else {
      g.raw_in = input;
      g.raw_h = (int)d.h;
      g.raw_w = (int)d.w;
    }
    if (lds) return check(conv_blocks4x4_launch(g, lds, device_cus(), (hipStream_t)s), "conv_blocks4x4_launch");
    return check(igemm_launch(p->mfma_kind, p->tile, true, g, (hipStream_t)s), "igemm_launch");
  }
  if (p->halo_lds)
    return check(conv_halo_launch(p->mfma_kind, g, p->halo_lds, p->n_cus, (hipStream_t)s), "conv_halo_launch");
  split_args(p, g);
  return check(igemm_launch(p->b_split ? KIND_F32X3P : p->mfma_kind, p->tile, true, g, (hipStream_t)s), "igemm_launch");
}

int pml_hip_gemm_pack_b(int64_t plan, const void* b, pml_hip_stream s) {
  Plan* p = (Plan*)(intptr_t)plan;
  if (!p || p->kind != PLAN_GEMM || !b) return fail("gemm_pack_b: bad argument");
  const pml_hip_gemm_desc& d = p->gemm;
  if (d.b_layout) return fail("gemm_pack_b: an [N][K] right-hand side needs no packing");
  if (check(transpose_pack(dt_size(d.in_dtype), b, p->bt, d.k, d.n, d.ldb, p->bt_ld, (hipStream_t)s), "transpose_pack"))
    return 1;
  if (p->b_split && check(split_rows_launch(p->bt, d.n, p->bt_ld, d.k, (hipStream_t)s), "split_rows_launch")) return 1;
  p->bt_is_split = p->b_split;
  p->packed = true;
  return 0;
}

int pml_hip_probe_mfma(int random_data, int iters, double* tflops, double* core_mhz) {
  if (iters <= 0 || iters > 100000) return fail("probe_mfma: iters out of range");
  const int blocks = device_cus();
  float* sink = nullptr;
  unsigned long long* clk = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  int rc = 1;
  do {
    if (check(hipMalloc((void**)&sink, 64), "hipMalloc") || check(hipMalloc((void**)&clk, 64), "hipMalloc")) break;
    if (check(hipEventCreate(&e0), "hipEventCreate") || check(hipEventCreate(&e1), "hipEventCreate")) break;
    if (check(mfma_probe_launch(blocks, 16, random_data, sink, clk, nullptr), "mfma_probe_launch")) break;  // warm-up
    if (check(hipEventRecord(e0, nullptr), "hipEventRecord")) break;
    if (check(mfma_probe_launch(blocks, iters, random_data, sink, clk, nullptr), "mfma_probe_launch")) break;
    if (check(hipEventRecord(e1, nullptr), "hipEventRecord") || check(hipEventSynchronize(e1), "hipEventSynchronize")) break;
    float ms = 0;
    if (check(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime")) break;
    unsigned long long host_clk[2] = {0, 0};
    if (check(hipMemcpy(host_clk, clk, sizeof host_clk, hipMemcpyDeviceToHost), "hipMemcpy")) break;
    const double mfmas = (double)iters * 4 * 8 * 8 * blocks;  // rounds x K-blocks x MFMAs per wavefront x wavefronts x workgroups
    if (tflops) *tflops = mfmas * 32768.0 / (ms * 1e-3) / 1e12;
    if (core_mhz) *core_mhz = host_clk[1] ? (double)host_clk[0] / ((double)host_clk[1] / 100.0) : 0.0;
    rc = 0;
  } while (false);
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  if (sink) (void)hipFree(sink);
  if (clk) (void)hipFree(clk);
  return rc;
}

const char* pml_hip_tile_name(int tile) { return tile >= 0 && tile < PML_HIP_TILE_COUNT_ ? kTileShort[tile] : nullptr; }
int pml_hip_tile_by_name(const char* name) {
  if (!name) return -1;
  for (int t = 0; t < PML_HIP_TILE_COUNT_; ++t)
    if (std::strcmp(name, kTileShort[t]) == 0) return t;
  return -1;
}

int pml_hip_tile_of_workgroup(int tiles_m, int tiles_n, int workgroup, int* tile_m, int* tile_n) {
  if (tiles_m <= 0 || tiles_n <= 0 || (int64_t)tiles_m * tiles_n >= ((int64_t)1 << 31) || workgroup < 0 ||
      workgroup >= tiles_m * tiles_n || !tile_m || !tile_n)
    return fail("tile_of_workgroup: bad argument");
  const TileOrder o = make_tile_order(tiles_m, tiles_n);
  tile_of(o, (unsigned)workgroup, tile_m, tile_n);
  return 0;
}

int pml_hip_gemm_pack_b2(int64_t plan, const void* b2, pml_hip_stream s) {
  Plan* p = (Plan*)(intptr_t)plan;
  if (!p || p->kind != PLAN_GEMM || !b2 || p->gemm.k2 <= 0) return fail("gemm_pack_b2: bad argument");
  const pml_hip_gemm_desc& d = p->gemm;
  if (d.b_layout) return fail("gemm_pack_b2: an [N][K] right-hand side needs no packing");
  if (check(transpose_pack(dt_size(d.in_dtype), b2, p->bt2, d.k2, d.n, d.ldb2, d.k2, (hipStream_t)s), "transpose_pack")) return 1;
  p->packed2 = true;
  return 0;
}

int pml_hip_conv2d_pack_filter(int64_t plan, const void* filter, pml_hip_stream s) {
  Plan* p = (Plan*)(intptr_t)plan;
  if (!p || p->kind != PLAN_CONV || !filter) return fail("conv2d_pack_filter: bad argument");
  const pml_hip_conv2d_desc& d = p->conv;
  if (check(pack_conv_filter(p, filter, (hipStream_t)s), "pack_conv_filter")) return 1;
  if (p->halo_lds && p->halo_variant == 3 && regfilter_takes_image((int)d.ow)) {
    // the register-filter kernel takes a constant filter in its own register order: no trip through LDS per launch
    if (!p->reg_image && check(hipMalloc(&p->reg_image, kRegfilterImageBytes), "hipMalloc")) return 1;
    if (check(regfilter_image_launch(p->bt, p->bt_ld * dt_size(d.in_dtype), p->reg_image, (hipStream_t)s), "regfilter_image_launch")) return 1;
  }
  p->packed = true;
  return 0;
}

// ---------------------------------------------------------------------------
// depthwise conv, pooling
// ---------------------------------------------------------------------------

int64_t pml_hip_dwconv2d_dispatch(const pml_hip_dwconv2d_desc* d) {
  if (!d) {
    fail("null descriptor");
    return 0;
  }
  if (d->dtype != PML_HIP_F32 && d->dtype != PML_HIP_BF16) {
    fail("dwconv2d: dtype must be F32 or BF16");
    return 0;
  }
  const int V = 16 / dt_size(d->dtype);
  if (d->c <= 0 || d->c % V != 0) {
    fail("dwconv2d: channels must cover whole 16-byte vectors");
    return 0;
  }
  if (d->n <= 0 || d->h <= 0 || d->w <= 0 || d->kh <= 0 || d->kw <= 0 || d->oh <= 0 || d->ow <= 0 ||
      d->stride_h <= 0 || d->stride_w <= 0 || d->dil_h <= 0 || d->dil_w <= 0 || !valid_tail(d->tail)) {
    fail("dwconv2d: bad geometry or tail");
    return 0;
  }
  if (d->out_pitch != 0 && d->out_pitch != d->c &&
      (d->out_pitch < d->c || d->out_pitch % V != 0 || d->tail.n_ops != 0 ||
       d->n * d->oh * d->ow * (int64_t)d->out_pitch >= ((int64_t)1 << 40))) {
    fail("dwconv2d: the output pitch must be at least c, a whole number of 16-byte vectors, and has no tail");
    return 0;
  }
  Plan* p = new Plan();
  p->kind = PLAN_DWCONV;
  p->dw = *d;
  char buf[200];
  std::snprintf(buf, sizeof buf, "dwconv2d %s n=%lld %lldx%lldx%lld k=%lldx%lld -> %lldx%lld (16B channel vectors)",
                d->dtype == PML_HIP_F32 ? "f32" : "bf16", (long long)d->n, (long long)d->h, (long long)d->w,
                (long long)d->c, (long long)d->kh, (long long)d->kw, (long long)d->oh, (long long)d->ow);
  p->text = buf;
  int64_t ysegs, seg_rows;
  if (dwconv2d_walks_rows(*d, device_cus(), &ysegs, &seg_rows)) {
    std::snprintf(buf, sizeof buf, ", window rows walked in registers (%lld runs of %lld rows)", (long long)ysegs, (long long)seg_rows);
    p->text += buf;
  }
  return (int64_t)(intptr_t)p;
}

int pml_hip_dwconv2d_invoke(int64_t plan, const void* input, const void* filter, void* output,
                            const void* const* operands, void* const* outs, pml_hip_stream s) {
  Plan* p = (Plan*)(intptr_t)plan;
  if (!p || p->kind != PLAN_DWCONV) return fail("dwconv2d_invoke: not a dwconv2d plan");
  if (!input || !output) return fail("dwconv2d_invoke: null operand");
  if (!filter && !p->dw_filter) return fail("dwconv2d_invoke: filter is null and no packed filter exists");
  if ((((uintptr_t)input | (uintptr_t)filter | (uintptr_t)output) & 15) != 0)
    return fail("dwconv2d_invoke: buffers must be 16-byte aligned");
  DwconvArgs a;
  std::memset(&a, 0, sizeof a);
  a.d = p->dw;
  a.in = input;
  a.filter = filter ? filter : p->dw_filter;
  a.paired_filter = filter ? nullptr : p->dw_paired;
  a.n_cus = device_cus();
  a.out = output;
  for (int i = 0; i < a.d.tail.n_operands; ++i) {
    if (!operands || !operands[i]) return fail("dwconv2d_invoke: missing tail operand");
    a.operands[i] = operands[i];
  }
  for (int i = 0; i < PML_HIP_MAX_EPI_OPERANDS; ++i) a.outs[i] = outs ? outs[i] : nullptr;
  return check(dwconv2d_launch(a, (hipStream_t)s), "dwconv2d_launch");
}

int pml_hip_dwconv2d_pack_filter(int64_t plan, const void* filter, pml_hip_stream s) {
  Plan* p = (Plan*)(intptr_t)plan;
  if (!p || p->kind != PLAN_DWCONV || !filter) return fail("dwconv2d_pack_filter: bad argument");
  const pml_hip_dwconv2d_desc& d = p->dw;
  const size_t bytes = (size_t)d.kh * d.kw * d.c * dt_size(d.dtype);
  if (!p->dw_filter && check(hipMalloc(&p->dw_filter, bytes), "hipMalloc")) return 1;
  if (check(hipMemcpyAsync(p->dw_filter, filter, bytes, hipMemcpyDeviceToDevice, (hipStream_t)s), "hipMemcpyAsync")) return 1;
  if (p->dw_paired) {
    (void)hipFree(p->dw_paired);
    p->dw_paired = nullptr;
  }
  if (!dwconv2d_takes_paired_filter(d)) return 0;
  // once per filter: its weights are looked at on the host (the paired kernel is for finite weights only) and re-laid there
  std::vector<uint16_t> host(bytes / 2);
  if (check(hipMemcpyAsync(host.data(), p->dw_filter, bytes, hipMemcpyDeviceToHost, (hipStream_t)s), "hipMemcpyAsync") ||
      check(hipStreamSynchronize((hipStream_t)s), "hipStreamSynchronize"))
    return 1;
  std::vector<uint32_t> packed((size_t)12 * (d.c / 8) * 4);
  if (!dwconv2d_pair_filter(host.data(), d.c, packed.data())) return 0;  // an infinite or NaN weight: the general kernel
  if (check(hipMalloc(&p->dw_paired, packed.size() * 4), "hipMalloc")) return 1;
  if (check(hipMemcpy(p->dw_paired, packed.data(), packed.size() * 4, hipMemcpyHostToDevice), "hipMemcpy")) {
    (void)hipFree(p->dw_paired);
    p->dw_paired = nullptr;
    return 1;
  }
  return 0;
}

int64_t pml_hip_pool2d_dispatch(const pml_hip_pool2d_desc* d) {
  if (!d) {
    fail("null descriptor");
    return 0;
  }
  if (d->dtype != PML_HIP_F32 && d->dtype != PML_HIP_BF16) {
    fail("pool2d: dtype must be F32 or BF16");
    return 0;
  }
  if (d->agg != PML_HIP_AGG_MAX && d->agg != PML_HIP_AGG_MIN && d->agg != PML_HIP_AGG_ADD) {
    fail("pool2d: aggregation must be max, min or add");
    return 0;
  }
  const int V = 16 / dt_size(d->dtype);
  if (d->c <= 0 || d->c % V != 0 || d->n <= 0 || d->h <= 0 || d->w <= 0 || d->kh <= 0 || d->kw <= 0 || d->oh <= 0 ||
      d->ow <= 0 || d->stride_h <= 0 || d->stride_w <= 0) {
    fail("pool2d: bad geometry (channels must cover whole 16-byte vectors)");
    return 0;
  }
  if (d->divisor != 0.f) {
    // (what pool_whole_kernel takes: pool2d_launch's own test)
    const int64_t chunks = (d->c / V + 31) / 32;
    const bool whole = d->agg == PML_HIP_AGG_ADD && d->oh == 1 && d->ow == 1 && d->kh == d->h && d->kw == d->w && d->pad_h == 0 &&
                       d->pad_w == 0 && !d->with_index && d->h * d->w >= 16 && d->n * chunks <= 0x7fffffff;
    if (!whole || !(d->divisor == d->divisor)) {
      fail("pool2d: a divisor goes with the sum over a whole image of at least 16 pixels only");
      return 0;
    }
  }
  Plan* p = new Plan();
  p->kind = PLAN_POOL;
  p->pool = *d;
  char buf[200];
  std::snprintf(buf, sizeof buf, "pool2d %s agg=%d n=%lld %lldx%lldx%lld k=%lldx%lld -> %lldx%lld%s",
                d->dtype == PML_HIP_F32 ? "f32" : "bf16", d->agg, (long long)d->n, (long long)d->h, (long long)d->w,
                (long long)d->c, (long long)d->kh, (long long)d->kw, (long long)d->oh, (long long)d->ow,
                d->with_index ? " +argmax" : "");
  p->text = buf;
  return (int64_t)(intptr_t)p;
}

int pml_hip_pool2d_invoke(int64_t plan, const void* input, void* output, void* index_output, pml_hip_stream s) {
  Plan* p = (Plan*)(intptr_t)plan;
  if (!p || p->kind != PLAN_POOL) return fail("pool2d_invoke: not a pool2d plan");
  if (!input || !output) return fail("pool2d_invoke: null operand");
  if (p->pool.with_index && !index_output) return fail("pool2d_invoke: the plan expects an index output");
  if ((((uintptr_t)input | (uintptr_t)output | (uintptr_t)index_output) & 15) != 0)
    return fail("pool2d_invoke: buffers must be 16-byte aligned");
  PoolArgs a;
  a.d = p->pool;
  a.in = input;
  a.out = output;
  a.idx = index_output;
  return check(pool2d_launch(a, (hipStream_t)s), "pool2d_launch");
}

// ---------------------------------------------------------------------------
// elementwise, select, index
// ---------------------------------------------------------------------------

int64_t pml_hip_eltwise_dispatch(const pml_hip_eltwise_desc* d) {
  if (!d) {
    fail("null descriptor");
    return 0;
  }
  if (d->rank < 0 || d->rank > PML_HIP_MAX_RANK) {
    fail("eltwise: rank out of range");
    return 0;
  }
  const pml_hip_epilogue& t = d->tail;
  if (t.n_ops < 0 || t.n_ops > PML_HIP_MAX_EPI_OPS || t.n_operands < 0 || t.n_operands > PML_HIP_MAX_EPI_OPERANDS) {
    fail("eltwise: malformed tail");
    return 0;
  }
  if (!valid_tail(t, /*allow64=*/true)) {
    fail("eltwise: a step of the chain names an unknown operation or an operand outside the operand list");
    return 0;
  }
  Plan* p = new Plan();
  p->kind = PLAN_ELTWISE;
  p->elt = *d;
  p->text = "eltwise chain of " + std::to_string(t.n_ops) + " steps, rank " + std::to_string(d->rank);
  return (int64_t)(intptr_t)p;
}

int pml_hip_eltwise_invoke(int64_t plan, const void* input, void* output, const void* const* operands,
                           void* const* outs, pml_hip_stream s) {
  Plan* p = (Plan*)(intptr_t)plan;
  if (!p || p->kind != PLAN_ELTWISE) return fail("eltwise_invoke: not an eltwise plan");
  if (!input || !output) return fail("eltwise_invoke: null operand");
  EltwiseArgs a;
  std::memset(&a, 0, sizeof a);
  a.d = p->elt;
  a.in = input;
  a.out = output;
  a.total = 1;
  for (int r = 0; r < a.d.rank; ++r) a.total *= a.d.sizes[r];
  bool wide = dt_size(a.d.in_dtype) == 8 || dt_size(a.d.out_dtype) == 8;
  for (int i = 0; i < a.d.tail.n_operands; ++i) {
    if (!operands || !operands[i]) return fail("eltwise_invoke: missing operand");
    a.operands[i] = operands[i];
    wide = wide || dt_size(a.d.tail.operand_dtype[i]) == 8;
  }
  for (int i = 0; i < a.d.tail.n_ops; ++i) wide = wide || dt_size(a.d.tail.ops[i].dtype) == 8;
  for (int i = 0; i < PML_HIP_MAX_EPI_OPERANDS; ++i) a.outs[i] = outs ? outs[i] : nullptr;
  a.wide = wide ? 1 : 0;
  return check(eltwise_launch(a, (hipStream_t)s), "eltwise_launch");
}

int pml_hip_select(const pml_hip_select_desc* d, const void* cond, const void* t, const void* f, void* out,
                   pml_hip_stream s) {
  if (!d || !cond || !t || !f || !out) return fail("select: null argument");
  if (d->rank < 0 || d->rank > PML_HIP_MAX_RANK) return fail("select: rank out of range");
  return check(select_launch(*d, cond, t, f, out, (hipStream_t)s), "select_launch");
}

int pml_hip_softmax(const pml_hip_softmax_desc* d, const void* x, void* y, pml_hip_stream s) {
  if (!d || !x || !y) return fail("softmax: null argument");
  if (d->dtype != PML_HIP_F32 && d->dtype != PML_HIP_BF16) return fail("softmax: dtype must be F32 or BF16");
  if (d->rows < 0 || d->cols < 0 || d->rows > 0x7fffffff) return fail("softmax: rows or cols out of range");
  return check(softmax_launch(*d, x, y, (hipStream_t)s), "softmax_launch");
}

int pml_hip_index(void* out, int32_t rank, const int64_t* sizes, int32_t axis, pml_hip_stream s) {
  if (!out || !sizes || rank <= 0 || axis < 0 || axis >= rank) return fail("index: bad argument");
  return check(index_launch(out, rank, sizes, axis, (hipStream_t)s), "index_launch");
}

// ---------------------------------------------------------------------------
// special operations
// ---------------------------------------------------------------------------

namespace {
bool sizes_ok(const int64_t* sizes, int rank) {
  for (int i = 0; i < rank; ++i)
    if (sizes[i] < 0) return false;
  return true;
}
int64_t count_of(const int64_t* sizes, int rank) {
  int64_t n = 1;
  for (int i = 0; i < rank; ++i) n *= sizes[i];
  return n;
}
}  // namespace

int pml_hip_gather(const pml_hip_gather_desc* d, const void* tensor, const void* indices, void* out, pml_hip_stream s) {
  if (!d || !tensor || !indices || !out) return fail("gather: null argument");
  if (d->rank < 1 || d->rank > PML_HIP_MAX_SPECIAL_RANK || d->idx_rank < 0 || d->idx_rank > PML_HIP_MAX_SPECIAL_RANK)
    return fail("gather: rank out of range");
  if (!sizes_ok(d->sizes, d->rank) || !sizes_ok(d->idx_sizes, d->idx_rank)) return fail("gather: negative size");
  if (dt_size(d->dtype) == 0 || dt_size(d->idx_dtype) == 0) return fail("gather: bad element type");
  if (d->mode == PML_HIP_GATHER_NORMAL) {
    if (d->axis < 0 || d->axis >= d->rank) return fail("gather: axis out of range");
    if (d->rank - 1 + d->idx_rank > PML_HIP_MAX_SPECIAL_RANK) return fail("gather: result rank out of range");
    if (dt_is_float(d->idx_dtype) && dt_is_float(d->dtype)) {
      if (d->interpolation < PML_HIP_INTERP_NEAREST || d->interpolation > PML_HIP_INTERP_CUBIC)
        return fail("gather: floating indices need an interpolation mode");
      if (d->interpolation == PML_HIP_INTERP_NEAREST && (d->nearest < 0 || d->nearest > PML_HIP_NEAREST_SIMPLE))
        return fail("gather: bad nearest mode");
      if (d->oob != PML_HIP_OOB_EDGE_PADDED_INPUT && d->oob != PML_HIP_OOB_RETURN_ZERO) return fail("gather: bad out-of-bounds mode");
    }
  } else if (d->mode == PML_HIP_GATHER_ND) {
    if (dt_is_float(d->idx_dtype)) return fail("gather: ND mode needs integer indices");
    if (d->idx_rank < 1) return fail("gather: ND mode needs indices of rank >= 1");
    const int64_t k = d->idx_sizes[d->idx_rank - 1];
    if (d->batch_dims < 0 || d->batch_dims > d->idx_rank - 1 || d->batch_dims + k > d->rank)
      return fail("gather: ND index depth out of range");
    if (d->idx_rank - 1 + d->rank - d->batch_dims - k > PML_HIP_MAX_SPECIAL_RANK) return fail("gather: result rank out of range");
    for (int i = 0; i < d->batch_dims; ++i)
      if (d->sizes[i] != d->idx_sizes[i]) return fail("gather: batch dimensions differ");
  } else {
    return fail("gather: bad mode");
  }
  return check(gather_launch(*d, tensor, indices, out, (hipStream_t)s), "gather_launch");
}

int pml_hip_scatter(const pml_hip_scatter_desc* d, const void* data, const void* indices, const void* updates, void* out,
                    pml_hip_stream s) {
  if (!d || !data || !indices || !updates || !out) return fail("scatter: null argument");
  if (out == data) return fail("scatter: the result must not alias the data");
  if (d->rank < 1 || d->rank > PML_HIP_MAX_SPECIAL_RANK || d->idx_rank < 1 || d->idx_rank > PML_HIP_MAX_SPECIAL_RANK ||
      d->upd_rank < 1 || d->upd_rank > PML_HIP_MAX_SPECIAL_RANK)
    return fail("scatter: rank out of range");
  if (!sizes_ok(d->sizes, d->rank) || !sizes_ok(d->idx_sizes, d->idx_rank) || !sizes_ok(d->upd_sizes, d->upd_rank))
    return fail("scatter: negative size");
  if (d->idx_dtype != PML_HIP_I32 && d->idx_dtype != PML_HIP_U32) return fail("scatter: indices must be si32 or ui32");
  if (dt_size(d->dtype) == 0) return fail("scatter: bad element type");
  if (d->axis < 0 || d->axis >= d->rank) return fail("scatter: axis out of range");
  // every update element must name a full coordinate of the result
  int dst_rank = 0;
  switch (d->mode) {
    case PML_HIP_SCATTER_UPDATE_ND: {
      const int64_t k = d->idx_sizes[d->idx_rank - 1];
      if (d->upd_rank < d->idx_rank - 1) return fail("scatter: updates have too few dimensions");
      dst_rank = (int)k + d->upd_rank - (d->idx_rank - 1);
      for (int i = 0; i + 1 < d->idx_rank; ++i)
        if (d->upd_sizes[i] != d->idx_sizes[i]) return fail("scatter: updates and indices disagree");
      break;
    }
    case PML_HIP_SCATTER_UPDATE_SLICE:
      if (d->upd_rank < d->axis + d->idx_rank) return fail("scatter: updates have too few dimensions");
      dst_rank = d->upd_rank - d->idx_rank + 1;
      for (int i = 0; i < d->idx_rank; ++i)
        if (d->upd_sizes[d->axis + i] != d->idx_sizes[i]) return fail("scatter: updates and indices disagree");
      break;
    case PML_HIP_SCATTER_NORMAL:
    case PML_HIP_SCATTER_UPDATE_ELT:
      if (d->upd_rank < d->idx_rank) return fail("scatter: updates have too few dimensions");
      dst_rank = d->upd_rank;
      for (int i = 0; i < d->idx_rank; ++i)
        if (d->upd_sizes[i] != d->idx_sizes[i]) return fail("scatter: updates and indices disagree");
      break;
    default: return fail("scatter: bad mode");
  }
  if (dst_rank != d->rank) return fail("scatter: updates do not address the result's rank");
  return check(scatter_launch(*d, data, indices, updates, out, (hipStream_t)s), "scatter_launch");
}

int pml_hip_prng(const void* state, int64_t count, void* values, void* new_state, pml_hip_stream s) {
  if (!state) return fail("prng: null state");
  if (count < 0) return fail("prng: negative count");
  if (!values && !new_state) return 0;
  return check(prng_launch(state, count, values, new_state, (hipStream_t)s), "prng_launch");
}

int pml_hip_argsort(const pml_hip_argsort_desc* d, const void* tensor, void* out, pml_hip_stream s) {
  if (!d || !tensor || !out) return fail("argsort: null argument");
  if (d->rank < 1 || d->rank > PML_HIP_MAX_SPECIAL_RANK) return fail("argsort: rank out of range");
  if (!sizes_ok(d->sizes, d->rank)) return fail("argsort: negative size");
  if (d->axis < 0 || d->axis >= d->rank) return fail("argsort: axis out of range");
  if (d->direction != 0 && d->direction != 1) return fail("argsort: bad direction");
  if (dt_size(d->dtype) == 0 || d->dtype == PML_HIP_BOOL) return fail("argsort: bad element type");
  if (d->sizes[d->axis] > PML_HIP_MAX_SORT_LINE)
    return fail("argsort: more than PML_HIP_MAX_SORT_LINE (16384) elements along the sorted axis");
  if (count_of(d->sizes, d->rank) == 0) return 0;
  return check(argsort_launch(*d, tensor, out, (hipStream_t)s), "argsort_launch");
}

// ---------------------------------------------------------------------------
// any contraction
// ---------------------------------------------------------------------------

int64_t pml_hip_contract_dispatch(const pml_hip_contract_desc* d) {
  if (!d) {
    fail("null descriptor");
    return 0;
  }
  if (d->n_idx < 0 || d->n_idx > PML_HIP_MAX_IDX || d->n_out_idx < 0 || d->n_out_idx > d->n_idx || d->n_forms < 0 ||
      d->n_forms > PML_HIP_MAX_FORMS || d->n_src < 1 || d->n_src > 3) {
    fail("contract: descriptor out of range");
    return 0;
  }
  int64_t outs = 1;
  for (int v = 0; v < d->n_out_idx; ++v) {
    if (d->hi[v] < d->lo[v]) {
      outs = 0;
      break;
    }
    outs *= d->hi[v] - d->lo[v] + 1;
  }
  if (outs != d->out_elems) {
    fail("contract: out_elems does not match the output index ranges");
    return 0;
  }
  for (int f = 0; f < d->n_forms; ++f) {
    if (d->forms[f].den <= 0 || d->forms[f].operand < -1 || d->forms[f].operand > d->n_src) {
      fail("contract: malformed form");
      return 0;
    }
  }
  if (d->combo == PML_HIP_COMBO_EQ && (d->dtype != PML_HIP_BOOL || d->n_src != 2)) {
    fail("contract: the eq combination takes two operands and gives a boolean result");
    return 0;
  }
  Plan* p = new Plan();
  p->kind = PLAN_CONTRACT;
  p->con = *d;
  p->text = "contract (thread per output element) agg=" + std::to_string(d->agg) + " combo=" + std::to_string(d->combo) +
            " idx=" + std::to_string(d->n_idx) + " outputs=" + std::to_string((long long)d->out_elems);
  return (int64_t)(intptr_t)p;
}

int pml_hip_contract_invoke(int64_t plan, const void* const* srcs, void* out, pml_hip_stream s) {
  Plan* p = (Plan*)(intptr_t)plan;
  if (!p || p->kind != PLAN_CONTRACT) return fail("contract_invoke: not a contract plan");
  if (!srcs || !out) return fail("contract_invoke: null operand");
  ContractArgs a;
  std::memset(&a, 0, sizeof a);
  a.d = p->con;
  for (int i = 0; i < a.d.n_src; ++i) {
    if (!srcs[i]) return fail("contract_invoke: null source");
    a.srcs[i] = srcs[i];
  }
  a.out = out;
  return check(contract_launch(a, (hipStream_t)s), "contract_launch");
}

size_t pml_hip_struct_size(int which) {
  switch (which) {
    case 0: return sizeof(pml_hip_epilogue);
    case 1: return sizeof(pml_hip_gemm_desc);
    case 2: return sizeof(pml_hip_conv2d_desc);
    case 3: return sizeof(pml_hip_dwconv2d_desc);
    case 4: return sizeof(pml_hip_pool2d_desc);
    case 5: return sizeof(pml_hip_eltwise_desc);
    case 6: return sizeof(pml_hip_select_desc);
    case 7: return sizeof(pml_hip_contract_desc);
    case 8: return sizeof(pml_hip_form);
    case 9: return sizeof(pml_hip_gather_desc);
    case 10: return sizeof(pml_hip_scatter_desc);
    case 11: return sizeof(pml_hip_argsort_desc);
    case 12: return sizeof(pml_hip_softmax_desc);
  }
  return 0;
}

int pml_hip_plan_free(int64_t plan) {
  delete (Plan*)(intptr_t)plan;
  return 0;
}

int pml_hip_plan_describe(int64_t plan, char* buf, size_t buf_len) {
  Plan* p = (Plan*)(intptr_t)plan;
  if (!p || !buf || buf_len == 0) return fail("plan_describe: bad argument");
  std::snprintf(buf, buf_len, "%s", p->text.c_str());
  return 0;
}

}  // extern "C"
