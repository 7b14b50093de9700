/*
 * pml_hip.h -- C ABI of the gfx950 kernel library that sits beneath the `hip`
 * runtime device, in the position the libxsmm shims occupy beneath `llvm_cpu`
 * in the reference (pmlc/rt/xsmm.cc:17-890).
 *
 * Shape of the interface follows the reference's dispatch-once / invoke-many
 * convention (pmlc/rt/xsmm.cc:17-56: `*_dispatch_*` returns an int64 handle at
 * compile time, `*_invoke_*` takes the handle plus raw pointers at run time).
 * Differences that the GPU forces: one invoke covers a whole contraction, not
 * one cache tile; pointers are device pointers; invokes are stream-ordered.
 *
 * Every function returns 0 on success and a non-zero status on failure unless
 * stated otherwise; pml_hip_last_error() gives the message for the calling
 * thread.  Plain C types only.
 *
 * A plan may own device memory that its invokes write: a right-hand side or filter
 * re-laid per invoke, a re-blocked input or patch matrix of a few-channel
 * convolution, the partial tiles of a K loop split over workgroups.  Invokes of ONE
 * plan must therefore not overlap (one stream, or streams ordered by events);
 * different plans are independent, and dispatching, packing and freeing plans is
 * safe from several threads.
 */
#ifndef PML_HIP_H_
#define PML_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types.  Values equal plaidml_datatype (plaidml/core/ffi.h:139-156);
 * bfloat16 is appended so that no existing value changes. */
enum {
  PML_HIP_BOOL = 4,
  PML_HIP_I8 = 5,
  PML_HIP_U8 = 6,
  PML_HIP_I16 = 7,
  PML_HIP_U16 = 8,
  PML_HIP_I32 = 9,
  PML_HIP_U32 = 10,
  PML_HIP_I64 = 11,
  PML_HIP_U64 = 12,
  PML_HIP_F16 = 13,
  PML_HIP_F32 = 14,
  PML_HIP_F64 = 15,
  PML_HIP_BF16 = 16
};

/* Aggregations and combinations of a contraction (pmlc/util/enums.td:9-33). */
enum { PML_HIP_AGG_ASSIGN = 0, PML_HIP_AGG_ADD = 1, PML_HIP_AGG_MAX = 2, PML_HIP_AGG_MIN = 3, PML_HIP_AGG_MUL = 4 };
enum { PML_HIP_COMBO_NONE = 0, PML_HIP_COMBO_ADD = 1, PML_HIP_COMBO_COND = 2, PML_HIP_COMBO_EQ = 3, PML_HIP_COMBO_MUL = 4 };

typedef void* pml_hip_stream; /* a hipStream_t; NULL is the default stream */
typedef void* pml_hip_event;  /* a hipEvent_t */

/* ---- library, device, memory, streams ------------------------------------
 * Counterpart of the process-level set-up the reference does in
 * pmlc::rt::registerXsmm (pmlc/rt/xsmm.cc:863-890, libxsmm_init) and of the host
 * buffers of pmlc/util/buffer.h:15-70, which here live in HBM. */
int pml_hip_init(int device_ordinal);
int pml_hip_device_count(void); /* number of devices, 0 if none; never fails */
int pml_hip_device_name(char* buf, size_t buf_len);
const char* pml_hip_last_error(void);

int pml_hip_malloc(void** dptr, size_t nbytes);
int pml_hip_free(void* dptr);
int pml_hip_host_alloc(void** hptr, size_t nbytes); /* pinned host memory */
int pml_hip_host_free(void* hptr);
int pml_hip_memcpy_h2d(void* dst, const void* src, size_t nbytes, pml_hip_stream s);
int pml_hip_memcpy_d2h(void* dst, const void* src, size_t nbytes, pml_hip_stream s);
int pml_hip_memcpy_d2d(void* dst, const void* src, size_t nbytes, pml_hip_stream s);
/* Fills with a 32-bit pattern using a kernel (safe to capture into a graph). */
int pml_hip_fill_u32(void* dptr, uint32_t pattern, size_t n_words, pml_hip_stream s);

int pml_hip_stream_create(pml_hip_stream* s);
int pml_hip_stream_destroy(pml_hip_stream s);
int pml_hip_stream_sync(pml_hip_stream s);
int pml_hip_event_create(pml_hip_event* e);
int pml_hip_event_destroy(pml_hip_event e);
int pml_hip_event_record(pml_hip_event e, pml_hip_stream s);
int pml_hip_event_sync(pml_hip_event e);
int pml_hip_event_elapsed_ms(pml_hip_event start, pml_hip_event stop, float* ms);

/* Replay of a fixed sequence of launches as one HIP graph: what the reference gets from jitting a whole program into
 * one function (pmlc/rt/jit_executable.cc:484-490 calls it once per run) -- here a run is many launches, and at small
 * batch the launches cost more than the kernels.  Between _begin and _end every launch on `s` (a stream made by
 * pml_hip_stream_create, never NULL) is recorded instead of run; every *_invoke of this library may be recorded once
 * it has run at least once on the same plan (first runs may allocate).  _end returns the replayable graph, or fails
 * (and leaves `s` usable) if something could not be recorded.  Pointers are baked in: replay with the same buffers. */
typedef void* pml_hip_graph;
int pml_hip_capture_begin(pml_hip_stream s);
int pml_hip_capture_end(pml_hip_stream s, pml_hip_graph* graph);
int pml_hip_graph_launch(pml_hip_graph graph, pml_hip_stream s);
int pml_hip_graph_destroy(pml_hip_graph graph);

/* ---- fused elementwise tail ------------------------------------------------
 * A chain of scalar operations applied to one running value per output
 * element.  It plays the role of the bias / ReLU variants of the reference
 * GEMM shims (plaidml_rt_xsmm_gemm_bias / _relu / _relu_beta1,
 * pmlc/rt/xsmm.cc:58-233) and of the TPP unary / binary kernels
 * (plaidml_rt_xsmm_unary_* :344-385, plaidml_rt_xsmm_binary_* :387-455), with the
 * scalar semantics of pmlc/conversion/tile_to_linalg/tile_to_linalg.cc:1227-1385.
 * After each step the value is rounded to that step's result type. */
enum {
  PML_HIP_EPI_ADD = 1,  /* v = v + x */
  PML_HIP_EPI_SUB,      /* v = v - x */
  PML_HIP_EPI_RSUB,     /* v = x - v */
  PML_HIP_EPI_MUL,      /* v = v * x */
  PML_HIP_EPI_DIV,      /* v = v / x */
  PML_HIP_EPI_RDIV,     /* v = x / v */
  PML_HIP_EPI_MAX,      /* v = (v < x) ? x : v */
  PML_HIP_EPI_MIN,      /* v = (v < x) ? v : x */
  PML_HIP_EPI_RELU,     /* v = (v < 0) ? 0 : v */
  PML_HIP_EPI_NEG,
  PML_HIP_EPI_EXP,
  PML_HIP_EPI_LOG,
  PML_HIP_EPI_SQRT,
  PML_HIP_EPI_TANH,
  PML_HIP_EPI_FLOOR,
  PML_HIP_EPI_CEIL,
  PML_HIP_EPI_ROUND,    /* C roundf: half away from zero */
  PML_HIP_EPI_CAST,     /* convert v to `dtype` (fp->int truncates toward zero) */
  PML_HIP_EPI_STORE,    /* store v to extra output `operand` (index into the outs array) */
  PML_HIP_EPI_CMP_LT,   /* v = (v < x), result BOOL */
  PML_HIP_EPI_CMP_GT,
  PML_HIP_EPI_CMP_LE,
  PML_HIP_EPI_CMP_GE,
  PML_HIP_EPI_CMP_EQ,
  PML_HIP_EPI_CMP_NE,
  PML_HIP_EPI_MAX_GT,   /* v = (v > x) ? v : x  (the lower bound of a clip) */
  /* float-only functions (tile.sin ... tile.erf lower to libm calls, pmlc/rt/llvm/builtin.cc:13-26) */
  PML_HIP_EPI_SIN,
  PML_HIP_EPI_COS,
  PML_HIP_EPI_TAN,
  PML_HIP_EPI_SINH,
  PML_HIP_EPI_COSH,
  PML_HIP_EPI_ASIN,
  PML_HIP_EPI_ACOS,
  PML_HIP_EPI_ATAN,
  PML_HIP_EPI_ASINH,
  PML_HIP_EPI_ACOSH,
  PML_HIP_EPI_ATANH,
  PML_HIP_EPI_ERF,
  PML_HIP_EPI_POW,      /* v = pow(v, x), float result types only */
  PML_HIP_EPI_RPOW,     /* v = pow(x, v) */
  PML_HIP_EPI_MOD,      /* v = v % x: fmod for floats, C remainder for integers (0 when x == 0) */
  PML_HIP_EPI_RMOD,     /* v = x % v */
  /* integer-only bit operations on the promoted type */
  PML_HIP_EPI_BIT_AND,
  PML_HIP_EPI_BIT_OR,
  PML_HIP_EPI_BIT_XOR,
  PML_HIP_EPI_BIT_NOT,  /* v = -1 - v */
  PML_HIP_EPI_SHL,      /* v = v << x */
  PML_HIP_EPI_RSHL,     /* v = x << v */
  PML_HIP_EPI_SHR,      /* v = v >> x: arithmetic when the step type is signed, logical when unsigned */
  PML_HIP_EPI_RSHR,     /* v = x >> v */
  /* truth-value operations: each side is first tested against zero (ordered for floats, so NaN counts
   * as false), result BOOL (LogicalOp / LogicalNotOp, pmlc/conversion/tile_to_linalg/tile_to_linalg.cc:311-370) */
  PML_HIP_EPI_LOGICAL_AND,
  PML_HIP_EPI_LOGICAL_OR,
  PML_HIP_EPI_LOGICAL_XOR,
  PML_HIP_EPI_LOGICAL_NOT, /* v = (v == 0) */
  PML_HIP_EPI_LAST_ = PML_HIP_EPI_LOGICAL_NOT
};

/* where the second operand x of a step comes from */
enum {
  PML_HIP_OPND_NONE = 0,
  PML_HIP_OPND_IMM = 1,    /* the immediate `imm` (converted to the step's type) */
  PML_HIP_OPND_TENSOR = 2  /* operands[`operand`], addressed by the per-call strides */
};

#define PML_HIP_MAX_EPI_OPS 12
#define PML_HIP_MAX_EPI_OPERANDS 6
#define PML_HIP_MAX_RANK 6

/* descriptor flag of gemm and conv2d (in_dtype F32 only): multiply fp32 operands as three bf16 products */
#define PML_HIP_FP32_AS_BF16X3 1

/* Schedule overrides, carried in `flags` of the gemm and conv2d descriptors beside the flag above (all zero: the
 * library's own choice per shape class).  They play the part of the per-contraction schedule the reference loads from
 * PLAIDML_SCHEDULE_PATH (pmlc/target/x86/pipeline.cc:267-272): a planner or a tuning run names the tiling of one
 * contraction without touching any process-wide state.
 *   bits 8..15  PML_HIP_FLAG_TILE(t): the output tile of the MFMA kernel, t one of PML_HIP_TILE_*
 *   bits 16..19 PML_HIP_FLAG_CONV(c): the convolution path, c one of PML_HIP_CONV_* (ignored by gemm)
 * A tile the element kind is not built for falls back to the nearest one that is; a convolution path the shape
 * does not qualify for is ignored.
 *   bits 20..24 PML_HIP_FLAG_MAXPOOL3x3S2(pt, pb, pl, pr) (conv2d only): a 3x3 stride-2 max-pool with 0 or 1 rows /
 *               columns of padding on each side runs over the convolution's result inside the launch, and `output`
 *               is the pooled tensor [n][(oh + pt + pb - 3) / 2 + 1][(ow + pl + pr - 3) / 2 + 1][co] -- bit for bit
 *               what pml_hip_pool2d (max) makes of the convolution's own output.  oh / ow stay the convolution's.
 *               Only where pml_hip_conv2d_takes_maxpool says so (the row-walking kernel of a few-channel stride-2
 *               bf16 convolution onto 64 channels with a plain tail: an image network's head); dispatch fails
 *               elsewhere.  Counterpart of the reference's producer / consumer fusion of such nests
 *               (pmlc/target/x86/pipeline.cc:304-322). */
enum {
  PML_HIP_TILE_64x64 = 0,      /* 4 wavefronts */
  PML_HIP_TILE_128x64,         /* 4 wavefronts of 64x32 */
  PML_HIP_TILE_128x128,        /* 4 wavefronts */
  PML_HIP_TILE_128x64_W8,      /* 8 wavefronts */
  PML_HIP_TILE_128x128_W8,     /* 8 wavefronts, three ring stages */
  PML_HIP_TILE_256x128_W16,    /* 16 wavefronts */
  PML_HIP_TILE_128x128_W8_S2,  /* 8 wavefronts, two ring stages (two workgroups per CU) */
  PML_HIP_TILE_64x64_W8_K2,    /* 8 wavefronts as two grids that split every slab's K-blocks */
  PML_HIP_TILE_256x256_W8,     /* 8 wavefronts of 128x64 */
  PML_HIP_TILE_128x64_N2,      /* 4 wavefronts of 32x64 (split fp32 kind only) */
  PML_HIP_TILE_192x384_W8,     /* 8 wavefronts of 96x96 (bf16 and int8) */
  PML_HIP_TILE_64x64_KSPLIT,   /* 64x64 tiles whose K loop is shared out among several workgroups, partial tiles added up by a second launch */
  PML_HIP_TILE_COUNT_
};
enum {
  PML_HIP_CONV_AUTO = 0,
  PML_HIP_CONV_IGEMM = 1,     /* implicit GEMM, never a resident-filter or row-walking kernel */
  PML_HIP_CONV_PATCHES = 2,   /* few-channel inputs through a patch matrix even where 2x2 pixel blocks would do */
  PML_HIP_CONV_LDSFILTER = 3, /* resident filter kept in LDS rather than in registers */
  PML_HIP_CONV_BLOCKS = 4     /* the row-walking stem kernel behind a separate re-blocking launch */
};
#define PML_HIP_FLAG_TILE(t) ((((t) + 1) & 0xff) << 8)
#define PML_HIP_FLAG_CONV(c) (((c) & 0xf) << 16)
#define PML_HIP_FLAG_TILE_OF(flags) ((((flags) >> 8) & 0xff) - 1) /* -1: none */
#define PML_HIP_FLAG_CONV_OF(flags) (((flags) >> 16) & 0xf)
#define PML_HIP_FLAG_MAXPOOL3x3S2(pt, pb, pl, pr) \
  ((1 << 20) | (((pt) & 1) << 21) | (((pb) & 1) << 22) | (((pl) & 1) << 23) | (((pr) & 1) << 24))
#define PML_HIP_FLAG_MAXPOOL_OF(flags) (((flags) >> 20) & 0x1f) /* 0: none; bit 0 set: fused, bits 1..4 = pt, pb, pl, pr */
/* Name of a tile as the plan dump and the `hip{tile=...}` target option spell it ("128x128w8s2"), NULL when out of range;
 * and the inverse (-1 for an unknown name).  Host arithmetic only. */
const char* pml_hip_tile_name(int tile);
int pml_hip_tile_by_name(const char* name);

typedef struct {
  int32_t opcode;
  int32_t dtype;        /* result element type of this step */
  int32_t operand_kind; /* PML_HIP_OPND_* */
  int32_t operand;      /* index into operands[] (TENSOR) or outs[] (STORE) */
  double imm;
} pml_hip_epi_op;

typedef struct {
  int32_t n_ops;
  int32_t n_operands;
  pml_hip_epi_op ops[PML_HIP_MAX_EPI_OPS];
  /* element type of each tensor operand */
  int32_t operand_dtype[PML_HIP_MAX_EPI_OPERANDS];
  /* For a 2-D (rows x cols) output as produced by gemm / conv2d: element strides
   * of each tensor operand along the row and the column of the output
   * (0 = broadcast).  A per-channel bias is {0, 1}. */
  int64_t operand_row_stride[PML_HIP_MAX_EPI_OPERANDS];
  int64_t operand_col_stride[PML_HIP_MAX_EPI_OPERANDS];
} pml_hip_epilogue;

/* ---- dense contraction: GEMM ------------------------------------------------
 * C[m,n] = tail( init[m,n] + sum_k A[m,k] * B[k,n] ), row-major with leading
 * dimensions, one launch per contraction.
 * Replaces plaidml_rt_xsmm_gemm_dispatch_f32 / _invoke_f32 and the bias / relu
 * variants (pmlc/rt/xsmm.cc:17-233), and the strided batch-reduce
 * plaidml_rt_xsmm_brgemm_* (:235-287).
 *   in_dtype F32  -> fp32 MFMA, fp32 accumulate; with PML_HIP_FP32_AS_BF16X3 in `flags` every operand value is
 *                    split into a bf16 head and a bf16 remainder in registers and each product is formed as
 *                    head*head + remainder*head + head*remainder on the bf16 matrix cores (fp32 accumulate):
 *                    about 2^-16 relative error per product instead of 2^-24, at several times the fp32 MFMA rate
 *   in_dtype BF16 -> bf16 MFMA, fp32 accumulate, result rounded once to acc_dtype's storage
 *   in_dtype I8   -> int8 MFMA, int32 accumulate (this is the `cast(A, INT32)` then
 *                    contract pattern of plaidml/edsl/tests/edsl_test.cc:509-545 applied to int8)
 * out_dtype is the element type of the contraction result (F32, BF16 or I32); the
 * tail then runs on that value and the final value is stored to C in the type of
 * the last step (or out_dtype when the tail is empty). */
typedef struct {
  int32_t in_dtype;
  int32_t out_dtype;
  int64_t m, n, k;
  int64_t lda, ldb, ldc;
  /* optional initial value (AddInitPattern, pmlc/dialect/tile/transforms/algebraic_opt.cc:30-75):
   * init_kind 0 = none, 1 = tensor addressed with init_row_stride / init_col_stride */
  int32_t init_kind;
  int32_t init_dtype;
  int64_t init_row_stride, init_col_stride;
  int32_t c_dtype;  /* element type stored to C (type after the tail) */
  int32_t b_layout; /* 0: B is [K][N] with leading dimension ldb; 1: B is [N][K] (K contiguous, ldb >= k) */
  pml_hip_epilogue tail;
  /* Optional second product summed into the same accumulators before the tail, C = tail(init + init2 + A.B + A2.B2):
   * what a residual block's projection shortcut and its main path's last 1x1 convolution compute together (the
   * reference fuses producer and consumer loop nests, pmlc/target/x86/pipeline.cc:304-322; here the two
   * contractions share one result tile).  k2 = 0: none.  A2 is [M][k2] with leading dimension lda2, or, with
   * a2_stride > 0, the rows a 1x1 convolution with that stride (no padding) reads from an NHWC image of
   * a2_h x a2_w pixels of lda2 elements each: row m = (image, oy, ox) of an a2_oh x a2_ow result starts at pixel
   * (oy * a2_stride, ox * a2_stride).  B2 is [k2][N] (leading dimension ldb2) or [N][k2] like B (b_layout).
   * init2_kind 1: a second per-column initial value, a contiguous vector of out_dtype.  bf16 GEMMs only. */
  int64_t k2, lda2, ldb2;
  int32_t a2_stride;
  int32_t init2_kind;
  int64_t a2_h, a2_w, a2_oh, a2_ow;
  int32_t flags; /* PML_HIP_FP32_AS_BF16X3, PML_HIP_FLAG_TILE(t), or 0 */
  int32_t reserved;
} pml_hip_gemm_desc;

int64_t pml_hip_gemm_dispatch(const pml_hip_gemm_desc* desc); /* 0 on failure */
int pml_hip_gemm_invoke(int64_t plan, const void* a, const void* b, void* c, const void* init,
                        const void* const* operands, void* const* outs, pml_hip_stream s);
/* Right-hand sides that are constants of the program (weights) are re-laid-out once, the way the
 * reference runs its `init` closure once when the executable is built
 * (pmlc/rt/jit_executable.cc:404-418): after pack_b, invoke may be given b == NULL. */
int pml_hip_gemm_pack_b(int64_t plan, const void* b, pml_hip_stream s);
/* The same pair for a plan with a second product (k2 > 0): invoke2 also takes its operands, pack_b2 re-lays-out a
 * constant B2 once (invoke2 may then be given b2 == NULL). */
int pml_hip_gemm_invoke2(int64_t plan, const void* a, const void* b, void* c, const void* init, const void* a2, const void* b2,
                         const void* init2, const void* const* operands, void* const* outs, pml_hip_stream s);
int pml_hip_gemm_pack_b2(int64_t plan, const void* b2, pml_hip_stream s);

/* Measurement aid (no counterpart in the reference): the bf16 rate the matrix cores of the current device sustain on
 * operands that stay in LDS -- the instruction mix of the large GEMM tile, no global memory -- with constant operand
 * values (random_data 0) or random ones of magnitude about 1 (random_data 1), and the core clock during the run.
 * Random values make the chip lower its clock: the second figure is the ceiling a GEMM on N(0,1) data can reach. */
int pml_hip_probe_mfma(int random_data, int iters, double* tflops, double* core_mhz);

/* 1 when this GEMM runs faster with its tail left to a separate element-wise launch than with the tail fused, 0
 * otherwise (also for a malformed descriptor).  Today: int8 GEMMs large enough for the 256x256 tile, which a tail that
 * runs in steps (a requantisation chain) cannot use -- 4096^3 with that tail fused takes 108 us, the plain GEMM 72 us
 * and the chain over its int32 result 16 us.  A planner asks before it fuses (the reference decides fusion per nest
 * in pmlc/target/x86/pipeline.cc:304-322 without a cost model).  Makes no device call. */
int pml_hip_gemm_tail_cheaper_apart(const pml_hip_gemm_desc* desc);

/* Test aid (host arithmetic only, no device call; no counterpart in the reference): the tile (row block, column block)
 * that workgroup `workgroup` of a tiles_m x tiles_n GEMM grid works on.  The order keeps the tiles an XCD holds at any
 * time a compact block of the grid; the tests check that it visits every tile exactly once. */
int pml_hip_tile_of_workgroup(int tiles_m, int tiles_n, int workgroup, int* tile_m, int* tile_n);

/* The GEMM above in one call that allocates nothing, neither on the host heap of the device runtime nor in
 * device memory: dispatch + invoke without a plan object.  It has no counterpart in the reference; it is for
 * callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  The transposed copy of a [K][N] right-hand side (b_layout 0), which a plan keeps in memory of its
 * own, lives in a fixed array in the library's device image instead: n * k * element size must not exceed
 * PML_HIP_STATIC_SCRATCH_BYTES, larger right-hand sides are rejected with an error text that says so
 * (b_layout 1 needs no copy and has no such limit; a right-hand side that the kernels read where it lies leaves the
 * array untouched -- fp32 with n and ldb multiples of four and 16-byte aligned, int8 with rows of whole 16-byte
 * vectors on problems where transposing reads cost less than the copy -- and the limit applies all the same).
 * Each GPU holds one such array for the life of the process and
 * every call on that GPU uses it: calls that overlap on one GPU (two streams, two threads) race on it.  The
 * result equals pml_hip_gemm_dispatch + pml_hip_gemm_invoke bit for bit (same tile choice, same kernels). */
#define PML_HIP_STATIC_SCRATCH_BYTES (32 * 1024 * 1024)
int pml_hip_gemm_run_static(const pml_hip_gemm_desc* desc, const void* a, const void* b, void* c, const void* init,
                            const void* const* operands, void* const* outs, pml_hip_stream s);

/* ---- dense contraction: 2-D convolution, NHWC (x) HWCK ------------------------
 * O[n,y,x,co] = tail( init + sum_{ky,kx,ci} I[n, sy*y + dy*ky - py, sx*x + dx*kx - px, ci] * F[ky,kx,ci,co] )
 * over the taps that fall inside the input (out-of-range taps are not part of
 * the index set: docs/usage/edsl_ops.rst:24-44).  The index formulas are the
 * ones plaidml/op/lib/ops.cc:1342-1450 emits for NXC / XCK layouts.
 * Replaces the offset batch-reduce shims plaidml_rt_xsmm_brgemm_offs_*
 * (pmlc/rt/xsmm.cc:289-342,457-861).  The tail sees the output as a
 * (n*oh*ow) x co matrix. */
typedef struct {
  int32_t in_dtype;
  int32_t out_dtype;
  int64_t n, h, w, ci;
  int64_t kh, kw, co;
  int64_t oh, ow;
  int64_t stride_h, stride_w;
  int64_t dil_h, dil_w;
  int64_t pad_h, pad_w; /* pad_before */
  int32_t init_kind;
  int32_t init_dtype;
  int64_t init_row_stride, init_col_stride;
  int32_t c_dtype;
  int32_t flags; /* PML_HIP_FP32_AS_BF16X3, PML_HIP_FLAG_TILE(t), PML_HIP_FLAG_CONV(c), or 0 */
  pml_hip_epilogue tail;
} pml_hip_conv2d_desc;

int64_t pml_hip_conv2d_dispatch(const pml_hip_conv2d_desc* desc);
/* 1 when a descriptor carrying PML_HIP_FLAG_MAXPOOL3x3S2 would be accepted by pml_hip_conv2d_dispatch (host arithmetic
 * only: a planner asks before it folds a pooling step into the convolution in front of it). */
int pml_hip_conv2d_takes_maxpool(const pml_hip_conv2d_desc* desc);
int pml_hip_conv2d_invoke(int64_t plan, const void* input, const void* filter, void* output, const void* init,
                          const void* const* operands, void* const* outs, pml_hip_stream s);
/* Same as pml_hip_gemm_pack_b for a constant filter: afterwards invoke may be given filter == NULL. */
int pml_hip_conv2d_pack_filter(int64_t plan, const void* filter, pml_hip_stream s);

/* ---- depthwise 2-D convolution, NHWC, channel multiplier 1 --------------------
 * O[n,y,x,c] = tail( sum_{ky,kx} I[n, sy*y + ky - py, sx*x + kx - px, c] * F[ky,kx,c,0] )
 * (GroupLayout IN_C + AutoGroupMode DEPTHWISE, plaidml/op/lib/ops.cc:1034-1045,1380-1384).
 * Bandwidth-bound; the reference runs it as scalar loops after
 * linalgx-regulate-depthwise (pmlc/dialect/linalgx/transforms/regulate_depthwise.cc:22-60). */
typedef struct {
  int32_t dtype; /* F32 or BF16 */
  /* Elements between the starts of two output pixels; 0 = c (dense).  A larger pitch (a multiple of 16 bytes, no
   * tail) lets a consumer that reads the result as GEMM rows see every row start on a 128-byte line; the bytes
   * between c and the pitch are not written. */
  int32_t out_pitch;
  int64_t n, h, w, c;
  int64_t kh, kw;
  int64_t oh, ow;
  int64_t stride_h, stride_w;
  int64_t dil_h, dil_w;
  int64_t pad_h, pad_w;
  pml_hip_epilogue tail; /* rows = n*oh*ow, cols = c */
} pml_hip_dwconv2d_desc;

int64_t pml_hip_dwconv2d_dispatch(const pml_hip_dwconv2d_desc* desc);
int pml_hip_dwconv2d_invoke(int64_t plan, const void* input, const void* filter, void* output,
                            const void* const* operands, void* const* outs, pml_hip_stream s);
/* Same as pml_hip_conv2d_pack_filter for a constant depthwise filter: the plan keeps a copy, and invoke may afterwards
 * be given filter == NULL.  A 3x3 bf16 filter whose weights are all finite is also re-laid for a kernel that multiplies
 * the taps of two filter rows in one instruction; the weights are looked at here, once, instead of in every launch.
 * Waits for the stream (the filter is read back to the host). */
int pml_hip_dwconv2d_pack_filter(int64_t plan, const void* filter, pml_hip_stream s);

/* ---- window reduction: 2-D pooling, NHWC --------------------------------------
 * O[n,y,x,c] = agg_{ky<kh,kx<kw} I[n, sy*y + ky - py, sx*x + kx - px, c] over in-range taps
 * (plaidml/op/lib/ops.cc:2562-2703).  With `with_index`, a second output receives
 * max_{taps with I == O} (ky*kw + kx) as int32: the cond/max argmax pattern of
 * plaidml/op/lib/ops.cc:505-521 restricted to the window (ties -> largest index;
 * a NaN tap is never selected). */
typedef struct {
  int32_t dtype; /* F32 or BF16 */
  int32_t agg;   /* PML_HIP_AGG_MAX / MIN / ADD */
  int64_t n, h, w, c;
  int64_t kh, kw;
  int64_t oh, ow;
  int64_t stride_h, stride_w;
  int64_t pad_h, pad_w;
  int32_t with_index;
  /* 0: none.  Otherwise the aggregate, rounded to `dtype`, is divided by this value and rounded again -- a mean written
   * as sum / count (plaidml/op/lib/ops.cc:1970-2003) in one launch.  ADD over the whole image only (kh = h, kw = w,
   * no padding, no index); any other descriptor with a divisor is rejected. */
  float divisor;
} pml_hip_pool2d_desc;

int64_t pml_hip_pool2d_dispatch(const pml_hip_pool2d_desc* desc);
int pml_hip_pool2d_invoke(int64_t plan, const void* input, void* output, void* index_output, pml_hip_stream s);

/* ---- standalone elementwise chain -----------------------------------------------
 * out[i] = tail(in[i]) over an N-d output with broadcasting operands; the
 * counterpart of plaidml_rt_xsmm_unary_* / _binary_* (pmlc/rt/xsmm.cc:344-455)
 * with the broadcast rule of buildBroadcastMap
 * (pmlc/conversion/tile_to_linalg/tile_to_linalg.cc:443-472). */
typedef struct {
  int32_t rank;
  int32_t in_dtype;
  int32_t out_dtype;
  int32_t reserved;
  int64_t sizes[PML_HIP_MAX_RANK];     /* output sizes */
  int64_t in_strides[PML_HIP_MAX_RANK]; /* element strides of the first input (0 = broadcast) */
  int64_t operand_strides[PML_HIP_MAX_EPI_OPERANDS][PML_HIP_MAX_RANK];
  pml_hip_epilogue tail; /* row/col strides unused here */
} pml_hip_eltwise_desc;

int64_t pml_hip_eltwise_dispatch(const pml_hip_eltwise_desc* desc);
int pml_hip_eltwise_invoke(int64_t plan, const void* input, void* output, const void* const* operands,
                           void* const* outs, pml_hip_stream s);

/* ---- softmax over the last axis -------------------------------------------------
 * y[r, c] = e[r, c] / sum_c e[r, c] with e[r, c] = exp(x[r, c] - max_c x[r, c]): the five operations the op library
 * composes a softmax from (plaidml/op/lib/ops.cc:3049-3098: contraction max, sub, exp, contraction add, div) in one
 * launch instead of four, every intermediate rounded to `dtype` as those operations round it (the maximum by
 * `v > acc ? v : acc` from -inf, the sum accumulated in fp32 and rounded once).  x and y are dense [rows][cols]. */
typedef struct {
  int32_t dtype; /* F32 or BF16 */
  int32_t reserved;
  int64_t rows, cols;
} pml_hip_softmax_desc;
int pml_hip_softmax(const pml_hip_softmax_desc* desc, const void* x, void* y, pml_hip_stream s);

/* three-input select(cond, t, f) with broadcasting (tile.select, SelectOp of
 * pmlc/conversion/tile_to_linalg/tile_to_linalg.cc:262-273) */
typedef struct {
  int32_t rank;
  int32_t cond_dtype;
  int32_t t_dtype, f_dtype, out_dtype;
  int32_t reserved;
  int64_t sizes[PML_HIP_MAX_RANK];
  int64_t cond_strides[PML_HIP_MAX_RANK], t_strides[PML_HIP_MAX_RANK], f_strides[PML_HIP_MAX_RANK];
} pml_hip_select_desc;
int pml_hip_select(const pml_hip_select_desc* desc, const void* cond, const void* t, const void* f, void* out,
                   pml_hip_stream s);

/* index(dims, axis) (tile.index, IndexOpConversion tile_to_linalg.cc:863-): int32 iota along `axis` */
int pml_hip_index(void* out, int32_t rank, const int64_t* sizes, int32_t axis, pml_hip_stream s);

/* ---- special operations --------------------------------------------------------
 * The three Tile operations that are not contractions or elementwise maps
 * (ArgSortOpConversion / GatherOpConversion / ScatterOpConversion,
 * pmlc/conversion/linalg_to_pxa/tile_to_pxa_special_patterns.cc:29-896).  Dense
 * row-major tensors; enum values follow plaidml/edsl/edsl.h:1034,1625-1642. */
#define PML_HIP_MAX_SPECIAL_RANK 8

enum { PML_HIP_INTERP_NEAREST = 0, PML_HIP_INTERP_LINEAR, PML_HIP_INTERP_CUBIC, PML_HIP_INTERP_NONE };
enum {
  PML_HIP_NEAREST_ROUND_PREFER_FLOOR = 0,
  PML_HIP_NEAREST_ROUND_PREFER_CEIL,
  PML_HIP_NEAREST_FLOOR,
  PML_HIP_NEAREST_CEIL,
  PML_HIP_NEAREST_SIMPLE,
  PML_HIP_NEAREST_NONE
};
enum { PML_HIP_GATHER_NORMAL = 0, PML_HIP_GATHER_ND = 1 };
enum { PML_HIP_OOB_EDGE_PADDED_INPUT = 0, PML_HIP_OOB_RETURN_ZERO = 1 };
enum { PML_HIP_SCATTER_NORMAL = 0, PML_HIP_SCATTER_UPDATE_SLICE, PML_HIP_SCATTER_UPDATE_ELT, PML_HIP_SCATTER_UPDATE_ND };

/* gather: NORMAL  out[a.., i.., b..] = tensor[a.., f(indices[i..]), b..] along `axis`; integer indices address
 * directly (no clamping, as in the reference), floating indices of a floating tensor interpolate (nearest /
 * linear / cubic, taps clamped to the edge, optionally zero outside), floating indices of an integer tensor
 * truncate.  ND  out[i.., b..] = tensor[batch.., indices[i.., 0..k-1].., b..] with `batch_dims` leading
 * dimensions shared by tensor and indices. */
typedef struct {
  int32_t dtype;     /* element type of tensor and result */
  int32_t idx_dtype; /* element type of indices */
  int32_t mode, interpolation, nearest, oob;
  int32_t axis, batch_dims;
  int32_t rank, idx_rank;
  double cube_coeff;
  int64_t sizes[PML_HIP_MAX_SPECIAL_RANK];     /* tensor */
  int64_t idx_sizes[PML_HIP_MAX_SPECIAL_RANK]; /* indices */
} pml_hip_gather_desc;
int pml_hip_gather(const pml_hip_gather_desc* desc, const void* tensor, const void* indices, void* out, pml_hip_stream s);

/* scatter: out = data, then every element of `updates` goes to the place its indices name: NORMAL adds
 * (duplicates accumulate; floating sums in arrival order), the UPDATE modes assign (duplicate targets are a
 * race there, as in the reference's parallel loop).  Indices are si32 / ui32.  `out` must not alias `data`. */
typedef struct {
  int32_t dtype;
  int32_t idx_dtype;
  int32_t mode, axis;
  int32_t rank, idx_rank, upd_rank, reserved;
  int64_t sizes[PML_HIP_MAX_SPECIAL_RANK];     /* data and result */
  int64_t idx_sizes[PML_HIP_MAX_SPECIAL_RANK];
  int64_t upd_sizes[PML_HIP_MAX_SPECIAL_RANK];
} pml_hip_scatter_desc;
int pml_hip_scatter(const pml_hip_scatter_desc* desc, const void* data, const void* indices, const void* updates, void* out,
                    pml_hip_stream s);

/* argsort along `axis`: out (si32, shape of the input) holds the positions of the input's elements in
 * ascending (direction 0) or descending (1) order; equal elements keep their input order (the reference's
 * stable selection sort with strict ordered compares). */
#define PML_HIP_MAX_SORT_LINE 16384 /* every element's rank is counted against the whole line: O(n^2) per line */
typedef struct {
  int32_t dtype;
  int32_t rank, axis, direction;
  int64_t sizes[PML_HIP_MAX_SPECIAL_RANK];
} pml_hip_argsort_desc;
int pml_hip_argsort(const pml_hip_argsort_desc* desc, const void* tensor, void* out, pml_hip_stream s);

/* prng: the three-component Tausworthe generator of the reference runtime (pmlc/rt/prng.cc:8-44).  `state` holds
 * three uint32 words; value i is (s0 ^ s1 ^ s2) / 2^32 of the state after i steps, `new_state` the state after
 * `count` steps.  Either output may be null.  The recurrences are linear over GF(2), so a thread reaches the start
 * of its run of values by applying precomputed powers of the step matrix instead of stepping from the beginning. */
int pml_hip_prng(const void* state, int64_t count, void* values, void* new_state, pml_hip_stream s);

/* ---- any contraction ---------------------------------------------------------
 * The loop-nest form a contraction takes after bounds computation: the
 * `affine.parallel` + `pxa.load` + `pxa.reduce` nest of
 * pmlc/conversion/linalg_to_pxa/linalg_to_pxa.cc:283-428 with residual
 * constraints as `affine.if`.  One GPU thread (or one wavefront, for long
 * reductions) owns one output element and walks the reduction box; used for
 * every contraction no specialised kernel matches, so that every Tile program
 * in scope runs on the device.
 *
 * Index variables are ordered output-first: the first n_out_idx variables
 * enumerate distinct output elements (their ranges multiply to the number of
 * threads), the remaining ones are reduced.  An access / constraint is a set of
 * linear forms (sum_i coef[i]*idx[i] + c0) / den that must be an integer q with
 * 0 <= q < size; a tuple failing any form is skipped. */
#define PML_HIP_MAX_IDX 12
#define PML_HIP_MAX_FORMS 32

typedef struct {
  int32_t coef[PML_HIP_MAX_IDX];
  int32_t c0;
  int32_t den;
  int32_t operand; /* 0 = output, 1.. = source, -1 = explicit constraint */
  int64_t size;
  int64_t stride; /* flat element stride of this dimension in its operand */
} pml_hip_form;

typedef struct {
  int32_t dtype;    /* element type of the result and of the arithmetic */
  int32_t agg;
  int32_t combo;
  int32_t n_idx;
  int32_t n_out_idx;
  int32_t n_src;
  int32_t n_forms;
  int32_t cmp_dtype; /* COMBO_COND, COMBO_EQ: element type the two comparands are compared in */
  int32_t src_dtype[3];
  int32_t has_init;  /* output buffer already holds the initial value; else the identity is used */
  int64_t lo[PML_HIP_MAX_IDX], hi[PML_HIP_MAX_IDX]; /* inclusive box */
  int64_t out_elems;
  double identity_f;  /* initial value when has_init == 0, floating result types */
  int64_t identity_i; /* same for integer result types (already narrowed to dtype) */
  pml_hip_form forms[PML_HIP_MAX_FORMS];
} pml_hip_contract_desc;

int64_t pml_hip_contract_dispatch(const pml_hip_contract_desc* desc);
int pml_hip_contract_invoke(int64_t plan, const void* const* srcs, void* out, pml_hip_stream s);

/* sizeof() of a descriptor struct as this library was compiled, so that a foreign-language
 * binding can verify its own layout: 0 epilogue, 1 gemm, 2 conv2d, 3 dwconv2d, 4 pool2d,
 * 5 eltwise, 6 select, 7 contract, 8 form, 9 gather, 10 scatter, 11 argsort, 12 softmax.  Returns 0 for an unknown id. */
size_t pml_hip_struct_size(int which);

/* Releases a plan returned by any *_dispatch. */
int pml_hip_plan_free(int64_t plan);
/* Writes a one-line description of the plan (kernel family, tile, grid) for plan dumps. */
int pml_hip_plan_describe(int64_t plan, char* buf, size_t buf_len);

#ifdef __cplusplus
}
#endif
#endif /* PML_HIP_H_ */
