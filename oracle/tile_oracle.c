/*
 * tile_oracle.c -- CPU restatement of the Tile contraction semantics.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker that the HIP path is
 * compared against; nothing in the shipped library links, loads or calls it.
 *
 * What it restates (reference file:line):
 *   - the valid index set of a contraction: every integer index tuple for
 *     which every access of the output and of every input is in bounds and
 *     every explicit constraint 0 <= poly < rhs holds
 *       docs/usage/edsl_ops.rst:24-44
 *       pmlc/dialect/tile/transforms/contraction.cc:229-248 (GatherConstraints)
 *     An access polynomial may carry a rational coefficient (the EDSL `/`);
 *     a tuple at which such a polynomial is not an integer is not valid
 *     (plaidml/edsl/tests/edsl_test.cc:2709-2719 FunkySum pins that).
 *   - combination in the result element type
 *       pmlc/conversion/tile_to_linalg/tile_to_linalg.cc:209-260 (StdOp),
 *       :430-441 (ContractionCondOp: (a == b) ? c : 0)
 *   - aggregation into the output element
 *       pmlc/conversion/pxa_to_affine/pxa_to_affine.cc:155-203
 *       max: v > acc ? v : acc    min: v < acc ? v : acc   (ordered compares,
 *       so a NaN value never replaces the accumulator)
 *   - integer arithmetic wraps in the element width (no widening of the
 *     accumulator; plaidml/edsl/examples/gemm.cc:66-77 GEMM_INT8 pins int8)
 *
 * The caller (tile_oracle.py) presents every source already converted to the
 * compute type and the output buffer already holding the initial value
 * (aggregation identity or the broadcast `init` tensor,
 * pmlc/conversion/tile_to_linalg/tile_to_linalg.cc:372-416,697-730).
 *
 * Pinned by tests/test_oracle_golden.py against the reference's own known-answer
 * vectors; see the header of tile_oracle.py for the list.
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>

#define MAX_IDX 16
#define MAX_ACC 4
#define MAX_RANK 8
#define MAX_CONS 64

enum { AGG_ASSIGN = 0, AGG_ADD = 1, AGG_MAX = 2, AGG_MIN = 3, AGG_MUL = 4 };
enum { COMBO_NONE = 0, COMBO_ADD = 1, COMBO_COND = 2, COMBO_EQ = 3, COMBO_MUL = 4 };
/* element types the interpreter computes in */
enum { T_F32 = 0, T_F64, T_I8, T_I16, T_I32, T_I64, T_U8, T_U16, T_U32, T_U64 };

/* One linear form  (sum_i coef[i]*idx[i] + c0) / den  that must be an integer q
 * with 0 <= q < size.  For accesses `stride` is the flat element stride of the
 * dimension; for explicit constraints stride is 0. */
typedef struct {
  int64_t coef[MAX_IDX];
  int64_t c0;
  int64_t den;
  int64_t size;
  int64_t stride;
  int operand; /* which access this form belongs to, -1 for a constraint */
} form_t;

typedef struct {
  int n_idx;
  int64_t lo[MAX_IDX], hi[MAX_IDX]; /* inclusive enumeration box */
  int n_forms;
  form_t forms[MAX_ACC * MAX_RANK + MAX_CONS];
  int n_operands; /* operand 0 is the output */
} nest_t;

static inline int64_t floordiv(int64_t a, int64_t b) {
  int64_t q = a / b, r = a % b;
  return (r != 0 && ((r < 0) != (b < 0))) ? q - 1 : q;
}

/* Tighten the enumeration box by interval propagation over all forms until a
 * fixed point.  Returns 0 if every index has finite bounds, -1 otherwise.
 * This only shrinks the box that is enumerated; membership is still decided
 * tuple by tuple, so a loose box costs time, never correctness. */
static int propagate_bounds(nest_t* n) {
  const int64_t INF = (int64_t)1 << 60;
  for (int i = 0; i < n->n_idx; i++) {
    n->lo[i] = -INF;
    n->hi[i] = INF;
  }
  for (int iter = 0; iter < 64; iter++) {
    int changed = 0;
    for (int f = 0; f < n->n_forms; f++) {
      form_t* fm = &n->forms[f];
      /* 0 <= sum coef*idx + c0 <= den*(size-1)   (den > 0) */
      int64_t lo_rhs = -fm->c0, hi_rhs = fm->den * (fm->size - 1) - fm->c0;
      for (int v = 0; v < n->n_idx; v++) {
        if (fm->coef[v] == 0) continue;
        /* bound the rest of the sum */
        int64_t rest_lo = 0, rest_hi = 0;
        int finite = 1;
        for (int u = 0; u < n->n_idx && finite; u++) {
          if (u == v || fm->coef[u] == 0) continue;
          if (n->lo[u] <= -INF || n->hi[u] >= INF) {
            finite = 0;
            break;
          }
          int64_t a = fm->coef[u] * n->lo[u], b = fm->coef[u] * n->hi[u];
          rest_lo += a < b ? a : b;
          rest_hi += a < b ? b : a;
        }
        if (!finite) continue;
        /* coef*x in [lo_rhs - rest_hi, hi_rhs - rest_lo] */
        int64_t a = lo_rhs - rest_hi, b = hi_rhs - rest_lo;
        int64_t c = fm->coef[v];
        int64_t nlo, nhi;
        if (c > 0) {
          nlo = -floordiv(-a, c); /* ceil(a/c) */
          nhi = floordiv(b, c);
        } else {
          nlo = -floordiv(-b, c); /* ceil(b/c), c<0 */
          nhi = floordiv(a, c);
        }
        if (nlo > n->lo[v]) {
          n->lo[v] = nlo;
          changed = 1;
        }
        if (nhi < n->hi[v]) {
          n->hi[v] = nhi;
          changed = 1;
        }
      }
    }
    if (!changed) break;
  }
  for (int i = 0; i < n->n_idx; i++) {
    if (n->lo[i] <= -INF || n->hi[i] >= INF) return -1;
  }
  return 0;
}

/* Evaluate all forms at idx; fill flat offsets per operand.  Returns 1 if the
 * tuple is valid. */
static inline int eval_forms(const nest_t* n, const int64_t* idx, int64_t* off) {
  for (int o = 0; o < n->n_operands; o++) off[o] = 0;
  for (int f = 0; f < n->n_forms; f++) {
    const form_t* fm = &n->forms[f];
    int64_t s = fm->c0;
    for (int v = 0; v < n->n_idx; v++) s += fm->coef[v] * idx[v];
    int64_t q = s;
    if (fm->den != 1) {
      if (s % fm->den != 0) return 0;
      q = s / fm->den;
    }
    if (q < 0 || q >= fm->size) return 0;
    if (fm->operand >= 0) off[fm->operand] += q * fm->stride;
  }
  return 1;
}

#define DEFINE_RUN(NAME, T, UT, IS_FLOAT)                                                       \
  static int64_t NAME(const nest_t* n, int agg, int combo, T* out, const void* const* srcs,   \
                      int cmp_is_float) {                                                      \
    int64_t idx[MAX_IDX];                                                                      \
    int64_t off[MAX_ACC + 1];                                                                  \
    int64_t count = 0;                                                                         \
    for (int i = 0; i < n->n_idx; i++) {                                                       \
      if (n->lo[i] > n->hi[i]) return 0;                                                       \
      idx[i] = n->lo[i];                                                                       \
    }                                                                                          \
    for (;;) {                                                                                 \
      if (eval_forms(n, idx, off)) {                                                           \
        T v;                                                                                   \
        const T* s0 = (const T*)srcs[0];                                                       \
        switch (combo) {                                                                       \
          case COMBO_NONE:                                                                     \
            v = s0[off[1]];                                                                    \
            break;                                                                             \
          case COMBO_ADD:                                                                      \
            v = (T)((UT)s0[off[1]] + (UT)((const T*)srcs[1])[off[2]]);                         \
            break;                                                                             \
          case COMBO_MUL:                                                                      \
            v = (T)((UT)s0[off[1]] * (UT)((const T*)srcs[1])[off[2]]);                         \
            break;                                                                             \
          case COMBO_COND: {                                                                   \
            /* comparands arrive as f64 (float compare) or i64 (integer compare) */            \
            int eq;                                                                            \
            if (cmp_is_float)                                                                  \
              eq = ((const double*)srcs[0])[off[1]] == ((const double*)srcs[1])[off[2]];       \
            else                                                                               \
              eq = ((const int64_t*)srcs[0])[off[1]] == ((const int64_t*)srcs[1])[off[2]];     \
            v = eq ? ((const T*)srcs[2])[off[3]] : (T)0;                                       \
            break;                                                                             \
          }                                                                                    \
          default:                                                                             \
            return -1;                                                                         \
        }                                                                                      \
        T* o = out + off[0];                                                                   \
        switch (agg) {                                                                         \
          case AGG_ASSIGN:                                                                     \
            *o = v;                                                                            \
            break;                                                                             \
          case AGG_ADD:                                                                        \
            *o = (T)((UT)*o + (UT)v);                                                          \
            break;                                                                             \
          case AGG_MUL:                                                                        \
            *o = (T)((UT)*o * (UT)v);                                                          \
            break;                                                                             \
          case AGG_MAX:                                                                        \
            *o = (v > *o) ? v : *o;                                                            \
            break;                                                                             \
          case AGG_MIN:                                                                        \
            *o = (v < *o) ? v : *o;                                                            \
            break;                                                                             \
          default:                                                                             \
            return -1;                                                                         \
        }                                                                                      \
        count++;                                                                               \
      }                                                                                        \
      /* odometer, last index fastest */                                                       \
      int d = n->n_idx - 1;                                                                    \
      for (; d >= 0; d--) {                                                                    \
        if (++idx[d] <= n->hi[d]) break;                                                       \
        idx[d] = n->lo[d];                                                                     \
      }                                                                                        \
      if (d < 0) break;                                                                        \
    }                                                                                          \
    return count;                                                                              \
  }

/* For floating types UT == T so the "unsigned" casts are no-ops; for integers
 * arithmetic is done in the unsigned type of the same width so that overflow
 * wraps (two's complement), then converted back. */
DEFINE_RUN(run_f32, float, float, 1)
DEFINE_RUN(run_f64, double, double, 1)
DEFINE_RUN(run_i8, int8_t, uint8_t, 0)
DEFINE_RUN(run_i16, int16_t, uint16_t, 0)
DEFINE_RUN(run_i32, int32_t, uint32_t, 0)
DEFINE_RUN(run_i64, int64_t, uint64_t, 0)
DEFINE_RUN(run_u8, uint8_t, uint8_t, 0)
DEFINE_RUN(run_u16, uint16_t, uint16_t, 0)
DEFINE_RUN(run_u32, uint32_t, uint32_t, 0)
DEFINE_RUN(run_u64, uint64_t, uint64_t, 0)

/*
 * tile_oracle_contract
 *   dtype        compute/result element type (T_*)
 *   agg, combo   AGG_*, COMBO_*
 *   n_idx        number of index variables
 *   n_operands   1 + number of sources (operand 0 = output)
 *   ranks        [n_operands] rank of each access
 *   sizes        concatenated dimension sizes of every operand
 *   coefs        per access dimension, n_idx+2 int64: coef[0..n_idx), c0, den
 *   n_cons       explicit constraints; cons_coefs same layout, cons_rhs the
 *                exclusive upper bound
 *   out          output buffer, pre-initialised
 *   srcs         source buffers (for COMBO_COND srcs[0], srcs[1] are double or
 *                int64 per cmp_is_float, srcs[2] is T)
 *   box_lo/hi    optional outputs [n_idx]: the enumeration box that was used
 * Returns the number of valid index tuples, -1 on a malformed request,
 * -2 if an index is unbounded.
 */
int64_t tile_oracle_contract(int dtype, int agg, int combo, int n_idx, int n_operands,
                             const int64_t* ranks, const int64_t* sizes, const int64_t* coefs,
                             int n_cons, const int64_t* cons_coefs, const int64_t* cons_rhs,
                             void* out, const void* const* srcs, int cmp_is_float,
                             int64_t* box_lo, int64_t* box_hi) {
  nest_t n;
  memset(&n, 0, sizeof(n));
  if (n_idx > MAX_IDX || n_operands > MAX_ACC || n_cons > MAX_CONS) return -1;
  n.n_idx = n_idx;
  n.n_operands = n_operands;
  int f = 0;
  const int64_t* sz = sizes;
  const int64_t* cf = coefs;
  for (int o = 0; o < n_operands; o++) {
    int r = (int)ranks[o];
    if (r > MAX_RANK) return -1;
    /* row-major strides */
    int64_t stride[MAX_RANK];
    int64_t s = 1;
    for (int d = r - 1; d >= 0; d--) {
      stride[d] = s;
      s *= sz[d];
    }
    for (int d = 0; d < r; d++) {
      form_t* fm = &n.forms[f++];
      for (int v = 0; v < n_idx; v++) fm->coef[v] = cf[v];
      fm->c0 = cf[n_idx];
      fm->den = cf[n_idx + 1];
      if (fm->den <= 0) return -1;
      fm->size = sz[d];
      fm->stride = stride[d];
      fm->operand = o;
      cf += n_idx + 2;
    }
    sz += r;
  }
  cf = cons_coefs;
  for (int c = 0; c < n_cons; c++) {
    form_t* fm = &n.forms[f++];
    for (int v = 0; v < n_idx; v++) fm->coef[v] = cf[v];
    fm->c0 = cf[n_idx];
    fm->den = cf[n_idx + 1];
    if (fm->den <= 0) return -1;
    fm->size = cons_rhs[c];
    fm->stride = 0;
    fm->operand = -1;
    cf += n_idx + 2;
  }
  n.n_forms = f;
  if (propagate_bounds(&n) != 0) return -2;
  if (box_lo && box_hi) {
    for (int i = 0; i < n_idx; i++) {
      box_lo[i] = n.lo[i];
      box_hi[i] = n.hi[i];
    }
  }
  switch (dtype) {
    case T_F32: return run_f32(&n, agg, combo, (float*)out, srcs, cmp_is_float);
    case T_F64: return run_f64(&n, agg, combo, (double*)out, srcs, cmp_is_float);
    case T_I8: return run_i8(&n, agg, combo, (int8_t*)out, srcs, cmp_is_float);
    case T_I16: return run_i16(&n, agg, combo, (int16_t*)out, srcs, cmp_is_float);
    case T_I32: return run_i32(&n, agg, combo, (int32_t*)out, srcs, cmp_is_float);
    case T_I64: return run_i64(&n, agg, combo, (int64_t*)out, srcs, cmp_is_float);
    case T_U8: return run_u8(&n, agg, combo, (uint8_t*)out, srcs, cmp_is_float);
    case T_U16: return run_u16(&n, agg, combo, (uint16_t*)out, srcs, cmp_is_float);
    case T_U32: return run_u32(&n, agg, combo, (uint32_t*)out, srcs, cmp_is_float);
    case T_U64: return run_u64(&n, agg, combo, (uint64_t*)out, srcs, cmp_is_float);
  }
  return -1;
}
