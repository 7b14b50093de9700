#include "hip_planner.h"

namespace pmlc::target::hip {

// fills init_* of a dense kernel from op.init; false if the broadcast pattern is not expressible
bool Planner::denseInit(const Op& op, int32_t* kind, int32_t* dtype, int64_t* rs, int64_t* cs, int* buf) {
  *kind = 0;
  *buf = -1;
  if (!op.init) return true;
  if (op.init->kind == Value::Literal) return false;
  if (!rowColStrides(op.init->shape, op.result->shape, rs, cs)) return false;
  *kind = 1;
  *dtype = hipType(op.init->shape.elementType);
  *buf = bufferFor(op.init);
  return true;
}

bool Planner::denseTypes(const Op& op, ValuePtr* a, ValuePtr* b, int* in_dt, int* out_dt) {
  const DataType rdt = op.result->shape.elementType;
  *a = op.operands[0];
  *b = op.operands[1];
  const DataType adt = (*a)->shape.elementType, bdt = (*b)->shape.elementType;
  // the matrix-core kernels address an operand with 32-bit byte offsets: larger ones take the general kernel
  const size_t kOffsetLimit = size_t(1) << 31;
  if ((*a)->shape.getByteSize() >= kOffsetLimit || (*b)->shape.getByteSize() >= kOffsetLimit) return false;
  if (adt == bdt && adt == rdt && (rdt == DataType::f32 || rdt == DataType::bf16)) {
    *in_dt = hipType(rdt);
    *out_dt = hipType(rdt);
    return true;
  }
  // cast(A, INT32) (x) cast(B, INT32) with int8 sources: int8 MFMA with int32 accumulation
  if (rdt == DataType::si32 && adt == DataType::si32 && bdt == DataType::si32) {
    const Op* ca = castProducer(*a, DataType::si8);
    const Op* cb = castProducer(*b, DataType::si8);
    if (ca && cb) {
      *a = ca->operands[0];
      *b = cb->operands[0];
      *in_dt = PML_HIP_I8;
      *out_dt = PML_HIP_I32;
      return true;
    }
  }
  return false;
}

bool Planner::tryGemm(size_t i) {
  const Op& op = prog_->ops[i];
  if (op.agg != AggKind::add || op.combo != ComboKind::mul || op.operands.size() != 2) return false;
  ValuePtr A, B;
  int in_dt, out_dt;
  if (!denseTypes(op, &A, &B, &in_dt, &out_dt)) return false;
  Normalised n = normalise(op);
  for (const auto& c : n.cons)
    if (!impliedByBox(op, c.lhs, c.rhs)) return false;
  std::vector<int64_t> so, sa, sb;
  int64_t bo, ba, bb;
  if (!indexStrides(n.acc[0], op.result->shape, &so, &bo) || !indexStrides(n.acc[1], op.operands[0]->shape, &sa, &ba) ||
      !indexStrides(n.acc[2], op.operands[1]->shape, &sb, &bb))
    return false;
  // every access must stay in range over the whole box (no padding in a GEMM)
  for (size_t s = 0; s < 3; ++s) {
    const TensorShape& shape = s == 0 ? op.result->shape : op.operands[s - 1]->shape;
    for (size_t d = 0; d < n.acc[s].size(); ++d)
      if (!impliedByBox(op, n.acc[s][d], shape.sizes[d])) return false;
  }
  struct Idx { size_t v; int64_t range, so, sa, sb; };
  std::vector<Idx> M, N, K;
  for (size_t v = 0; v < n.nIdx; ++v) {
    if (!n.active[v]) continue;
    if (op.lower[v] != 0) return false;
    Idx x{v, op.upper[v] + 1, so[v], sa[v], sb[v]};
    const bool o = so[v] != 0, a = sa[v] != 0, b = sb[v] != 0;
    if (o && a && !b) M.push_back(x);
    else if (o && !a && b) N.push_back(x);
    else if (!o && a && b) K.push_back(x);
    else return false;
    if (so[v] < 0 || sa[v] < 0 || sb[v] < 0) return false;
  }
  if (K.empty()) return false;
  // a group collapses to one dimension if, ordered by stride, each stride equals the next stride x range
  auto collapse = [](std::vector<Idx>& g, int64_t Idx::*field, int64_t* ld) {
    std::sort(g.begin(), g.end(), [&](const Idx& x, const Idx& y) { return x.*field > y.*field; });
    for (size_t k = 0; k + 1 < g.size(); ++k)
      if (g[k].*field != g[k + 1].*field * g[k + 1].range) return false;
    *ld = g.empty() ? 0 : g.back().*field;
    return true;
  };
  auto sameOrder = [](const std::vector<Idx>& x, std::vector<Idx> y, int64_t Idx::*field) {
    std::sort(y.begin(), y.end(), [&](const Idx& p, const Idx& q) { return p.*field > q.*field; });
    for (size_t k = 0; k < x.size(); ++k)
      if (x[k].v != y[k].v) return false;
    return true;
  };
  int64_t ldc = 0, lda = 0, ncs = 0, kas = 0, ldb = 0, kbs = 0, nbs = 0;
  if (!collapse(M, &Idx::so, &ldc) || !sameOrder(M, M, &Idx::sa)) return false;
  {
    std::vector<Idx> t = M;
    if (!collapse(t, &Idx::sa, &lda)) return false;
    for (size_t k = 0; k < M.size(); ++k)
      if (t[k].v != M[k].v) return false;
  }
  {
    std::vector<Idx> t = N;
    if (!collapse(N, &Idx::so, &ncs) || !collapse(t, &Idx::sb, &nbs)) return false;
    for (size_t k = 0; k < N.size(); ++k)
      if (t[k].v != N[k].v) return false;
  }
  {
    std::vector<Idx> t = K;
    if (!collapse(K, &Idx::sa, &kas) || !collapse(t, &Idx::sb, &kbs)) return false;
    for (size_t k = 0; k < K.size(); ++k)
      if (t[k].v != K[k].v) return false;
  }
  int64_t m = 1, nn = 1, kk = 1;
  for (const Idx& x : M) m *= x.range;
  for (const Idx& x : N) nn *= x.range;
  for (const Idx& x : K) kk *= x.range;
  // the m x n block must be the whole result: elements the contraction never reaches hold the
  // aggregation identity (or the initial value), which only the general path writes
  if (bo != 0 || m * nn != op.result->shape.elements()) return false;
  if (N.empty()) { ncs = 1; nbs = 1; }   // matrix-vector: one column
  if (M.empty()) { ldc = nn; lda = kk; }  // vector-matrix: one row
  if (ncs != 1 || kas != 1) return false;
  bool b_is_nk;
  if (nbs == 1 || N.empty()) {
    b_is_nk = false;  // B[k][n]
    ldb = kbs;
    if (N.empty()) ldb = std::max<int64_t>(kbs, 1);
    if (ldb < nn) return false;
  } else if (kbs == 1) {
    b_is_nk = true;  // B[n][k]
    ldb = nbs;
    if (ldb < kk) return false;
  } else {
    return false;
  }
  if (ldc < nn || lda < kk) return false;
  const int es = in_dt == PML_HIP_F32 ? 4 : (in_dt == PML_HIP_BF16 ? 2 : 1);
  if ((kk * es) % 16 != 0 || (lda * es) % 16 != 0 || (ba * es) % 16 != 0) return false;
  if (b_is_nk && ((ldb * es) % 16 != 0 || (bb * es) % 16 != 0)) return false;

  Step s;
  s.kind = Step::Gemm;
  pml_hip_gemm_desc& d = s.gemm;
  d.in_dtype = in_dt;
  d.out_dtype = out_dt;
  d.m = m;
  d.n = nn;
  d.k = kk;
  d.lda = lda;
  d.ldb = ldb;
  d.ldc = ldc;
  d.b_layout = b_is_nk ? 1 : 0;
  if (opt_.fp32_as_bf16x3 && in_dt == PML_HIP_F32) d.flags = PML_HIP_FP32_AS_BF16X3;
  if (!denseInit(op, &d.init_kind, &d.init_dtype, &d.init_row_stride, &d.init_col_stride, &s.init)) return false;
  // the tail and the row/col operand addressing assume a dense rows x cols output
  TailBuild tb;
  tb.final_value = op.result;
  tb.final_dtype = op.result->shape.elementType;
  const bool dense_out = ldc == nn && bo == 0 && op.result->shape.getRank() >= 1 && op.result->shape.sizes.back() == nn;
  if (dense_out) extendTail(&tb, op.result, i, /*two_d=*/true, /*allow64=*/false);
  if (d.init_kind && !dense_out && !(d.init_row_stride == 0 && d.init_col_stride <= 1)) return unconsume(tb), false;
  d.tail = tb.tail;
  d.c_dtype = hipType(tb.final_dtype);
  if (tb.tail.n_ops && pml_hip_gemm_tail_cheaper_apart(&d)) {
    // the kernel library multiplies this shape faster under a plain tail: the chain stays with the
    // element-wise operations that follow (which fuse among themselves)
    unconsume(tb);
    tb = TailBuild();
    tb.final_value = op.result;
    tb.final_dtype = op.result->shape.elementType;
    d.tail = tb.tail;
    d.c_dtype = hipType(tb.final_dtype);
  }
  s.a = bufferFor(A);
  s.b = bufferFor(B);
  s.c = bufferFor(tb.final_value);
  s.a_off = ba;
  s.b_off = bb;
  s.c_off = bo;
  s.b_is_nk = b_is_nk;
  s.b_constant = B->kind == Value::Constant;
  attachTail(&s, tb);
  s.flops = 2.0 * m * nn * kk;
  s.bytes = static_cast<double>(m * kk + kk * nn) * es + static_cast<double>(m * nn) * util::byteSize(tb.final_dtype);
  std::stringstream ss;
  ss << "gemm " << util::mnemonic(static_cast<DataType>(in_dt)) << (d.flags & PML_HIP_FP32_AS_BF16X3 ? " (as 3 bf16 products)" : "")
     << " m=" << m << " n=" << nn << " k=" << kk << (b_is_nk ? " B=[n][k]" : " B=[k][n]") << (s.b_constant ? " (constant, packed once)" : "")
     << (d.init_kind ? " +init" : "") << tailText(tb) << " -> " << tb.final_value->shape.str();
  s.text = ss.str();
  plan_->steps.push_back(s);
  return true;
}

bool Planner::spatialForm(const Affine& a, const std::vector<bool>& in_out, const std::vector<bool>& active, Spatial* sp) {
  if (a.den != 1) return false;
  sp->pad = -a.c0;
  for (size_t v = 0; v < a.coef.size(); ++v) {
    if (!a.coef[v]) continue;
    if (!active[v]) return false;
    if (in_out[v]) {
      if (sp->out_idx >= 0) return false;
      sp->out_idx = static_cast<int>(v);
      sp->stride = a.coef[v];
    } else {
      if (sp->tap_idx >= 0) return false;
      sp->tap_idx = static_cast<int>(v);
      sp->dil = a.coef[v];
    }
  }
  return sp->stride > 0 && sp->dil > 0;
}

// The output access of a window kernel: every dimension is its own plain index over the whole extent; a
// dimension of size 1 (batch 1, a 1x1 plane) has had its index folded to the constant 0 and gets index -1.
bool Planner::windowOutput(const Op& op, const Normalised& n, const TensorShape& os, int oi[4], std::vector<bool>* in_out) {
  for (int k = 0; k < 4; ++k) {
    if (os.sizes[k] == 1 && n.acc[0][k].isConstant() && n.acc[0][k].c0 == 0) {
      oi[k] = -1;
      continue;
    }
    oi[k] = n.acc[0][k].plainIndex();
    if (oi[k] < 0 || (*in_out)[oi[k]] || op.lower[oi[k]] != 0 || op.upper[oi[k]] != os.sizes[k] - 1) return false;
    (*in_out)[oi[k]] = true;
  }
  return true;
}

// out[n,y,x,co] += I[n, sy*y + dy*ky - py, sx*x + dx*kx - px, ci] * F[ky,kx,ci,co]
bool Planner::tryConv(size_t i) {
  const Op& op = prog_->ops[i];
  if (op.agg != AggKind::add || op.combo != ComboKind::mul || op.operands.size() != 2) return false;
  ValuePtr I, F;
  int in_dt, out_dt;
  if (!denseTypes(op, &I, &F, &in_dt, &out_dt)) return false;
  const TensorShape &os = op.result->shape, &is = op.operands[0]->shape, &fs = op.operands[1]->shape;
  if (os.getRank() != 4 || is.getRank() != 4 || fs.getRank() != 4) return false;
  Normalised n = normalise(op);
  for (const auto& c : n.cons)
    if (!impliedByBox(op, c.lhs, c.rhs)) return false;
  // output: four distinct plain indices covering the whole output
  int oi[4];
  std::vector<bool> in_out(n.nIdx, false);
  for (int d = 0; d < 4; ++d) {
    if (os.sizes[d] == 1 && n.acc[0][d].isConstant() && n.acc[0][d].c0 == 0) {
      oi[d] = -1;
      continue;
    }
    oi[d] = n.acc[0][d].plainIndex();
    if (oi[d] < 0 || in_out[oi[d]]) return false;
    if (op.lower[oi[d]] != 0 || op.upper[oi[d]] != os.sizes[d] - 1) return false;
    in_out[oi[d]] = true;
  }
  // input batch and channel
  auto plainOrZero = [&](const Affine& a, int64_t size, int* idx) {
    if (size == 1 && a.isConstant() && a.c0 == 0) {
      *idx = -1;
      return true;
    }
    *idx = a.plainIndex();
    return *idx >= 0;
  };
  int in_n, in_c, f_ci, f_co, f_ky, f_kx;
  if (!plainOrZero(n.acc[1][0], is.sizes[0], &in_n) || in_n != oi[0]) return false;
  if (!plainOrZero(n.acc[1][3], is.sizes[3], &in_c)) return false;
  if (!plainOrZero(n.acc[2][0], fs.sizes[0], &f_ky) || !plainOrZero(n.acc[2][1], fs.sizes[1], &f_kx)) return false;
  if (!plainOrZero(n.acc[2][2], fs.sizes[2], &f_ci) || !plainOrZero(n.acc[2][3], fs.sizes[3], &f_co)) return false;
  if (f_ci != in_c || f_co != oi[3]) return false;
  if (in_c >= 0 && (in_out[in_c] || op.lower[in_c] != 0 || op.upper[in_c] != is.sizes[3] - 1)) return false;
  if (is.sizes[3] != fs.sizes[2] || fs.sizes[3] != os.sizes[3]) return false;
  Spatial sy, sx;
  if (!spatialForm(n.acc[1][1], in_out, n.active, &sy) || !spatialForm(n.acc[1][2], in_out, n.active, &sx)) return false;
  if (sy.out_idx != oi[1] || sx.out_idx != oi[2] || sy.tap_idx != f_ky || sx.tap_idx != f_kx) return false;
  if (f_ky >= 0 && (op.lower[f_ky] != 0 || op.upper[f_ky] != fs.sizes[0] - 1)) return false;
  if (f_kx >= 0 && (op.lower[f_kx] != 0 || op.upper[f_kx] != fs.sizes[1] - 1)) return false;
  // every active index must have been given a role
  std::set<int> roles = {oi[0], oi[1], oi[2], oi[3], in_c, f_ky, f_kx};
  for (size_t v = 0; v < n.nIdx; ++v)
    if (n.active[v] && !roles.count(static_cast<int>(v))) return false;
  const int es = in_dt == PML_HIP_F32 ? 4 : (in_dt == PML_HIP_BF16 ? 2 : 1);
  // (channel counts that do not fill 16-byte vectors are handled inside the kernel library: patch matrix + GEMM)

  Step s;
  s.kind = Step::Conv2d;
  pml_hip_conv2d_desc& d = s.conv;
  d.in_dtype = in_dt;
  d.out_dtype = out_dt;
  d.n = is.sizes[0];
  d.h = is.sizes[1];
  d.w = is.sizes[2];
  d.ci = is.sizes[3];
  d.kh = fs.sizes[0];
  d.kw = fs.sizes[1];
  d.co = fs.sizes[3];
  d.oh = os.sizes[1];
  d.ow = os.sizes[2];
  d.stride_h = sy.stride;
  d.stride_w = sx.stride;
  d.dil_h = sy.dil;
  d.dil_w = sx.dil;
  d.pad_h = sy.pad;
  d.pad_w = sx.pad;
  if (opt_.fp32_as_bf16x3 && in_dt == PML_HIP_F32) d.flags = PML_HIP_FP32_AS_BF16X3;
  if (os.sizes[0] != d.n) return false;
  if (!denseInit(op, &d.init_kind, &d.init_dtype, &d.init_row_stride, &d.init_col_stride, &s.init)) return false;
  TailBuild tb;
  extendTail(&tb, op.result, i, /*two_d=*/true, /*allow64=*/false);
  d.tail = tb.tail;
  d.c_dtype = hipType(tb.final_dtype);
  s.a = bufferFor(I);
  s.b = bufferFor(F);
  s.c = bufferFor(tb.final_value);
  s.b_constant = F->kind == Value::Constant;
  attachTail(&s, tb);
  // algorithmic FLOPs: 2 x valid (output, tap) pairs
  auto valid = [](int64_t out, int64_t in, int64_t k, int64_t st, int64_t dl, int64_t pad) {
    int64_t cnt = 0;
    for (int64_t o = 0; o < out; ++o)
      for (int64_t t = 0; t < k; ++t) {
        const int64_t x = o * st + t * dl - pad;
        if (x >= 0 && x < in) ++cnt;
      }
    return cnt;
  };
  s.flops = 2.0 * d.n * valid(d.oh, d.h, d.kh, d.stride_h, d.dil_h, d.pad_h) * valid(d.ow, d.w, d.kw, d.stride_w, d.dil_w, d.pad_w) *
            d.ci * d.co;
  s.bytes = static_cast<double>(is.elements() + fs.elements()) * es + static_cast<double>(os.elements()) * util::byteSize(tb.final_dtype);
  std::stringstream ss;
  ss << "conv2d " << util::mnemonic(static_cast<DataType>(in_dt)) << (d.flags & PML_HIP_FP32_AS_BF16X3 ? " (as 3 bf16 products) " : " ") << is.str() << " (*) " << fs.str() << " stride=" << d.stride_h
     << "x" << d.stride_w << " pad=" << d.pad_h << "," << d.pad_w << (s.b_constant ? " (constant filter, packed once)" : "")
     << (d.init_kind ? " +init" : "") << tailText(tb) << " -> " << tb.final_value->shape.str();
  s.text = ss.str();
  plan_->steps.push_back(s);
  return true;
}

// out[n,y,x,c] += I[n, sy*y + dy*ky - py, sx*x + dx*kx - px, c] * F[ky,kx,c,0]
bool Planner::tryDepthwise(size_t i) {
  const Op& op = prog_->ops[i];
  if (op.agg != AggKind::add || op.combo != ComboKind::mul || op.operands.size() != 2 || op.init) return false;
  const DataType dt = op.result->shape.elementType;
  if (dt != DataType::f32 && dt != DataType::bf16) return false;
  if (op.operands[0]->shape.elementType != dt || op.operands[1]->shape.elementType != dt) return false;
  const TensorShape &os = op.result->shape, &is = op.operands[0]->shape, &fs = op.operands[1]->shape;
  if (os.getRank() != 4 || is.getRank() != 4 || fs.getRank() != 4 || fs.sizes[3] != 1) return false;
  Normalised n = normalise(op);
  for (const auto& c : n.cons)
    if (!impliedByBox(op, c.lhs, c.rhs)) return false;
  int oi[4];
  std::vector<bool> in_out(n.nIdx, false);
  if (!windowOutput(op, n, os, oi, &in_out)) return false;
  if (!sameIndex(n.acc[1][0], oi[0]) || !sameIndex(n.acc[1][3], oi[3]) || !sameIndex(n.acc[2][2], oi[3])) return false;
  if (!(n.acc[2][3].isConstant() && n.acc[2][3].c0 == 0)) return false;
  if (is.sizes[3] != os.sizes[3] || fs.sizes[2] != os.sizes[3] || is.sizes[0] != os.sizes[0]) return false;
  Spatial sy, sx;
  if (!spatialForm(n.acc[1][1], in_out, n.active, &sy) || !spatialForm(n.acc[1][2], in_out, n.active, &sx)) return false;
  auto tapOk = [&](const Affine& a, int64_t size, int tap) {
    if (size == 1 && a.isConstant() && a.c0 == 0) return tap < 0;
    return a.plainIndex() == tap && tap >= 0 && op.lower[tap] == 0 && op.upper[tap] == size - 1;
  };
  if (sy.out_idx != oi[1] || sx.out_idx != oi[2] || !tapOk(n.acc[2][0], fs.sizes[0], sy.tap_idx) ||
      !tapOk(n.acc[2][1], fs.sizes[1], sx.tap_idx))
    return false;
  std::set<int> roles = {oi[0], oi[1], oi[2], oi[3], sy.tap_idx, sx.tap_idx};
  for (size_t v = 0; v < n.nIdx; ++v)
    if (n.active[v] && !roles.count(static_cast<int>(v))) return false;
  const int V = 16 / static_cast<int>(util::byteSize(dt));
  if (os.sizes[3] % V != 0) return false;
  Step s;
  s.kind = Step::Dwconv2d;
  pml_hip_dwconv2d_desc& d = s.dw;
  d.dtype = hipType(dt);
  d.n = is.sizes[0];
  d.h = is.sizes[1];
  d.w = is.sizes[2];
  d.c = is.sizes[3];
  d.kh = fs.sizes[0];
  d.kw = fs.sizes[1];
  d.oh = os.sizes[1];
  d.ow = os.sizes[2];
  d.stride_h = sy.stride;
  d.stride_w = sx.stride;
  d.dil_h = sy.dil;
  d.dil_w = sx.dil;
  d.pad_h = sy.pad;
  d.pad_w = sx.pad;
  TailBuild tb;
  extendTail(&tb, op.result, i, /*two_d=*/true, /*allow64=*/false);
  if (tb.final_dtype != dt) return unconsume(tb);  // this kernel stores its own element type
  d.tail = tb.tail;
  s.a = bufferFor(op.operands[0]);
  s.b = bufferFor(op.operands[1]);
  s.c = bufferFor(tb.final_value);
  s.b_constant = op.operands[1]->kind == Value::Constant;
  attachTail(&s, tb);
  s.flops = 2.0 * os.elements() * d.kh * d.kw;
  s.bytes = static_cast<double>(is.elements() + os.elements() + fs.elements()) * util::byteSize(dt);
  s.text = "dwconv2d " + std::string(util::mnemonic(dt)) + " " + is.str() + " k=" + std::to_string(d.kh) + "x" + std::to_string(d.kw) +
           " stride=" + std::to_string(d.stride_h) + (s.b_constant ? " (constant filter, packed once)" : "") + tailText(tb) + " -> " +
           tb.final_value->shape.str();
  plan_->steps.push_back(s);
  return true;
}

// out[n,y,x,c] = agg I[n, sy*y + ky - py, sx*x + kx - px, c],  ky < KH, kx < KW
bool Planner::poolGeometry(const Op& op, const Normalised& n, pml_hip_pool2d_desc* d, Spatial* sy, Spatial* sx) {
  const TensorShape &os = op.result->shape, &is = op.operands[0]->shape;
  if (os.getRank() != 4 || is.getRank() != 4) return false;
  int oi[4];
  std::vector<bool> in_out(n.nIdx, false);
  if (!windowOutput(op, n, os, oi, &in_out)) return false;
  if (!sameIndex(n.acc[1][0], oi[0]) || !sameIndex(n.acc[1][3], oi[3])) return false;
  if (is.sizes[0] != os.sizes[0] || is.sizes[3] != os.sizes[3]) return false;
  if (!spatialForm(n.acc[1][1], in_out, n.active, sy) || !spatialForm(n.acc[1][2], in_out, n.active, sx)) return false;
  if (sy->out_idx != oi[1] || sx->out_idx != oi[2] || sy->dil != 1 || sx->dil != 1) return false;
  // window extents come from the explicit constraints k < K; a tap index without one is not a pooling window
  int64_t kh = 1, kw = 1;
  bool have_h = sy->tap_idx < 0, have_w = sx->tap_idx < 0;
  for (const auto& c : op.constraints) {
    const int p = c.lhs.plainIndex();
    if (p < 0) return false;
    if (p == sy->tap_idx) {
      kh = c.rhs;
      have_h = true;
    } else if (p == sx->tap_idx) {
      kw = c.rhs;
      have_w = true;
    } else if (!impliedByBox(op, c.lhs, c.rhs)) {
      return false;
    }
  }
  if (!have_h || !have_w) return false;
  d->n = is.sizes[0];
  d->h = is.sizes[1];
  d->w = is.sizes[2];
  d->c = is.sizes[3];
  d->kh = kh;
  d->kw = kw;
  d->oh = os.sizes[1];
  d->ow = os.sizes[2];
  d->stride_h = sy->stride;
  d->stride_w = sx->stride;
  d->pad_h = sy->pad;
  d->pad_w = sx->pad;
  return true;
}

// out[n,c] (or out[n,0,0,c]) = agg over all (y,x) of I[n,y,x,c]: a pooling window that is the whole image
bool Planner::tryGlobalPool(size_t i) {
  const Op& op = prog_->ops[i];
  if (op.combo != ComboKind::none || op.operands.size() != 1 || op.init) return false;
  if (op.agg != AggKind::max && op.agg != AggKind::min && op.agg != AggKind::add) return false;
  const DataType dt = op.result->shape.elementType;
  if ((dt != DataType::f32 && dt != DataType::bf16) || op.operands[0]->shape.elementType != dt) return false;
  const TensorShape &os = op.result->shape, &is = op.operands[0]->shape;
  if (is.getRank() != 4) return false;
  const bool keep = os.getRank() == 4;
  if (!keep && os.getRank() != 2) return false;
  if (keep && (os.sizes[1] != 1 || os.sizes[2] != 1)) return false;
  if (os.sizes.front() != is.sizes[0] || os.sizes.back() != is.sizes[3]) return false;
  Normalised n = normalise(op);
  for (const auto& c : n.cons)
    if (!impliedByBox(op, c.lhs, c.rhs)) return false;
  const bool one_image = is.sizes[0] == 1;  // the batch index of a single image is folded to the constant 0
  const int on = one_image ? -1 : n.acc[0].front().plainIndex(), oc = n.acc[0].back().plainIndex();
  if ((!one_image && on < 0) || oc < 0 || on == oc) return false;
  if (one_image && !sameIndex(n.acc[0].front(), -1)) return false;
  if (keep && !(n.acc[0][1].isConstant() && n.acc[0][1].c0 == 0 && n.acc[0][2].isConstant() && n.acc[0][2].c0 == 0)) return false;
  const int iy = n.acc[1][1].plainIndex(), ix = n.acc[1][2].plainIndex();
  if (!sameIndex(n.acc[1][0], on) || n.acc[1][3].plainIndex() != oc || iy < 0 || ix < 0 || iy == ix || iy == on ||
      iy == oc || ix == on || ix == oc)
    return false;
  const int idx[4] = {on, iy, ix, oc};
  for (int k = 0; k < 4; ++k)
    if (idx[k] >= 0 && (op.lower[idx[k]] != 0 || op.upper[idx[k]] != is.sizes[k] - 1)) return false;
  for (size_t v = 0; v < n.nIdx; ++v)
    if (n.active[v] && static_cast<int>(v) != on && static_cast<int>(v) != oc && static_cast<int>(v) != iy &&
        static_cast<int>(v) != ix)
      return false;
  const int V = 16 / static_cast<int>(util::byteSize(dt));
  if (is.sizes[3] % V != 0) return false;
  Step s;
  s.kind = Step::Pool2d;
  pml_hip_pool2d_desc& d = s.pool;
  d.dtype = hipType(dt);
  d.agg = hipAgg(op.agg);
  d.n = is.sizes[0];
  d.h = is.sizes[1];
  d.w = is.sizes[2];
  d.c = is.sizes[3];
  d.kh = d.h;
  d.kw = d.w;
  d.oh = d.ow = 1;
  d.stride_h = d.stride_w = 1;
  d.pad_h = d.pad_w = 0;
  s.a = bufferFor(op.operands[0]);
  // A mean is written as sum / count: the division by a literal, when it is all that follows and the kernel that
  // sums whole images will run (at least 16 pixels), rides in the same launch.
  ValuePtr result = op.result;
  std::string divided;
  if (op.agg == AggKind::add && d.h * d.w >= 16) {
    TailBuild tb;
    extendTail(&tb, op.result, i, /*two_d=*/true, /*allow64=*/false);
    const bool one_division = tb.tail.n_ops == 1 && tb.tail.ops[0].opcode == PML_HIP_EPI_DIV &&
                              tb.tail.ops[0].operand_kind == PML_HIP_OPND_IMM && tb.tail.ops[0].dtype == hipType(dt) &&
                              tb.final_dtype == dt && tb.outs.empty() && tb.tail.ops[0].imm != 0 &&
                              static_cast<double>(static_cast<float>(tb.tail.ops[0].imm)) == tb.tail.ops[0].imm;
    if (one_division) {
      d.divisor = static_cast<float>(tb.tail.ops[0].imm);
      result = tb.final_value;
      divided = tailText(tb);
    } else {
      unconsume(tb);
    }
  }
  s.c = bufferFor(result);
  s.bytes = static_cast<double>(is.elements() + os.elements()) * util::byteSize(dt);
  s.text = "pool2d " + tile::toString(op.agg) + " " + std::string(util::mnemonic(dt)) + " " + is.str() +
           " over the whole image" + divided + " -> " + os.str();
  plan_->steps.push_back(s);
  return true;
}

bool Planner::tryPool(size_t i) {
  const Op& op = prog_->ops[i];
  if (op.combo != ComboKind::none || op.operands.size() != 1 || op.init) return false;
  if (op.agg != AggKind::max && op.agg != AggKind::min && op.agg != AggKind::add) return false;
  const DataType dt = op.result->shape.elementType;
  if ((dt != DataType::f32 && dt != DataType::bf16) || op.operands[0]->shape.elementType != dt) return false;
  Normalised n = normalise(op);
  Step s;
  s.kind = Step::Pool2d;
  Spatial sy, sx;
  if (!poolGeometry(op, n, &s.pool, &sy, &sx)) return false;
  const int V = 16 / static_cast<int>(util::byteSize(dt));
  if (s.pool.c % V != 0) return false;
  s.pool.dtype = hipType(dt);
  s.pool.agg = hipAgg(op.agg);
  s.a = bufferFor(op.operands[0]);
  s.c = bufferFor(op.result);
  // window argmax: AM = max(cond(R[window], M[out], IX[ky,kx])) with IX = ky*KW + kx, same geometry
  if (op.agg == AggKind::max) {
    auto uit = users_.find(op.result.get());
    if (uit != users_.end()) {
      for (size_t ui : uit->second) {
        if (consumed_.count(ui)) continue;
        if (matchWindowArgmax(ui, op, s.pool)) {
          s.pool.with_index = 1;
          s.out2 = bufferFor(prog_->ops[ui].result);
          consumed_.insert(ui);
          break;
        }
      }
    }
  }
  const TensorShape& is = op.operands[0]->shape;
  s.bytes = static_cast<double>(is.elements() + op.result->shape.elements()) * util::byteSize(dt) +
            (s.pool.with_index ? 4.0 * op.result->shape.elements() : 0.0);
  s.text = "pool2d " + tile::toString(op.agg) + " " + std::string(util::mnemonic(dt)) + " " + is.str() + " k=" +
           std::to_string(s.pool.kh) + "x" + std::to_string(s.pool.kw) + " stride=" + std::to_string(s.pool.stride_h) +
           (s.pool.with_index ? " +window argmax" : "") + " -> " + op.result->shape.str();
  plan_->steps.push_back(s);
  return true;
}

// IX is (index(dims,0) * KW + index(dims,1)) over dims [KH, KW]
bool Planner::isWindowIota(const ValuePtr& ix, int64_t kh, int64_t kw) {
  if (ix->shape.sizes != std::vector<int64_t>{kh, kw} || ix->shape.elementType != DataType::si32) return false;
  auto prod = [&](const ValuePtr& v) -> const Op* {
    auto it = producer_.find(v.get());
    return it == producer_.end() ? nullptr : &prog_->ops[it->second];
  };
  const Op* add = prod(ix);
  if (!add || add->kind != Op::Eltwise || add->fn != "add" || add->operands.size() != 2) return false;
  for (int side = 0; side < 2; ++side) {
    const Op* mul = prod(add->operands[side]);
    const Op* i1 = prod(add->operands[1 - side]);
    if (!mul || !i1 || i1->kind != Op::Index || i1->axis != 1) continue;
    if (mul->kind != Op::Eltwise || mul->fn != "mul" || mul->operands.size() != 2) continue;
    for (int ms = 0; ms < 2; ++ms) {
      const Op* i0 = prod(mul->operands[ms]);
      const ValuePtr& lit = mul->operands[1 - ms];
      if (i0 && i0->kind == Op::Index && i0->axis == 0 && lit->kind == Value::Literal && !util::isFloat(lit->shape.elementType) &&
          static_cast<int64_t>(lit->literalAsDouble()) == kw)
        return true;
    }
  }
  return false;
}

bool Planner::matchWindowArgmax(size_t ui, const Op& pool, const pml_hip_pool2d_desc& pd) {
  Op& u = prog_->ops[ui];
  if (u.kind != Op::Contraction || u.agg != AggKind::max || u.combo != ComboKind::cond || u.operands.size() != 3 || u.init) return false;
  if (u.operands[0] != pool.operands[0] || u.operands[1] != pool.result) return false;
  if (u.result->shape.elementType != DataType::si32 || u.result->shape.sizes != pool.result->shape.sizes) return false;
  if (!u.boundsComputed) tile::computeBounds(&u);
  if (emptyBox(u)) return false;
  Normalised n = normalise(u);
  // geometry of the R access must equal the pool's; M access must be the plain output access
  pml_hip_pool2d_desc d{};
  Spatial sy, sx;
  Op probe = u;  // poolGeometry reads operands[0] and explicit constraints only
  // the window extents of this contraction come from IX's shape instead of explicit constraints
  if (n.acc[3].size() != 2) return false;
  const int ky = n.acc[3][0].plainIndex(), kx = n.acc[3][1].plainIndex();
  {
    // re-use the spatial matcher by hand
    std::vector<bool> in_out(n.nIdx, false);
    int oi[4];
    if (!windowOutput(u, n, u.result->shape, oi, &in_out)) return false;
    for (int k = 0; k < 4; ++k)
      if (!sameIndex(n.acc[2][k], oi[k])) return false;
    if (!sameIndex(n.acc[1][0], oi[0]) || !sameIndex(n.acc[1][3], oi[3])) return false;
    if (!spatialForm(n.acc[1][1], in_out, n.active, &sy) || !spatialForm(n.acc[1][2], in_out, n.active, &sx)) return false;
    if (sy.out_idx != oi[1] || sx.out_idx != oi[2] || sy.dil != 1 || sx.dil != 1) return false;
    if (sy.tap_idx != ky || sx.tap_idx != kx) return false;
  }
  (void)probe;
  (void)d;
  if (sy.stride != pd.stride_h || sx.stride != pd.stride_w || sy.pad != pd.pad_h || sx.pad != pd.pad_w) return false;
  if (!u.constraints.empty()) return false;
  return isWindowIota(u.operands[2], pd.kh, pd.kw);
}

// agg over the last axis of one dense operand, nothing else: O[x0, .., 0] = agg_{x_last} I[x0, .., x_last]
bool Planner::reducesLastAxis(const Op& op, AggKind agg) {
  if (op.kind != Op::Contraction || op.agg != agg || op.combo != ComboKind::none || op.operands.size() != 1 || op.init) return false;
  if (!op.constraints.empty() || op.accesses.size() != 2) return false;
  const TensorShape &is = op.operands[0]->shape, &os = op.result->shape;
  const size_t r = is.getRank();
  if (r < 1 || os.getRank() != r || op.idxNames.size() != r || op.accesses[0].size() != r || op.accesses[1].size() != r) return false;
  if (os.elementType != is.elementType || os.sizes[r - 1] != 1) return false;
  std::vector<bool> seen(r, false);
  for (size_t d = 0; d < r; ++d) {
    const int v = op.accesses[1][d].plainIndex();
    if (v < 0 || seen[v]) return false;
    seen[v] = true;
    if (op.lower[v] != 0 || op.upper[v] != is.sizes[d] - 1) return false;  // the whole tensor
    if (d + 1 < r) {
      if (os.sizes[d] != is.sizes[d] || op.accesses[0][d].plainIndex() != v) return false;
    } else if (!(op.accesses[0][d].isConstant() && op.accesses[0][d].c0 == 0)) {
      return false;
    }
  }
  return true;
}

// The op library's softmax (plaidml/op/lib/ops.cc:3049-3098) -- M = max over the last axis, E = exp(X - M), S = sum of
// E over the last axis, E / S -- with every intermediate value used by nothing else: one launch of the softmax kernel
// in place of two reductions and two elementwise launches.  `i` is the max contraction.
bool Planner::trySoftmax(size_t i) {
  Op& mx = prog_->ops[i];
  if (!reducesLastAxis(mx, AggKind::max)) return false;
  const ValuePtr X = mx.operands[0];
  const DataType dt = X->shape.elementType;
  if (dt != DataType::f32 && dt != DataType::bf16) return false;
  // the only user of a value that is no program output, or npos
  auto only_user = [&](const ValuePtr& v) -> size_t {
    if (outputs_.count(v.get())) return std::string::npos;
    const auto it = users_.find(v.get());
    if (it == users_.end() || it->second.empty()) return std::string::npos;
    for (size_t u : it->second)
      if (u != it->second.front() || consumed_.count(u)) return std::string::npos;
    return it->second.front();
  };
  auto same_shape = [&](const ValuePtr& v) { return v->shape.sizes == X->shape.sizes && v->shape.elementType == dt; };
  const size_t si = only_user(mx.result);
  if (si == std::string::npos) return false;
  const Op& sub = prog_->ops[si];
  if (sub.kind != Op::Eltwise || sub.fn != "sub" || sub.operands.size() != 2 || sub.operands[0] != X || sub.operands[1] != mx.result ||
      !same_shape(sub.result))
    return false;
  const size_t ei = only_user(sub.result);
  if (ei == std::string::npos) return false;
  const Op& ex = prog_->ops[ei];
  if (ex.kind != Op::Eltwise || ex.fn != "exp" || ex.operands.size() != 1 || !same_shape(ex.result)) return false;
  const ValuePtr E = ex.result;
  if (outputs_.count(E.get())) return false;
  const auto eu = users_.find(E.get());
  if (eu == users_.end()) return false;
  std::set<size_t> e_users(eu->second.begin(), eu->second.end());
  if (e_users.size() != 2) return false;
  size_t sum_i = std::string::npos, div_i = std::string::npos;
  for (size_t u : e_users) {
    if (consumed_.count(u)) return false;
    if (prog_->ops[u].kind == Op::Contraction)
      sum_i = u;
    else
      div_i = u;
  }
  if (sum_i == std::string::npos || div_i == std::string::npos) return false;
  Op& sm = prog_->ops[sum_i];
  if (!sm.boundsComputed) tile::computeBounds(&sm);
  if (!reducesLastAxis(sm, AggKind::add) || sm.operands[0] != E) return false;
  const Op& dv = prog_->ops[div_i];
  if (dv.kind != Op::Eltwise || dv.fn != "div" || dv.operands.size() != 2 || dv.operands[0] != E || dv.operands[1] != sm.result ||
      !same_shape(dv.result))
    return false;
  if (only_user(sm.result) != div_i) return false;
  const size_t r = X->shape.getRank();
  Step s;
  s.kind = Step::Softmax;
  s.sm.dtype = hipType(dt);
  s.sm.cols = X->shape.sizes[r - 1];
  s.sm.rows = X->shape.sizes[r - 1] ? static_cast<int64_t>(X->shape.elements()) / X->shape.sizes[r - 1] : 0;
  s.a = bufferFor(X);
  s.c = bufferFor(dv.result);
  for (size_t k : {si, ei, sum_i, div_i}) consumed_.insert(k);
  s.bytes = 2.0 * static_cast<double>(X->shape.elements()) * util::byteSize(dt);
  s.text = "softmax " + std::string(util::mnemonic(dt)) + " over the last axis of " + X->shape.str() + " -> " + dv.result->shape.str();
  plan_->steps.push_back(s);
  return true;
}

}  // namespace pmlc::target::hip
