#include "hip_planner.h"

namespace pmlc::target::hip {

std::shared_ptr<Plan> Planner::run() {
  rewriteSelectMinMax();
  tile::eliminateDeadOps(prog_);
  analyse();
  for (size_t i = 0; i < prog_->inputs.size(); ++i) {
    BufferInfo b;
    b.kind = BufferInfo::Input;
    b.index = static_cast<int>(i);
    b.bytes = prog_->inputs[i]->shape.getByteSize();
    b.name = prog_->inputs[i]->name;
    plan_->buffers.push_back(b);
    bufferOf_[prog_->inputs[i].get()] = static_cast<int>(plan_->buffers.size()) - 1;
    plan_->input_buffers.push_back(static_cast<int>(plan_->buffers.size()) - 1);
  }
  // outputs: the first occurrence of a Temp value owns an Output buffer; anything else is copied
  plan_->output_buffers.assign(prog_->outputs.size(), -1);
  std::vector<std::pair<size_t, ValuePtr>> copies;
  for (size_t i = 0; i < prog_->outputs.size(); ++i) {
    const ValuePtr& v = prog_->outputs[i];
    BufferInfo b;
    b.kind = BufferInfo::Output;
    b.index = static_cast<int>(i);
    b.bytes = v->shape.getByteSize();
    b.name = v->name;
    plan_->buffers.push_back(b);
    const int id = static_cast<int>(plan_->buffers.size()) - 1;
    plan_->output_buffers[i] = id;
    if (v->kind == Value::Temp && !bufferOf_.count(v.get()))
      bufferOf_[v.get()] = id;
    else
      copies.emplace_back(i, v);
  }
  for (size_t i = 0; i < prog_->ops.size(); ++i) {
    if (consumed_.count(i)) continue;
    emit(i);
  }
  for (const auto& c : copies) {
    Step s;
    s.kind = Step::Copy;
    s.a = bufferFor(c.second);
    s.c = plan_->output_buffers[c.first];
    s.copy_bytes = c.second->shape.getByteSize();
    s.text = "copy -> output #" + std::to_string(c.first);
    plan_->steps.push_back(s);
  }
  if (opt_.fuse && opt_.specialise) fuseSecondProducts();
  if (opt_.specialise) padDepthwiseResults();
  if (opt_.fuse && opt_.specialise) fusePoolIntoConv();
  pruneDeadSteps();
  applySchedule();
  return plan_;
}

// Tiling overrides, per program (target options) and per step (schedule file): they travel to the kernel library in
// the descriptors' schedule bits.  Runs last, so that a step is keyed by the text the plan dump shows for it.
int Planner::convPathByName(const std::string& name) {
  static const char* const names[] = {"auto", "igemm", "patches", "ldsfilter", "blocks"};
  for (int i = 0; i < 5; ++i)
    if (name == names[i]) return i;
  throw std::runtime_error("Invalid convolution path '" + name + "' (igemm, patches, ldsfilter or blocks)");
}

int Planner::tileByName(const std::string& name) {
  const int t = pml_hip_tile_by_name(name.c_str());
  if (t < 0) throw std::runtime_error("Invalid tile '" + name + "' (64x64, 128x64, 128x128, 128x64w8, 128x128w8, 128x128w8s2, 256x128w16, 64x64w8k2, 256x256w8, 128x64n2, 192x384w8, 64x64ks)");
  return t;
}

Planner::Rule Planner::parseRule(const std::string& text) {  // "tile=...,conv=..."
  Rule r;
  std::stringstream ss(text);
  for (std::string item; std::getline(ss, item, ',');) {
    const auto eq = item.find('=');
    const std::string key = item.substr(0, eq), value = eq == std::string::npos ? "" : item.substr(eq + 1);
    if (key == "tile")
      r.tile = tileByName(value);
    else if (key == "conv")
      r.conv = convPathByName(value);
    else
      throw std::runtime_error("Invalid schedule entry '" + item + "' (tile=... or conv=...)");
  }
  return r;
}

void Planner::applySchedule() {
  Rule all;
  if (!opt_.tile.empty()) all.tile = tileByName(opt_.tile);
  if (!opt_.conv.empty()) all.conv = convPathByName(opt_.conv);
  std::map<std::string, Rule> rules;
  if (!opt_.schedule_path.empty()) {
    std::ifstream f(opt_.schedule_path);
    if (!f) throw std::runtime_error("Cannot read the schedule file " + opt_.schedule_path);
    for (std::string line; std::getline(f, line);) {
      const auto open = line.rfind(" {"), lead = line.find("] ");
      if (line.empty() || line.back() != '}' || open == std::string::npos || lead == std::string::npos || lead > open) continue;
      rules[line.substr(lead + 2, open - lead - 2)] = parseRule(line.substr(open + 2, line.size() - open - 3));
    }
  }
  for (Step& s : plan_->steps) {
    if (s.kind != Step::Gemm && s.kind != Step::Conv2d) continue;
    Rule r = all;
    const auto it = rules.find(s.text);
    if (it != rules.end()) {
      if (it->second.tile >= 0) r.tile = it->second.tile;
      if (it->second.conv > 0) r.conv = it->second.conv;
    }
    if (s.kind == Step::Gemm) r.conv = 0;
    int32_t& flags = s.kind == Step::Gemm ? s.gemm.flags : s.conv.flags;
    if (r.conv > 0 && s.kind == Step::Conv2d && PML_HIP_FLAG_MAXPOOL_OF(flags)) {
      // (a convolution that pools its result inside the launch keeps the path that can)
      pml_hip_conv2d_desc probe = s.conv;
      probe.flags |= PML_HIP_FLAG_CONV(r.conv);
      if (!pml_hip_conv2d_takes_maxpool(&probe)) r.conv = 0;
    }
    std::string text;
    if (r.tile >= 0) {
      flags |= PML_HIP_FLAG_TILE(r.tile);
      text += std::string("tile=") + pml_hip_tile_name(r.tile);
    }
    if (r.conv > 0) {
      static const char* const names[] = {"auto", "igemm", "patches", "ldsfilter", "blocks"};
      flags |= PML_HIP_FLAG_CONV(r.conv);
      text += std::string(text.empty() ? "" : ",") + "conv=" + names[r.conv];
    }
    if (!text.empty()) s.schedule = " {" + text + "}";
  }
}

void Planner::analyse() {
  users_.clear();
  producer_.clear();
  outputs_.clear();
  for (size_t i = 0; i < prog_->ops.size(); ++i) {
    const Op& op = prog_->ops[i];
    producer_[op.result.get()] = i;
    for (const ValuePtr& v : op.operands) users_[v.get()].push_back(i);
    if (op.init) users_[op.init.get()].push_back(i);
  }
  for (const ValuePtr& v : prog_->outputs) outputs_.insert(v.get());
}

// select(cmp_lt(a, b), b, a) -> max(a, b);  select(cmp_lt(a, b), a, b) -> min(a, b)
void Planner::rewriteSelectMinMax() {
  std::map<const Value*, size_t> producer;
  std::map<const Value*, int> uses;
  for (size_t i = 0; i < prog_->ops.size(); ++i) {
    producer[prog_->ops[i].result.get()] = i;
    for (const ValuePtr& v : prog_->ops[i].operands) uses[v.get()]++;
  }
  for (const ValuePtr& v : prog_->outputs) uses[v.get()]++;
  for (Op& op : prog_->ops) {
    if (op.kind != Op::Eltwise || op.fn != "select" || op.operands.size() != 3) continue;
    auto it = producer.find(op.operands[0].get());
    if (it == producer.end()) continue;
    const Op& cmp = prog_->ops[it->second];
    if (cmp.kind != Op::Eltwise || (cmp.fn != "cmp_lt" && cmp.fn != "cmp_gt") || cmp.operands.size() != 2) continue;
    const ValuePtr &a = cmp.operands[0], &b = cmp.operands[1];
    // the running value of a chain has to be the first comparand
    if (a->kind == Value::Literal) continue;
    const ValuePtr &t = op.operands[1], &f = op.operands[2];
    auto same = [](const ValuePtr& x, const ValuePtr& y) {
      if (x == y) return true;
      // two scalar literals / rank-0 constants with the same value count as the same operand
      // (an untyped literal takes the type of the tensor it meets, so `x > -127.0` and `cast(-127.0, f32)` agree)
      if (x->kind == Value::Literal && y->kind == Value::Literal) {
        const DataType xt = x->shape.elementType, yt = y->shape.elementType;
        if (xt != yt && !util::isAmbiguous(xt) && !util::isAmbiguous(yt)) return false;
        return x->literalAsDouble() == y->literalAsDouble();
      }
      return false;
    };
    // the comparison happens in the promoted type of (a, b); min/max in the chain must compute the same
    if (a->shape.elementType != b->shape.elementType && a->kind != Value::Literal && b->kind != Value::Literal) continue;
    if (cmp.fn == "cmp_gt") {
      // select(a > b, a, b): the lower bound of op::clip
      if (same(t, a) && same(f, b)) {
        op.fn = "maxgt";
        op.operands = {a, b};
      }
    } else if (same(t, b) && same(f, a)) {
      op.fn = "max";
      op.operands = {a, b};
    } else if (same(t, a) && same(f, b)) {
      op.fn = "min";
      op.operands = {a, b};
    }
  }
}

int Planner::newBuffer(BufferInfo::Kind kind, size_t bytes, const std::string& name) {
  BufferInfo b;
  b.kind = kind;
  b.bytes = bytes;
  b.name = name;
  plan_->buffers.push_back(b);
  return static_cast<int>(plan_->buffers.size()) - 1;
}

int Planner::bufferFor(const ValuePtr& v) {
  auto it = bufferOf_.find(v.get());
  if (it != bufferOf_.end()) return it->second;
  int id = -1;
  switch (v->kind) {
    case Value::Constant:
      id = newBuffer(BufferInfo::Constant, v->constant->size(), v->name);
      plan_->buffers[id].constant = v->constant;
      break;
    case Value::Temp:
      id = newBuffer(BufferInfo::Temp, v->shape.getByteSize(), v->name);
      break;
    case Value::Literal:
      throw std::runtime_error("internal: a scalar literal has no buffer");
    case Value::Input:
      throw std::runtime_error("internal: unknown program input");
  }
  bufferOf_[v.get()] = id;
  return id;
}

// a one-element constant of type dt holding the given value
int Planner::scalarConstant(DataType dt, double f, int64_t i) {
  TensorShape shape(dt);
  auto buf = std::make_shared<util::SimpleBuffer>(shape);
  char* p = buf->data();
  switch (dt) {
    case DataType::f32: { float x = static_cast<float>(f); std::memcpy(p, &x, 4); break; }
    case DataType::f64: std::memcpy(p, &f, 8); break;
    case DataType::bf16: {
      float x = static_cast<float>(f);
      uint32_t u;
      std::memcpy(&u, &x, 4);
      uint16_t h = (u & 0x7fffffffu) > 0x7f800000u ? static_cast<uint16_t>((u >> 16) | 0x40)
                                                   : static_cast<uint16_t>((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
      std::memcpy(p, &h, 2);
      break;
    }
    case DataType::f16: throw std::runtime_error("float16 constants are not supported by the hip target");
    default: std::memcpy(p, &i, util::byteSize(dt)); break;
  }
  const int id = newBuffer(BufferInfo::Constant, buf->size(), "scalar");
  plan_->buffers[id].constant = buf;
  return id;
}


std::string Plan::dump() const {
  std::stringstream ss;
  ss << "hip plan: " << steps.size() << " launches, " << buffers.size() << " buffers\n";
  for (size_t i = 0; i < steps.size(); ++i) ss << "  [" << i << "] " << steps[i].text << steps[i].schedule << "\n";
  return ss.str();
}

std::shared_ptr<Plan> buildPlan(tile::Program* program, const Options& options) {
  Planner p(program, options);
  return p.run();
}

}  // namespace pmlc::target::hip
