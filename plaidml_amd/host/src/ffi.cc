// The stable C ABI of libplaidml.so: core, edsl, op and exec entry points
// (plaidml/{core,edsl,op,exec}/ffi.h).  Each function wraps its body so that a
// C++ exception becomes plaidml_error{1, message} and the declared default is
// returned (reference convention: plaidml/core/internal.h:40-70).
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <mutex>
#include <sstream>

#include "ast.h"
#include "ffi_internal.h"
#include "hip_plan.h"
#include "hip_runtime.h"
#include "tile.h"
#include "util.h"

using namespace pmlc;  // NOLINT
using pmlc::ast::DimNode;
using pmlc::ast::ExprNode;
using pmlc::ast::PolyNode;
using pmlc::util::DataType;
using pmlc::util::TensorShape;

namespace pmlc::util {

std::string getEnvVar(const std::string& key, const std::string& def) {
  const char* v = std::getenv(key.c_str());
  return v ? std::string(v) : def;
}

int verbosity() {
  const std::string v = getEnvVar("PLAIDML_VERBOSE");
  return v.empty() ? 0 : std::atoi(v.c_str());
}

Settings* Settings::Instance() {
  static Settings s;
  static bool init = false;
  if (!init) {
    init = true;
    std::string path = getEnvVar("PLAIDML_SETTINGS");
    if (path.empty()) path = getEnvVar("HOME", ".") + "/.plaidml2";
    s.settings_["PLAIDML_SETTINGS"] = path;
  }
  return &s;
}
std::string Settings::get(const std::string& key) const {
  std::string env = getEnvVar(key);
  if (!env.empty()) return env;
  auto it = settings_.find(key);
  return it == settings_.end() ? std::string() : it->second;
}
void Settings::set(const std::string& key, const std::string& value) {
  settings_[key] = value;
  setenv(key.c_str(), value.c_str(), 1);
}
void Settings::load() {
  const std::string path = get("PLAIDML_SETTINGS");
  std::ifstream file(path);
  if (!file) return;
  settings_.clear();
  for (std::string line; std::getline(file, line);) {
    auto pos = line.find('=');
    if (pos == std::string::npos) continue;
    std::string key = line.substr(0, pos), value = line.substr(pos + 1);
    std::string env = getEnvVar(key);
    set(key, env.empty() ? value : env);
  }
  settings_["PLAIDML_SETTINGS"] = path;
}
void Settings::save() {
  std::ofstream file(get("PLAIDML_SETTINGS"));
  for (const auto& kv : settings_)
    if (kv.first != "PLAIDML_SETTINGS") file << kv.first << "=" << kv.second << std::endl;
}

}  // namespace pmlc::util

namespace {

template <typename T, typename F>
T ffi_wrap(plaidml_error* err, T def, F fn) {
  try {
    err->code = 0;
    err->msg = nullptr;
    return fn();
  } catch (const std::exception& ex) {
    err->code = 1;
    err->msg = new plaidml_string{ex.what()};
    return def;
  } catch (...) {
    err->code = 1;
    err->msg = new plaidml_string{"C++ exception"};
    return def;
  }
}
template <typename F>
void ffi_wrap_void(plaidml_error* err, F fn) {
  try {
    err->code = 0;
    err->msg = nullptr;
    fn();
  } catch (const std::exception& ex) {
    err->code = 1;
    err->msg = new plaidml_string{ex.what()};
  } catch (...) {
    err->code = 1;
    err->msg = new plaidml_string{"C++ exception"};
  }
}

plaidml_strings* makeStrings(const std::vector<std::string>& v) {
  auto* ret = new plaidml_strings{v.size(), new plaidml_string*[v.size()]};
  for (size_t i = 0; i < v.size(); ++i) ret->elts[i] = new plaidml_string{v[i]};
  return ret;
}
plaidml_integers* makeIntegers(const std::vector<int64_t>& v) {
  auto* ret = new plaidml_integers{v.size(), new int64_t[v.size()]};
  for (size_t i = 0; i < v.size(); ++i) ret->elts[i] = v[i];
  return ret;
}
plaidml_shapes* makeShapes(const std::vector<tile::ValuePtr>& values) {
  auto* ret = new plaidml_shapes{values.size(), new plaidml_shape*[values.size()]};
  for (size_t i = 0; i < values.size(); ++i) ret->elts[i] = new plaidml_shape{values[i]->shape};
  return ret;
}

ast::AffineOp affineOp(plaidml_int_op op) {
  switch (op) {
    case PLAIDML_INT_OP_NEG: return ast::AffineOp::Neg;
    case PLAIDML_INT_OP_ADD: return ast::AffineOp::Add;
    case PLAIDML_INT_OP_SUB: return ast::AffineOp::Sub;
    case PLAIDML_INT_OP_MUL: return ast::AffineOp::Mul;
    case PLAIDML_INT_OP_DIV: return ast::AffineOp::Div;
    case PLAIDML_INT_OP_MAX: return ast::AffineOp::Max;
    case PLAIDML_INT_OP_MIN: return ast::AffineOp::Min;
  }
  throw std::runtime_error("Unknown polynomial op");
}

std::atomic<uint64_t> g_next_index_id{1};

// target string "name{key=value,...}" (reference pmlc/compiler/program.cc:176-185)
void parseTarget(const std::string& text, std::string* name, std::map<std::string, std::string>* opts) {
  auto brace = text.find('{');
  *name = text.substr(0, brace);
  if (brace == std::string::npos) return;
  auto end = text.rfind('}');
  if (end == std::string::npos || end < brace) throw std::runtime_error("Invalid target options: " + text);
  std::stringstream ss(text.substr(brace + 1, end - brace - 1));
  for (std::string item; std::getline(ss, item, ',');) {
    auto eq = item.find('=');
    if (eq == std::string::npos)
      (*opts)[item] = "1";
    else
      (*opts)[item.substr(0, eq)] = item.substr(eq + 1);
  }
}

bool truthy(const std::string& v) { return !(v == "0" || v == "false" || v == "off" || v.empty()); }

void compileProgram(tile::Program* program, const std::string& requested, bool /*debug*/) {
  std::string target = requested;
  if (target.empty()) target = util::Settings::Instance()->get("PLAIDML_TARGET");
  if (target.empty()) target = "hip";
  std::string name;
  std::map<std::string, std::string> opts;
  parseTarget(target, &name, &opts);
  if (name != "hip") throw std::runtime_error("Could not find compiler target: " + name);
  target::hip::Options options;
  if (opts.count("fuse")) options.fuse = truthy(opts["fuse"]);
  if (opts.count("specialise")) options.specialise = truthy(opts["specialise"]);
  if (opts.count("specialize")) options.specialise = truthy(opts["specialize"]);
  if (opts.count("fp32")) {
    if (opts["fp32"] == "bf16x3")
      options.fp32_as_bf16x3 = true;
    else if (opts["fp32"] != "mfma")
      throw std::runtime_error("Invalid target option fp32=" + opts["fp32"] + " (mfma or bf16x3)");
  }
  if (opts.count("tile")) options.tile = opts["tile"];
  if (opts.count("conv")) options.conv = opts["conv"];
  if (opts.count("graph")) options.graph = truthy(opts["graph"]);
  options.schedule_path = util::Settings::Instance()->get("PLAIDML_SCHEDULE_PATH");
  program->passes.resize(1);  // keep only the "tile" text when compiling again
  tile::foldAddIntoInit(program);
  program->passes.emplace_back("tile-algebraic-opt", program->str());
  tile::computeBounds(program);
  program->passes.emplace_back("tile-compute-bounds", program->str());
  auto plan = target::hip::buildPlan(program, options);
  program->passes.emplace_back("hip-plan", plan->dump());
  program->compiled = plan;
  program->target = "hip";
  // PLAIDML_DUMP=<dir>: one file per pass, NN_pass.txt
  const std::string dump = util::Settings::Instance()->get("PLAIDML_DUMP");
  if (!dump.empty()) {
    for (size_t i = 0; i < program->passes.size(); ++i) {
      char num[16];
      std::snprintf(num, sizeof num, "%02zu_", i);
      std::ofstream f(dump + "/" + program->name + "_" + num + program->passes[i].first + ".txt");
      f << program->passes[i].second;
    }
  }
  if (util::verbosity() >= 1) std::fprintf(stderr, "%s", plan->dump().c_str());
}

}  // namespace

extern "C" {

// ---------------------------------------------------------------------------------------
// core
// ---------------------------------------------------------------------------------------

const char* plaidml_string_ptr(plaidml_string* str) { return str->str.c_str(); }
void plaidml_string_free(plaidml_string* str) { delete str; }

void plaidml_init(plaidml_error* err) {
  static std::once_flag once;
  ffi_wrap_void(err, [&] { std::call_once(once, [] { util::Settings::Instance(); }); });
}
void plaidml_shutdown(plaidml_error* err) { ffi_wrap_void(err, [] {}); }
const char* plaidml_version(plaidml_error* err) {
  return ffi_wrap<const char*>(err, nullptr, [] { return "1.0.0+hip.gfx950"; });
}

void plaidml_integers_free(plaidml_error* err, plaidml_integers* ints) {
  ffi_wrap_void(err, [&] {
    delete[] ints->elts;
    delete ints;
  });
}
// The list frees only its array; each element handle belongs to the caller
// (reference plaidml/core/ffi.cc:84-91,158-174).
void plaidml_strings_free(plaidml_error* err, plaidml_strings* strs) {
  ffi_wrap_void(err, [&] {
    delete[] strs->elts;
    delete strs;
  });
}
void plaidml_kvps_free(plaidml_error* err, plaidml_kvps* kvps) {
  ffi_wrap_void(err, [&] {
    delete[] kvps->elts;
    delete kvps;
  });
}
void plaidml_shapes_free(plaidml_error* err, plaidml_shapes* shapes) {
  ffi_wrap_void(err, [&] {
    delete[] shapes->elts;
    delete shapes;
  });
}

plaidml_kvps* plaidml_settings_list(plaidml_error* err) {
  return ffi_wrap<plaidml_kvps*>(err, nullptr, [&] {
    const auto& all = util::Settings::Instance()->all();
    auto* ret = new plaidml_kvps{all.size(), new plaidml_kvp[all.size()]};
    size_t i = 0;
    for (const auto& kv : all) {
      ret->elts[i].key = new plaidml_string{kv.first};
      ret->elts[i].value = new plaidml_string{kv.second};
      ++i;
    }
    return ret;
  });
}
plaidml_string* plaidml_settings_get(plaidml_error* err, const char* key) {
  return ffi_wrap<plaidml_string*>(err, nullptr, [&] { return new plaidml_string{util::Settings::Instance()->get(key)}; });
}
void plaidml_settings_set(plaidml_error* err, const char* key, const char* value) {
  ffi_wrap_void(err, [&] { util::Settings::Instance()->set(key, value); });
}
void plaidml_settings_load(plaidml_error* err) { ffi_wrap_void(err, [] { util::Settings::Instance()->load(); }); }
void plaidml_settings_save(plaidml_error* err) { ffi_wrap_void(err, [] { util::Settings::Instance()->save(); }); }

void plaidml_shape_free(plaidml_error* err, plaidml_shape* shape) { ffi_wrap_void(err, [&] { delete shape; }); }
plaidml_shape* plaidml_shape_alloc(plaidml_error* err, plaidml_datatype dtype, size_t rank, const int64_t* sizes,
                                   const int64_t* strides) {
  return ffi_wrap<plaidml_shape*>(err, nullptr, [&] {
    if (dtype <= PLAIDML_DATA_INVALID || dtype > PLAIDML_DATA_BFLOAT16) throw std::runtime_error("Invalid dtype");
    TensorShape shape(static_cast<DataType>(dtype));
    shape.sizes.assign(sizes, sizes + rank);
    if (strides) shape.strides.assign(strides, strides + rank);
    return new plaidml_shape{shape};
  });
}
plaidml_shape* plaidml_shape_clone(plaidml_error* err, plaidml_shape* shape) {
  return ffi_wrap<plaidml_shape*>(err, nullptr, [&] { return new plaidml_shape{shape->shape}; });
}
plaidml_string* plaidml_shape_repr(plaidml_error* err, plaidml_shape* shape) {
  return ffi_wrap<plaidml_string*>(err, nullptr, [&] { return new plaidml_string{shape->shape.str()}; });
}
size_t plaidml_shape_get_rank(plaidml_error* err, plaidml_shape* shape) {
  return ffi_wrap<size_t>(err, 0, [&] { return shape->shape.getRank(); });
}
plaidml_datatype plaidml_shape_get_dtype(plaidml_error* err, plaidml_shape* shape) {
  return ffi_wrap<plaidml_datatype>(err, PLAIDML_DATA_INVALID,
                                    [&] { return static_cast<plaidml_datatype>(shape->shape.elementType); });
}
plaidml_integers* plaidml_shape_get_sizes(plaidml_error* err, plaidml_shape* shape) {
  return ffi_wrap<plaidml_integers*>(err, nullptr, [&] { return makeIntegers(shape->shape.sizes); });
}
plaidml_integers* plaidml_shape_get_strides(plaidml_error* err, plaidml_shape* shape) {
  return ffi_wrap<plaidml_integers*>(err, nullptr, [&] {
    return makeIntegers(shape->shape.strides.empty() ? shape->shape.denseStrides() : shape->shape.strides);
  });
}
uint64_t plaidml_shape_get_nbytes(plaidml_error* err, plaidml_shape* shape) {
  return ffi_wrap<uint64_t>(err, 0, [&] { return static_cast<uint64_t>(shape->shape.getByteSize()); });
}

plaidml_buffer* plaidml_buffer_alloc(plaidml_error* err, plaidml_shape* shape) {
  return ffi_wrap<plaidml_buffer*>(err, nullptr,
                                   [&] {
                                     // large buffers in page-locked memory when a GPU is visible: exec copies to and
                                     // from them at the link's rate (65536: below that the copy's set-up dominates)
                                     if (shape->shape.getByteSize() >= 65536) {
                                       try {
                                         return new plaidml_buffer{
                                             std::make_shared<util::ForeignBuffer>(shape->shape, rt::pinnedAlloc, rt::pinnedFree)};
                                       } catch (const std::bad_alloc&) {
                                       }
                                     }
                                     return new plaidml_buffer{std::make_shared<util::SimpleBuffer>(shape->shape)};
                                   });
}
plaidml_buffer* plaidml_buffer_adopt(plaidml_error* err, plaidml_shape* shape, char* data, size_t size) {
  return ffi_wrap<plaidml_buffer*>(
      err, nullptr, [&] { return new plaidml_buffer{std::make_shared<util::AdoptedBuffer>(shape->shape, data, size)}; });
}
void plaidml_buffer_free(plaidml_error* err, plaidml_buffer* buffer) { ffi_wrap_void(err, [&] { delete buffer; }); }
plaidml_buffer* plaidml_buffer_clone(plaidml_error* err, plaidml_buffer* buffer) {
  return ffi_wrap<plaidml_buffer*>(err, nullptr, [&] { return new plaidml_buffer{buffer->buffer}; });
}
plaidml_shape* plaidml_buffer_shape(plaidml_error* err, plaidml_buffer* buffer) {
  return ffi_wrap<plaidml_shape*>(err, nullptr, [&] { return new plaidml_shape{buffer->buffer->shape()}; });
}
char* plaidml_buffer_data(plaidml_error* err, plaidml_buffer* buffer) {
  return ffi_wrap<char*>(err, nullptr, [&] { return buffer->buffer->data(); });
}
size_t plaidml_buffer_size(plaidml_error* err, plaidml_buffer* buffer) {
  return ffi_wrap<size_t>(err, 0, [&] { return buffer->buffer->size(); });
}

void plaidml_program_free(plaidml_error* err, plaidml_program* program) { ffi_wrap_void(err, [&] { delete program; }); }
plaidml_string* plaidml_program_repr(plaidml_error* err, plaidml_program* program) {
  return ffi_wrap<plaidml_string*>(err, nullptr, [&] { return new plaidml_string{program->program->passes.at(0).second}; });
}
plaidml_shapes* plaidml_program_get_inputs(plaidml_error* err, plaidml_program* program) {
  return ffi_wrap<plaidml_shapes*>(err, nullptr, [&] { return makeShapes(program->program->inputs); });
}
plaidml_shapes* plaidml_program_get_outputs(plaidml_error* err, plaidml_program* program) {
  return ffi_wrap<plaidml_shapes*>(err, nullptr, [&] { return makeShapes(program->program->outputs); });
}
plaidml_kvps* plaidml_program_get_passes(plaidml_error* err, plaidml_program* program) {
  return ffi_wrap<plaidml_kvps*>(err, nullptr, [&] {
    const auto& passes = program->program->passes;
    auto* ret = new plaidml_kvps{passes.size(), new plaidml_kvp[passes.size()]};
    for (size_t i = 0; i < passes.size(); ++i) {
      ret->elts[i].key = new plaidml_string{passes[i].first};
      ret->elts[i].value = new plaidml_string{passes[i].second};
    }
    return ret;
  });
}
void plaidml_program_compile(plaidml_error* err, plaidml_program* program, bool debug, const char* target) {
  ffi_wrap_void(err, [&] { compileProgram(program->program.get(), target ? target : "", debug); });
}
plaidml_buffer* plaidml_program_save(plaidml_error* err, plaidml_program*, size_t, const char**, const char**) {
  return ffi_wrap<plaidml_buffer*>(err, nullptr, [&]() -> plaidml_buffer* {
    throw std::runtime_error("Target 'hip' does not have 'save' support.");
  });
}

// ---------------------------------------------------------------------------------------
// edsl
// ---------------------------------------------------------------------------------------

void plaidml_edsl_init(plaidml_error* err) { ffi_wrap_void(err, [] {}); }

void plaidml_poly_expr_free(plaidml_error* err, plaidml_poly_expr* expr) { ffi_wrap_void(err, [&] { delete expr; }); }
plaidml_string* plaidml_poly_expr_repr(plaidml_error* err, plaidml_poly_expr* expr) {
  return ffi_wrap<plaidml_string*>(err, nullptr, [&] { return new plaidml_string{expr->node->str()}; });
}
plaidml_poly_expr* plaidml_poly_expr_dim(plaidml_error* err, plaidml_dim_expr* expr) {
  return ffi_wrap<plaidml_poly_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<PolyNode>(PolyNode::Dim);
    node->dimRef = expr->node;
    return new plaidml_poly_expr{node};
  });
}
plaidml_poly_expr* plaidml_poly_expr_index(plaidml_error* err, const char* name) {
  return ffi_wrap<plaidml_poly_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<PolyNode>(PolyNode::Index);
    node->name = name ? name : "";
    node->id = g_next_index_id++;
    return new plaidml_poly_expr{node};
  });
}
plaidml_poly_expr* plaidml_poly_expr_literal(plaidml_error* err, int64_t value) {
  return ffi_wrap<plaidml_poly_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<PolyNode>(PolyNode::Literal);
    node->value = value;
    return new plaidml_poly_expr{node};
  });
}
plaidml_poly_expr* plaidml_poly_expr_op(plaidml_error* err, plaidml_int_op op, size_t nargs, plaidml_poly_expr** args) {
  return ffi_wrap<plaidml_poly_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<PolyNode>(PolyNode::Op);
    node->op = affineOp(op);
    for (size_t i = 0; i < nargs; ++i) node->operands.push_back(args[i]->node);
    if (node->operands.size() != (op == PLAIDML_INT_OP_NEG ? 1u : 2u)) throw std::runtime_error("Invalid number of operands in polynomial op");
    return new plaidml_poly_expr{node};
  });
}

void plaidml_dim_expr_free(plaidml_error* err, plaidml_dim_expr* expr) { ffi_wrap_void(err, [&] { delete expr; }); }
plaidml_string* plaidml_dim_expr_repr(plaidml_error* err, plaidml_dim_expr* expr) {
  return ffi_wrap<plaidml_string*>(err, nullptr, [&] { return new plaidml_string{expr->node->str()}; });
}
plaidml_dim_expr* plaidml_dim_expr_none(plaidml_error* err) {
  return ffi_wrap<plaidml_dim_expr*>(err, nullptr, [&] { return new plaidml_dim_expr{std::make_shared<DimNode>(DimNode::None)}; });
}
plaidml_dim_expr* plaidml_dim_expr_int(plaidml_error* err, int64_t value) {
  return ffi_wrap<plaidml_dim_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<DimNode>(DimNode::Literal);
    node->value = value;
    return new plaidml_dim_expr{node};
  });
}
plaidml_dim_expr* plaidml_dim_expr_op(plaidml_error* err, plaidml_int_op op, size_t nargs, plaidml_dim_expr** args) {
  return ffi_wrap<plaidml_dim_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<DimNode>(DimNode::Op);
    node->op = affineOp(op);
    for (size_t i = 0; i < nargs; ++i) node->operands.push_back(args[i]->node);
    if (node->operands.size() != (op == PLAIDML_INT_OP_NEG ? 1u : 2u)) throw std::runtime_error("Invalid number of operands in dim op");
    return new plaidml_dim_expr{node};
  });
}

void plaidml_expr_free(plaidml_error* err, plaidml_expr* expr) { ffi_wrap_void(err, [&] { delete expr; }); }
void* plaidml_expr_ptr(plaidml_error* err, plaidml_expr* expr) {
  return ffi_wrap<void*>(err, nullptr, [&] { return static_cast<void*>(expr->node.get()); });
}
plaidml_datatype plaidml_expr_get_dtype(plaidml_error* err, plaidml_expr* expr) {
  return ffi_wrap<plaidml_datatype>(err, PLAIDML_DATA_INVALID, [&] {
    ast::Evaluator ev;
    return static_cast<plaidml_datatype>(ev.getShape(expr->node).elementType);
  });
}
size_t plaidml_expr_get_rank(plaidml_error* err, plaidml_expr* expr) {
  return ffi_wrap<size_t>(err, 0, [&] {
    ast::Evaluator ev;
    return ev.getShape(expr->node).getRank();
  });
}
plaidml_shape* plaidml_expr_get_shape(plaidml_error* err, plaidml_expr* expr) {
  return ffi_wrap<plaidml_shape*>(err, nullptr, [&] {
    ast::Evaluator ev;
    return new plaidml_shape{ev.getShape(expr->node)};
  });
}
void plaidml_expr_bind_dims(plaidml_error* err, plaidml_expr* expr, size_t rank, plaidml_dim_expr** dims) {
  ffi_wrap_void(err, [&] {
    std::vector<ast::DimNodePtr*> into(rank);
    for (size_t i = 0; i < rank; ++i) into[i] = &dims[i]->node;
    ast::Evaluator ev;
    ev.bindDims(expr->node, into);
  });
}
plaidml_string* plaidml_expr_repr(plaidml_error* err, plaidml_expr* expr) {
  return ffi_wrap<plaidml_string*>(err, nullptr, [&] { return new plaidml_string{expr->node->str()}; });
}
plaidml_expr* plaidml_expr_clone(plaidml_error* err, plaidml_expr* expr) {
  return ffi_wrap<plaidml_expr*>(err, nullptr, [&] { return new plaidml_expr{expr->node}; });
}
plaidml_dim_expr* plaidml_expr_get_dim(plaidml_error* err, plaidml_expr* expr) {
  return ffi_wrap<plaidml_dim_expr*>(err, nullptr, [&] {
    if (expr->node->kind != ExprNode::Dim) throw std::runtime_error("plaidml_expr_get_dim can only be used on a dim expression");
    return new plaidml_dim_expr{expr->node->dimNode};
  });
}
plaidml_expr* plaidml_expr_dim(plaidml_error* err, plaidml_dim_expr* expr) {
  return ffi_wrap<plaidml_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<ExprNode>(ExprNode::Dim);
    node->dimNode = expr->node;
    return new plaidml_expr{node};
  });
}
plaidml_expr* plaidml_expr_input(plaidml_error* err, plaidml_shape* shape, const char* name) {
  return ffi_wrap<plaidml_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<ExprNode>(ExprNode::Input);
    node->shape = shape->shape;
    node->shape.strides.clear();
    node->name = name ? name : "";
    return new plaidml_expr{node};
  });
}
plaidml_expr* plaidml_expr_constant(plaidml_error* err, plaidml_buffer* buffer, const char* name) {
  return ffi_wrap<plaidml_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<ExprNode>(ExprNode::ConstTensor);
    node->buffer = buffer->buffer;
    node->name = name ? name : "";
    return new plaidml_expr{node};
  });
}
plaidml_expr* plaidml_expr_uint(plaidml_error* err, uint64_t value) {
  return ffi_wrap<plaidml_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<ExprNode>(ExprNode::ConstUnsigned);
    node->uvalue = value;
    return new plaidml_expr{node};
  });
}
plaidml_expr* plaidml_expr_int(plaidml_error* err, int64_t value) {
  return ffi_wrap<plaidml_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<ExprNode>(ExprNode::ConstSigned);
    node->ivalue = value;
    return new plaidml_expr{node};
  });
}
plaidml_expr* plaidml_expr_float(plaidml_error* err, double value) {
  return ffi_wrap<plaidml_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<ExprNode>(ExprNode::ConstFloat);
    node->fvalue = value;
    return new plaidml_expr{node};
  });
}
plaidml_expr* plaidml_expr_element(plaidml_error* err, plaidml_expr* expr, size_t ordinal) {
  return ffi_wrap<plaidml_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<ExprNode>(ExprNode::Element);
    node->expr = expr->node;
    node->ordinal = ordinal;
    return new plaidml_expr{node};
  });
}
plaidml_expr* plaidml_expr_intrinsic(plaidml_error* err, const char* fn, size_t nargs, plaidml_expr** args, const char* name) {
  return ffi_wrap<plaidml_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<ExprNode>(ExprNode::Intrinsic);
    node->op = fn;
    node->name = name ? name : "";
    for (size_t i = 0; i < nargs; ++i) node->operands.push_back(args[i]->node);
    ast::Evaluator ev;
    ev.verify(node);
    return new plaidml_expr{node};
  });
}
plaidml_expr* plaidml_expr_cast(plaidml_error* err, plaidml_expr* tensor, plaidml_datatype dtype) {
  return ffi_wrap<plaidml_expr*>(err, nullptr, [&] {
    if (dtype <= PLAIDML_DATA_FLOATX || dtype > PLAIDML_DATA_BFLOAT16) throw std::runtime_error("Invalid dtype for cast");
    auto node = std::make_shared<ExprNode>(ExprNode::Cast);
    node->expr = tensor->node;
    node->dtype = static_cast<DataType>(dtype);
    return new plaidml_expr{node};
  });
}
plaidml_expr* plaidml_expr_pragma(plaidml_error* err, plaidml_expr* tensor, const char* op, size_t, plaidml_attr**) {
  return ffi_wrap<plaidml_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<ExprNode>(ExprNode::Pragma);
    node->expr = tensor->node;
    node->op = op;
    return new plaidml_expr{node};
  });
}
void plaidml_exprs_free(plaidml_error* err, plaidml_exprs* exprs) {
  ffi_wrap_void(err, [&] {
    delete[] exprs->elts;
    delete exprs;
  });
}
// Layers only group operations for readers of the program text: begin returns a token, end hands the
// outputs back unchanged.
plaidml_expr* plaidml_expr_layer_begin(plaidml_error* err, const char* op, size_t, plaidml_expr**, size_t, plaidml_attr**) {
  return ffi_wrap<plaidml_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<ExprNode>(ExprNode::Pragma);
    node->op = op ? op : "layer";
    return new plaidml_expr{node};
  });
}
plaidml_exprs* plaidml_expr_layer_end(plaidml_error* err, plaidml_expr*, size_t noutputs, plaidml_expr** outputs) {
  return ffi_wrap<plaidml_exprs*>(err, nullptr, [&] {
    auto* ret = new plaidml_exprs{noutputs, new plaidml_expr*[noutputs]};
    for (size_t i = 0; i < noutputs; ++i) ret->elts[i] = new plaidml_expr{outputs[i]->node};
    return ret;
  });
}

plaidml_expr* plaidml_expr_contraction(plaidml_error* err, plaidml_agg_op agg_op, plaidml_combo_op combo_op, size_t rank,
                                       plaidml_poly_expr** idxs, plaidml_dim_expr** dims, plaidml_expr* init,
                                       const char* name) {
  return ffi_wrap<plaidml_expr*>(err, nullptr, [&] {
    auto node = std::make_shared<ExprNode>(ExprNode::Contraction);
    node->name = name ? name : "";
    switch (agg_op) {
      case PLAIDML_AGG_OP_ASSIGN: node->aggKind = ast::AggKind::assign; break;
      case PLAIDML_AGG_OP_MAX: node->aggKind = ast::AggKind::max; break;
      case PLAIDML_AGG_OP_MIN: node->aggKind = ast::AggKind::min; break;
      case PLAIDML_AGG_OP_PROD: node->aggKind = ast::AggKind::mul; break;
      case PLAIDML_AGG_OP_SUM: node->aggKind = ast::AggKind::add; break;
      default: throw std::runtime_error("Unsupported agg_op");
    }
    switch (combo_op) {
      case PLAIDML_COMBO_OP_ADD: node->comboKind = ast::ComboKind::add; break;
      case PLAIDML_COMBO_OP_COND: node->comboKind = ast::ComboKind::cond; break;
      case PLAIDML_COMBO_OP_EQ: node->comboKind = ast::ComboKind::eq; break;
      case PLAIDML_COMBO_OP_MUL: node->comboKind = ast::ComboKind::mul; break;
      case PLAIDML_COMBO_OP_NONE: node->comboKind = ast::ComboKind::none; break;
      default: throw std::runtime_error("Unsupported combo_op");
    }
    for (size_t i = 0; i < rank; ++i) {
      node->sinkIdxs.push_back(idxs[i]->node);
      node->sinkDims.push_back(dims[i]->node);
    }
    if (init) node->init = init->node;
    return new plaidml_expr{node};
  });
}
void plaidml_contraction_add_operand(plaidml_error* err, plaidml_expr* expr, plaidml_expr* tensor, size_t rank,
                                     plaidml_poly_expr** idxs) {
  ffi_wrap_void(err, [&] {
    if (expr->node->kind != ExprNode::Contraction) throw std::bad_cast();
    ast::PolyMap map;
    map.ref = tensor->node;
    for (size_t i = 0; i < rank; ++i) map.idxs.push_back(idxs[i]->node);
    expr->node->srcs.push_back(map);
  });
}
void plaidml_contraction_add_constraint(plaidml_error* err, plaidml_expr* expr, plaidml_poly_expr* lhs, plaidml_dim_expr* rhs) {
  ffi_wrap_void(err, [&] {
    if (expr->node->kind != ExprNode::Contraction) throw std::bad_cast();
    expr->node->constraints.push_back(ast::Constraint{lhs->node, rhs->node});
  });
}
void plaidml_contraction_build(plaidml_error* err, plaidml_expr* expr) {
  ffi_wrap_void(err, [&] {
    ast::Evaluator ev;
    ev.verify(expr->node);
  });
}

void plaidml_tuple_free(plaidml_error* err, plaidml_tuple* tuple) {
  ffi_wrap_void(err, [&] {
    delete[] tuple->elts;
    delete tuple;
  });
}
void plaidml_value_free(plaidml_error* err, plaidml_value* value) { ffi_wrap_void(err, [&] { delete value; }); }
plaidml_value* plaidml_value_clone(plaidml_error* err, plaidml_value* value) {
  return ffi_wrap<plaidml_value*>(err, nullptr, [&] { return new plaidml_value{*value}; });
}
plaidml_value_kind plaidml_value_get_kind(plaidml_error* err, plaidml_value* value) {
  return ffi_wrap<plaidml_value_kind>(err, PLAIDML_VALUE_NONE, [&] { return value->kind; });
}
plaidml_value* plaidml_value_none(plaidml_error* err) {
  return ffi_wrap<plaidml_value*>(err, nullptr, [&] { return new plaidml_value{}; });
}
plaidml_value* plaidml_value_dim(plaidml_error* err, plaidml_dim_expr* expr) {
  return ffi_wrap<plaidml_value*>(err, nullptr, [&] {
    auto* v = new plaidml_value{};
    v->kind = PLAIDML_VALUE_DIM;
    v->dim = expr->node;
    return v;
  });
}
plaidml_value* plaidml_value_expr(plaidml_error* err, plaidml_expr* expr) {
  return ffi_wrap<plaidml_value*>(err, nullptr, [&] {
    if (!expr) throw std::runtime_error("plaidml_value_expr requires non-null expr");
    auto* v = new plaidml_value{};
    v->kind = PLAIDML_VALUE_EXPR;
    v->expr = expr->node;
    return v;
  });
}
plaidml_value* plaidml_value_float(plaidml_error* err, double value) {
  return ffi_wrap<plaidml_value*>(err, nullptr, [&] {
    auto* v = new plaidml_value{};
    v->kind = PLAIDML_VALUE_FLOAT;
    v->f = value;
    return v;
  });
}
plaidml_value* plaidml_value_int(plaidml_error* err, int64_t value) {
  return ffi_wrap<plaidml_value*>(err, nullptr, [&] {
    auto* v = new plaidml_value{};
    v->kind = PLAIDML_VALUE_INT;
    v->i = value;
    return v;
  });
}
plaidml_value* plaidml_value_str(plaidml_error* err, const char* value) {
  return ffi_wrap<plaidml_value*>(err, nullptr, [&] {
    auto* v = new plaidml_value{};
    v->kind = PLAIDML_VALUE_STR;
    v->s = value ? value : "";
    return v;
  });
}
plaidml_value* plaidml_value_tuple(plaidml_error* err, size_t nelts, plaidml_value** elts) {
  return ffi_wrap<plaidml_value*>(err, nullptr, [&] {
    auto* v = new plaidml_value{};
    v->kind = PLAIDML_VALUE_TUPLE;
    for (size_t i = 0; i < nelts; ++i) v->tuple.push_back(std::make_shared<plaidml_value>(*elts[i]));
    return v;
  });
}
plaidml_dim_expr* plaidml_value_dim_get(plaidml_error* err, plaidml_value* value) {
  return ffi_wrap<plaidml_dim_expr*>(err, nullptr, [&] {
    if (value->kind != PLAIDML_VALUE_DIM) throw std::runtime_error("Value is not a dim");
    return new plaidml_dim_expr{value->dim};
  });
}
plaidml_expr* plaidml_value_expr_get(plaidml_error* err, plaidml_value* value) {
  return ffi_wrap<plaidml_expr*>(err, nullptr, [&] {
    if (value->kind != PLAIDML_VALUE_EXPR) throw std::runtime_error("Value is not an expr");
    return new plaidml_expr{value->expr};
  });
}
double plaidml_value_float_get(plaidml_error* err, plaidml_value* value) {
  return ffi_wrap<double>(err, 0.0, [&] {
    if (value->kind == PLAIDML_VALUE_INT) return static_cast<double>(value->i);
    if (value->kind != PLAIDML_VALUE_FLOAT) throw std::runtime_error("Value is not a float");
    return value->f;
  });
}
int64_t plaidml_value_int_get(plaidml_error* err, plaidml_value* value) {
  return ffi_wrap<int64_t>(err, 0, [&] {
    if (value->kind != PLAIDML_VALUE_INT) throw std::runtime_error("Value is not an int");
    return value->i;
  });
}
plaidml_string* plaidml_value_str_get(plaidml_error* err, plaidml_value* value) {
  return ffi_wrap<plaidml_string*>(err, nullptr, [&] {
    if (value->kind != PLAIDML_VALUE_STR) throw std::runtime_error("Value is not a str");
    return new plaidml_string{value->s};
  });
}
plaidml_tuple* plaidml_value_tuple_get(plaidml_error* err, plaidml_value* value) {
  return ffi_wrap<plaidml_tuple*>(err, nullptr, [&] {
    if (value->kind != PLAIDML_VALUE_TUPLE) throw std::runtime_error("Value is not a tuple");
    auto* ret = new plaidml_tuple{value->tuple.size(), new plaidml_value*[value->tuple.size()]};
    for (size_t i = 0; i < value->tuple.size(); ++i) ret->elts[i] = new plaidml_value{*value->tuple[i]};
    return ret;
  });
}
plaidml_string* plaidml_value_repr(plaidml_error* err, plaidml_value* value) {
  return ffi_wrap<plaidml_string*>(err, nullptr, [&] { return new plaidml_string{value->str()}; });
}

plaidml_strings* plaidml_targets_get(plaidml_error* err) {
  return ffi_wrap<plaidml_strings*>(err, nullptr, [&] { return makeStrings({"hip"}); });
}

plaidml_program* plaidml_build(plaidml_error* err, const char* name, size_t ninputs, plaidml_expr** inputs,
                               plaidml_shape** shapes, size_t noutputs, plaidml_expr** outputs) {
  return ffi_wrap<plaidml_program*>(err, nullptr, [&] {
    std::vector<ast::ExprNodePtr> in, out;
    for (size_t i = 0; i < ninputs; ++i) {
      if (shapes && shapes[i] && inputs[i]->node->kind == ExprNode::Input) {
        // explicit input shapes override the placeholders' (used to fix dynamic dimensions)
        inputs[i]->node->shape = shapes[i]->shape;
        inputs[i]->node->shape.strides.clear();
      }
      in.push_back(inputs[i]->node);
    }
    for (size_t i = 0; i < noutputs; ++i) out.push_back(outputs[i]->node);
    return new plaidml_program{tile::buildProgram(name ? name : "", in, out)};
  });
}

// ---------------------------------------------------------------------------------------
// exec
// ---------------------------------------------------------------------------------------

void plaidml_exec_init(plaidml_error* err) {
  static std::once_flag once;
  ffi_wrap_void(err, [&] { std::call_once(once, [] { rt::initRuntimes(); }); });
}

plaidml_strings* plaidml_devices_get(plaidml_error* err) {
  return ffi_wrap<plaidml_strings*>(err, nullptr, [&] {
    rt::initRuntimes();
    return makeStrings(rt::listDevices());
  });
}

plaidml_executable* plaidml_jit(plaidml_error* err, plaidml_program* program, const char* device) {
  return ffi_wrap<plaidml_executable*>(err, nullptr, [&] {
    rt::initRuntimes();
    std::string id = device ? device : "";
    if (id.empty()) id = util::Settings::Instance()->get("PLAIDML_DEVICE");
    if (id.empty()) id = "hip.0";
    if (!program->program->compiled) compileProgram(program->program.get(), "", false);
    auto dev = rt::getDevice(id);
    auto* exec = new plaidml_executable{};
    exec->program = program->program;
    exec->exec = dev->compile(program->program);
    return exec;
  });
}

void plaidml_executable_free(plaidml_error* err, plaidml_executable* exec) { ffi_wrap_void(err, [&] { delete exec; }); }

double plaidml_executable_run(plaidml_error* err, plaidml_executable* exec, size_t ninputs, plaidml_buffer** inputs,
                              size_t noutputs, plaidml_buffer** outputs) {
  return ffi_wrap<double>(err, 0.0, [&] {
    const auto& prog = *exec->program;
    if (prog.inputs.size() != ninputs) {
      throw std::runtime_error("Program expects " + std::to_string(prog.inputs.size()) + " inputs, but " +
                               std::to_string(ninputs) + " were specified");
    }
    if (prog.outputs.size() != noutputs) {
      throw std::runtime_error("Program expects " + std::to_string(prog.outputs.size()) + " outputs, but " +
                               std::to_string(noutputs) + " were specified");
    }
    std::vector<util::BufferPtr> in, out;
    for (size_t i = 0; i < ninputs; ++i) {
      TensorShape actual = inputs[i]->buffer->shape();
      actual.strides.clear();
      if (actual != prog.inputs[i]->shape) {
        throw std::runtime_error("Shape mismatch for input buffer #" + std::to_string(i) + ", expected '" +
                                 prog.inputs[i]->shape.str() + "' but '" + actual.str() + "' was specified");
      }
      in.push_back(inputs[i]->buffer);
    }
    for (size_t i = 0; i < noutputs; ++i) {
      TensorShape actual = outputs[i]->buffer->shape();
      actual.strides.clear();
      if (actual != prog.outputs[i]->shape) {
        throw std::runtime_error("Shape mismatch for output buffer #" + std::to_string(i) + ", expected '" +
                                 prog.outputs[i]->shape.str() + "' but '" + actual.str() + "' was specified");
      }
      out.push_back(outputs[i]->buffer);
    }
    return exec->exec->invoke(in, out);
  });
}

// Not part of the reference ABI: timing breakdown of the calling thread's most recent run, for benchmarks.
void plaidml_hip_last_run_stats(double* kernel_ms, double* h2d_ms, double* d2h_ms, size_t* launches) {
  rt::InvokeStats s = rt::lastInvokeStats();
  if (kernel_ms) *kernel_ms = s.kernel_ms;
  if (h2d_ms) *h2d_ms = s.h2d_ms;
  if (d2h_ms) *d2h_ms = s.d2h_ms;
  if (launches) *launches = s.launches;
}

// Device memory of the executable behind the calling thread's most recent run: the arena its temporaries share,
// what they would take unshared, and everything it holds on the device (arena + inputs + outputs + constants).
void plaidml_hip_last_run_memory(size_t* arena_bytes, size_t* unshared_temp_bytes, size_t* device_bytes) {
  rt::InvokeStats s = rt::lastInvokeStats();
  if (arena_bytes) *arena_bytes = s.arena_bytes;
  if (unshared_temp_bytes) *unshared_temp_bytes = s.unshared_temp_bytes;
  if (device_bytes) *device_bytes = s.device_bytes;
}

// 1 when that run replayed its launches as one recorded HIP graph, 0 when it launched them one by one.
int plaidml_hip_last_run_replayed(void) { return rt::lastInvokeStats().replayed ? 1 : 0; }
// Why not, when recording was tried and failed ("" otherwise); valid until the calling thread's next run.
const char* plaidml_hip_last_run_graph_note(void) {
  thread_local std::string note;
  note = rt::lastInvokeStats().graph_note;
  return note.c_str();
}

// Per-launch device milliseconds of that run (filled only when PLAIDML_PROFILE=1 was set during it): copies up
// to `capacity` values to `ms` and returns how many launches the run had timed.
size_t plaidml_hip_last_run_step_ms(size_t capacity, double* ms) {
  rt::InvokeStats s = rt::lastInvokeStats();
  for (size_t i = 0; i < s.step_ms.size() && i < capacity && ms; ++i) ms[i] = s.step_ms[i];
  return s.step_ms.size();
}

}  // extern "C"
