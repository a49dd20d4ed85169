// C facade over the code generator (declared in include/kcg_codegen.h).
#include "kcg_codegen.h"

#include <cstdlib>
#include <cstring>
#include <string>

#include "backend/KernelFamilies.h"

using namespace KernelCodeGen;

namespace {
void copyErr(const std::string& msg, char* err, size_t cap) {
  if (!err || cap == 0) return;
  size_t n = msg.size() < cap - 1 ? msg.size() : cap - 1;
  memcpy(err, msg.data(), n);
  err[n] = '\0';
}

char* dupString(const std::string& s) {
  char* p = (char*)malloc(s.size() + 1);
  if (p) memcpy(p, s.c_str(), s.size() + 1);
  return p;
}

void fillInfo(const hipgen::KernelLaunchInfo& in, kcg_launch_info* out) {
  memset(out, 0, sizeof *out);
  strncpy(out->name, in.name.c_str(), sizeof(out->name) - 1);
  for (int i = 0; i < 3; ++i) {
    out->grid[i] = in.grid[i];
    out->block[i] = in.block[i];
  }
  out->lds_bytes = in.ldsBytes;
  out->num_args = in.numArgs;
  out->num_scalars = in.numScalars;
  out->workspace_bytes = (uint64_t)in.workspaceBytes;
  out->flops = in.flops;
  out->bytes = in.bytes;
}
}  // namespace

extern "C" {

const char* kcg_prelude(void) { return hipgen::prelude().c_str(); }

int kcg_emit_kernel(const char* family, const char* name, const char* const* ikeys, const int64_t* ivals, int ni,
                    const char* const* fkeys, const double* fvals, int nf, const char* const* skeys,
                    const char* const* svals, int ns, char** src_out, kcg_launch_info* info, char* err,
                    size_t err_cap) {
  if (err && err_cap) err[0] = '\0';
  if (!family || !name || !src_out || !info || ni < 0 || nf < 0 || ns < 0 || (ni && (!ikeys || !ivals)) ||
      (nf && (!fkeys || !fvals)) || (ns && (!skeys || !svals))) {
    copyErr("invalid argument", err, err_cap);
    return KCG_ERR_INVALID_ARGUMENT;
  }
  *src_out = nullptr;
  try {
    hipgen::KernelSpec spec;
    spec.family = family;
    spec.name = name;
    for (int i = 0; i < ni; ++i) spec.p[ikeys[i]] = ivals[i];
    for (int i = 0; i < nf; ++i) spec.f[fkeys[i]] = fvals[i];
    for (int i = 0; i < ns; ++i) spec.s[skeys[i]] = svals[i];
    std::string src, msg;
    hipgen::KernelLaunchInfo li;
    if (!hipgen::emitKernel(spec, src, li, msg)) {
      copyErr(msg, err, err_cap);
      return KCG_ERR_INVALID_ARGUMENT;
    }
    char* out = dupString(src);
    if (!out) return KCG_ERR_OUT_OF_HOST_MEMORY;
    *src_out = out;
    fillInfo(li, info);
    return KCG_OK;
  } catch (const std::exception& e) {
    copyErr(e.what(), err, err_cap);
    return KCG_ERR_INVALID_ARGUMENT;
  }
}

void kcg_free_string(char* s) { free(s); }

}  // extern "C"

// ---------------------------------------------------------------------------
// generator facade
// ---------------------------------------------------------------------------
#include <sstream>

#include "IR/Interpreter.h"
#include "KernelCodeGen.h"

struct kcg_generator_s {
  std::unique_ptr<KernelCodeGenerator> gen;
  ComputeDAG* graph = nullptr;
  std::vector<mlir::Value> values;
  mlir::ModuleOp optimized;
  bool hasOptimized = false;
  std::string source, text, error, scratch, adaptorText, configsText;
  std::string lowering = "families";
  int64_t numPlaceholders = 0;
};

namespace {

// The builders report problems on stderr; capture that text for the caller.
struct StderrCapture {
  std::ostringstream captured;
  std::streambuf* old;
  StderrCapture() : old(std::cerr.rdbuf(captured.rdbuf())) {}
  ~StderrCapture() { std::cerr.rdbuf(old); }
  std::string str() const { return captured.str(); }
};

int addValue(kcg_generator_s* g, mlir::Value v, const StderrCapture& cap) {
  if (!v) {
    g->error = cap.str().empty() ? "operator builder failed" : cap.str();
    return -1;
  }
  g->values.push_back(v);
  return (int)g->values.size() - 1;
}

bool valid(kcg_generator_s* g, std::initializer_list<int> ids) {
  if (!g || !g->graph) {
    if (g) g->error = "no graph: call kcg_generator_create_graph first";
    return false;
  }
  for (int id : ids)
    if (id < 0 || id >= (int)g->values.size()) {
      g->error = "unknown value id " + std::to_string(id);
      return false;
    }
  return true;
}

mlir::ModuleOp pick(kcg_generator_s* g, int which) {
  if (which == 1 && g->hasOptimized) return g->optimized;
  return g->graph ? g->graph->module : mlir::ModuleOp();
}

template <typename Fn>
int guarded(kcg_generator_s* g, Fn&& fn) {
  try {
    return fn();
  } catch (const std::exception& e) {
    g->error = e.what();
    return -1;
  }
}

}  // namespace

extern "C" {

kcg_generator_t kcg_generator_create(const char* platform) {
  try {
    auto* g = new kcg_generator_s;
    g->gen = std::make_unique<KernelCodeGenerator>(platform ? platform : "ROCm");
    return g;
  } catch (...) {
    return nullptr;
  }
}

void kcg_generator_destroy(kcg_generator_t g) { delete g; }

int kcg_generator_create_graph(kcg_generator_t g, const char* name) {
  if (!g) return -1;
  return guarded(g, [&] {
    g->graph = &g->gen->createGraph(name ? name : "graph");
    g->values.clear();
    g->numPlaceholders = 0;
    g->hasOptimized = false;
    return 0;
  });
}

const char* kcg_generator_error(kcg_generator_t g) { return g ? g->error.c_str() : "null generator"; }

void kcg_generator_set_log_mode(kcg_generator_t g, int level) {
  if (g) g->gen->setLogMode(level == 0 ? Log::Debug : Log::Release);
}

int kcg_placeholder(kcg_generator_t g, const int64_t* shape, int rank, const char* dtype) {
  if (!valid(g, {}) || !shape || rank <= 0 || !dtype) { if (g) g->error = "invalid argument"; return -1; }
  return guarded(g, [&] {
    StderrCapture cap;
    mlir::Value v = g->graph->create<PlaceHolder>(std::vector<int64_t>(shape, shape + rank), std::string(dtype));
    // the caller's placeholders are numbered, so that a plan of the module can tell them from the buffers
    // that operator builders and fusions allocate at module level
    if (v && v.getDefiningOp())
      v.getDefiningOp()->setAttr("kcg.placeholder", g->graph->builder.getI64IntegerAttr(g->numPlaceholders++));
    return addValue(g, v, cap);
  });
}

int kcg_matmul(kcg_generator_t g, int a, int b, const char* dtype) {
  if (!valid(g, {a, b})) return -1;
  return guarded(g, [&] {
    StderrCapture cap;
    return addValue(g, g->graph->create<Matmul>(g->values[a], g->values[b], std::string(dtype ? dtype : "")), cap);
  });
}

int kcg_batched_matmul(kcg_generator_t g, int a, int layout_a, int b, int layout_b, const char* dtype) {
  if (!valid(g, {a, b})) return -1;
  return guarded(g, [&] {
    StderrCapture cap;
    return addValue(g, g->graph->create<BatchedMatmul>(g->values[a], layout_a ? Layout::colMajor : Layout::rowMajor, g->values[b],
                                                       layout_b ? Layout::colMajor : Layout::rowMajor, std::string(dtype ? dtype : "")), cap);
  });
}

int kcg_matmul_scaled(kcg_generator_t g, int a, int b, int scale_a, int scale_b, const char* dtype) {
  if (!valid(g, {a, b, scale_a, scale_b})) return -1;
  return guarded(g, [&] {
    StderrCapture cap;
    return addValue(g, g->graph->create<Matmul>(g->values[a], g->values[b], g->values[scale_a], g->values[scale_b],
                                                std::string(dtype ? dtype : "")), cap);
  });
}

int kcg_batched_matmul_scaled(kcg_generator_t g, int a, int layout_a, int b, int layout_b, int scale_a, int scale_b, const char* dtype) {
  if (!valid(g, {a, b, scale_a, scale_b})) return -1;
  return guarded(g, [&] {
    StderrCapture cap;
    return addValue(g, g->graph->create<BatchedMatmul>(g->values[a], layout_a ? Layout::colMajor : Layout::rowMajor, g->values[b],
                                                       layout_b ? Layout::colMajor : Layout::rowMajor, g->values[scale_a],
                                                       g->values[scale_b], std::string(dtype ? dtype : "")), cap);
  });
}

int kcg_softmax(kcg_generator_t g, int x, int axis, int memory_space, const char* dtype) {
  if (!valid(g, {x})) return -1;
  return guarded(g, [&] {
    StderrCapture cap;
    return addValue(g, g->graph->create<Softmax>(g->values[x], axis, static_cast<MemorySpace>(memory_space), std::string(dtype ? dtype : "")), cap);
  });
}

int kcg_relu(kcg_generator_t g, int x, int memory_space, const char* dtype) {
  if (!valid(g, {x})) return -1;
  return guarded(g, [&] {
    StderrCapture cap;
    return addValue(g, g->graph->create<Relu>(g->values[x], static_cast<MemorySpace>(memory_space), std::string(dtype ? dtype : "")), cap);
  });
}

int kcg_elementwise(kcg_generator_t g, int x, const char* operation, int memory_space, const char* dtype) {
  if (!valid(g, {x}) || !operation) return -1;
  return guarded(g, [&] {
    StderrCapture cap;
    return addValue(g, g->graph->create<ElementWise>(g->values[x], std::string(operation), static_cast<MemorySpace>(memory_space),
                                                     std::string(dtype ? dtype : "")), cap);
  });
}

int kcg_binary(kcg_generator_t g, int a, int b, const char* operation, int memory_space, const char* dtype) {
  if (!valid(g, {a, b}) || !operation) return -1;
  return guarded(g, [&] {
    StderrCapture cap;
    return addValue(g, g->graph->create<Binary>(g->values[a], g->values[b], std::string(operation),
                                                static_cast<MemorySpace>(memory_space), std::string(dtype ? dtype : "")), cap);
  });
}

int kcg_gather(kcg_generator_t g, int x, int indices, int64_t axis, const char* dtype) {
  if (!valid(g, {x, indices})) return -1;
  return guarded(g, [&] {
    StderrCapture cap;
    return addValue(g, g->graph->create<Gather>(g->values[x], g->values[indices], axis, std::string(dtype ? dtype : "")), cap);
  });
}

int kcg_layernorm(kcg_generator_t g, int x, int scale, int bias, int64_t axis, float eps, int memory_space, const char* dtype) {
  if (!valid(g, {x, scale, bias})) return -1;
  return guarded(g, [&] {
    StderrCapture cap;
    return addValue(g, g->graph->create<LayerNorm>(g->values[x], g->values[scale], g->values[bias], axis, eps,
                                                   static_cast<MemorySpace>(memory_space), std::string(dtype ? dtype : "")), cap);
  });
}

int kcg_add_optimizer(kcg_generator_t g, const char* name) {
  if (!g || !name) return -1;
  std::string n = name;
  std::unique_ptr<Optimizer> opt;
  if (n == "Matmul") opt = std::make_unique<MatmulOptimizer>();
  else if (n == "BatchMatmul") opt = std::make_unique<BatchMatmulOptimizer>();
  else if (n == "ElementWise") opt = std::make_unique<ElementWiseOptimizer>();
  else if (n == "LayerNorm") opt = std::make_unique<LayerNormOptimizer>();
  else if (n == "FMHA") opt = std::make_unique<FMHAOptimizer>();
  else if (n == "Binary") opt = std::make_unique<BinaryOptimizer>();
  else if (n == "Gather") opt = std::make_unique<GatherOptimizer>();
  else if (n == "Softmax") opt = std::make_unique<SoftmaxOptimizer>();
  else { g->error = "unknown optimizer '" + n + "'"; return -1; }
  g->gen->opts.push_back(std::move(opt));
  return 0;
}

int kcg_set_configs(kcg_generator_t g, const char* optimizer, int count, const int* sizes, const char* const* keys, const int* values) {
  if (!g || !optimizer || count < 0 || (count && (!sizes || !keys || !values))) return -1;
  KernelCodeGenerator::ConfigList list;
  int pos = 0;
  for (int i = 0; i < count; ++i) {
    std::map<std::string, int> m;
    for (int j = 0; j < sizes[i]; ++j, ++pos) m[keys[pos]] = values[pos];
    list.push_back(m);
  }
  if (!g->gen->setConfigs(optimizer, list)) { g->error = std::string("unknown optimizer '") + optimizer + "'"; return -1; }
  return 0;
}

const char* kcg_get_configs(kcg_generator_t g, const char* optimizer) {
  if (!g || !optimizer) return nullptr;
  const KernelCodeGenerator::ConfigList* list = g->gen->getConfigs(optimizer);
  if (!list) { g->error = std::string("unknown optimizer '") + optimizer + "'"; return nullptr; }
  std::ostringstream os;
  for (auto& candidate : *list) {
    bool first = true;
    for (auto& kv : candidate) {
      os << (first ? "" : " ") << kv.first << "=" << kv.second;
      first = false;
    }
    os << "\n";
  }
  g->configsText = os.str();
  return g->configsText.c_str();
}

int kcg_optimize(kcg_generator_t g) {
  if (!valid(g, {})) return -1;
  return guarded(g, [&] {
    StderrCapture cap;
    g->optimized = g->gen->optimize(*g->graph);
    g->hasOptimized = true;
    g->scratch = cap.str();  // notes about functions that were not scheduled
    return 0;
  });
}

const char* kcg_codegen(kcg_generator_t g) {
  if (!valid(g, {})) return nullptr;
  if (!g->hasOptimized) { g->error = "call kcg_optimize first"; return nullptr; }
  try {
    StderrCapture cap;
    g->gen->setLowering(g->lowering);
    g->source = g->gen->codegen(g->optimized);
    if (!g->gen->error().empty()) { g->error = g->gen->error(); return nullptr; }
    return g->source.c_str();
  } catch (const std::exception& e) {
    g->error = e.what();
    return nullptr;
  }
}

int kcg_set_lowering(kcg_generator_t g, const char* mode) {
  if (!valid(g, {}) || !mode) return 1;
  const std::string m = mode;
  if (m != "families" && m != "schedule" && m != "families-only") {
    g->error = "lowering is \"families\", \"families-only\" or \"schedule\"";
    return 1;
  }
  g->lowering = m;
  g->gen->setLowering(m);      // also what a later kcg_optimize rates its candidates with
  return 0;
}

const char* kcg_adaptor(kcg_generator_t g, const char* kernel_file) {
  if (!valid(g, {}) || !kernel_file) return nullptr;
  try {
    g->adaptorText = g->gen->adaptor(kernel_file);
    return g->adaptorText.c_str();
  } catch (const std::exception& e) {
    g->error = e.what();
    return nullptr;
  }
}

int kcg_num_kernels(kcg_generator_t g) { return g ? (int)g->gen->launchInfos().size() : -1; }

int kcg_kernel_info(kcg_generator_t g, int index, kcg_launch_info* info) {
  if (!g || !info || index < 0 || index >= (int)g->gen->launchInfos().size()) return -1;
  fillInfo(g->gen->launchInfos()[index], info);
  return 0;
}

const char* kcg_kernel_function(kcg_generator_t g, int index) {
  if (!g || index < 0 || index >= (int)g->gen->launchInfos().size()) return nullptr;
  return g->gen->launchInfos()[index].function.c_str();
}

const char* kcg_kernel_lowering(kcg_generator_t g, int index) {
  if (!g || index < 0 || index >= (int)g->gen->launchInfos().size()) return nullptr;
  return g->gen->launchInfos()[index].lowering.c_str();
}

int kcg_kernel_arg_bytes(kcg_generator_t g, int index, int64_t* bytes, int cap) {
  if (!g || !bytes || index < 0 || index >= (int)g->gen->launchInfos().size()) return -1;
  auto& v = g->gen->launchInfos()[index].argBytes;
  for (int i = 0; i < (int)v.size() && i < cap; ++i) bytes[i] = v[i];
  return (int)v.size();
}

int kcg_kernel_arg_types(kcg_generator_t g, int index, int* types, int cap) {
  if (!g || !types || index < 0 || index >= (int)g->gen->launchInfos().size()) return -1;
  auto& v = g->gen->launchInfos()[index].argTypes;
  for (int i = 0; i < (int)v.size() && i < cap; ++i) types[i] = v[i];
  return (int)v.size();
}

int kcg_num_skipped(kcg_generator_t g) { return g ? (int)g->gen->skippedFunctions().size() : -1; }

const char* kcg_skipped_function(kcg_generator_t g, int index) {
  if (!g || index < 0 || index >= (int)g->gen->skippedFunctions().size()) return nullptr;
  return g->gen->skippedFunctions()[index].c_str();
}

int kcg_num_evaluations(kcg_generator_t g) { return g ? (int)g->gen->evaluations().size() : -1; }

int kcg_evaluation(kcg_generator_t g, int index, const char** optimizer, int* config_index, int* kernels,
                   float* latency_ms, int* kept, const char** note) {
  if (!g || index < 0 || index >= (int)g->gen->evaluations().size()) return -1;
  auto& e = g->gen->evaluations()[index];
  if (optimizer) *optimizer = e.optimizer.c_str();
  if (config_index) *config_index = e.configIndex;
  if (kernels) *kernels = e.kernels;
  if (latency_ms) *latency_ms = e.latencyMs;
  if (kept) *kept = e.kept;
  if (note) *note = e.note.c_str();
  return 0;
}

int kcg_evaluation_config(kcg_generator_t g, int index, const char* key) {
  if (!g || !key || index < 0 || index >= (int)g->gen->evaluations().size()) return -1;
  auto& c = g->gen->evaluations()[index].config;
  auto it = c.find(key);
  return it == c.end() ? -1 : it->second;
}

float kcg_evaluate(kcg_generator_t g) {
  if (!valid(g, {})) return -1.0f;
  if (!g->hasOptimized) { g->error = "call kcg_optimize first"; return -1.0f; }
  try {
    std::string note;
    int kernels = 0;
    const float ms = g->gen->evaluate(g->optimized, &kernels, &note);
    if (ms == FLT_MAX) { g->error = note; return -1.0f; }
    return ms;
  } catch (const std::exception& e) {
    g->error = e.what();
    return -1.0f;
  }
}

const char* kcg_module_plan(kcg_generator_t g, int which) {
  if (!valid(g, {})) return nullptr;
  try {
    mlir::ModuleOp module = pick(g, which);
    std::vector<mlir::Value> known;           // value of buffer id
    auto idOf = [&](mlir::Value v) {
      for (size_t i = 0; i < known.size(); ++i)
        if (known[i] == v) return (int)i;
      return -1;
    };
    auto describe = [&](std::ostringstream& os, mlir::Value v, int64_t placeholder) {
      auto type = v.getType().cast<mlir::MemRefType>();
      os << "{\"id\": " << known.size() << ", \"shape\": [";
      for (int64_t i = 0; i < type.getRank(); ++i) os << (i ? ", " : "") << type.getShape()[i];
      const unsigned bits = type.getElementType().isIndex() ? 64 : type.getElementType().getIntOrFloatBitWidth();
      os << "], \"dtype\": \"" << toStr(type.getElementType()) << "\", \"bytes\": " << type.getNumElements() * ((bits + 7) / 8)
         << ", \"input\": " << placeholder << "}";
      known.push_back(v);
    };
    std::ostringstream buffers, calls;
    bool firstBuffer = true, firstCall = true;
    for (auto& op : module.getBody()->getOperations()) {
      if (auto alloc = mlir::dyn_cast<mlir::memref::AllocOp>(op)) {
        buffers << (firstBuffer ? "" : ", ");
        mlir::Attribute mark = alloc->getAttr("kcg.placeholder");
        describe(buffers, alloc.getResult(), mark ? mark.i : -1);
        firstBuffer = false;
      } else if (auto call = mlir::dyn_cast<mlir::func::CallOp>(op)) {
        calls << (firstCall ? "" : ", ") << "{\"callee\": \"" << call.getCallee() << "\", \"operands\": [";
        firstCall = false;
        bool firstOperand = true;
        for (mlir::Value v : call.getOperands()) {
          calls << (firstOperand ? "" : ", ") << idOf(v);
          firstOperand = false;
        }
        // in place when the callee returns one of its arguments
        int result = -1;
        bool scheduled = false;
        module.walk<mlir::WalkOrder::PreOrder>([&](mlir::func::FuncOp f) {
          if (f.getSymName() != call.getCallee() || f.empty()) return;
          mlir::Attribute state = f->getAttr("func.state");
          scheduled = state && state.s == "gpu";
          mlir::Operation& ret = f.front().back();
          if (ret.getNumOperands() && ret.getOperand(0).isa<mlir::BlockArgument>())
            result = idOf(call.getOperand(ret.getOperand(0).cast<mlir::BlockArgument>().getArgNumber()));
        });
        if (call->getNumResults()) {
          if (result < 0) {
            result = (int)known.size();
            buffers << (firstBuffer ? "" : ", ");
            describe(buffers, call.getResult(0), -1);
            firstBuffer = false;
          } else {
            // later calls name the call's result value: it is the operand's buffer
            known.push_back(call.getResult(0));
            buffers << (firstBuffer ? "" : ", ") << "{\"id\": " << known.size() - 1 << ", \"alias\": " << result << "}";
            firstBuffer = false;
          }
        }
        calls << "], \"result\": " << result << ", \"scheduled\": " << (scheduled ? "true" : "false") << "}";
      }
    }
    g->text = "{\"buffers\": [" + buffers.str() + "], \"calls\": [" + calls.str() + "]}";
    return g->text.c_str();
  } catch (const std::exception& e) {
    g->error = e.what();
    return nullptr;
  }
}

const char* kcg_dump(kcg_generator_t g, int which) {
  if (!valid(g, {})) return nullptr;
  std::ostringstream os;
  pick(g, which)->print(os);
  g->text = os.str();
  return g->text.c_str();
}

int kcg_verify(kcg_generator_t g, int which) {
  if (!valid(g, {})) return -1;
  std::string msg;
  if (mlir::failed(mlir::verify(pick(g, which), &msg))) { g->error = msg; return 1; }
  return 0;
}

const char* kcg_function_state(kcg_generator_t g, int which, const char* function) {
  if (!valid(g, {}) || !function) return "";
  mlir::ModuleOp m = pick(g, which);
  auto f = Analyzer::getTargetFunction(m, function);
  if (!f) return "";
  g->scratch = f->getAttr("func.state").s;
  return g->scratch.c_str();
}

int64_t kcg_interpret(kcg_generator_t g, int which, const float* const* inputs, const int64_t* sizes, int num_inputs,
                      float* out, int64_t out_cap) {
  if (!valid(g, {}) || num_inputs < 0 || (num_inputs && (!inputs || !sizes)) || !out) return -1;
  try {
    mlir::ModuleOp m = pick(g, which);
    std::vector<HostTensor> ph;
    int idx = 0;
    for (auto& op : m.getBody()->getOperations()) {
      if (idx >= num_inputs) break;
      if (op.getKind() != mlir::OpKind::Alloc || op.hasAttr("kcg.result")) continue;
      auto mt = op.getResult(0).getType().cast<mlir::MemRefType>();
      HostTensor t{mt.getShape().vec(), mt.getElementType(), {}};
      if (sizes[idx] != t.numElements()) { g->error = "input " + std::to_string(idx) + " has the wrong number of elements"; return -1; }
      t.data.resize((size_t)sizes[idx]);
      for (int64_t i = 0; i < sizes[idx]; ++i) t.data[(size_t)i] = roundToType((double)inputs[idx][i], mt.getElementType());
      ph.push_back(std::move(t));
      ++idx;
    }
    Interpreter interp(m);
    auto results = interp.runGraph(ph);
    if (results.empty()) { g->error = "the graph has no calls"; return -1; }
    if (interp.sharedHazards) {
      g->error = "the schedule races on the GPU (" + std::to_string(interp.sharedHazards) + " accesses): " + interp.firstHazard;
      return -1;
    }
    auto& last = results.back();
    const int64_t n = std::min<int64_t>(out_cap, (int64_t)last.data.size());
    for (int64_t i = 0; i < n; ++i) out[i] = (float)last.data[(size_t)i];
    return n;
  } catch (const std::exception& e) {
    g->error = e.what();
    return -1;
  }
}

int kcg_fmha_map_evaluate(const char* name, const int64_t* inputs, int num_inputs, int64_t* out, int out_cap) {
  if (!name || num_inputs < 0 || (num_inputs > 0 && !inputs) || out_cap < 0 || (out_cap > 0 && !out)) return -1;
  static const char* const tiled[] = {"loadTileQ", "loadTileK", "storeTileQ", "storeTileK", "loadFragQ", "loadFragK", "brIdxS",
                                      "bcIdxS", "storeTileP", "readTileS", "loadFactor", "loadTileV", "storeTileV", "loadFragP",
                                      "loadFragV", "brIdxO", "storeTileO"};
  static const char* const rows[] = {"loadTileQ", "storeTileO", "loadTileK", "loadTileV", "score"};
  bool known = false;
  if (KernelCodeGen::FMHAOptimizer::tiledConfig()) { for (const char* n : tiled) known |= !strcmp(n, name); }
  else { for (const char* n : rows) known |= !strcmp(n, name); }
  if (!known) return -1;
  mlir::OpBuilder builder;
  KernelCodeGen::FMHAOptimizer opt;
  mlir::AffineMap map = opt.getAffineMap(name, builder);
  if ((int)map.getNumDims() != num_inputs) return -2;
  std::vector<int64_t> res = map.evaluate(std::vector<int64_t>(inputs, inputs + num_inputs));
  if ((int)res.size() > out_cap) return -3;
  for (size_t i = 0; i < res.size(); ++i) out[i] = res[i];
  return (int)res.size();
}

}  // extern "C"
