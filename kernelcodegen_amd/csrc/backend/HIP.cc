// HIPGen: scheduled functions -> gfx950 kernels (declared in include/Backend/HIP.h).
#include "Backend/HIP.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <sstream>

#include "Optimizer/Analyzer.h"
#include "Optimizer/Optimizer.h"
#include "backend/KernelFamilies.h"
#include "backend/ScheduleEmitter.h"
#include "kcg_hip.h"
#include "log.h"

namespace KernelCodeGen {

using namespace mlir;

namespace {

struct Lowering {
  func::FuncOp f;
  std::string op;
  std::vector<AffineParallelOp> levels;  // [grid, block]
  std::string error;
  // the refusal in `error` says that the family has no form for this operator instance (an element type, a kind of
  // broadcast), as opposed to a configuration it cannot build (tile sizes, launch shape)
  bool noForm = false;
  // what the host adaptor checks the kernel against (KernelLaunchInfo::check and friends)
  std::string check;
  std::vector<int64_t> checkInts;
  std::vector<double> checkFloats;
  double fillLo = -1.0, fillHi = 1.0;

  int64_t cfg(const std::string& key, int64_t dflt = 0) const {
    Attribute a = f->getAttr("kcg.cfg." + key);
    return a ? a.i : dflt;
  }
};

int64_t bytesOf(Type memref) {
  auto mt = memref.cast<MemRefType>();
  return mt.getNumElements() * ((mt.getElementType().getIntOrFloatBitWidth() + 7) / 8);
}

// Element type -> KCG_DT_* code of kcg_hip.h (index values are 64-bit on the device, i1 results one byte).
int dtypeCode(Type t) {
  if (t.isF32()) return KCG_DT_F32;
  if (t.isBF16()) return KCG_DT_BF16;
  if (t.isa<Float8E4M3FNType>()) return KCG_DT_F8E4M3;
  if (t.isF16()) return KCG_DT_F16;
  if (t.isF64()) return KCG_DT_F64;
  if (t.isIndex()) return KCG_DT_I64;
  switch (t.getIntOrFloatBitWidth()) {
    case 64: return KCG_DT_I64;
    case 32: return KCG_DT_I32;
    case 16: return KCG_DT_I16;
    default: return KCG_DT_I8;
  }
}
int dtypeOf(Type memref) { return dtypeCode(memref.cast<MemRefType>().getElementType()); }

std::string gemmFamily(Type element, std::string& err) {
  if (element.isF32()) return "gemm_f32";
  if (element.isF64()) return "gemm_f64";
  if (element.isBF16() || element.isF16()) return "gemm_bf16";     // one family for both 16-bit float types
  if (element.isa<Float8E4M3FNType>()) return "gemm_fp8";
  err = "GEMM operand type is not f64, f32, f16, bf16 or f8E4M3FN";
  return "";
}

// Arrangement of `waves` wavefronts over a BM x BN tile: as square as the tile
// allows, every wavefront owning whole 32 x 32 MFMA tiles.
bool waveGrid(int64_t bm, int64_t bn, int64_t waves, int64_t& wm, int64_t& wn) {
  bool found = false;
  int64_t bestSkew = 0;
  for (int64_t a = 1; a <= waves; ++a) {
    if (waves % a) continue;
    const int64_t b = waves / a;
    if (bm % (32 * a) || bn % (32 * b)) continue;
    const int64_t skew = std::llabs((bm / a) - (bn / b));
    if (!found || skew < bestSkew) { found = true; bestSkew = skew; wm = a; wn = b; }
  }
  return found;
}

bool lowerGemm(Lowering& L, hipgen::KernelSpec& spec) {
  auto args = L.f.getArguments();
  auto typeA = args[0].getType().cast<MemRefType>(), typeB = args[1].getType().cast<MemRefType>();
  auto typeC = L.f.getFunctionType().getResult(0).cast<MemRefType>();
  spec.family = gemmFamily(typeA.getElementType(), L.error);
  if (spec.family.empty()) { L.noForm = true; return false; }
  if (typeA.getElementType() != typeB.getElementType()) { L.noForm = true; L.error = "GEMM operands differ in element type"; return false; }
  const int64_t rank = typeA.getRank();
  bool ta = false, tb = false;
  if (L.op == "BatchMatmul") {
    BatchMatmulDescriptor d;
    if (!identifyBatchMatmul(L.f.getSymName(), d)) { L.error = "function name is not a BatchMatmul descriptor"; return false; }
    ta = d.transA; tb = d.transB;
  }
  int64_t batch = 1;
  for (int64_t i = 0; i + 2 < rank; ++i) batch *= typeA.getShape()[i];
  const int64_t m = typeC.getShape()[rank - 2], n = typeC.getShape()[rank - 1];
  const int64_t k = ta ? typeA.getShape()[rank - 2] : typeA.getShape()[rank - 1];
  // tile sizes: from the schedule.  Grid extents give M/BM and N/BN, the block extent the thread count.
  auto grid = L.levels[0].getConstantUpperBounds();
  auto block = L.levels[1].getConstantUpperBounds();
  const size_t gd = grid.size();
  // the recorded tile sizes, else what the grid says; an extent that is no multiple of the tile has one more
  // workgroup for the rest
  const int64_t bm = L.cfg("BLOCK_SIZE_M", m / grid[gd - 2]), bn = L.cfg("BLOCK_SIZE_N", n / grid[gd - 1]);
  if (bm <= 0 || bn <= 0 || (m + bm - 1) / bm != grid[gd - 2] || (n + bn - 1) / bn != grid[gd - 1]) {
    L.error = "grid extents disagree with the recorded tile sizes";
    return false;
  }
  int64_t threads = 1;
  for (auto e : block) threads *= e;
  if (threads % 64) { L.error = "workgroup size is not a multiple of the 64-wide wavefront"; return false; }
  int64_t wm = 1, wn = 1;
  if (!waveGrid(bm, bn, threads / 64, wm, wn)) { L.error = "tile does not split into 32x32 MFMA tiles per wavefront"; return false; }
  int64_t bk = L.cfg("BLOCK_SIZE_K", 16);
  spec.p = {{"M", m}, {"N", n}, {"K", k}, {"BATCH", batch}, {"TA", ta}, {"TB", tb}, {"BM", bm}, {"BN", bn}, {"BK", bk},
            {"WM", wm}, {"WN", wn}, {"GROUP_M", L.cfg("GROUP_SIZE_M", 8)}};
  if (spec.family == "gemm_f64" && !typeC.getElementType().isF64()) { L.noForm = true; L.error = "an f64 GEMM returns f64"; return false; }
  if (spec.family != "gemm_f32" && spec.family != "gemm_f64") spec.p["OUT_BF16"] = typeC.getElementType().getIntOrFloatBitWidth() == 16;
  if (typeA.getElementType().isF16()) {
    spec.p["F16"] = 1;
    if (spec.p["OUT_BF16"] && !typeC.getElementType().isF16()) { L.noForm = true; L.error = "a 16-bit GEMM result must have the operands' type"; return false; }
  } else if (spec.family == "gemm_bf16" && spec.p["OUT_BF16"] && !typeC.getElementType().isBF16()) {
    L.noForm = true; L.error = "a 16-bit GEMM result must have the operands' type";
    return false;
  }
  if (L.f->hasAttr("kcg.fused_relu")) spec.p["RELU"] = 1;
  if (Attribute scales = L.f->getAttr("kcg.scales")) {
    // per-tensor scales as graph values (one fp32 each in device memory): the fp8 family reads them through pointers
    // that stand where the function has them, (A, B, scaleA, scaleB) -> C or (A, B, C, scaleA, scaleB)
    if (spec.family != "gemm_fp8") { L.noForm = true; L.error = "only the fp8 GEMM family applies per-tensor scales"; return false; }
    spec.p["SCALE_PTR"] = scales.i == 2 ? 2 : 1;
    return true;        // no host-side check routine knows where the scales lie: the adaptor times this kernel only
  }
  L.check = "gemm";
  L.checkInts = {m, n, k, batch, ta, tb, spec.get("RELU", 0)};
  return true;
}

bool lowerElementWise(Lowering& L, hipgen::KernelSpec& spec) {
  auto in = L.f.getArgument(0).getType().cast<MemRefType>();
  auto out = L.f.getFunctionType().getResult(0).cast<MemRefType>();
  const std::string name = L.f.getSymName();
  const std::string opName = name.substr(0, name.find("_Elementwise"));
  auto ctype = [&](Type t) -> std::string {
    if (t.isF32()) return "float";
    if (t.isF16()) return "_Float16";
    if (t.isBF16()) return "__bf16";
    if (t.isa<IntegerType>() && t.getIntOrFloatBitWidth() == 32) return "int";
    return "";
  };
  spec.family = "elementwise";
  spec.s["OP"] = opName;
  spec.s["IN_T"] = ctype(in.getElementType());
  spec.s["OUT_T"] = ctype(out.getElementType());
  if (spec.s["IN_T"].empty() || spec.s["OUT_T"].empty()) { L.noForm = true; L.error = "elementwise element type is not f32 / f16 / i32"; return false; }
  // in place when the function returns its argument
  Operation& ret = L.f.front().back();
  const bool inplace = ret.getOperand(0) == Value(L.f.getArgument(0));
  spec.p = {{"N", in.getNumElements()}, {"INPLACE", inplace}};
  if (in.getNumElements() % 4 == 0) spec.p["VW"] = L.cfg("VECTORIZE_WIDTH", 4) == 4 ? 4 : 1;
  static const char* names[] = {"Tanh", "Sqrt", "Log", "Relu", "Gelu", "Cast"};
  int64_t code = -1;
  for (int i = 0; i < 6; ++i)
    if (opName == names[i]) code = i;
  L.check = "elementwise";
  L.checkInts = {in.getNumElements(), code};
  if (opName == "Sqrt" || opName == "Log") { L.fillLo = 0.05; L.fillHi = 9.0; }
  if (opName == "Cast") { L.fillLo = -1000.0; L.fillHi = 1000.0; }
  return true;
}

bool lowerLayerNorm(Lowering& L, hipgen::KernelSpec& spec) {
  auto in = L.f.getArgument(0).getType().cast<MemRefType>();
  auto scale = L.f.getArgument(1).getType().cast<MemRefType>();
  auto bias = L.f.getArgument(2).getType().cast<MemRefType>();
  const int64_t half = in.getElementType().isF16() ? 1 : (in.getElementType().isBF16() ? 2 : 0);      // 16-bit storage, fp32 arithmetic
  if (!in.getElementType().isF32() && !half) { L.noForm = true; L.error = "LayerNorm element type is neither f32, f16 nor bf16"; return false; }
  if (scale.getElementType() != in.getElementType() || bias.getElementType() != in.getElementType()) {
    L.noForm = true; L.error = "LayerNorm scale and bias must have the input's element type";
    return false;
  }
  const int64_t rows = L.levels[0].getConstantUpperBounds()[0];
  const int64_t n = in.getNumElements() / rows;
  // epsilon: the float constant added to the variance right before the sqrt
  double eps = 1e-5;
  bool found = false;
  L.f->walk([&](Operation* o) {
    if (o->getKind() != OpKind::Sqrt) return;
    Operation* add = o->getOperand(0).getDefiningOp();
    if (!add || add->getKind() != OpKind::AddF) return;
    for (Value v : add->getOperands())
      if (auto c = v.getDefiningOp<arith::ConstantOp>()) { eps = c.getValue().f; found = true; }
  }, WalkOrder::PreOrder);
  if (!found) { L.error = "LayerNorm epsilon constant not found"; return false; }
  spec.family = "layernorm";
  spec.p = {{"ROWS", rows}, {"N", n}, {"NG", scale.getNumElements()}, {"NB", bias.getNumElements()},
            {"GELU", L.f->hasAttr("kcg.fused_gelu")}, {"F16", half}};
  // broadcast with inner size-1 dims is not a plain "index mod length" pattern
  auto plain = [&](MemRefType t) {
    auto s = t.getShape();
    for (size_t i = 0; i < s.size(); ++i)
      if (s[s.size() - 1 - i] != in.getShape()[in.getRank() - 1 - i]) return false;
    return true;
  };
  if (!plain(scale) || !plain(bias)) { L.noForm = true; L.error = "LayerNorm scale/bias broadcast over size-1 dims is not supported by the kernel"; return false; }
  spec.f["EPS"] = eps;
  const int64_t tpr = L.levels[1].getConstantUpperBounds()[0];
  if (tpr >= 64 && (tpr & (tpr - 1)) == 0 && tpr <= 1024) spec.p["TPR"] = tpr;
  if (L.cfg("VECTORIZE_WIDTH", 4) == 1) spec.p["VW"] = 1;
  L.check = "layernorm";
  L.checkInts = {rows, n, scale.getNumElements(), bias.getNumElements(), spec.get("GELU", 0)};
  L.checkFloats = {(double)(float)eps};
  return true;
}

bool lowerBinary(Lowering& L, hipgen::KernelSpec& spec) {
  auto a = L.f.getArgument(0).getType().cast<MemRefType>(), b = L.f.getArgument(1).getType().cast<MemRefType>();
  auto out = L.f.getFunctionType().getResult(0).cast<MemRefType>();
  const std::string name = L.f.getSymName();
  const std::string opName = name.substr(0, name.find("_Binary"));
  const bool compare = opName == "Equal" || opName == "Greater";
  const bool half = a.getElementType().isF16();
  const bool outOk = compare ? (out.getElementType().isa<IntegerType>() && out.getElementType().getIntOrFloatBitWidth() == 1)
                             : out.getElementType() == a.getElementType();
  if ((!a.getElementType().isF32() && !half) || b.getElementType() != a.getElementType() || !outOk) {
    L.noForm = true; L.error = "the binary kernel takes two fp32 or two f16 operands (and gives their type, or i1 for a comparison)";
    return false;
  }
  spec.family = "binary";
  spec.p["F16"] = half;
  spec.s["OP"] = opName;
  // row-major element strides of an operand seen through the result's dimensions: 0 where the
  // operand has extent 1 or no dimension at all
  auto strides = [&](MemRefType t) {
    const int64_t rank = out.getRank(), r = t.getRank();
    std::vector<int64_t> s((size_t)rank, 0);
    int64_t run = 1;
    for (int64_t i = 0; i < r; ++i) {
      const int64_t extent = t.getShape()[r - 1 - i];
      if (extent != 1) s[(size_t)(rank - 1 - i)] = run;
      run *= extent;
    }
    return s;
  };
  auto join = [](const std::vector<int64_t>& v) {
    std::string text;
    for (size_t i = 0; i < v.size(); ++i) text += (i ? "," : "") + std::to_string(v[i]);
    return text;
  };
  std::vector<int64_t> dims(out.getShape().begin(), out.getShape().end());
  spec.s["DIMS"] = join(dims);
  spec.s["SA"] = join(strides(a));
  spec.s["SB"] = join(strides(b));
  Operation& ret = L.f.front().back();
  spec.p["INPLACE"] = ret.getOperand(0).isa<BlockArgument>();
  if (L.cfg("VECTORIZE_WIDTH", 4) == 1) spec.p["VW"] = 1;
  static const char* names[] = {"Add", "Sub", "Mul", "Div", "Pow", "Equal", "Greater"};
  int64_t code = -1;
  for (int i = 0; i < 7; ++i)
    if (opName == names[i]) code = i;
  if (dims.size() <= 6) {
    L.check = "binary";
    L.checkInts = {(int64_t)dims.size(), code};
    auto sa = strides(a), sb = strides(b);
    for (size_t d = 0; d < 6; ++d) L.checkInts.push_back(d < dims.size() ? dims[d] : 1);
    for (size_t d = 0; d < 6; ++d) L.checkInts.push_back(d < dims.size() ? sa[d] : 0);
    for (size_t d = 0; d < 6; ++d) L.checkInts.push_back(d < dims.size() ? sb[d] : 0);
    L.fillLo = 0.5; L.fillHi = 2.0;      // keeps Div and Pow away from poles
  }
  return true;
}

bool lowerSoftmax(Lowering& L, hipgen::KernelSpec& spec) {
  auto in = L.f.getArgument(0).getType().cast<MemRefType>();
  const int64_t half = in.getElementType().isF16() ? 1 : (in.getElementType().isBF16() ? 2 : 0);      // 16-bit storage, fp32 arithmetic
  if (!in.getElementType().isF32() && !half) { L.noForm = true; L.error = "the softmax kernel takes fp32, f16 or bf16 operands"; return false; }
  const int64_t rows = L.levels[0].getConstantUpperBounds()[0];
  const int64_t n = in.getShape().back();
  if (rows * n != in.getNumElements()) { L.error = "softmax grid extent disagrees with the operand shape"; return false; }
  Operation& ret = L.f.front().back();
  if (!ret.getOperand(0).isa<BlockArgument>()) { L.error = "softmax is expected to update its operand in place"; return false; }
  spec.family = "softmax";
  spec.p = {{"ROWS", rows}, {"N", n}, {"INPLACE", 1}, {"F16", half}};
  const int64_t tpr = L.levels[1].getConstantUpperBounds()[0];
  if (tpr >= 64 && (tpr & (tpr - 1)) == 0 && tpr <= 1024) spec.p["TPR"] = tpr;
  if (L.cfg("VECTORIZE_WIDTH", 4) == 1) spec.p["VW"] = 1;
  L.check = "softmax";
  L.checkInts = {rows, n};
  L.fillLo = -4.0; L.fillHi = 4.0;
  return true;
}

bool lowerGather(Lowering& L, hipgen::KernelSpec& spec) {
  auto in = L.f.getArgument(0).getType().cast<MemRefType>(), idx = L.f.getArgument(1).getType().cast<MemRefType>();
  auto out = L.f.getFunctionType().getResult(0).cast<MemRefType>();
  if (!idx.getElementType().isIndex()) { L.error = "gather indices are not of index type"; return false; }
  const int64_t axis = L.cfg("AXIS", -1);
  if (axis < 0 || axis >= in.getRank()) { L.error = "gather axis is not recorded on the function"; return false; }
  int64_t outer = 1, inner = 1;
  for (int64_t d = 0; d < axis; ++d) outer *= in.getShape()[d];
  for (int64_t d = axis + 1; d < in.getRank(); ++d) inner *= in.getShape()[d];
  const int64_t nidx = idx.getNumElements();
  if (out.getNumElements() != outer * nidx * inner) { L.error = "gather result shape disagrees with input, indices and axis"; return false; }
  spec.family = "gather";
  spec.p = {{"OUTER", outer}, {"AXIS", in.getShape()[axis]}, {"NIDX", nidx}, {"INNER", inner},
            {"ESIZE", (int64_t)bytesOf(MemRefType::get({1}, in.getElementType()))}};
  L.check = "gather";
  L.checkInts = {outer, in.getShape()[axis], nidx, inner * spec.p["ESIZE"]};
  L.fillLo = 0.0; L.fillHi = (double)in.getShape()[axis];     // the index operand; the table is drawn from the same range
  return true;
}

bool lowerFMHA(Lowering& L, hipgen::KernelSpec& spec) {
  auto q = L.f.getArgument(0).getType().cast<MemRefType>();
  auto o = L.f.getArgument(3).getType().cast<MemRefType>();
  const bool half = q.getElementType().isF16(), single = q.getElementType().isF32();
  if (!q.getElementType().isBF16() && !half && !single) {
    L.noForm = true; L.error = "the fused attention kernels take f32, bf16 or f16 operands";
    return false;
  }
  if (single ? !o.getElementType().isF32() : (o.getElementType() != q.getElementType() && !o.getElementType().isF32())) {
    L.noForm = true; L.error = "the fused attention kernels return the operands' type or f32";
    return false;
  }
  auto s = q.getShape();
  if (s[3] % 32 || s[3] > 256) {
    L.noForm = true; L.error = "the fused attention kernels take head dims that are multiples of 32, up to 256";
    return false;
  }
  if (single) {
    // fp32 graphs (the reference's own attention, test/test.cc:107-147): both products on the fp32 MFMA.  The tile
    // sizes of the schedule (thread tiles of a scalar outer product) say nothing about MFMA tiles; the family chooses.
    spec.family = "fmha_f32";
    spec.p = {{"B", s[0]}, {"H", s[1]}, {"S", s[2]}, {"D", s[3]}, {"CAUSAL", L.cfg("CAUSAL")}};
  } else {
    spec.family = "fmha_bf16";      // one family for both 16-bit float types
    spec.p = {{"B", s[0]}, {"H", s[1]}, {"S", s[2]}, {"D", s[3]}, {"CAUSAL", L.cfg("CAUSAL")},
              {"OUT_BF16", o.getElementType() == q.getElementType()}, {"F16", half}};
  }
  const int64_t br = L.cfg("TILED", 0) ? 0 : L.cfg("BLOCK_SIZE", 0);   // queries per workgroup; the kernel picks its own when this does not fit
  if (!single && br >= 32 && br <= 512 && br % 32 == 0 && s[2] % br == 0) spec.p["BR"] = br;
  spec.f["SCALE"] = L.cfg("SCALE_RSQRT_D") ? 1.0 / std::sqrt((double)s[3]) : 1.0;
  L.check = "fmha";
  L.checkInts = {s[0], s[1], s[2], s[3], L.cfg("CAUSAL") != 0};
  L.checkFloats = {spec.f["SCALE"]};
  return true;
}

}  // namespace

std::string HIPGen(ModuleOp& module, std::vector<KernelLaunchInfo>& infos, std::string* error,
                   std::vector<std::string>* skipped) {
  infos.clear();
  // Functions that the module body no longer calls (the operators a fusion has replaced) get no kernel.  A
  // module without any call (functions built by hand) translates all of its scheduled functions.
  std::vector<std::string> called;
  for (auto& op : module.getBody()->getOperations())
    if (auto call = dyn_cast<func::CallOp>(op)) called.push_back(call.getCallee());
  if (skipped) {
    // operators that are called from the module body but that no optimizer has scheduled
    skipped->clear();
    for (auto& op : module.getBody()->getOperations())
      if (auto call = dyn_cast<func::CallOp>(op)) {
        bool scheduled = false;
        module.walk<WalkOrder::PreOrder>([&](func::FuncOp f) {
          if (f.getSymName() != call.getCallee()) return;
          Attribute state = f->getAttr("func.state");
          scheduled = state && state.s == "gpu";
        });
        if (!scheduled) skipped->push_back(call.getCallee());
      }
  }
  std::ostringstream body;
  int kernelCounter = 0;  // restarts at every call
  bool failed = false;
  std::string firstError;
  module.walk<WalkOrder::PreOrder>([&](func::FuncOp f) {
    if (failed || f.empty()) return;
    Attribute state = f->getAttr("func.state");
    if (!state || state.s != "gpu") return;
    if (!called.empty() && std::find(called.begin(), called.end(), f.getSymName()) == called.end()) return;
    Lowering L;
    L.f = f;
    L.op = f->getAttr("kcg.op").s;
    for (auto& op : f.front().getOperations())
      if (auto grid = dyn_cast<AffineParallelOp>(op)) {
        L.levels.push_back(grid);
        for (auto& inner : grid.getBody()->getOperations())
          if (auto blk = dyn_cast<AffineParallelOp>(inner)) { L.levels.push_back(blk); break; }
        break;
      }
    hipgen::KernelSpec spec;
    spec.name = "kernel" + std::to_string(kernelCounter);
    bool ok = false;
    bool known = true;
    if (L.levels.size() != 2) L.error = "function has no grid / workgroup parallel levels";
    else if (L.op == "Matmul" || L.op == "BatchMatmul") ok = lowerGemm(L, spec);
    else if (L.op == "ElementWise") ok = lowerElementWise(L, spec);
    else if (L.op == "LayerNorm") ok = lowerLayerNorm(L, spec);
    else if (L.op == "FMHA") ok = lowerFMHA(L, spec);
    else if (L.op == "Binary") ok = lowerBinary(L, spec);
    else if (L.op == "Gather") ok = lowerGather(L, spec);
    else if (L.op == "Softmax") ok = lowerSoftmax(L, spec);
    else { known = false; L.error = "no gfx950 kernel family for operator '" + L.op + "'"; }
    // Which lowering: a kernel family sized by the schedule, or the schedule itself, statement by statement.  The
    // second is what a function without an operator tag gets (a schedule scripted by hand), and what
    // kcg.lowering = "schedule" on the function or on the module asks for.
    Attribute want = f->getAttr("kcg.lowering");
    if (!want) want = module->getAttr("kcg.lowering");
    const bool bySchedule = (want && want.s == "schedule") || !known;
    const bool familiesOnly = want && want.s == "families-only";
    std::string text, emitError;
    KernelLaunchInfo info;
    if (!bySchedule && ok && !hipgen::emitKernel(spec, text, info, emitError)) { ok = false; L.error = emitError; }
    if (L.levels.size() == 2 && (bySchedule || (!ok && !familiesOnly))) {
      // Also the way out when a family refuses the function (an element type it has no form for, such as f64):
      // the schedule itself always says what to compute.  The operator's description for the host-side check
      // (L.check and friends) stays when the family got as far as writing it.
      const std::string familyError = bySchedule ? "" : L.error;
      // A family that has no form for the function is the expected case; one that refuses a configuration (tile
      // sizes, the LDS limit) leaves the caller with a far slower kernel than it asked for, and says so.
      if (!bySchedule && !L.noForm)
        fprintf(stderr, "kcg warning: %s: kernel family refused (%s); lowering its schedule statement by statement instead\n",
                f.getSymName().c_str(), L.error.c_str());
      if (!ok) { L.check.clear(); L.checkInts.clear(); L.checkFloats.clear(); }
      text.clear();
      ok = hipgen::emitSchedule(f, spec.name, text, info, emitError);
      if (!ok) L.error = (familyError.empty() ? "" : familyError + "; ") + "schedule lowering: " + emitError;
      info.lowering = familyError.empty() ? "schedule" : "schedule (" + familyError + ")";
    } else {
      info.lowering = "family " + spec.family;
    }
    if (!ok) {
      failed = true;
      firstError = f.getSymName() + ": " + L.error;
      return;
    }
    info.function = f.getSymName();
    for (auto a : f.getArguments()) {
      info.argBytes.push_back(bytesOf(a.getType()));
      info.argTypes.push_back(dtypeOf(a.getType()));
    }
    // outputs that the function allocates itself follow the inputs
    Operation& ret = f.front().back();
    for (Value r : ret.getOperands()) {
      if (!r.isa<BlockArgument>()) {
        info.argBytes.push_back(bytesOf(r.getType()));
        info.argTypes.push_back(dtypeOf(r.getType()));
        if (info.outputArg < 0) info.outputArg = (int)info.argBytes.size() - 1;
      } else if (info.outputArg < 0) {
        info.outputArg = (int)r.cast<BlockArgument>().getArgNumber();     // the result is written into an argument
      }
    }
    if (info.workspaceBytes > 0) {
      info.workspaceArg = (int)info.argBytes.size();
      info.argBytes.push_back(info.workspaceBytes);
      info.argTypes.push_back(KCG_DT_I32);
    }
    info.check = L.check;
    info.checkInts = L.checkInts;
    info.checkFloats = L.checkFloats;
    info.fillLo = L.fillLo;
    info.fillHi = L.fillHi;
    if (info.argBytes.size() + info.numScalars != info.numArgs) {   // trailing fp32 scalars are not buffers
      failed = true;
      firstError = f.getSymName() + ": kernel takes " + std::to_string(info.numArgs - info.numScalars) + " pointers but the function has " +
                   std::to_string(info.argBytes.size()) + " buffers";
      return;
    }
    // launch geometry, outer to inner (z, y, x) like the reference's comment
    body << "// " << f.getSymName() << "\n";
    body << "// grid dims:(" << info.grid[2] << ", " << info.grid[1] << ", " << info.grid[0] << ", ), block dims:("
         << info.block[2] << ", " << info.block[1] << ", " << info.block[0] << ", )\n";
    body << text << "\n";
    infos.push_back(info);
    ++kernelCounter;
  });
  if (failed) {
    infos.clear();
    if (error) *error = firstError;
    else llvm::errs() << "HIPGen: " << firstError << "\n";
    return "";
  }
  std::string source = hipgen::prelude() + "\n" + body.str();
  if (KCGLog::level == Log::Debug) llvm::errs() << source;
  return source;
}

std::string HIPGen(ModuleOp& module) {
  std::vector<KernelLaunchInfo> infos;
  return HIPGen(module, infos, nullptr, nullptr);
}

}  // namespace KernelCodeGen
