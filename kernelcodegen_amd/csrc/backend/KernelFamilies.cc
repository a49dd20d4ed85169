#include "backend/KernelFamilies.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <sstream>
#include <vector>

// Generated at build time from backend/kernels/*.hip: one raw string per file.
#include "backend/kernels/_templates_gen.inc"

namespace KernelCodeGen {
namespace hipgen {

namespace {

struct Defines {
  std::vector<std::pair<std::string, std::string>> items;
  void add(const std::string& k, const std::string& v) { items.emplace_back(k, v); }
  void add(const std::string& k, int64_t v) { items.emplace_back(k, std::to_string(v)); }
  std::string wrap(const char* body) const {
    std::ostringstream os;
    for (auto& kv : items) os << "#define " << kv.first << " " << kv.second << "\n";
    os << body << "\n";
    for (auto& kv : items) os << "#undef " << kv.first << "\n";
    return os.str();
  }
};

std::string floatLiteral(double v) {
  char buf[64];
  snprintf(buf, sizeof buf, "%af", (double)(float)v);  // hex float: exact fp32 value
  return buf;
}

int64_t ceilDiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

int64_t nextPow2(int64_t v) {
  int64_t p = 1;
  while (p < v) p <<= 1;
  return p;
}

bool need(const KernelSpec& s, std::initializer_list<const char*> keys, std::string& err) {
  for (auto k : keys)
    if (!s.has(k)) {
      err = "kernel family '" + s.family + "' needs parameter " + k;
      return false;
    }
  return true;
}

bool positive(const KernelSpec& s, std::initializer_list<const char*> keys, std::string& err) {
  for (auto k : keys)
    if (s.get(k, 0) <= 0) {
      err = std::string("parameter ") + k + " must be positive";
      return false;
    }
  return true;
}

// ---------------------------------------------------------------------------
bool emitLayerNorm(KernelSpec& s, std::string& src, KernelLaunchInfo& info, std::string& err) {
  if (!need(s, {"ROWS", "N"}, err) || !positive(s, {"ROWS", "N"}, err)) return false;
  const int64_t rows = s.p["ROWS"], n = s.p["N"];
  const int64_t ng = s.get("NG", n), nb = s.get("NB", n);
  if (ng <= 0 || nb <= 0 || n % ng || n % nb) {
    err = "layernorm: scale/bias length must divide the normalised length";
    return false;
  }
  int64_t vw = s.get("VW", (n % 4 == 0 && ng % 4 == 0 && nb % 4 == 0) ? 4 : 1);
  if (vw != 1 && vw != 4) { err = "layernorm: VW must be 1 or 4"; return false; }
  if (vw == 4 && (n % 4 || ng % 4 || nb % 4)) { err = "layernorm: VW=4 needs lengths divisible by 4"; return false; }
  int64_t tpr = s.get("TPR", 0);
  if (rows > 0xFFFFFFFFLL) { err = "layernorm: too many rows"; return false; }
  if (tpr == 0) {
    // four vectors per lane measured best for 4096-float rows, with and without the GELU
    tpr = nextPow2(ceilDiv(n, vw * 4));
    if (tpr < 64) tpr = 64;
    if (tpr > 512) tpr = 512;
  }
  if (tpr < 64 || tpr > 1024 || (tpr & (tpr - 1))) { err = "layernorm: TPR must be a power of two in [64,1024]"; return false; }
  int64_t vpt = ceilDiv(n, tpr * vw);
  if (vpt > 8 && !s.has("TPR")) {  // widen the team: up to 8 vectors per lane leave room for gamma, beta and a prefetched row
    tpr = 1024;
    vpt = ceilDiv(n, tpr * vw);
  }
  const bool f16 = s.get("F16", 0) != 0;
  const double esize = f16 ? 2.0 : 4.0;
  if (vpt > 32) {
    // the group does not fit the register file of one workgroup: three streamed passes
    const int64_t block = 1024;
    s.p["VW"] = vw; s.p["TPR"] = block; s.p["RPB"] = 1; s.p["VPT"] = 0; s.p["NG"] = ng; s.p["NB"] = nb;
    Defines d;
    d.add("LS_NAME", s.name);
    d.add("LS_ROWS", rows);
    d.add("LS_N", std::to_string(n) + "L");
    d.add("LS_NG", ng);
    d.add("LS_NB", nb);
    d.add("LS_EPS", floatLiteral(s.f.count("EPS") ? s.f["EPS"] : 1e-5));
    d.add("LS_BLOCK", block);
    d.add("LS_VW", vw);
    d.add("LS_GELU", s.get("GELU", 0) ? 1 : 0);
    d.add("LS_F16", s.get("F16", 0));
    src = d.wrap(kTpl_layernorm_stream);
    info.name = s.name;
    info.grid[0] = (uint32_t)rows;
    info.block[0] = (uint32_t)block;
    info.numArgs = 4;
    info.flops = 8.0 * (double)rows * (double)n;
    info.bytes = 2.0 * (double)rows * (double)n * esize + (double)(ng + nb) * esize;
    return true;
  }
  int64_t rpb = s.get("RPB", tpr >= 256 ? 1 : 256 / tpr);
  if (rpb < 1 || rpb * tpr > 1024) { err = "layernorm: RPB*TPR must be in [64,1024]"; return false; }
  s.p["VW"] = vw; s.p["TPR"] = tpr; s.p["RPB"] = rpb; s.p["VPT"] = vpt; s.p["NG"] = ng; s.p["NB"] = nb;

  Defines d;
  d.add("LN_NAME", s.name);
  d.add("LN_ROWS", rows);
  d.add("LN_N", n);
  d.add("LN_NG", ng);
  d.add("LN_NB", nb);
  d.add("LN_EPS", floatLiteral(s.f.count("EPS") ? s.f["EPS"] : 1e-5));
  d.add("LN_TPR", tpr);
  d.add("LN_RPB", rpb);
  d.add("LN_VW", vw);
  d.add("LN_VPT", vpt);
  d.add("LN_GELU", s.get("GELU", 0) ? 1 : 0);
  d.add("LN_F16", s.get("F16", 0));
  // Two persistent workgroups per CU, each walking the row groups with stride GRID and loading its next
  // row before it reduces the current one: measured on operands that are not in the last-level cache
  // (three rotating buffer sets), 16384 x 4096 runs at 6.1 TB/s this way against 5.5 TB/s with one
  // workgroup per row; a plain copy reaches 6.3-6.4 TB/s under the same conditions.
  const int64_t groups = ceilDiv(rows, rpb);
  int64_t grid = s.get("GRID", 0);
  if (grid <= 0) grid = vpt <= 8 ? 512 : groups;      // rows too long to prefetch keep one workgroup per group
  if (grid > groups) grid = groups;
  if (grid > 0x7FFFFFFFLL) grid = 0x7FFFFFFFLL;
  s.p["GRID"] = grid;
  d.add("LN_GRID", grid);
  d.add("LN_STREAM", s.get("STREAM", 1) ? 1 : 0);
  d.add("LN_LEAN", s.get("LEAN", vpt > 8 ? 1 : 0) ? 1 : 0);
  // one reduction per row (merged means and sums of squared deviations) where every lane holds the same number of values
  const bool onePass = s.get("ONEPASS", 0) != 0 && n % (tpr * vw) == 0;
  s.p["ONEPASS"] = onePass;
  d.add("LN_ONEPASS", onePass ? 1 : 0);
  src = d.wrap(kTpl_layernorm);

  info.name = s.name;
  info.grid[0] = (uint32_t)grid;
  info.block[0] = (uint32_t)(tpr * rpb);
  info.numArgs = 4;
  info.flops = 8.0 * (double)rows * (double)n;
  info.bytes = 2.0 * (double)rows * (double)n * esize + (double)(ng + nb) * esize;
  return true;
}

// ---------------------------------------------------------------------------
bool parseList(const std::string& text, std::vector<int64_t>& out) {
  out.clear();
  std::stringstream ss(text);
  std::string item;
  while (std::getline(ss, item, ',')) {
    if (item.empty()) return false;
    char* end = nullptr;
    const long long v = std::strtoll(item.c_str(), &end, 10);
    if (*end) return false;
    out.push_back(v);
  }
  return !out.empty();
}

std::string joinList(const std::vector<int64_t>& v) {
  std::string s;
  for (size_t i = 0; i < v.size(); ++i) s += (i ? ", " : "") + std::to_string(v[i]) + "L";
  return s;
}

bool emitBinary(KernelSpec& s, std::string& src, KernelLaunchInfo& info, std::string& err) {
  static const char* names[] = {"Add", "Sub", "Mul", "Div", "Pow", "Equal", "Greater"};
  int op = -1;
  for (int i = 0; i < 7; ++i)
    if (s.s.count("OP") && s.s["OP"] == names[i]) op = i;
  if (op < 0) { err = "binary: OP must be Add, Sub, Mul, Div, Pow, Equal or Greater"; return false; }
  const bool compare = op >= 5;     // one byte per result element
  std::vector<int64_t> dims, sa, sb;
  if (!s.s.count("DIMS") || !s.s.count("SA") || !s.s.count("SB") || !parseList(s.s["DIMS"], dims) ||
      !parseList(s.s["SA"], sa) || !parseList(s.s["SB"], sb) || sa.size() != dims.size() || sb.size() != dims.size()) {
    err = "binary: DIMS, SA and SB must be comma separated lists of one length";
    return false;
  }
  if (dims.size() > 6) { err = "binary: rank above 6"; return false; }
  int64_t total = 1, elemsA = 1, elemsB = 1;
  for (size_t d = 0; d < dims.size(); ++d) {
    if (dims[d] <= 0 || sa[d] < 0 || sb[d] < 0) { err = "binary: extents must be positive and strides non-negative"; return false; }
    total *= dims[d];
    if (sa[d]) elemsA *= dims[d];
    if (sb[d]) elemsB *= dims[d];
  }
  const bool inplace = s.get("INPLACE", 0) != 0;
  if (inplace && elemsA != total) { err = "binary: an in-place result needs an unbroadcast left operand"; return false; }
  if (inplace && compare) { err = "binary: a comparison cannot overwrite its fp32 operand"; return false; }
  const int64_t inner = dims.back();
  const bool lastOk = (sa.back() == 1 || sa.back() == 0) && (sb.back() == 1 || sb.back() == 0);
  if (!lastOk) { err = "binary: the innermost stride of an operand must be 1 or 0"; return false; }
  // 128-bit accesses need every operand row to start on a 16-byte boundary
  bool aligned = inner % 4 == 0;
  for (size_t d = 0; d + 1 < dims.size(); ++d) aligned = aligned && sa[d] % 4 == 0 && sb[d] % 4 == 0;
  int64_t vw = s.get("VW", aligned ? 4 : 1);
  if (vw != 1 && vw != 4) { err = "binary: VW must be 1 or 4"; return false; }
  if (vw == 4 && !aligned) { err = "binary: VW=4 needs rows that are multiples of four elements"; return false; }
  int64_t block = s.get("BLOCK", 512);
  if (block < 64 || block > 1024 || block % 64) { err = "binary: bad BLOCK"; return false; }
  if (ceilDiv(total, vw * block) > 0x7FFFFFFFLL) { err = "binary: too many elements"; return false; }
  s.p["VW"] = vw; s.p["BLOCK"] = block;

  Defines d;
  d.add("BN_NAME", s.name);
  d.add("BN_RANK", (int64_t)dims.size());
  d.add("BN_DIMS", joinList(dims));
  d.add("BN_SA", joinList(sa));
  d.add("BN_SB", joinList(sb));
  d.add("BN_OP", op);
  d.add("BN_VW", vw);
  d.add("BN_BLOCK", block);
  d.add("BN_INPLACE", inplace ? 1 : 0);
  d.add("BN_F16", s.get("F16", 0) ? 1 : 0);
  // An operand that is not broadcast is read once: non-temporal loads for it (bit 0: X, bit 1: Y); a broadcast one is
  // read again and again out of the cache and keeps plain loads (16384 x 4096 plus a row: 84.3 us with the hint on X
  // alone, 86.0 without, 86.5 with it on both).  Not for an in-place result, whose operand is written back.
  const int64_t stream = s.get("STREAM", inplace ? 0 : ((elemsA == total ? 1 : 0) | (elemsB == total ? 2 : 0))) & 3;
  s.p["STREAM"] = stream;
  d.add("BN_STREAM", stream);
  src = d.wrap(kTpl_binary);

  info.name = s.name;
  info.grid[0] = (uint32_t)ceilDiv(total, vw * block);
  info.block[0] = (uint32_t)block;
  info.numArgs = inplace ? 2 : 3;
  info.flops = (double)total;
  const double esize = s.get("F16", 0) ? 2.0 : 4.0;
  info.bytes = esize * ((double)elemsA + (double)elemsB) + (compare ? 1.0 : esize) * (double)total;
  return true;
}

bool emitSoftmax(KernelSpec& s, std::string& src, KernelLaunchInfo& info, std::string& err) {
  if (!need(s, {"ROWS", "N"}, err) || !positive(s, {"ROWS", "N"}, err)) return false;
  const int64_t rows = s.p["ROWS"], n = s.p["N"];
  int64_t vw = s.get("VW", n % 4 == 0 ? 4 : 1);
  if (vw != 1 && vw != 4) { err = "softmax: VW must be 1 or 4"; return false; }
  if (vw == 4 && n % 4) { err = "softmax: VW=4 needs a row length divisible by 4"; return false; }
  int64_t tpr = s.get("TPR", 0);
  if (tpr == 0) {
    tpr = nextPow2(ceilDiv(n, vw * 4));      // about four vectors per lane
    if (tpr < 64) tpr = 64;
    if (tpr > 1024) tpr = 1024;
  }
  if (tpr < 64 || tpr > 1024 || (tpr & (tpr - 1))) { err = "softmax: TPR must be a power of two in [64,1024]"; return false; }
  const int64_t vpt = ceilDiv(n, tpr * vw);
  if (vpt > 32) {
    // rows too long for registers (a vocabulary of 150 000 logits, say): one workgroup per row, two streamed passes
    if (rows > 0x7FFFFFFFLL) { err = "softmax: too many rows"; return false; }
    const bool inplaceLong = s.get("INPLACE", 1) != 0;
    s.p["VW"] = vw; s.p["TPR"] = 1024; s.p["RPB"] = 1; s.p["VPT"] = 0; s.p["INPLACE"] = inplaceLong;
    Defines d;
    d.add("SS_NAME", s.name);
    d.add("SS_ROWS", rows); d.add("SS_N", n);
    d.add("SS_BLOCK", 1024); d.add("SS_VW", vw);
    d.add("SS_INPLACE", inplaceLong ? 1 : 0);
    d.add("SS_F16", s.get("F16", 0));
    src = d.wrap(kTpl_softmax_stream);
    info.name = s.name;
    info.grid[0] = (uint32_t)rows;
    info.block[0] = 1024;
    info.numArgs = inplaceLong ? 1 : 2;
    info.flops = 4.0 * (double)rows * (double)n;
    info.bytes = 2.0 * (double)rows * (double)n * (s.get("F16", 0) ? 2.0 : 4.0);
    return true;
  }
  int64_t rpb = s.get("RPB", tpr >= 256 ? 1 : 256 / tpr);
  if (rpb < 1 || rpb * tpr > 1024) { err = "softmax: RPB*TPR must be in [64,1024]"; return false; }
  const int64_t groups = ceilDiv(rows, rpb);
  if (groups > 0x7FFFFFFFLL) { err = "softmax: too many rows"; return false; }
  const bool inplace = s.get("INPLACE", 1) != 0;
  s.p["VW"] = vw; s.p["TPR"] = tpr; s.p["RPB"] = rpb; s.p["VPT"] = vpt; s.p["INPLACE"] = inplace;

  Defines d;
  d.add("SM_NAME", s.name);
  d.add("SM_ROWS", rows); d.add("SM_N", n);
  d.add("SM_TPR", tpr); d.add("SM_RPB", rpb); d.add("SM_VW", vw); d.add("SM_VPT", vpt);
  d.add("SM_INPLACE", inplace ? 1 : 0);
  d.add("SM_STREAM", s.get("STREAM", 1) ? 1 : 0);
  d.add("SM_F16", s.get("F16", 0));
  src = d.wrap(kTpl_softmax);

  info.name = s.name;
  info.grid[0] = (uint32_t)groups;
  info.block[0] = (uint32_t)(tpr * rpb);
  info.numArgs = inplace ? 1 : 2;
  info.flops = 4.0 * (double)rows * (double)n;
  info.bytes = 2.0 * (double)rows * (double)n * (s.get("F16", 0) ? 2.0 : 4.0);
  return true;
}

bool emitGather(KernelSpec& s, std::string& src, KernelLaunchInfo& info, std::string& err) {
  if (!need(s, {"OUTER", "AXIS", "NIDX", "INNER", "ESIZE"}, err) || !positive(s, {"OUTER", "AXIS", "NIDX", "INNER", "ESIZE"}, err))
    return false;
  const int64_t outer = s.p["OUTER"], axis = s.p["AXIS"], nidx = s.p["NIDX"], inner = s.p["INNER"], esize = s.p["ESIZE"];
  if (esize != 1 && esize != 2 && esize != 4 && esize != 8) { err = "gather: ESIZE must be 1, 2, 4 or 8 bytes"; return false; }
  const int64_t row = inner * esize;
  int64_t vb = 16;
  while (vb > 2 && row % vb) vb /= 2;
  if (row % vb) { err = "gather: rows of an odd number of bytes are not supported"; return false; }
  const int64_t block = s.get("BLOCK", 256);
  if (block < 64 || block > 1024 || block % 64) { err = "gather: bad BLOCK"; return false; }
  const double units = (double)outer * (double)nidx * (double)(row / vb);
  if (units / (double)block > 2147483647.0) { err = "gather: too many elements"; return false; }
  // two units per lane when there is work for every CU several times over (32000 x 4096 bf16 table, 16384 rows
  // picked, operands in HBM: 0.82 of the HBM peak against 0.78 with one unit, 0.75 with four)
  const int64_t unroll = s.get("UNROLL", units >= 2.0 * (double)block * 2048.0 ? 2 : 1);
  if (unroll < 1 || unroll > 16) { err = "gather: UNROLL must be in [1,16]"; return false; }
  s.p["BLOCK"] = block; s.p["VB"] = vb; s.p["UNROLL"] = unroll;

  Defines d;
  d.add("GA_NAME", s.name);
  d.add("GA_OUTER", outer); d.add("GA_AXIS", axis); d.add("GA_NIDX", nidx);
  d.add("GA_ROW", row); d.add("GA_VB", vb); d.add("GA_BLOCK", block); d.add("GA_UNROLL", unroll);
  src = d.wrap(kTpl_gather);

  info.name = s.name;
  info.grid[0] = (uint32_t)ceilDiv(outer * nidx * (row / vb), block * unroll);
  info.block[0] = (uint32_t)block;
  info.numArgs = 3;
  info.flops = 0.0;
  info.bytes = 2.0 * (double)outer * (double)nidx * (double)row + 8.0 * (double)nidx;   // rows read and written, indices
  return true;
}

// ---------------------------------------------------------------------------
int elementwiseOpCode(const std::string& op) {
  static const char* names[] = {"Tanh", "Sqrt", "Log", "Relu", "Gelu", "Cast"};
  for (int i = 0; i < 6; ++i)
    if (op == names[i]) return i;
  return -1;
}

int ctypeSize(const std::string& t) {
  if (t == "float" || t == "int") return 4;
  if (t == "double" || t == "long") return 8;
  if (t == "short" || t == "_Float16" || t == "__bf16") return 2;
  return 0;
}

bool emitElementwise(KernelSpec& s, std::string& src, KernelLaunchInfo& info, std::string& err) {
  if (!need(s, {"N"}, err) || !positive(s, {"N"}, err)) return false;
  const int64_t n = s.p["N"];
  int op = s.has("OP") ? (int)s.p["OP"] : elementwiseOpCode(s.s.count("OP") ? s.s["OP"] : "");
  if (op < 0 || op > 5) { err = "elementwise: unknown operation"; return false; }
  std::string inT = s.s.count("IN_T") ? s.s["IN_T"] : "float";
  std::string outT = s.s.count("OUT_T") ? s.s["OUT_T"] : "float";
  if (!ctypeSize(inT) || !ctypeSize(outT)) { err = "elementwise: unsupported element type"; return false; }
  // the maps compute in fp32; operands and results are fp32, IEEE half or bfloat16 (converted on the way in and out)
  const bool floatIO = (inT == "float" || inT == "_Float16" || inT == "__bf16") && inT == outT;
  if (op != 5 && !floatIO) { err = "elementwise: only Cast changes the element type; the other maps take float, _Float16 or __bf16"; return false; }
  const bool inplace = s.get("INPLACE", 0) != 0;
  if (inplace && ctypeSize(inT) != ctypeSize(outT)) { err = "elementwise: in-place needs equal element sizes"; return false; }
  int64_t vw = s.get("VW", n % 4 == 0 ? 4 : 1);
  if (vw != 1 && vw != 4) { err = "elementwise: VW must be 1 or 4"; return false; }
  if (vw == 4 && n % 4) { err = "elementwise: VW=4 needs N divisible by 4"; return false; }
  int64_t block = s.get("BLOCK", 512), unroll = s.get("UNROLL", 1);
  if (block < 64 || block > 1024 || block % 64 || unroll < 1 || unroll > 16) { err = "elementwise: bad BLOCK/UNROLL"; return false; }
  s.p["VW"] = vw; s.p["BLOCK"] = block; s.p["UNROLL"] = unroll; s.p["OP"] = op;

  Defines d;
  d.add("EW_NAME", s.name);
  d.add("EW_N", std::to_string(n) + "L");
  d.add("EW_OP", op);
  d.add("EW_VW", vw);
  d.add("EW_BLOCK", block);
  d.add("EW_UNROLL", unroll);
  d.add("EW_STREAM", s.get("STREAM", 1) ? 1 : 0);
  d.add("EW_INPLACE", inplace ? 1 : 0);
  d.add("EW_IN_T", inT);
  d.add("EW_OUT_T", outT);
  src = d.wrap(kTpl_elementwise);

  info.name = s.name;
  info.grid[0] = (uint32_t)ceilDiv(n, vw * block * unroll);
  info.block[0] = (uint32_t)block;
  info.numArgs = inplace ? 1 : 2;
  info.flops = (op == 4 ? 10.0 : 1.0) * (double)n;
  info.bytes = (double)n * (ctypeSize(inT) + ctypeSize(outT));
  return true;
}

// ---------------------------------------------------------------------------
bool gemmCommon(KernelSpec& s, std::string& err, int64_t& m, int64_t& n, int64_t& k, int64_t& batch) {
  if (!need(s, {"M", "N", "K"}, err) || !positive(s, {"M", "N", "K"}, err)) return false;
  m = s.p["M"]; n = s.p["N"]; k = s.p["K"];
  batch = s.get("BATCH", 1);
  if (batch < 1 || batch > 65535) { err = "gemm: BATCH must be in [1,65535]"; return false; }
  if (m > (1LL << 30) || n > (1LL << 30) || k > (1LL << 30)) { err = "gemm: dimension too large"; return false; }
  return true;
}

bool checkTile(const KernelSpec& s, int64_t bm, int64_t bn, int64_t bk, int64_t wm, int64_t wn, int64_t kmul,
               std::string& err) {
  if (wm < 1 || wn < 1 || wm * wn > 16 || bm % (32 * wm) || bn % (32 * wn) || bk % kmul || bm <= 0 || bn <= 0 ||
      bk <= 0) {
    err = s.family + ": tile BM/BN must be multiples of 32*WM / 32*WN and BK a multiple of " + std::to_string(kmul);
    return false;
  }
  return true;
}

bool emitGemmF32(KernelSpec& s, std::string& src, KernelLaunchInfo& info, std::string& err) {
  int64_t m, n, k, batch;
  if (!gemmCommon(s, err, m, n, k, batch)) return false;
  // The largest square tile that still gives every CU a workgroup (measured on 4096^3, 2048^3, 1024^3 and
  // 16 x 1024^3: 256^2 with 16 wavefronts, 128^2 with 16 and a deeper k-tile, 64^2 with 4 and a deeper k-tile).
  int64_t tile = 64;
  for (int64_t t : {256, 128}) {
    if (m < t || n < t) continue;
    if ((double)ceilDiv(m, t) * (double)ceilDiv(n, t) * (double)batch >= 256.0) { tile = t; break; }
  }
  int64_t bm = s.get("BM", tile), bn = s.get("BN", tile);
  int64_t bk = s.get("BK", bm <= 128 && bn <= 128 ? 32 : 16);
  int64_t wm = s.get("WM", bm >= 128 ? 4 : 2), wn = s.get("WN", bn >= 128 ? 4 : 2), gm = s.get("GROUP_M", 8);
  if (!checkTile(s, bm, bn, bk, wm, wn, 4, err)) return false;
  const int64_t pad = s.get("PAD", 4);
  if (pad < 0 || pad % 4) { err = "gemm_f32: PAD must be a multiple of 4 floats"; return false; }
  const int64_t lds = 2 * bk * ((bm + pad) + (bn + pad)) * 4;
  if (lds > 160 * 1024) { err = "gemm_f32: tile needs more than 160 KiB of LDS"; return false; }
  const bool edge = (m % bm) || (n % bn) || (k % bk);
  s.p["BM"] = bm; s.p["BN"] = bn; s.p["BK"] = bk; s.p["WM"] = wm; s.p["WN"] = wn; s.p["GROUP_M"] = gm;

  // Whole tiles with BK = 16 or 32 of two row-major operands: the kernel that loads both tiles straight into LDS
  // (kernels/gemm_f32_d2l.hip)
  const bool d2l = s.get("D2L", 1) != 0 && !s.get("TA", 0) && !s.get("TB", 0) && (bk == 16 || bk == 32) && !edge && bm % 64 == 0 &&
                   (bn == 64 || bn == 128 || bn == 256) && bm % (32 * wm) == 0 && bn % (32 * wn) == 0 && (bm + bn) * bk * 8 <= 160 * 1024;
  s.p["D2L"] = d2l;
  // WK = 2: two groups of WM x WN wavefronts split the steps of every k-tile and add their partial sums through LDS at
  // the end (the kernel says why); needs k-tiles of 32, at most 16 wavefronts in all and results that fit the LDS tiles
  const bool wkFits = d2l && bk == 32 && wm * wn * 2 <= 16 && bm * bn * 4 <= (bm + bn) * bk * 8;
  // 64 x 64 x 32 tiles of four wavefronts on a launch that gives a CU at most one workgroup: two groups and three buffers
  // (1024^3: 19.7 against 20.7-21.1 us, 512 x 512 x 2048: 35.6 against 37.8 us; either one alone is slower, 22.5 and 23.7 us;
  // with several workgroups per CU, 1536^3, the groups change nothing and the launch keeps the plain form)
  const bool small = wkFits && bm == 64 && bn == 64 && wm * wn == 4 && (m / bm) * (n / bn) * batch <= 256;
  const int64_t wk = s.get("WK", small ? 2 : 1);
  if (wk != 1 && !(wk == 2 && wkFits)) { err = "gemm_f32: WK is 1 or 2; 2 needs whole tiles of two row-major operands, BK = 32, at most eight wavefronts per group and BM * BN <= 64 (BM + BN)"; return false; }
  s.p["WK"] = wk;
  // NBUF LDS buffers per operand (the loads of k-tile kt + NBUF - 1 start with k-tile kt): more than two where a k-tile is
  // shorter than a load's way from the L2; every wavefront must then issue the same number of loads per k-tile
  const int64_t nbuf = s.get("NBUF", small && wk == 2 ? 3 : 2);
  const int64_t blocks = (bm + bn) * bk * 4 / 1024;
  if (nbuf != 2 && !(d2l && (nbuf == 3 || nbuf == 4) && blocks % (wm * wn * wk) == 0 && nbuf * (bm + bn) * bk * 4 <= 160 * 1024)) {
    err = "gemm_f32: NBUF is 2, or 3 or 4 for whole tiles of two row-major operands whose k-tile is a whole number of 1 KiB blocks per wavefront and fits the LDS that many times";
    return false;
  }
  s.p["NBUF"] = nbuf;
  if (d2l) {
    Defines d;
    d.add("GL_NAME", s.name);
    d.add("GL_M", m); d.add("GL_N", n); d.add("GL_K", k); d.add("GL_BATCH", batch);
    d.add("GL_BM", bm); d.add("GL_BN", bn); d.add("GL_BK", bk); d.add("GL_WM", wm); d.add("GL_WN", wn);
    d.add("GL_WK", wk);
    d.add("GL_NBUF", nbuf);
    d.add("GL_GROUP_M", gm);
    d.add("GL_RELU", s.get("RELU", 0) ? 1 : 0);
    src = d.wrap(kTpl_gemm_f32_d2l);
    info.name = s.name;
    info.grid[0] = (uint32_t)((m / bm) * (n / bn));
    info.grid[1] = (uint32_t)batch;
    info.block[0] = (uint32_t)(64 * wm * wn * wk);
    info.numArgs = 3;
    info.flops = 2.0 * (double)batch * (double)m * (double)n * (double)k;
    info.bytes = 4.0 * (double)batch * ((double)m * k + (double)k * n + (double)m * n);
    return true;
  }

  Defines d;
  d.add("GM_NAME", s.name);
  d.add("GM_M", m); d.add("GM_N", n); d.add("GM_K", k); d.add("GM_BATCH", batch);
  d.add("GM_TA", s.get("TA", 0) ? 1 : 0); d.add("GM_TB", s.get("TB", 0) ? 1 : 0);
  d.add("GM_BM", bm); d.add("GM_BN", bn); d.add("GM_BK", bk);
  d.add("GM_WM", wm); d.add("GM_WN", wn); d.add("GM_GROUP_M", gm);
  d.add("GM_EDGE", edge ? 1 : 0);
  d.add("GM_RELU", s.get("RELU", 0) ? 1 : 0);
  d.add("GM_PAD", pad);
  src = d.wrap(kTpl_gemm_f32);

  info.name = s.name;
  info.grid[0] = (uint32_t)(ceilDiv(m, bm) * ceilDiv(n, bn));
  info.grid[1] = (uint32_t)batch;
  info.block[0] = (uint32_t)(64 * wm * wn);
  info.numArgs = 3;
  info.flops = 2.0 * (double)batch * (double)m * (double)n * (double)k;
  info.bytes = 4.0 * (double)batch * ((double)m * k + (double)k * n + (double)m * n);
  return true;
}

// Default workgroup tile of the bf16 and fp8 GEMMs: the largest of 256x256, 128x128, 128x64 and 64x64 that still
// gives each of the 256 CUs a workgroup (measured on 1024^3 ... 8192^3, 512x4096x4096 and 4096x4096x512: the
// choice is within a few per cent of the best tile everywhere, where a fixed 256x256 loses up to 2x on 2048^3).
static void defaultGemmTile(int64_t m, int64_t n, int64_t batch, int64_t& bm, int64_t& bn) {
  static const int64_t cand[4][2] = {{256, 256}, {128, 128}, {128, 64}, {64, 64}};
  bm = bn = 64;
  for (const auto& c : cand)
    if ((double)ceilDiv(m, c[0]) * (double)ceilDiv(n, c[1]) * (double)batch >= 256.0) {
      bm = c[0];
      bn = c[1];
      return;
    }
}

// fp64 GEMM on v_mfma_f64_16x16x4_f64.  128 x 128 x 16 tiles; 64 x 64 tiles where the larger ones would leave
// compute units without a workgroup.
bool emitGemmF64(KernelSpec& s, std::string& src, KernelLaunchInfo& info, std::string& err) {
  int64_t m, n, k, batch;
  if (!gemmCommon(s, err, m, n, k, batch)) return false;
  // measured at 4096^3 with 16 wavefronts: 128 x 256 tiles 68 TF (0.87 of the 78.6 TF peak), 256 x 128 66 TF,
  // 128 x 128 63.5 TF, 64 x 64 (four wavefronts) 54 TF; k-tiles of 8 or 32 instead of 16: 55 TF
  static const int64_t cand[3][2] = {{128, 256}, {128, 128}, {64, 64}};
  int64_t tm = 64, tn = 64;
  for (const auto& c : cand)
    if (m >= c[0] && n >= c[1] && (double)ceilDiv(m, c[0]) * (double)ceilDiv(n, c[1]) * (double)batch >= 256.0) { tm = c[0]; tn = c[1]; break; }
  int64_t bm = s.get("BM", tm), bn = s.get("BN", s.has("BM") ? s.get("BM", tn) : tn), bk = s.get("BK", 16);
  // wavefronts of 32 x 32 results (four MFMA tiles): 16 of them on a 128 x 128 tile measured 63 TF at 4096^3, 0.81
  // of the 78.6 TF peak, where four wavefronts of 64 x 64 reach 44 TF (one wavefront per SIMD hides no latency)
  int64_t wm = s.get("WM", std::max<int64_t>(1, std::min<int64_t>(4, bm / 32)));
  int64_t wn = s.get("WN", std::max<int64_t>(1, std::min<int64_t>(4, bn / 32))), gm = s.get("GROUP_M", 8);
  if (wm < 1 || wn < 1 || wm * wn > 16 || bm <= 0 || bn <= 0 || bm % (16 * wm) || bn % (16 * wn) || bk < 8 || bk % 8) {
    err = "gemm_f64: tile BM/BN must be multiples of 16*WM / 16*WN and BK a multiple of 8";
    return false;
  }
  if ((bm / wm / 16) * (bn / wn / 16) > 24) { err = "gemm_f64: more than 24 MFMA tiles per wavefront do not fit the registers"; return false; }
  const int64_t lds = 2 * (bm + bn) * (bk + 2) * 8;      // both tiles with k innermost, rows of BK + 2 doubles
  if (lds > 160 * 1024) { err = "gemm_f64: tile needs more than 160 KiB of LDS"; return false; }
  const bool edge = (m % bm) || (n % bn) || (k % bk);
  s.p["BM"] = bm; s.p["BN"] = bn; s.p["BK"] = bk; s.p["WM"] = wm; s.p["WN"] = wn; s.p["GROUP_M"] = gm;

  // Whole tiles with BK = 16 of two row-major operands: the kernel that loads both tiles straight into LDS
  // (kernels/gemm_f64_d2l.hip)
  const bool d2l = s.get("D2L", 1) != 0 && !s.get("TA", 0) && !s.get("TB", 0) && bk == 16 && !edge && bm % 64 == 0 && (bn == 128 || bn == 256) &&
                   bm % (16 * wm) == 0 && bn % (32 * wn) == 0 && 2 * (bm * 128 + 16 * bn * 8) <= 160 * 1024;
  s.p["D2L"] = d2l;
  if (d2l) {
    Defines d;
    d.add("GE_NAME", s.name);
    d.add("GE_M", m); d.add("GE_N", n); d.add("GE_K", k); d.add("GE_BATCH", batch);
    d.add("GE_BM", bm); d.add("GE_BN", bn); d.add("GE_WM", wm); d.add("GE_WN", wn);
    d.add("GE_GROUP_M", gm);
    d.add("GE_RELU", s.get("RELU", 0) ? 1 : 0);
    src = d.wrap(kTpl_gemm_f64_d2l);
    info.name = s.name;
    info.grid[0] = (uint32_t)((m / bm) * (n / bn));
    info.grid[1] = (uint32_t)batch;
    info.block[0] = (uint32_t)(64 * wm * wn);
    info.numArgs = 3;
    info.flops = 2.0 * (double)batch * (double)m * (double)n * (double)k;
    info.bytes = 8.0 * (double)batch * ((double)m * k + (double)k * n + (double)m * n);
    return true;
  }

  Defines d;
  d.add("GD_NAME", s.name);
  d.add("GD_M", m); d.add("GD_N", n); d.add("GD_K", k); d.add("GD_BATCH", batch);
  d.add("GD_TA", s.get("TA", 0) ? 1 : 0); d.add("GD_TB", s.get("TB", 0) ? 1 : 0);
  d.add("GD_BM", bm); d.add("GD_BN", bn); d.add("GD_BK", bk);
  d.add("GD_WM", wm); d.add("GD_WN", wn); d.add("GD_GROUP_M", gm);
  d.add("GD_EDGE", edge ? 1 : 0);
  d.add("GD_RELU", s.get("RELU", 0) ? 1 : 0);
  src = d.wrap(kTpl_gemm_f64);

  info.name = s.name;
  info.grid[0] = (uint32_t)(ceilDiv(m, bm) * ceilDiv(n, bn));
  info.grid[1] = (uint32_t)batch;
  info.block[0] = (uint32_t)(64 * wm * wn);
  info.numArgs = 3;
  info.flops = 2.0 * (double)batch * (double)m * (double)n * (double)k;
  info.bytes = 8.0 * (double)batch * ((double)m * k + (double)k * n + (double)m * n);
  return true;
}

// Tail split of a tiled GEMM (see kernels/gemm_bf16.hip): SK_UNITS extra workgroups share the k-iterations of
// the tiles behind the first SK_FULL ones and leave partial sums in a workspace.  Only on request (SK_UNITS > 0):
// on the 4096 x 11008 x 4096 product it measured slower than one workgroup per tile (0.53 against 0.34 ms).  The
// tiles of a round that run side by side read the same A and B panels at the same k and share them in the L2;
// runs that start at different k read their operands alone.  And the partly filled last round costs little to
// begin with: 256, 512 and 688 workgroups of that kernel take 0.123, 0.242 and 0.343 ms, the last 176 tiles
// 0.100 ms on CUs that then have more of the chip's power and bandwidth each.
bool chooseTailSplit(const KernelSpec& s, int64_t tiles, int64_t kt, int64_t batch, int64_t& full, int64_t& units,
                     std::string& err) {
  full = 0;
  units = s.get("SK_UNITS", 0);
  if (units <= 0) {
    units = 0;
    return true;
  }
  full = s.get("SK_FULL", tiles / units * units == tiles ? tiles - units : tiles / units * units);
  const int64_t tail = tiles - full;
  const bool xcd = units % 8 == 0 && full % 8 == 0 && tail % 8 == 0 && tiles % 8 == 0;
  const int64_t groups = xcd ? 8 : 1;
  int64_t per = ceilDiv((tail / groups) * kt, units / groups);
  per += per & 1;      // whole pairs of k-iterations: the kernel's k loop runs in pairs
  if (batch != 1 || units > 4096 || full < 0 || tail < 1 || tail > 1024 || per > kt || kt % 2) {
    err = s.family + ": tail split needs one batch, 1..1024 tail tiles, an even number of k-tiles and at most one tile's "
                     "k-iterations per unit";
    return false;
  }
  return true;
}

bool emitGemmBf16(KernelSpec& s, std::string& src, KernelLaunchInfo& info, std::string& err) {
  int64_t m, n, k, batch;
  if (!gemmCommon(s, err, m, n, k, batch)) return false;
  int64_t dm, dn;
  defaultGemmTile(m, n, batch, dm, dn);
  int64_t bm = s.get("BM", dm);
  int64_t bn = s.get("BN", dn);
  int64_t bk = s.get("BK", 64);
  // 256x256 tiles run as 8 wavefronts (two per SIMD, 64x128 each) so that one wavefront's
  // LDS and global-memory instructions issue under the other's MFMAs
  int64_t wm = s.get("WM", bm >= 256 && bn >= 256 ? 4 : 2), wn = s.get("WN", 2), gm = s.get("GROUP_M", 8);
  if (!checkTile(s, bm, bn, bk, wm, wn, 16, err)) return false;
  // A tiles k-contiguous with 16 bytes of padding a row; B tiles the same, or [k][n] rows with 32 bytes of padding
  // pad of an sB[k][n] row: the 32 lanes that a transposing read serves together take four k rows of 64 bytes, which fall
  // on disjoint banks when the row pitch is 64 modulo 256 (SQ_LDS_BANK_CONFLICT: 22.5 M cycles per launch of the
  // 4096 x 11008 x 4096 product with a pad of 32, none with 64)
  int64_t bpad = s.get("BPAD", (bn * 2) % 256 == 0 ? 64 : 32);
  if (bpad < 0 || bpad % 16) { err = "gemm_bf16: BPAD must be a multiple of 16 bytes"; return false; }
  const bool edge = (m % bm) || (n % bn) || (k % bk);
  // the 16x16x32 MFMA (see the kernel): whole 64-deep k-tiles, A contiguous along k, B contiguous along k or read
  // through the transposing LDS reads, loads without guards
  const bool m16Fits = bk == 64 && !s.get("TA", 0) && (s.get("TB", 0) || s.get("BTR", 1)) && !edge && k % 8 == 0 && n % 8 == 0 &&
                       (wm * wn) % 2 == 0 && bm % (8 * wm * wn) == 0 && bn % (8 * wm * wn) == 0 && s.get("STAGES", 1) == 1 &&
                       s.get("SK_UNITS", 0) <= 0 && bm / wm % 16 == 0 && bn / wn % 16 == 0;
  // direct loads into LDS (global_load_lds_dwordx4, see the kernel): every wavefront moves a whole, even number of
  // 1 KiB blocks per operand tile; row-major weights need the 256-column tile and eight wavefronts
  const int64_t waves = wm * wn;
  const bool d2lFits = m16Fits && bm % (16 * waves) == 0 &&
                       (s.get("TB", 0) ? bn % (16 * waves) == 0 : (bn == 256 && waves == 8));
  // Default on the 256 x 256 tile with eight wavefronts, where it was measured: with direct loads 0.295-0.303 ms on
  // 4096 x 11008 x 4096 in either weight layout against 0.310-0.315 ms ([N][K]) and 0.338-0.346 ms ([K][N]) for the
  // 32x32x16 form; through registers 0.320-0.328 ms for [K][N] (also 4-8 % ahead on 4096^3, 8192^3 and
  // 2048 x 8192 x 2048) and level with the other form for [N][K].
  const bool m16 = s.get("M16", m16Fits && d2lFits && bm == 256 && bn == 256 && waves == 8 && s.get("D2L", 1)) != 0;
  s.p["M16"] = m16;
  if (m16 && !m16Fits) { err = "gemm_bf16: M16 needs full 64-deep tiles, TA = 0, one staging set and no tail split"; return false; }
  const bool d2l = m16 && s.get("D2L", d2lFits) != 0;
  s.p["D2L"] = d2l;
  if (d2l && !d2lFits) { err = "gemm_bf16: D2L needs M16 and whole 1 KiB blocks per wavefront (row-major weights: BN = 256, eight wavefronts)"; return false; }
  // the 16x16x32 form's transposing reads take eight consecutive k rows of 32 bytes together: the pitch must be an odd
  // multiple of 32 bytes (through registers; direct loads leave the rows unpadded and swizzle them instead)
  if (m16 && !s.has("BPAD")) bpad = 32;
  if (d2l) bpad = 0;
  const int64_t rowA = m16 ? bk * 2 : bk * 2 + 16;
  const int64_t ldsB = s.get("TB", 0) ? bn * rowA : bk * (bn * 2 + bpad);
  const int64_t lds = 2 * bm * rowA + 2 * ldsB;
  if (lds > 160 * 1024) { err = "gemm_bf16: tile needs more than 160 KiB of LDS"; return false; }
  const bool outBf16 = s.get("OUT_BF16", 0) != 0;
  // staging register sets = tiles in flight from global memory; two only fit small wave tiles
  const int64_t stages = s.get("STAGES", 1);
  if (stages != 1 && stages != 2) { err = "gemm_bf16: STAGES must be 1 or 2"; return false; }
  s.p["BM"] = bm; s.p["BN"] = bn; s.p["BK"] = bk; s.p["WM"] = wm; s.p["WN"] = wn; s.p["GROUP_M"] = gm;
  s.p["STAGES"] = stages;
  // with one wavefront per SIMD the memory instructions have to be interleaved with the MFMAs explicitly
  const bool interleave = s.get("INTERLEAVE", wm * wn <= 4) != 0;
  s.p["INTERLEAVE"] = interleave;
  const int64_t tiles = ceilDiv(m, bm) * ceilDiv(n, bn);
  int64_t skFull = 0, skUnits = 0;
  if (stages != 1 || k % bk) s.p["SK_UNITS"] = s.has("SK_UNITS") && s.get("SK_UNITS", 0) ? -1 : 0;   // needs whole k-tiles, one staging set
  if (s.get("SK_UNITS", 0) < 0) { err = "gemm_bf16: tail split needs K a multiple of BK and STAGES = 1"; return false; }
  if (!chooseTailSplit(s, tiles, ceilDiv(k, bk), batch, skFull, skUnits, err)) return false;
  s.p["SK_UNITS"] = skUnits; s.p["SK_FULL"] = skFull;

  Defines d;
  d.add("GB_NAME", s.name);
  d.add("GB_M", m); d.add("GB_N", n); d.add("GB_K", k); d.add("GB_BATCH", batch);
  d.add("GB_TA", s.get("TA", 0) ? 1 : 0); d.add("GB_TB", s.get("TB", 0) ? 1 : 0);
  d.add("GB_BM", bm); d.add("GB_BN", bn); d.add("GB_BK", bk);
  d.add("GB_WM", wm); d.add("GB_WN", wn); d.add("GB_GROUP_M", gm);
  d.add("GB_EDGE", edge ? 1 : 0);
  d.add("GB_OUT_BF16", outBf16 ? 1 : 0);
  d.add("GB_RELU", s.get("RELU", 0) ? 1 : 0);
  d.add("GB_STAGES", stages);
  d.add("GB_INTERLEAVE", interleave ? 1 : 0);
  d.add("GB_F16", s.get("F16", 0) ? 1 : 0);
  d.add("GB_BPAD", bpad);
  if (m16) d.add("GB_M16", 1);
  if (d2l) d.add("GB_D2L", 1);
  if (m16 && s.has("M16_DEAL")) d.add("GB_M16_DEAL", s.get("M16_DEAL", 0) ? 1 : 0);
  // 16-bit results of whole 256 x 256 tiles in the 16x16x32 form leave through LDS as whole rows (see the kernel)
  const bool stageOk = m16 && bm == 256 && bn == 256 && wm == 4 && wn == 2 && !edge && skUnits == 0;
  const int64_t stageC = stageOk ? std::max<int64_t>(0, std::min<int64_t>(2, s.get("STAGE_C", outBf16 ? 2 : 0))) : 0;
  s.p["STAGE_C"] = stageC;
  if (stageC) d.add("GB_STAGE_C", stageC);
  if (s.has("BTR") && !s.get("TB", 0)) d.add("GB_BTR", s.get("BTR", 1) ? 1 : 0);
  // start of the walk along k staggered between the XCDs: default on for two k-contiguous operands (see the kernel)
  if (s.has("KROT")) d.add("GB_KROT_ON", s.get("KROT", 0) ? 1 : 0);
  if (s.get("SETPRIO", 0) > 0) d.add("GB_SETPRIO", std::min<int64_t>(3, s.get("SETPRIO", 0)));
  if (s.get("STAGGER", 0) > 0) d.add("GB_STAGGER", s.get("STAGGER", 0));
  d.add("GB_SK_UNITS", skUnits);
  d.add("GB_SK_FULL", skFull);
  src = d.wrap(kTpl_gemm_bf16);

  info.name = s.name;
  info.grid[0] = (uint32_t)(skUnits > 0 ? skFull + skUnits : tiles);
  info.grid[1] = (uint32_t)batch;
  info.block[0] = (uint32_t)(64 * wm * wn);
  info.numArgs = skUnits > 0 ? 4 : 3;
  if (skUnits > 0) {
    info.workspaceBytes = 4096 + skUnits * 2 * bm * bn * 4;
    info.workspaceArg = 3;
  }
  info.flops = 2.0 * (double)batch * (double)m * (double)n * (double)k;
  info.bytes = (double)batch * (2.0 * ((double)m * k + (double)k * n) + (outBf16 ? 2.0 : 4.0) * (double)m * n);
  return true;
}

bool emitGemmFp8(KernelSpec& s, std::string& src, KernelLaunchInfo& info, std::string& err) {
  int64_t m, n, k, batch;
  if (!gemmCommon(s, err, m, n, k, batch)) return false;
  const bool ta = s.get("TA", 0) != 0, tb = s.get("TB", 0) != 0;
  int64_t dm, dn;
  defaultGemmTile(m, n, batch, dm, dn);
  int64_t bm = s.get("BM", dm);
  int64_t bn = s.get("BN", dn);
  int64_t bk = s.get("BK", 128);
  // eight wavefronts from 128x128 up (2048^3: 1180 against 980 TFLOP/s with four)
  int64_t wm = s.get("WM", bm >= 128 && bn >= 128 ? 4 : 2), wn = s.get("WN", 2), gm = s.get("GROUP_M", 8);
  if (!checkTile(s, bm, bn, bk, wm, wn, 64, err)) return false;
  // Full 256 x 256 x 128 tiles of two k-contiguous operands: the kernel on v_mfma_f32_16x16x128 with direct loads into
  // LDS (kernels/gemm_fp8_d2l.hip), unless one of the other kernel's switches is asked for
  // Measured against the other kernel (M 4096-8192, N 4096-14336): 7-20 % faster for K up to 4096
  // (4096 x 11008 x 4096: 0.151 against 0.173 ms); beyond that level to 5 % faster on launches of more than one round
  // of tiles (8192^3: 0.419 against 0.441 ms) and 1-4 % slower on single rounds, which stay with the other.  Launches of more
  // than one round of tiles get the non-temporal result stores and the staggered start, which only pay together (see
  // the kernel); a single round is fastest without either.
  const bool legacyKnob = s.has("PREFETCH") || s.has("ROTATE") || s.has("PINGPONG") || s.has("STAGES") || (s.has("BTR") && !s.get("BTR", 1));
  const bool oneRound = ceilDiv(m, 256) * ceilDiv(n, 256) * batch <= 256;
  if (s.get("D2L", !legacyKnob && (k <= 4096 || !oneRound)) && !ta && (tb || s.get("BTR", 1)) && n % 16 == 0 && bm == 256 && bn == 256 && bk == 128 && wm == 4 && wn == 2 &&
      m % 256 == 0 && n % 256 == 0 && k % 128 == 0) {
    const int64_t scalePtr = s.get("SCALE_PTR", 0);
    if (scalePtr < 0 || scalePtr > 2) { err = "gemm_fp8: SCALE_PTR is 0 (scalar arguments), 1 (A, B, C, pointers) or 2 (A, B, pointers, C)"; return false; }
    const bool outBf16 = s.get("OUT_BF16", 0) != 0;
    // Strips of tile rows: workgroup ids are renumbered so that each of the 8 XCDs works through one contiguous run of
    // tiles; when such a run is a whole number of tile rows (at most four), the strip is the run, and all XCDs walk the
    // same columns of B at the same time (4096 x 11008 x 4096, two rows: 0.160 against 0.168 ms with strips of eight,
    // 0.164 with four); four rows otherwise (level with or ahead of eight on every shape measured).
    if (!s.has("GROUP_M")) {
      const int64_t tm = m / 256, tn = n / 256, run = tm * tn / 8;
      gm = (tm * tn) % 8 == 0 && run % tn == 0 && run / tn >= 1 && run / tn <= 4 ? run / tn : 4;
    }
    s.p["TA"] = 0; s.p["TB"] = tb; s.p["D2L"] = 1; s.p["BTR"] = !tb;
    s.p["BM"] = bm; s.p["BN"] = bn; s.p["BK"] = bk; s.p["WM"] = wm; s.p["WN"] = wn; s.p["GROUP_M"] = gm;
    Defines d;
    d.add("G8_NAME", s.name);
    d.add("G8_M", m); d.add("G8_N", n); d.add("G8_K", k); d.add("G8_BATCH", batch);
    d.add("G8_GROUP_M", gm);
    d.add("G8_OUT_BF16", outBf16 ? 1 : 0);
    d.add("G8_RELU", s.get("RELU", 0) ? 1 : 0);
    d.add("G8_SCALE_PTR", scalePtr);
    d.add("G8_BTR", tb ? 0 : 1);
    const int64_t tilesAll = (m / 256) * (n / 256);
    const bool persist = s.get("PERSIST", 0) != 0 && batch == 1 && (k / 128) % 2 == 0 && tilesAll > 256;
    s.p["PERSIST"] = persist;
    if (persist) d.add("G8_PERSIST", 1);
    const bool rounds = (m / 256) * (n / 256) * batch > 256;                   // more than one round of tiles
    // The results go through LDS and leave as whole rows of the tile (STAGE_C) unless the workgroups are persistent:
    // 4096 x 11008 x 4096 0.151 against 0.160 ms, 2 to 8 % on other shapes of more than one round, level on single
    // rounds.  The staggered start then does best at half its former width.  A bf16 result, of which a lane would
    // otherwise store two bytes of a row, gains most: 0.156 ms against 0.190, and against 0.171 for the other kernel.
    const int64_t stageC = s.get("STAGE_C", 1) != 0 && !persist;
    const int64_t ntStore = s.get("NT_STORE", rounds && (stageC || !outBf16) ? 1 : 0) != 0, stagger = std::max<int64_t>(0, std::min<int64_t>(16, s.get("STAGGER", rounds ? (stageC ? 1 : 2) : 0)));
    s.p["NT_STORE"] = ntStore; s.p["STAGGER"] = stagger;
    d.add("G8_NT_STORE", ntStore);
    d.add("G8_STAGGER", stagger);
    s.p["STAGE_C"] = stageC;
    d.add("G8_STAGE_C", stageC);
    src = d.wrap(kTpl_gemm_fp8_d2l);
    info.name = s.name;
    info.grid[0] = (uint32_t)(persist ? 256 : (m / 256) * (n / 256));
    info.grid[1] = (uint32_t)batch;
    info.block[0] = 512;
    info.numArgs = 5;
    info.numScalars = scalePtr ? 0 : 2;
    info.flops = 2.0 * (double)batch * (double)m * (double)n * (double)k;
    info.bytes = (double)batch * ((double)m * k + (double)k * n + (outBf16 ? 2.0 : 4.0) * (double)m * n);
    return true;
  }
  if (s.get("D2L", 0) && s.has("D2L")) { err = "gemm_fp8: D2L needs full 256 x 256 x 128 tiles, TA = 0 and TB = 1"; return false; }
  s.p["D2L"] = 0;
  // a B stored [K][N] lies in LDS as it lies in memory and is transposed by the LDS reads (BTR = 0: in registers on the way in)
  const bool btr = !tb && s.get("BTR", 1) != 0;
  s.p["BTR"] = btr;
  const int64_t lds = 2 * bm * (bk + 16) + (btr ? 2 * bk * (bn + 32) : 2 * bn * (bk + 16));
  if (lds > 160 * 1024) { err = "gemm_fp8: tile needs more than 160 KiB of LDS"; return false; }
  const bool edge = (m % bm) || (n % bn) || (k % bk);
  const bool outBf16 = s.get("OUT_BF16", 0) != 0;
  const int64_t stages = s.get("STAGES", 1);
  if (stages != 1 && stages != 2) { err = "gemm_fp8: STAGES must be 1 or 2"; return false; }
  // a second fragment set costs 8 registers per 32-row fragment: only small wave tiles can afford it
  const bool prefetch = s.get("PREFETCH", (bm / wm / 32 + bn / wn / 32) <= 4) != 0;
  s.p["PREFETCH"] = prefetch;
  s.p["TA"] = ta; s.p["TB"] = tb;
  s.p["BM"] = bm; s.p["BN"] = bn; s.p["BK"] = bk; s.p["WM"] = wm; s.p["WN"] = wn; s.p["GROUP_M"] = gm;
  s.p["STAGES"] = stages;

  Defines d;
  d.add("GF_NAME", s.name);
  d.add("GF_M", m); d.add("GF_N", n); d.add("GF_K", k); d.add("GF_BATCH", batch);
  d.add("GF_TA", ta ? 1 : 0); d.add("GF_TB", tb ? 1 : 0);
  d.add("GF_BM", bm); d.add("GF_BN", bn); d.add("GF_BK", bk);
  d.add("GF_WM", wm); d.add("GF_WN", wn); d.add("GF_GROUP_M", gm);
  d.add("GF_EDGE", edge ? 1 : 0);
  d.add("GF_OUT_BF16", outBf16 ? 1 : 0);
  d.add("GF_RELU", s.get("RELU", 0) ? 1 : 0);
  d.add("GF_STAGES", stages);
  d.add("GF_PREFETCH", prefetch ? 1 : 0);
  // fragments re-read behind their last use (no second set): where there is no room for a second set and a tile has
  // at least two k-steps
  // (default: with row-major [K][N] weights, where it measured 2-4 % faster at 4096 x 11008 x 4096; no difference with
  // [N][K] weights)
  const bool rotate = !prefetch && bk >= 128 && s.get("ROTATE", btr ? 1 : 0) != 0;
  s.p["ROTATE"] = rotate;
  d.add("GF_ROTATE", rotate ? 1 : 0);
  // the two wavefronts of a SIMD half a k-tile out of step (one k-step per tile, eight wavefronts, nothing guarded)
  const bool guarded = edge || (k % 16) || (ta && m % 16) || (!tb && n % 16);
  const bool pingpong = s.get("PINGPONG", 0) != 0 && bk == 64 && wm * wn == 8 && !guarded && !prefetch && k / bk >= stages + 2;
  s.p["PINGPONG"] = pingpong;
  d.add("GF_PINGPONG", pingpong ? 1 : 0);
  d.add("GF_BTR", btr ? 1 : 0);
  // where the two per-tensor scales come from: trailing scalars, or one fp32 each in device memory (graph values)
  const int64_t scalePtr = s.get("SCALE_PTR", 0);
  if (scalePtr < 0 || scalePtr > 2) { err = "gemm_fp8: SCALE_PTR is 0 (scalar arguments), 1 (A, B, C, pointers) or 2 (A, B, pointers, C)"; return false; }
  d.add("GF_SCALE_PTR", scalePtr);
  if (s.get("STAGGER", 0) > 0) d.add("GF_STAGGER", s.get("STAGGER", 0));
  src = d.wrap(kTpl_gemm_fp8);

  info.name = s.name;
  info.grid[0] = (uint32_t)(ceilDiv(m, bm) * ceilDiv(n, bn));
  info.grid[1] = (uint32_t)batch;
  info.block[0] = (uint32_t)(64 * wm * wn);
  info.numArgs = 5;       // A, B, C, scale_a, scale_b
  info.numScalars = scalePtr ? 0 : 2;
  info.flops = 2.0 * (double)batch * (double)m * (double)n * (double)k;
  info.bytes = (double)batch * ((double)m * k + (double)k * n + (outBf16 ? 2.0 : 4.0) * (double)m * n);
  return true;
}

bool emitFmhaBf16(KernelSpec& s, std::string& src, KernelLaunchInfo& info, std::string& err) {
  if (!need(s, {"B", "H", "S", "D"}, err) || !positive(s, {"B", "H", "S", "D"}, err)) return false;
  const int64_t b = s.p["B"], h = s.p["H"], sl = s.p["S"], dh = s.p["D"];
  if (dh % 32 || dh > 256) { err = "fmha_bf16: head dim must be a multiple of 32, at most 256"; return false; }
  int64_t br = s.get("BR", 0), bc = s.get("BC", 0);
  // A sequence length that the tiles do not divide is taken too (the kernel guards its last query and key tiles); the
  // automatic choice prefers tiles that divide it, and for a length with no such tile takes the sizes of its magnitude.
  // Large tiles with a guarded edge are faster than small ones that divide the length: 32 queries per workgroup (one
  // wavefront) for a length like 4000 ran at a fifth of the speed of 256 with the last tile partly filled.
  if (br <= 0) {
    if (sl % 256 == 0) br = 256;
    else if (sl % 128 == 0) br = 128;
    else if (sl % 64 == 0 && sl <= 512) br = 64;
    else br = sl > 128 ? 256 : (sl > 64 ? 128 : (sl > 32 ? 64 : 32));
  }
  if (bc <= 0) {
    bc = sl > 32 ? 64 : 32;
    if (2 * bc * (dh * 2 + 16) + 3 * bc * (dh * 2 + 32) > 160 * 1024) bc = 32;   // head dim 256: 64-key tiles do not fit the LDS
  }
  if (br % 32 || br > 512 || bc % 32) { err = "fmha_bf16: BR must be a multiple of 32 (at most 512) and BC a multiple of 32"; return false; }
  // 64 queries per wavefront (every LDS fragment feeds two MFMAs, one wavefront per SIMD with the whole
  // register file) when that still leaves four wavefronts and the step-pipelined loop applies
  int64_t qw = s.get("QW", 0);
  if (qw <= 0) qw = 1;
  if ((qw != 1 && qw != 2) || br % (32 * qw)) { err = "fmha_bf16: QW must be 1 or 2 and BR a multiple of 32 * QW"; return false; }
  const bool ragged = sl % br != 0 || sl % bc != 0;
  if (ragged && (double)sl * (double)dh * 2.0 >= 4294967296.0) {
    err = "fmha_bf16: a sequence length that is no multiple of the tiles needs heads below 4 GiB";
    return false;
  }
  if ((double)ceilDiv(sl, br) * (double)b * (double)h > 2147483647.0) { err = "fmha_bf16: too many workgroups"; return false; }
  if (s.f.count("SCALE") && !(s.f["SCALE"] > 0.0)) { err = "fmha_bf16: the softmax scale must be positive"; return false; }
  const int64_t vpad = s.get("VPAD", 32);
  if (vpad < 0 || vpad % 16) { err = "fmha_bf16: VPAD must be a multiple of 16 bytes"; return false; }
  const int64_t lds = 2 * bc * (dh * 2 + 16) + 3 * bc * (dh * 2 + vpad);   // two K buffers, three V buffers
  if (lds > 160 * 1024) { err = "fmha_bf16: tile needs more than 160 KiB of LDS"; return false; }
  const bool causal = s.get("CAUSAL", 0) != 0, outBf16 = s.get("OUT_BF16", 1) != 0;
  const double scale = s.f.count("SCALE") ? s.f["SCALE"] : 1.0;
  s.p["BR"] = br; s.p["BC"] = bc; s.p["QW"] = qw; s.p["CAUSAL"] = causal; s.p["OUT_BF16"] = outBf16;
  s.f["SCALE"] = scale;

  Defines d;
  d.add("FA_NAME", s.name);
  d.add("FA_B", b); d.add("FA_H", h); d.add("FA_S", sl); d.add("FA_D", dh);
  d.add("FA_BR", br); d.add("FA_BC", bc); d.add("FA_QW", qw);
  d.add("FA_CAUSAL", causal ? 1 : 0);
  d.add("FA_C", floatLiteral(scale * 1.4426950408889634));
  d.add("FA_OUT_BF16", outBf16 ? 1 : 0);
  d.add("FA_F16", s.get("F16", 0) ? 1 : 0);
  d.add("FA_VPAD", vpad);
  // K and V tiles straight from global memory into LDS (see the kernel): head dim 128, 64-key tiles, eight wavefronts of
  // 32 queries, whole tiles.  On request for now.
  const bool d2lFits = dh == 128 && bc == 64 && br == 256 && qw == 1 && !ragged;
  const bool d2l = s.get("D2L", 0) != 0;
  if (d2l && !d2lFits) { err = "fmha_bf16: D2L needs head dim 128, BC = 64, BR = 256, QW = 1 and a sequence length that is a multiple of 256"; return false; }
  s.p["D2L"] = d2l;
  if (d2l) d.add("FA_D2L", 1);
  // causal: a workgroup takes a pair of query tiles with the same total number of key tiles, unless asked not to:
  // PAIR = 1 of one head (an even number of query tiles), PAIR = 2 of two heads (an even number of heads; see the kernel)
  // (across two heads by default: the same speed as within one head, 641 against 763 MB of HBM traffic at B8 H32 S2048 D128)
  int64_t pairMode = causal ? s.get("PAIR", (b * h) % 2 == 0 ? 2 : 1) : 0;
  if (pairMode == 2 && (b * h) % 2) pairMode = 1;
  if (pairMode == 1 && ceilDiv(sl, br) % 2) pairMode = 0;
  if (pairMode < 0 || pairMode > 2) { err = "fmha_bf16: PAIR is 0, 1 or 2"; return false; }
  const bool pair = pairMode != 0;
  s.p["PAIR"] = pairMode;
  d.add("FA_PAIR", pairMode);
  // One workgroup per compute unit that works through its query tiles one after the other and fetches the next one's
  // first tiles while it finishes the current one, where every job has the same length (no mask, or pairs) and an even
  // number of key tiles (the fetch sits in the iteration known at compile time to be the last).
  const int64_t nq = ceilDiv(sl, br), items = (pairMode == 2 ? nq * (b * h / 2) : (pair ? nq / 2 : nq) * b * h);
  const bool even = !ragged && (causal ? br % (2 * bc) == 0 : (sl / bc) % 2 == 0);
  // Only where the steady-state form of the iteration exists (64-key tiles, head dim a multiple of 64): measured with the
  // general form alone (head dim 96, 256) the persistent kernel is up to 1.8 times slower than one job per workgroup.
  const bool steady = bc == 64 && dh % 64 == 0 && qw == 1;
  const bool persist = s.get("PERSIST", steady ? 1 : 0) != 0 && (!causal || pair) && even && items > 256;
  s.p["PERSIST"] = persist;
  d.add("FA_PERSIST", persist ? 1 : 0);
  // The result tile goes through LDS to be written in whole rows, where that was measured to pay: not for the pairs of
  // query tiles under a causal mask unless the workgroup is persistent (the second pass runs while the first one's
  // scattered stores drain, and the detour costs time).
  if (s.get("STAGE_O", causal && !persist ? 0 : 1) == 0) d.add("FA_STAGE_O", "0");
  // two wavefronts per SIMD: one workgroup of 8 wavefronts, or two smaller ones when the LDS holds both
  int64_t occ = s.get("OCC", 0);
  if (occ <= 0) occ = (br >= 256 || qw == 2 || 2 * lds > 160 * 1024) ? 1 : 2;
  s.p["OCC"] = occ;
  d.add("FA_OCC", occ);
  src = d.wrap(kTpl_fmha_bf16);

  info.name = s.name;
  info.grid[0] = (uint32_t)(persist ? 256 : items);      // persistent: the compute units of an MI355X
  info.block[0] = (uint32_t)(2 * br / qw);
  info.numArgs = 4;
  // two products of S x S x D per head; a causal mask leaves half of each
  info.flops = 4.0 * (double)b * h * (double)sl * sl * dh * (causal ? 0.5 : 1.0);
  info.bytes = (double)b * h * sl * dh * (3 * 2.0 + (outBf16 ? 2.0 : 4.0));
  return true;
}

bool emitFmhaF32(KernelSpec& s, std::string& src, KernelLaunchInfo& info, std::string& err) {
  if (!need(s, {"B", "H", "S", "D"}, err) || !positive(s, {"B", "H", "S", "D"}, err)) return false;
  const int64_t b = s.p["B"], h = s.p["H"], sl = s.p["S"], dh = s.p["D"];
  if (dh % 32 || dh > 256) { err = "fmha_f32: head dim must be a multiple of 32, at most 256"; return false; }
  // queries per workgroup (32 per wavefront): four wavefronts, fewer for short sequences
  int64_t br = s.get("BR", 0);
  if (br <= 0) br = sl >= 128 ? 128 : (sl > 64 ? 128 : (sl > 32 ? 64 : 32));
  if (br % 32 || br > 512) { err = "fmha_f32: BR must be a multiple of 32, at most 512"; return false; }
  // keys per LDS tile: 64 for head dims above 64 while two workgroups' tiles fit the LDS together, else 32 (measured at
  // B8 H32 S2048: head dim 64 135 against 131 TFLOP/s with 32-key tiles, head dim 128 the same either way)
  int64_t bc = s.get("BC", 0);
  // whole tiles of head dim 64 or 128 can have their K and V tiles straight from global memory into two LDS buffers each
  // (see the kernel): the default at head dim 128 (B8 H32 S2048 causal: 2.70 against 2.80 ms); at head dim 64, where a
  // workgroup's loads are short next to its MFMAs, the two workgroups of a CU hide them as well (2.06 against 2.02 ms)
  const bool d2lShape = (dh == 64 || dh == 128) && sl % br == 0;
  bool d2l = s.get("D2L", dh == 128 ? 1 : 0) != 0 && d2lShape;
  auto ldsOf = [&](int64_t keys) { return d2l ? 4 * keys * dh * 4 : keys * ((dh + 4) + (dh + 8)) * 4; };
  if (bc <= 0) bc = (sl > 32 && dh > 64 && 2 * ldsOf(64) <= 160 * 1024) ? 64 : 32;
  if (bc % 32 || bc <= 0) { err = "fmha_f32: BC must be a multiple of 32"; return false; }
  if (d2l && sl % bc) d2l = false;
  if (ldsOf(bc) > 160 * 1024) { err = "fmha_f32: the key tile needs more than 160 KiB of LDS"; return false; }
  if ((double)ceilDiv(sl, br) * (double)b * (double)h > 2147483647.0) { err = "fmha_f32: too many workgroups"; return false; }
  if ((double)sl * (double)dh >= 2147483648.0) { err = "fmha_f32: a head must have fewer than 2^31 elements"; return false; }
  if (s.f.count("SCALE") && !(s.f["SCALE"] > 0.0)) { err = "fmha_f32: the softmax scale must be positive"; return false; }
  const bool causal = s.get("CAUSAL", 0) != 0;
  const double scale = s.f.count("SCALE") ? s.f["SCALE"] : 1.0;
  // registers: Q fragments and the output accumulators take D / 2 each; beyond D = 128 a wavefront needs the whole file
  int64_t occ = s.get("OCC", 0);
  if (occ <= 0) occ = (dh > 128 || 2 * ldsOf(bc) > 160 * 1024) ? 1 : 2;
  // under the mask a workgroup may take two query tiles of its head, the longest with the shortest (see the kernel)
  const int64_t nq = ceilDiv(sl, br);
  const bool pairFits = causal && nq % 2 == 0;
  // the default once the halved grid still gives every CU its two workgroups (B8 H32 S2048 causal: head dim 128 2.19
  // against 2.70 ms, head dim 64 1.18 against 1.45 ms; on grids smaller than the part it costs parallelism: 20 workgroups
  // instead of 40 at B1 H5 S1024 take 0.129 against 0.114 ms)
  const bool pair = s.get("PAIR", pairFits && (nq / 2) * b * h >= 512 ? 1 : 0) != 0;
  if (pair && !pairFits) { err = "fmha_f32: PAIR needs the causal mask and an even number of query tiles"; return false; }
  s.p["BR"] = br; s.p["BC"] = bc; s.p["CAUSAL"] = causal; s.p["OCC"] = occ; s.p["D2L"] = d2l; s.p["PAIR"] = pair;
  s.f["SCALE"] = scale;

  Defines d;
  d.add("FF_NAME", s.name);
  d.add("FF_PAIR", pair ? 1 : 0);
  d.add("FF_B", b); d.add("FF_H", h); d.add("FF_S", sl); d.add("FF_D", dh);
  d.add("FF_WAVES", br / 32); d.add("FF_BC", bc);
  d.add("FF_CAUSAL", causal ? 1 : 0);
  d.add("FF_C", floatLiteral(scale * 1.4426950408889634));
  d.add("FF_OCC", occ);
  d.add("FF_D2L", d2l ? 1 : 0);
  src = d.wrap(kTpl_fmha_f32);

  info.name = s.name;
  info.grid[0] = (uint32_t)((pair ? nq / 2 : nq) * b * h);
  info.block[0] = (uint32_t)(2 * br);
  info.numArgs = 4;
  info.flops = 4.0 * (double)b * h * (double)sl * sl * dh * (causal ? 0.5 : 1.0);
  info.bytes = (double)b * h * sl * dh * 4 * 4.0;
  return true;
}

}  // namespace

const std::string& prelude() {
  static const std::string text(kTpl_common);
  return text;
}

bool emitKernel(KernelSpec& spec, std::string& src, KernelLaunchInfo& info, std::string& err) {
  src.clear();
  err.clear();
  info = KernelLaunchInfo();
  if (spec.name.empty()) { err = "kernel name is empty"; return false; }
  for (char c : spec.name)
    if (!(isalnum((unsigned char)c) || c == '_')) { err = "kernel name must be a C identifier"; return false; }
  if (spec.family == "layernorm") return emitLayerNorm(spec, src, info, err);
  if (spec.family == "elementwise") return emitElementwise(spec, src, info, err);
  if (spec.family == "binary") return emitBinary(spec, src, info, err);
  if (spec.family == "gather") return emitGather(spec, src, info, err);
  if (spec.family == "softmax") return emitSoftmax(spec, src, info, err);
  if (spec.family == "gemm_f32") return emitGemmF32(spec, src, info, err);
  if (spec.family == "gemm_f64") return emitGemmF64(spec, src, info, err);
  if (spec.family == "gemm_bf16") return emitGemmBf16(spec, src, info, err);
  if (spec.family == "gemm_fp8") return emitGemmFp8(spec, src, info, err);
  if (spec.family == "fmha_bf16") return emitFmhaBf16(spec, src, info, err);
  if (spec.family == "fmha_f32") return emitFmhaF32(spec, src, info, err);
  err = "unknown kernel family '" + spec.family + "'";
  return false;
}

}  // namespace hipgen
}  // namespace KernelCodeGen
