// A reference user's program against this build's headers: the call sequences
// of the reference's own test/test.cc (:8-49 operators, :115-143 flash
// attention; shapes from :20,:28-31,:37-43,:122-133) with platform "ROCm", then
// the emitted text is compiled for gfx950 through the C ABI (no GPU needed).
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <string>
#include <vector>

#include "KernelCodeGen.h"
#include "kcg_hip.h"

using namespace KernelCodeGen;

static int failures = 0;
#define CHECK(cond)                                                        \
  do {                                                                     \
    if (!(cond)) {                                                         \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);        \
      ++failures;                                                          \
    }                                                                      \
  } while (0)

static bool compiles(const std::string& src) {
  void* code = nullptr;
  size_t size = 0;
  char log[4096];
  int rc = kcg_hip_compile_to_code(src.c_str(), nullptr, 0, &code, &size, log, sizeof log);
  if (rc != 0) std::printf("compile log: %s\n", log);
  if (code) kcg_hip_free_code(code);
  return rc == 0 && size > 1000;
}

static void test_elementwise_cast() {
  KernelCodeGenerator generator("ROCm");
  auto graph = generator.createGraph("demo");
  generator.setLogMode(Log::Release);
  generator.opts.push_back(std::move(std::make_unique<ElementWiseOptimizer>()));
  auto A = graph.create<PlaceHolder>(std::vector<int64_t>{2, 768, 768}, std::string{"float32"});
  auto cast = graph.create<ElementWise>(A, "Cast", MemorySpace::global, "int32");
  (void)cast;
  auto module = generator.optimize(graph);
  auto&& sourceCode = generator.codegen(module);
  CHECK(sourceCode.find("extern \"C\" __global__") != std::string::npos);
  CHECK(sourceCode.find("kernel0") != std::string::npos);
  CHECK(generator.launchInfos().size() == 1);
  CHECK(generator.launchInfos()[0].numArgs == 2);
  CHECK(compiles(sourceCode));
  std::printf("ok elementwise_cast\n");
}

static void test_layernorm() {
  KernelCodeGenerator generator("ROCm");
  auto graph = generator.createGraph("demo");
  generator.setLogMode(Log::Release);
  generator.opts.push_back(std::move(std::make_unique<LayerNormOptimizer>()));
  auto A = graph.create<PlaceHolder>(std::vector<int64_t>{2, 768, 768}, std::string{"float32"});
  int64_t axis_ = 1;
  float eps = 1e-5;
  auto scale = graph.create<PlaceHolder>(std::vector<int64_t>{768, 768}, std::string{"float32"});
  auto bias = graph.create<PlaceHolder>(std::vector<int64_t>{768, 768}, std::string{"float32"});
  auto layernorm = graph.create<LayerNorm>(A, scale, bias, axis_, eps);
  (void)layernorm;
  auto module = generator.optimize(graph);
  auto&& sourceCode = generator.codegen(module);
  CHECK(generator.launchInfos().size() == 1);
  CHECK(generator.launchInfos()[0].function == "LayerNorm_2_768_768_axis_1");
  CHECK(generator.launchInfos()[0].numArgs == 4);          // X, scale, bias, Y
  CHECK(compiles(sourceCode));
  std::printf("ok layernorm\n");
}

static void test_matmul_and_save() {
  KernelCodeGenerator generator("ROCm");
  auto graph = generator.createGraph("matmul_demo");
  generator.setLogMode(Log::Release);
  generator.opts.push_back(std::move(std::make_unique<MatmulOptimizer>()));
  int m = 2048, n = 2048, k = 1024;
  auto A = graph.create<PlaceHolder>(std::vector<int64_t>{m, k}, std::string{"float32"});
  auto B = graph.create<PlaceHolder>(std::vector<int64_t>{k, n}, std::string{"float32"});
  auto C = graph.create<Matmul>(A, B);
  (void)C;
  auto module = generator.optimize(graph);
  auto&& sourceCode = generator.codegen(module);
  CHECK(generator.launchInfos().size() == 1);
  const auto& info = generator.launchInfos()[0];
  CHECK(info.name == "kernel0" && info.function == "Matmul_m2048n2048k1024");
  CHECK(info.grid[0] * info.grid[1] * info.grid[2] == (2048 / 128) * (2048 / 128));
  CHECK(sourceCode.find("// grid dims:(") != std::string::npos);
  CHECK(compiles(sourceCode));
  const char* tmp = std::getenv("TMPDIR");
  std::string path = std::string(tmp ? tmp : "/tmp") + "/kcg_test_api_matmul.hip";
  generator.save(sourceCode, path);
  std::ifstream in(path);
  std::string back((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
  CHECK(back == sourceCode);
  std::remove(path.c_str());
  // the module snapshots of the tuning loop
  generator.backupModule(module);
  generator.saveBestModule(module);
  generator.resetModule(module);
  CHECK(!generator.codegen(module).empty());
  std::printf("ok matmul_and_save\n");
}

static void test_batched_matmul_column_major_and_unscheduled() {
  // test/test.cc:41-43: Q K^T of an attention block, B column-major
  {
    KernelCodeGenerator generator("ROCm");
    auto graph = generator.createGraph("demo");
    generator.setLogMode(Log::Release);
    generator.opts.push_back(std::move(std::make_unique<BatchMatmulOptimizer>()));
    auto A = graph.create<PlaceHolder>(std::vector<int64_t>{256, 2048, 64}, std::string{"float32"});
    auto B = graph.create<PlaceHolder>(std::vector<int64_t>{256, 2048, 64}, std::string{"float32"});
    auto C = graph.create<BatchedMatmul>(A, Layout::rowMajor, B, Layout::colMajor);
    (void)C;
    auto module = generator.optimize(graph);
    auto&& sourceCode = generator.codegen(module);
    CHECK(generator.launchInfos().size() == 1);
    if (!generator.launchInfos().empty()) {
      const auto& info = generator.launchInfos()[0];
      CHECK(info.function == "BatchMatmul_256_m2048_n2048_k64_NT");
      CHECK(info.grid[1] == 256);                         // batch on grid.y
    }
    CHECK(sourceCode.find("#define GM_TB 1") != std::string::npos);
    CHECK(compiles(sourceCode));
  }
  // a shape the tile does not divide gets the guarded schedule and a kernel of the GEMM family, which guards its
  // own edges ...
  {
    KernelCodeGenerator generator("ROCm");
    auto graph = generator.createGraph("demo");
    generator.setLogMode(Log::Release);
    generator.opts.push_back(std::move(std::make_unique<BatchMatmulOptimizer>()));
    auto A = graph.create<PlaceHolder>(std::vector<int64_t>{4, 100, 33}, std::string{"float32"});
    auto B = graph.create<PlaceHolder>(std::vector<int64_t>{4, 33, 77}, std::string{"float32"});
    auto C = graph.create<BatchedMatmul>(A, Layout::rowMajor, B, Layout::rowMajor);
    (void)C;
    auto module = generator.optimize(graph);
    auto&& sourceCode = generator.codegen(module);
    CHECK(generator.launchInfos().size() == 1 && generator.error().empty());
    if (!generator.launchInfos().empty()) {
      CHECK(generator.launchInfos()[0].lowering == "family gemm_f32");
      CHECK(generator.launchInfos()[0].grid[1] == 4);
    }
    CHECK(sourceCode.find("#define GM_M 100") != std::string::npos && compiles(sourceCode));
  }
  // ... unless RAGGED = 0 asks for the reference's behaviour: no schedule, the function stays a host nest and the
  // backend emits no kernel for it (and does not fail)
  {
    KernelCodeGenerator generator("ROCm");
    auto graph = generator.createGraph("demo");
    generator.setLogMode(Log::Release);
    generator.opts.push_back(std::move(std::make_unique<BatchMatmulOptimizer>()));
    auto A = graph.create<PlaceHolder>(std::vector<int64_t>{4, 100, 33}, std::string{"float32"});
    auto B = graph.create<PlaceHolder>(std::vector<int64_t>{4, 33, 77}, std::string{"float32"});
    auto C = graph.create<BatchedMatmul>(A, Layout::rowMajor, B, Layout::rowMajor);
    (void)C;
    auto configs = *generator.getConfigs("BatchMatmul");
    for (auto& c : configs) c["RAGGED"] = 0;
    CHECK(generator.setConfigs("BatchMatmul", configs));
    auto module = generator.optimize(graph);
    generator.codegen(module);
    CHECK(generator.launchInfos().empty());
    CHECK(generator.error().empty());
  }
  std::printf("ok batched_matmul\n");
}

static void test_flash_attention() {
  KernelCodeGenerator generator("ROCm");
  auto graph = generator.createGraph("flash_attn_demo");
  generator.setLogMode(Log::Release);
  generator.opts.push_back(std::move(std::make_unique<FMHAOptimizer>()));
  int64_t batch_size = 8, head_num = 32, seq_len = 2048, head_dim = 128;
  auto Q = graph.create<PlaceHolder>(std::vector<int64_t>{batch_size, head_num, seq_len, head_dim}, std::string{"bfloat16"});
  auto K = graph.create<PlaceHolder>(std::vector<int64_t>{batch_size, head_num, seq_len, head_dim}, std::string{"bfloat16"});
  auto V = graph.create<PlaceHolder>(std::vector<int64_t>{batch_size, head_num, seq_len, head_dim}, std::string{"bfloat16"});
  auto S = graph.create<BatchedMatmul>(Q, Layout::rowMajor, K, Layout::colMajor);
  auto P = graph.create<Softmax>(S, -1, MemorySpace::inplace);
  auto O = graph.create<BatchedMatmul>(P, Layout::rowMajor, V, Layout::rowMajor);
  (void)O;
  auto module = generator.optimize(graph);
  auto&& sourceCode = generator.codegen(module);
  CHECK(generator.launchInfos().size() == 1);
  if (!generator.launchInfos().empty()) {
    const auto& info = generator.launchInfos()[0];
    CHECK(info.function.rfind("Fused_Multi_Head_Attention_8_32_SL2048_HD128", 0) == 0);
    CHECK(info.numArgs == 4);                                 // Q, K, V, O
    // 2048 query tiles of 256 rows: more than the part has compute units, so 256 persistent workgroups take eight each
    CHECK(info.block[0] == 512 && info.grid[0] == 256);
  }
  CHECK(sourceCode.find("mfma_f32_32x32x16_bf16") != std::string::npos);
  CHECK(compiles(sourceCode));
  std::printf("ok flash_attention\n");
}

static void test_other_platform_is_an_error() {
  KernelCodeGenerator generator("CUDA");
  auto graph = generator.createGraph("demo");
  generator.setLogMode(Log::Release);
  auto A = graph.create<PlaceHolder>(std::vector<int64_t>{64, 64}, std::string{"float32"});
  auto R = graph.create<Relu>(A, MemorySpace::inplace);
  (void)R;
  auto module = generator.optimize(graph);
  CHECK(generator.codegen(module).empty());
  CHECK(!generator.error().empty());
  std::printf("ok other_platform\n");
}

// test/test.cc:33-35 builds Binary and Gather next to each other; here both, and a Softmax that no attention
// fusion takes, go all the way to kernels, and the adaptor names each of them.
static void test_binary_gather_softmax_and_adaptor() {
  KernelCodeGenerator generator("ROCm");
  auto graph = generator.createGraph("demo");
  generator.setLogMode(Log::Release);
  generator.opts.push_back(std::move(std::make_unique<BinaryOptimizer>()));
  generator.opts.push_back(std::move(std::make_unique<GatherOptimizer>()));
  generator.opts.push_back(std::move(std::make_unique<SoftmaxOptimizer>()));
  auto A = graph.create<PlaceHolder>(std::vector<int64_t>{16, 1, 1, 256}, std::string{"float32"});
  auto B = graph.create<PlaceHolder>(std::vector<int64_t>{1, 128, 256}, std::string{"float32"});
  auto C = graph.create<Binary>(A, B, "Add");
  CHECK(C != nullptr);
  auto table = graph.create<PlaceHolder>(std::vector<int64_t>{1000, 64}, std::string{"float32"});
  auto idx = graph.create<PlaceHolder>(std::vector<int64_t>{4, 8}, std::string{"index"});
  auto rows = graph.create<Gather>(table, idx, 0);
  CHECK(rows != nullptr);
  auto P = graph.create<Softmax>(rows, -1, MemorySpace::inplace);
  CHECK(P != nullptr);
  auto module = generator.optimize(graph);
  auto source = generator.codegen(module);
  CHECK(generator.error().empty());
  CHECK(generator.launchInfos().size() == 3);
  CHECK(compiles(source));
  auto host = generator.adaptor("kernels.hip");
  for (auto& k : generator.launchInfos()) CHECK(host.find("\"" + k.function + "\"") != std::string::npos);
  CHECK(host.find("kcg_hip_time_rotating") != std::string::npos);
  // every kernel carries the operator the generated program checks it against, and its element types
  for (auto& k : generator.launchInfos()) {
    CHECK(!k.check.empty() && k.outputArg >= 0 && k.argTypes.size() == k.argBytes.size());
    CHECK(host.find("\"" + k.function + "\", \"" + k.check + "\"") != std::string::npos);
  }
  CHECK(generator.skippedFunctions().empty());
  // the search's record: one entry per optimizer and configuration
  CHECK(generator.evaluations().size() >= 3);
  std::printf("ok binary_gather_softmax_adaptor\n");
}

// The helper members the reference's optimizer classes declare publicly (include/Optimizer/Optimizer.h:89-108,
// 159-164, 191-192, 221-224, 267): a program that names them compiles and links against the library.  What each
// of them does is checked in tests/cpp/test_rewriter.cc.
static void test_public_optimizer_members_link() {
  KernelCodeGenerator generator("ROCm");
  auto graph = generator.createGraph("members");
  mlir::OpBuilder& builder = graph.builder;
  auto big = graph.create<PlaceHolder>(std::vector<int64_t>{2, 20, 256}, std::string{"float32"});
  auto small = graph.create<PlaceHolder>(std::vector<int64_t>{1, 256}, std::string{"float32"});
  BinaryOptimizer binary;
  BinaryOptimizer::BinaryOpData data;
  binary.getBinaryOpData(big, small, data);
  CHECK(data.type == BinaryOptimizer::BinaryType::hasOneOrder && data.oneDimNums == 1 && data.needDimNums == 1);
  CHECK(binary.getAffineMap("MaxLoadOrStore", builder, {3, 5120, 256, 256, 80}).getNumResults() == 3);
  CHECK(binary.getMinLoadOperands(3, llvm::SmallVector<mlir::Value>{big, small}, nullptr).size() == 2);
  CHECK(GatherOptimizer().getAffineMap("PointLoadOrStore", builder).getNumDims() == 1);
  CHECK(FMHAOptimizer().getAffineMap("loadTileK", builder).getNumResults() == 4);
  // member pointers of the rewrites: taking their addresses needs the definitions at link time
  auto combine = &LayerNormOptimizer::combineParallel;
  auto read = &LayerNormOptimizer::read;
  auto extract = &LayerNormOptimizer::extractOpsFromLoop;
  auto write = &LayerNormOptimizer::write;
  auto reduce = &LayerNormOptimizer::reduceUnrollOptimize;
  auto unroll = &LayerNormOptimizer::elementWiseUnrollOptimize;
  auto hoist = &GatherOptimizer::oneIndexLoad;
  auto softmax = &FMHAOptimizer::softmaxIR;
  auto twoD = &BatchMatmulOptimizer::threadLevelOneToTwo;
  CHECK(combine && read && extract && write && reduce && unroll && hoist && softmax && twoD);
  std::printf("ok public_optimizer_members\n");
}

int main() {
  test_public_optimizer_members_link();
  test_elementwise_cast();
  test_layernorm();
  test_matmul_and_save();
  test_batched_matmul_column_major_and_unscheduled();
  test_flash_attention();
  test_other_platform_is_an_error();
  test_binary_gather_softmax_and_adaptor();
  if (failures) {
    std::printf("%d FAILED\n", failures);
    return 1;
  }
  std::printf("ALL OK\n");
  return 0;
}
