// KernelCodeGenerator::adaptor(): the generated host program (declared in include/KernelCodeGen.h).
// The reference's flow ends with an adaptor and an out-of-tree harness that compiles the saved kernel file,
// checks the result ("correctness") and compares latencies (test/test.cc:69-104, performance/output.log:1-40).
// Here the generator writes that harness itself: a plain C program over include/kcg_hip.h.
#include <sstream>

#include "KernelCodeGen.h"

namespace KernelCodeGen {

namespace {

// Everything of the program that does not depend on the kernels: operand generation, one check routine per
// operator (a plain C evaluation of the operator on a sample of the result, in double precision, from the
// very operands that were uploaded), timing on three operand sets in turn, the report.
const char* const kAdaptorBody = R"KCGADAPTOR(
#define CHECK(call) do { int rc_ = (call); if (rc_) { fprintf(stderr, "%s: %s\n", #call, kcg_hip_strerror(rc_)); return 1; } } while (0)

typedef struct { double err, ref; long n; } acc_t;
static void note(acc_t *a, double got, double want) {
  const double e = fabs(got - want);
  if (!(e <= a->err)) a->err = e;              /* a NaN sticks */
  if (fabs(want) > a->ref) a->ref = fabs(want);
  a->n++;
}
static double elem(const void *p, size_t i, int type) {
  float f = 0.0f;
  if (type == KCG_DT_F64) return ((const double *)p)[i];
  if (type == KCG_DT_I64) return (double)((const long long *)p)[i];
  kcg_host_to_f32((const char *)p + i * kcg_dtype_size(type), &f, 1, type);
  return f;
}
static unsigned long long lcg_state = 0x4B4347ull;
static size_t pick(size_t extent) {             /* a sample position in [0, extent) */
  lcg_state = lcg_state * 6364136223846793005ull + 1442695040888963407ull;
  return (size_t)((lcg_state >> 20) % extent);
}
static double gelu_tanh(double y) { return 0.5 * y * (1.0 + tanh(0.797884 * (y + 0.044715 * y * y * y))); }

/* C[b] = op(A[b]) op(B[b]) (* scale_a * scale_b), optionally max(0, .):  ci = M N K BATCH TA TB RELU */
static void check_gemm(const launch_t *l, void **h, const void *out, const float *scalars, acc_t *a) {
  const long long M = l->ci[0], N = l->ci[1], K = l->ci[2], B = l->ci[3], ta = l->ci[4], tb = l->ci[5], relu = l->ci[6];
  const double scale = l->num_scalars == 2 ? (double)scalars[0] * (double)scalars[1] : 1.0;
  for (int s = 0; s < 384; ++s) {
    const long long b = s < 4 ? (s & 1) * (B - 1) : (long long)pick((size_t)B);
    const long long i = s < 4 ? (s & 2 ? M - 1 : 0) : (long long)pick((size_t)M);
    const long long j = s < 4 ? (s & 1 ? N - 1 : 0) : (long long)pick((size_t)N);
    double sum = 0.0;
    for (long long k = 0; k < K; ++k) {
      const double x = elem(h[0], (size_t)(b * M * K + (ta ? k * M + i : i * K + k)), l->types[0]);
      const double y = elem(h[1], (size_t)(b * K * N + (tb ? j * K + k : k * N + j)), l->types[1]);
      sum += x * y;
    }
    sum *= scale;
    if (relu && sum < 0.0) sum = 0.0;
    note(a, elem(out, (size_t)(b * M * N + i * N + j), l->types[l->output]), sum);
  }
}

/* y = gamma (x - mean) / sqrt(var + eps) + beta over rows of N, biased variance; GELU on top when asked:
 * ci = ROWS N NG NB GELU, cf = eps */
static void check_layernorm(const launch_t *l, void **h, const void *out, acc_t *a) {
  const long long rows = l->ci[0], N = l->ci[1], NG = l->ci[2], NB = l->ci[3], gelu = l->ci[4];
  for (int s = 0; s < 8; ++s) {
    const long long r = s == 0 ? 0 : (s == 1 ? rows - 1 : (long long)pick((size_t)rows));
    double mean = 0.0, var = 0.0;
    for (long long c = 0; c < N; ++c) mean += elem(h[0], (size_t)(r * N + c), l->types[0]);
    mean /= (double)N;
    for (long long c = 0; c < N; ++c) { const double d = elem(h[0], (size_t)(r * N + c), l->types[0]) - mean; var += d * d; }
    const double den = sqrt(var / (double)N + l->cf[0]);
    for (long long c = 0; c < N; ++c) {
      double y = elem(h[1], (size_t)(c % NG), l->types[1]) * ((elem(h[0], (size_t)(r * N + c), l->types[0]) - mean) / den) +
                 elem(h[2], (size_t)(c % NB), l->types[2]);
      if (gelu) y = gelu_tanh(y);
      note(a, elem(out, (size_t)(r * N + c), l->types[l->output]), y);
    }
  }
}

/* ci = N OP (0 Tanh, 1 Sqrt, 2 Log, 3 Relu, 4 Gelu, 5 Cast) */
static void check_elementwise(const launch_t *l, void **h, const void *out, acc_t *a) {
  const long long N = l->ci[0], op = l->ci[1];
  for (int s = 0; s < 4096; ++s) {
    const size_t i = s == 0 ? 0 : (s == 1 ? (size_t)N - 1 : pick((size_t)N));
    const double x = elem(h[0], i, l->types[0]);
    double y = x;
    switch (op) {
      case 0: y = tanh(x); break;
      case 1: y = sqrt(x); break;
      case 2: y = log(x); break;
      case 3: y = x > 0.0 ? x : 0.0; break;
      case 4: y = gelu_tanh(x); break;
      case 5: y = l->types[l->output] == KCG_DT_F32 ? x : trunc(x); break;
    }
    note(a, elem(out, i, l->types[l->output]), y);
  }
}

/* softmax over rows of N: ci = ROWS N */
static void check_softmax(const launch_t *l, void **h, const void *out, acc_t *a) {
  const long long rows = l->ci[0], N = l->ci[1];
  for (int s = 0; s < 8; ++s) {
    const long long r = s == 0 ? 0 : (s == 1 ? rows - 1 : (long long)pick((size_t)rows));
    double top = -INFINITY, sum = 0.0;
    for (long long c = 0; c < N; ++c) { const double x = elem(h[0], (size_t)(r * N + c), l->types[0]); if (x > top) top = x; }
    for (long long c = 0; c < N; ++c) sum += exp(elem(h[0], (size_t)(r * N + c), l->types[0]) - top);
    for (long long c = 0; c < N; ++c)
      note(a, elem(out, (size_t)(r * N + c), l->types[l->output]), exp(elem(h[0], (size_t)(r * N + c), l->types[0]) - top) / sum);
  }
}

/* O = softmax(scale Q K^T [keys up to the query only]) V per (batch, head): ci = B H S D CAUSAL, cf = scale */
static void check_fmha(const launch_t *l, void **h, const void *out, acc_t *a) {
  const long long B = l->ci[0], H = l->ci[1], S = l->ci[2], D = l->ci[3], causal = l->ci[4];
  double *p = (double *)malloc((size_t)S * sizeof(double));
  if (!p) return;
  for (int s = 0; s < 8; ++s) {
    const long long bh = s < 2 ? s * (B * H - 1) : (long long)pick((size_t)(B * H));
    const long long q = s == 0 ? 0 : (s == 1 ? S - 1 : (long long)pick((size_t)S));
    const long long keys = causal ? q + 1 : S;
    const size_t base = (size_t)(bh * S * D);
    double top = -INFINITY, sum = 0.0;
    for (long long j = 0; j < keys; ++j) {
      double dot = 0.0;
      for (long long d = 0; d < D; ++d)
        dot += elem(h[0], base + (size_t)(q * D + d), l->types[0]) * elem(h[1], base + (size_t)(j * D + d), l->types[1]);
      p[j] = dot * l->cf[0];
      if (p[j] > top) top = p[j];
    }
    for (long long j = 0; j < keys; ++j) { p[j] = exp(p[j] - top); sum += p[j]; }
    for (long long d = 0; d < D; ++d) {
      double o = 0.0;
      for (long long j = 0; j < keys; ++j) o += p[j] * elem(h[2], base + (size_t)(j * D + d), l->types[2]);
      note(a, elem(out, base + (size_t)(q * D + d), l->types[l->output]), o / sum);
    }
  }
  free(p);
}

/* z = x op y with broadcasting: ci = RANK OP dims[6] strides_x[6] strides_y[6]; OP: 0 Add 1 Sub 2 Mul 3 Div 4 Pow
 * 5 Equal 6 Greater (the last two give one byte per element) */
static void check_binary(const launch_t *l, void **h, const void *out, acc_t *a) {
  const long long rank = l->ci[0], op = l->ci[1];
  const long long *dims = l->ci + 2, *sx = l->ci + 8, *sy = l->ci + 14;
  size_t total = 1;
  for (long long d = 0; d < rank; ++d) total *= (size_t)dims[d];
  for (int s = 0; s < 4096; ++s) {
    const size_t i = s == 0 ? 0 : (s == 1 ? total - 1 : pick(total));
    size_t rest = i, ix = 0, iy = 0;
    for (long long d = rank - 1; d >= 0; --d) {
      const size_t c = rest % (size_t)dims[d];
      rest /= (size_t)dims[d];
      ix += c * (size_t)sx[d];
      iy += c * (size_t)sy[d];
    }
    const double x = elem(h[0], ix, l->types[0]), y = elem(h[1], iy, l->types[1]);
    double z = 0.0;
    switch (op) {
      case 0: z = x + y; break;
      case 1: z = x - y; break;
      case 2: z = x * y; break;
      case 3: z = x / y; break;
      case 4: z = pow(x, y); break;
      case 5: z = x == y; break;
      case 6: z = x > y; break;
    }
    note(a, elem(out, i, l->types[l->output]), z);
  }
}

/* out[o][i][:] = in[o][idx[i]][:], rows of ROWBYTES bytes: ci = OUTER AXIS NIDX ROWBYTES; err counts rows that differ */
static void check_gather(const launch_t *l, void **h, const void *out, acc_t *a) {
  const long long outer = l->ci[0], axis = l->ci[1], nidx = l->ci[2], row = l->ci[3];
  for (int s = 0; s < 256; ++s) {
    const long long o = (long long)pick((size_t)outer), i = s == 0 ? 0 : (s == 1 ? nidx - 1 : (long long)pick((size_t)nidx));
    long long j = ((const long long *)h[1])[i];
    j = j < 0 ? 0 : (j >= axis ? axis - 1 : j);
    const int same = memcmp((const char *)out + (size_t)((o * nidx + i) * row), (const char *)h[0] + (size_t)((o * axis + j) * row),
                            (size_t)row) == 0;
    note(a, same ? 1.0 : 0.0, 1.0);
  }
}

int main(int argc, char **argv) {
  const int iters = argc > 1 ? atoi(argv[1]) : 20;
  int failures = 0;
  FILE *f = fopen(kernel_file, "rb");
  if (!f) { fprintf(stderr, "cannot open %s\n", kernel_file); return 1; }
  fseek(f, 0, SEEK_END);
  long size = ftell(f);
  fseek(f, 0, SEEK_SET);
  char *source = (char *)malloc((size_t)size + 1);
  if (!source || fread(source, 1, (size_t)size, f) != (size_t)size) { fprintf(stderr, "cannot read %s\n", kernel_file); return 1; }
  source[size] = 0;
  fclose(f);
  static char log[1 << 16];
  kcg_module_t module;
  CHECK(kcg_hip_init(0));
  if (kcg_hip_compile(source, NULL, 0, &module, log, sizeof log)) { fputs(log, stderr); return 1; }
  for (size_t n = 0; n < sizeof launches / sizeof launches[0]; ++n) {
    const launch_t *l = &launches[n];
    if (l->num_buffers > MAX_BUFFERS || l->num_scalars > 2) { fprintf(stderr, "%s: too many arguments\n", l->name); return 1; }
    kcg_kernel_t kernel;
    CHECK(kcg_hip_get_kernel(module, l->name, &kernel));
    /* operands: stream i + 1 of the seeded generator, U(fill_lo, fill_hi); e4m3 operands are spread over the
     * format's range (x 448 / max|.|) and the two per-tensor scales undo that */
    const double top = fabs(l->fill_lo) > fabs(l->fill_hi) ? fabs(l->fill_lo) : fabs(l->fill_hi);
    void *host[MAX_BUFFERS];
    size_t set_bytes = 0;
    for (int i = 0; i < l->num_buffers; ++i) {
      host[i] = malloc(l->bytes[i]);
      if (!host[i]) { fprintf(stderr, "%s: out of host memory\n", l->name); return 1; }
      if (i == l->workspace) memset(host[i], 0, l->bytes[i]);     /* scratch shared by the workgroups: counters start at zero */
      else
        CHECK(kcg_host_fill(host[i], l->bytes[i] / kcg_dtype_size(l->types[i]), l->types[i], KCG_DIST_UNIFORM, 0x4B4347ull,
                            (uint64_t)(i + 1), (float)l->fill_lo, (float)l->fill_hi,
                            l->types[i] == KCG_DT_F8E4M3 ? (float)(448.0 / top) : 1.0f));
      set_bytes += l->bytes[i];
    }
    float scalars[2] = {(float)(top / 448.0), (float)(top / 448.0)};
    const int num_sets = set_bytes * 3 <= ((size_t)6 << 30) ? 3 : 1;
    void *buffers[3][MAX_BUFFERS];
    void *args[3][MAX_BUFFERS + 2];
    void **arg_sets[3];
    for (int s = 0; s < num_sets; ++s) {
      for (int i = 0; i < l->num_buffers; ++i) {
        CHECK(kcg_hip_malloc(&buffers[s][i], l->bytes[i]));
        CHECK(kcg_hip_memcpy_h2d(buffers[s][i], host[i], l->bytes[i]));
        args[s][i] = &buffers[s][i];
      }
      for (int i = 0; i < l->num_scalars; ++i) args[s][l->num_buffers + i] = &scalars[i];
      arg_sets[s] = args[s];
    }
    /* one launch, checked against the operator evaluated on the host */
    acc_t acc = {0.0, 0.0, 0};
    double tolerance = 0.0;
    if (l->check[0] && l->output >= 0) {
      CHECK(kcg_hip_launch(kernel, l->grid, l->block, l->lds_bytes, NULL, args[0]));
      CHECK(kcg_hip_device_synchronize());
      void *out = malloc(l->bytes[l->output]);
      if (!out) { fprintf(stderr, "%s: out of host memory\n", l->name); return 1; }
      CHECK(kcg_hip_memcpy_d2h(out, buffers[0][l->output], l->bytes[l->output]));
      const int narrow_in = l->types[0] != KCG_DT_F32 && l->types[0] != KCG_DT_F64;
      const int narrow_out = l->types[l->output] == KCG_DT_BF16 || l->types[l->output] == KCG_DT_F16;
      tolerance = narrow_out ? 1e-2 : (narrow_in ? 1e-3 : 1e-4);
      if (!strcmp(l->check, "gemm")) check_gemm(l, host, out, scalars, &acc);
      else if (!strcmp(l->check, "layernorm")) check_layernorm(l, host, out, &acc);
      else if (!strcmp(l->check, "elementwise")) check_elementwise(l, host, out, &acc);
      else if (!strcmp(l->check, "softmax")) check_softmax(l, host, out, &acc);
      else if (!strcmp(l->check, "fmha")) { check_fmha(l, host, out, &acc); tolerance = 2e-2; }
      else if (!strcmp(l->check, "binary")) check_binary(l, host, out, &acc);
      else if (!strcmp(l->check, "gather")) { check_gather(l, host, out, &acc); tolerance = 0.0; }
      free(out);
      if (l->output < l->num_buffers)          /* an in-place operator has overwritten its operand */
        CHECK(kcg_hip_memcpy_h2d(buffers[0][l->output], host[l->output], l->bytes[l->output]));
    }
    float ms = 0.0f;
    CHECK(kcg_hip_time_rotating(kernel, l->grid, l->block, l->lds_bytes, NULL, arg_sets, num_sets, 3, 20.0f, 5, iters, &ms, NULL));
    printf("%s (%s) Latency = %g ms", l->name, l->function, ms);
    if (l->flops > 0) printf(", %g TFLOP/s", l->flops / (ms * 1e-3) / 1e12);
    if (l->hbm_bytes > 0) printf(", %g GB/s of algorithmic traffic", l->hbm_bytes / (ms * 1e-3) / 1e9);
    if (acc.n > 0) {
      const double rel = acc.ref > 0.0 ? acc.err / acc.ref : acc.err;
      const int ok = rel <= tolerance;             /* false for a NaN */
      printf(", max rel err = %.3g over %ld sampled results (tolerance %g), correctness: %s", rel, acc.n, tolerance,
             ok ? "Done" : "FAILED");
      failures += !ok;
    } else {
      printf(", correctness: not checked");
    }
    printf("\n");
    for (int s = 0; s < num_sets; ++s)
      for (int i = 0; i < l->num_buffers; ++i) CHECK(kcg_hip_free(buffers[s][i]));
    for (int i = 0; i < l->num_buffers; ++i) free(host[i]);
  }
  CHECK(kcg_hip_module_destroy(module));
  free(source);
  return failures ? 2 : 0;
}
)KCGADAPTOR";

}  // namespace

std::string KernelCodeGenerator::adaptor(const std::string& kernelFile) const {
  std::ostringstream os;
  os << "/* Generated by KernelCodeGenerator::adaptor(): checks and times the kernels of \"" << kernelFile << "\". */\n"
     << "#include <math.h>\n#include <stdint.h>\n#include <stdio.h>\n#include <stdlib.h>\n#include <string.h>\n#include \"kcg_hip.h\"\n\n"
     << "#define MAX_BUFFERS 8\n"
     << "typedef struct {\n  const char *name, *function, *check;\n  uint32_t grid[3], block[3], lds_bytes;\n"
     << "  int num_buffers, num_scalars, output, workspace;\n  size_t bytes[MAX_BUFFERS];\n  int types[MAX_BUFFERS];\n"
     << "  double flops, hbm_bytes, fill_lo, fill_hi;\n  long long ci[24];\n  double cf[2];\n} launch_t;\n\n"
     << "static const char *kernel_file = \"";
  for (char c : kernelFile) { if (c == '\\' || c == '"') os << '\\'; os << c; }
  os << "\";\nstatic const launch_t launches[] = {\n";
  os.precision(17);
  for (const auto& k : lastLaunchInfos) {
    os << "  {\"" << k.name << "\", \"" << k.function << "\", \"" << k.check << "\", {" << k.grid[0] << ", " << k.grid[1] << ", "
       << k.grid[2] << "}, {" << k.block[0] << ", " << k.block[1] << ", " << k.block[2] << "}, " << k.ldsBytes << ", "
       << k.argBytes.size() << ", " << k.numScalars << ", " << k.outputArg << ", " << k.workspaceArg << ", {";
    for (size_t i = 0; i < k.argBytes.size(); ++i) os << (i ? ", " : "") << k.argBytes[i];
    os << "}, {";
    for (size_t i = 0; i < k.argTypes.size(); ++i) os << (i ? ", " : "") << k.argTypes[i];
    os << "}, " << k.flops << ", " << k.bytes << ", " << k.fillLo << ", " << k.fillHi << ", {";
    for (size_t i = 0; i < k.checkInts.size() && i < 24; ++i) os << (i ? ", " : "") << k.checkInts[i] << "LL";
    if (k.checkInts.empty()) os << "0";
    os << "}, {";
    for (size_t i = 0; i < k.checkFloats.size() && i < 2; ++i) os << (i ? ", " : "") << k.checkFloats[i];
    if (k.checkFloats.empty()) os << "0";
    os << "}},\n";
  }
  os << "};\n" << kAdaptorBody;
  return os.str();
}

}  // namespace KernelCodeGen
