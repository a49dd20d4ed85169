// C-ABI runtime over hipRTC and hipModule for the emitted gfx950 kernels.
// Declared in include/kcg_hip.h.  Host code only; no device code lives here.
#include "kcg_hip.h"

#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>

#include <dirent.h>
#include <dlfcn.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "runtime/kcg_handles.h"

namespace {

inline int hipErr(hipError_t e) { return e == hipSuccess ? KCG_OK : (KCG_ERR_DOMAIN_HIP | (int)e); }
inline int rtcErr(hiprtcResult r) { return r == HIPRTC_SUCCESS ? KCG_OK : (KCG_ERR_DOMAIN_HIPRTC | (int)r); }

// The kernels are compiled by the ROCm installation's hipRTC, whatever else the process has loaded.  A host
// program may carry a hipRTC of its own under the same soname (the PyTorch wheel bundles one, with an older
// compiler whose code for the same kernel source runs up to 20 % differently); the loader would then hand that
// one to every later user.  The installation's library (and the code-object manager it opens) is therefore
// loaded into a link-map namespace of its own.  KCG_HIPRTC_LIBRARY names another file; if the isolated load
// fails, the process-wide libhiprtc is used.
struct Rtc {
  decltype(&hiprtcCreateProgram) createProgram = nullptr;
  decltype(&hiprtcCompileProgram) compileProgram = nullptr;
  decltype(&hiprtcGetProgramLogSize) getProgramLogSize = nullptr;
  decltype(&hiprtcGetProgramLog) getProgramLog = nullptr;
  decltype(&hiprtcGetCodeSize) getCodeSize = nullptr;
  decltype(&hiprtcGetCode) getCode = nullptr;
  decltype(&hiprtcDestroyProgram) destroyProgram = nullptr;
  decltype(&hiprtcGetErrorString) getErrorString = nullptr;
  decltype(&hiprtcVersion) version = nullptr;
  std::string origin;       // file the functions come from and how it was loaded
  bool ok = false;
  char ***privateEnviron = nullptr;   // `environ` of the C library inside the private namespace, if there is one
};

bool bindRtc(void *handle, Rtc &t) {
  auto sym = [&](const char *name) { return dlsym(handle, name); };
  t.createProgram = (decltype(t.createProgram))sym("hiprtcCreateProgram");
  t.compileProgram = (decltype(t.compileProgram))sym("hiprtcCompileProgram");
  t.getProgramLogSize = (decltype(t.getProgramLogSize))sym("hiprtcGetProgramLogSize");
  t.getProgramLog = (decltype(t.getProgramLog))sym("hiprtcGetProgramLog");
  t.getCodeSize = (decltype(t.getCodeSize))sym("hiprtcGetCodeSize");
  t.getCode = (decltype(t.getCode))sym("hiprtcGetCode");
  t.destroyProgram = (decltype(t.destroyProgram))sym("hiprtcDestroyProgram");
  t.getErrorString = (decltype(t.getErrorString))sym("hiprtcGetErrorString");
  t.version = (decltype(t.version))sym("hiprtcVersion");
  return t.createProgram && t.compileProgram && t.getProgramLogSize && t.getProgramLog && t.getCodeSize &&
         t.getCode && t.destroyProgram && t.getErrorString && t.version;
}

const Rtc &rtc() {
  static Rtc table;
  static std::once_flag once;
  std::call_once(once, [] {
    std::string path;
    if (const char *e = getenv("KCG_HIPRTC_LIBRARY")) path = e;
    if (path.empty()) {
      const char *root = getenv("ROCM_PATH");
      path = std::string(root && *root ? root : "/opt/rocm") + "/lib/libhiprtc.so.7";
    }
    if (void *h = dlmopen(LM_ID_NEWLM, path.c_str(), RTLD_NOW | RTLD_LOCAL)) {
      if (bindRtc(h, table)) {
        table.origin = path + " (own namespace)";
        table.ok = true;
        table.privateEnviron = (char ***)dlsym(h, "environ");
        return;
      }
    }
    if (void *h = dlopen("libhiprtc.so.7", RTLD_NOW | RTLD_LOCAL)) {
      if (bindRtc(h, table)) {
        table.origin = "libhiprtc.so.7 (as the process resolves it)";
        table.ok = true;
        return;
      }
    }
    table.origin = "hipRTC not found";
  });
  // A namespace of its own has a C library of its own, whose `environ` still points at the array the process
  // had when the namespace was made; a setenv since then may have moved the array.  hipRTC reads the
  // environment on most of its entry points, so every use of the table hands it the current array first.
  if (table.privateEnviron) *table.privateEnviron = environ;
  return table;
}

// SHA-256 (FIPS 180-4) of a byte string, as lower-case hex: the key of the on-disk code-object cache.
std::string sha256Hex(const std::string &data) {
  static const uint32_t K[64] = {
      0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5, 0xd807aa98, 0x12835b01,
      0x243185be, 0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174, 0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc,
      0x2de92c6f, 0x4a7484aa, 0x5cb0a9dc, 0x76f988da, 0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147,
      0x06ca6351, 0x14292967, 0x27b70a85, 0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85,
      0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3, 0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070, 0x19a4c116, 0x1e376c08,
      0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f, 0x682e6ff3, 0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208,
      0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};
  uint32_t h[8] = {0x6a09e667, 0xbb67ae85, 0x3c6ef372, 0xa54ff53a, 0x510e527f, 0x9b05688c, 0x1f83d9ab, 0x5be0cd19};
  std::string msg = data;
  const uint64_t bitLen = (uint64_t)data.size() * 8;
  msg.push_back((char)0x80);
  while (msg.size() % 64 != 56) msg.push_back('\0');
  for (int i = 7; i >= 0; --i) msg.push_back((char)(bitLen >> (8 * i)));
  auto rotr = [](uint32_t x, int n) { return (x >> n) | (x << (32 - n)); };
  for (size_t off = 0; off < msg.size(); off += 64) {
    uint32_t w[64];
    for (int i = 0; i < 16; ++i) {
      const unsigned char *b = (const unsigned char *)msg.data() + off + 4 * i;
      w[i] = ((uint32_t)b[0] << 24) | ((uint32_t)b[1] << 16) | ((uint32_t)b[2] << 8) | (uint32_t)b[3];
    }
    for (int i = 16; i < 64; ++i) {
      const uint32_t s0 = rotr(w[i - 15], 7) ^ rotr(w[i - 15], 18) ^ (w[i - 15] >> 3);
      const uint32_t s1 = rotr(w[i - 2], 17) ^ rotr(w[i - 2], 19) ^ (w[i - 2] >> 10);
      w[i] = w[i - 16] + s0 + w[i - 7] + s1;
    }
    uint32_t a = h[0], b = h[1], c = h[2], d = h[3], e = h[4], f = h[5], g = h[6], hh = h[7];
    for (int i = 0; i < 64; ++i) {
      const uint32_t t1 = hh + (rotr(e, 6) ^ rotr(e, 11) ^ rotr(e, 25)) + ((e & f) ^ (~e & g)) + K[i] + w[i];
      const uint32_t t2 = (rotr(a, 2) ^ rotr(a, 13) ^ rotr(a, 22)) + ((a & b) ^ (a & c) ^ (b & c));
      hh = g; g = f; f = e; e = d + t1; d = c; c = b; b = a; a = t1 + t2;
    }
    h[0] += a; h[1] += b; h[2] += c; h[3] += d; h[4] += e; h[5] += f; h[6] += g; h[7] += hh;
  }
  char hex[65];
  for (int i = 0; i < 8; ++i) snprintf(hex + 8 * i, 9, "%08x", h[i]);
  return std::string(hex, 64);
}

// KCG_CACHE_DIR, or "_cache" beside the shared object this function lives in.
std::string cacheDir() {
  if (const char *e = getenv("KCG_CACHE_DIR"))
    if (*e) return e;
  Dl_info where;
  if (dladdr((const void *)&sha256Hex, &where) && where.dli_fname) {
    std::string path = where.dli_fname;
    const size_t slash = path.rfind('/');
    return (slash == std::string::npos ? std::string(".") : path.substr(0, slash)) + "/_cache";
  }
  return "_cache";
}

// The cache directory is bounded: after a new object is written, the oldest objects (by modification time) are
// removed until the directory's *.hsaco files add up to at most nine tenths of KCG_CACHE_MAX_MB (default 1024; 0 or a
// negative value: no bound).  A config search writes one object per candidate, which is what fills it.
void trimCache(const std::string &dir, const std::string &keep) {
  long long cap = 1024;
  if (const char *e = getenv("KCG_CACHE_MAX_MB"))
    if (*e) cap = atoll(e);
  if (cap <= 0) return;
  cap *= 1024 * 1024;
  DIR *d = opendir(dir.c_str());
  if (!d) return;
  struct Entry { time_t mtime; long long size; std::string path; };
  std::vector<Entry> entries;
  long long total = 0;
  while (const dirent *e = readdir(d)) {
    const std::string name = e->d_name;
    if (name.size() < 6 || name.compare(name.size() - 6, 6, ".hsaco") != 0) continue;
    const std::string path = dir + "/" + name;
    struct stat st;
    if (stat(path.c_str(), &st) != 0 || !S_ISREG(st.st_mode)) continue;
    total += (long long)st.st_size;
    if (path != keep) entries.push_back({st.st_mtime, (long long)st.st_size, path});
  }
  closedir(d);
  if (total <= cap) return;
  std::sort(entries.begin(), entries.end(), [](const Entry &a, const Entry &b) {
    return a.mtime != b.mtime ? a.mtime < b.mtime : a.path < b.path;
  });
  for (const Entry &e : entries) {
    if (total <= cap / 10 * 9) break;
    if (remove(e.path.c_str()) == 0) total -= e.size;
  }
}

void copyLog(const std::string &text, char *log, size_t cap) {
  if (!log || cap == 0) return;
  size_t n = text.size() < cap - 1 ? text.size() : cap - 1;
  memcpy(log, text.data(), n);
  log[n] = '\0';
}

}  // namespace

extern "C" {

int kcg_hip_init(int device) {
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) return hipErr(e);
  if (n <= 0 || device < 0 || device >= n) return KCG_ERR_NO_DEVICE;
  e = hipSetDevice(device);
  if (e != hipSuccess) return hipErr(e);
  e = hipFree(nullptr);  // forces context creation
  if (e != hipSuccess) return hipErr(e);
  return kcg_scratch_setup();   // this device's address of the library's scratch array (kcg_hip_launch_scratch)
}

int kcg_hip_device_count(int *count) {
  if (!count) return KCG_ERR_INVALID_ARGUMENT;
  *count = 0;
  hipError_t e = hipGetDeviceCount(count);
  if (e == hipErrorNoDevice) { *count = 0; return KCG_OK; }
  return hipErr(e);
}

int kcg_hip_device_name(int device, char *name, size_t cap) {
  if (!name || cap == 0) return KCG_ERR_INVALID_ARGUMENT;
  hipDeviceProp_t prop;
  hipError_t e = hipGetDeviceProperties(&prop, device);
  if (e != hipSuccess) return hipErr(e);
  snprintf(name, cap, "%s (%s)", prop.name, prop.gcnArchName);
  return KCG_OK;
}

// The options every compilation gets in front of the caller's.  They are part of the on-disk cache's key: a
// library that changes them does not find the code objects of one that had others.
// "-packed-fp32-ops" switched off keeps hipcc from forming packed fp32 ops out of scalar float code.
static const char *const kBuiltinOptions[] = {"--offload-arch=gfx950", "-O3", "-Xclang", "-target-feature",
                                              "-Xclang", "-packed-fp32-ops"};

int kcg_hip_compile_to_code(const char *src, const char *const *opts, int nopts,
                            void **code, size_t *code_size, char *log, size_t log_cap) {
  if (log && log_cap) log[0] = '\0';
  if (!src || !code || !code_size || nopts < 0 || (nopts > 0 && !opts)) return KCG_ERR_INVALID_ARGUMENT;
  *code = nullptr;
  *code_size = 0;
  const Rtc &R = rtc();
  if (!R.ok) {
    copyLog("no usable libhiprtc: " + R.origin, log, log_cap);
    return KCG_ERR_NO_COMPILER;
  }
  hiprtcProgram prog;
  hiprtcResult r = R.createProgram(&prog, src, "kcg_kernels.hip", 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) return rtcErr(r);
  std::vector<const char *> all(std::begin(kBuiltinOptions), std::end(kBuiltinOptions));
  for (int i = 0; i < nopts; ++i) all.push_back(opts[i]);
  r = R.compileProgram(prog, (int)all.size(), all.data());
  size_t logSize = 0;
  R.getProgramLogSize(prog, &logSize);
  if (logSize > 1) {
    std::string text(logSize, '\0');
    R.getProgramLog(prog, &text[0]);
    copyLog(text, log, log_cap);
  }
  if (r != HIPRTC_SUCCESS) {
    R.destroyProgram(&prog);
    return rtcErr(r);
  }
  size_t size = 0;
  r = R.getCodeSize(prog, &size);
  if (r != HIPRTC_SUCCESS) { R.destroyProgram(&prog); return rtcErr(r); }
  void *buf = malloc(size);
  if (!buf) { R.destroyProgram(&prog); return KCG_ERR_OUT_OF_HOST_MEMORY; }
  r = R.getCode(prog, (char *)buf);
  R.destroyProgram(&prog);
  if (r != HIPRTC_SUCCESS) { free(buf); return rtcErr(r); }
  *code = buf;
  *code_size = size;
  return KCG_OK;
}

void kcg_hip_free_code(void *code) { free(code); }

int kcg_hip_cache_dir(char *path, size_t cap) {
  if (!path || cap == 0) return KCG_ERR_INVALID_ARGUMENT;
  const std::string dir = cacheDir();
  if (dir.size() + 1 > cap) return KCG_ERR_LOG_TRUNCATED;
  memcpy(path, dir.c_str(), dir.size() + 1);
  return KCG_OK;
}

int kcg_hip_compile_to_code_cached(const char *src, const char *const *opts, int nopts, int refresh,
                                   void **code, size_t *code_size, char *log, size_t log_cap) {
  if (log && log_cap) log[0] = '\0';
  if (!src || !code || !code_size || nopts < 0 || (nopts > 0 && !opts)) return KCG_ERR_INVALID_ARGUMENT;
  char compiler[512];
  if (kcg_hip_compiler_info(compiler, sizeof compiler) != KCG_OK) compiler[0] = '\0';
  std::string key(compiler);
  key.push_back('\0');
  key += src;
  for (const char *o : kBuiltinOptions) {      // the full option vector the compiler sees, not only the caller's part
    key.push_back('\0');
    key += o;
  }
  for (int i = 0; i < nopts; ++i) {
    key.push_back('\0');
    key += opts[i];
  }
  const std::string dir = cacheDir();
  const std::string path = dir + "/" + sha256Hex(key).substr(0, 32) + ".hsaco";
  if (!refresh) {
    if (FILE *f = fopen(path.c_str(), "rb")) {
      fseek(f, 0, SEEK_END);
      const long size = ftell(f);
      fseek(f, 0, SEEK_SET);
      void *buf = size > 0 ? malloc((size_t)size) : nullptr;
      const bool ok = buf && fread(buf, 1, (size_t)size, f) == (size_t)size;
      fclose(f);
      if (ok) {
        *code = buf;
        *code_size = (size_t)size;
        return KCG_OK;
      }
      free(buf);
    }
  }
  int rc = kcg_hip_compile_to_code(src, opts, nopts, code, code_size, log, log_cap);
  if (rc != KCG_OK) return rc;
  // written under a private name and renamed: readers never see a partial file
  mkdir(dir.c_str(), 0777);
  const std::string tmp = path + ".tmp" + std::to_string((long)getpid());
  if (FILE *f = fopen(tmp.c_str(), "wb")) {
    const bool ok = fwrite(*code, 1, *code_size, f) == *code_size;
    if (fclose(f) == 0 && ok) {
      if (rename(tmp.c_str(), path.c_str()) == 0) trimCache(dir, path);
    } else {
      remove(tmp.c_str());
    }
  }
  return KCG_OK;
}

int kcg_hip_compile_cached(const char *src, const char *const *opts, int nopts,
                           kcg_module_t *out, char *log, size_t log_cap) {
  if (!out) return KCG_ERR_INVALID_ARGUMENT;
  *out = nullptr;
  void *code = nullptr;
  size_t size = 0;
  int rc = kcg_hip_compile_to_code_cached(src, opts, nopts, 0, &code, &size, log, log_cap);
  if (rc != KCG_OK) return rc;
  rc = kcg_hip_load_code(code, size, out);
  free(code);
  return rc;
}

int kcg_hip_compiler_info(char *text, size_t cap) {
  if (!text || cap == 0) return KCG_ERR_INVALID_ARGUMENT;
  const Rtc &R = rtc();
  int major = 0, minor = 0;
  if (R.ok) R.version(&major, &minor);
  snprintf(text, cap, "hipRTC %d.%d from %s", major, minor, R.origin.c_str());
  return R.ok ? KCG_OK : KCG_ERR_NO_COMPILER;
}

int kcg_hip_load_code(const void *code, size_t code_size, kcg_module_t *out) {
  if (!code || code_size == 0 || !out) return KCG_ERR_INVALID_ARGUMENT;
  *out = nullptr;
  kcg_module_s *m = new (std::nothrow) kcg_module_s;
  if (!m) return KCG_ERR_OUT_OF_HOST_MEMORY;
  hipError_t e = hipModuleLoadData(&m->mod, code);
  if (e != hipSuccess) { delete m; return hipErr(e); }
  *out = m;
  return KCG_OK;
}

int kcg_hip_compile(const char *src, const char *const *opts, int nopts,
                    kcg_module_t *out, char *log, size_t log_cap) {
  if (!out) return KCG_ERR_INVALID_ARGUMENT;
  *out = nullptr;
  void *code = nullptr;
  size_t size = 0;
  int rc = kcg_hip_compile_to_code(src, opts, nopts, &code, &size, log, log_cap);
  if (rc != KCG_OK) return rc;
  rc = kcg_hip_load_code(code, size, out);
  free(code);
  return rc;
}

int kcg_hip_get_kernel(kcg_module_t module, const char *name, kcg_kernel_t *out) {
  if (!module || !name || !out) return KCG_ERR_INVALID_ARGUMENT;
  *out = nullptr;
  hipFunction_t fn;
  hipError_t e = hipModuleGetFunction(&fn, module->mod, name);
  if (e != hipSuccess) return hipErr(e);
  kcg_kernel_s *k = new (std::nothrow) kcg_kernel_s;
  if (!k) return KCG_ERR_OUT_OF_HOST_MEMORY;
  k->fn = fn;
  module->kernels.push_back(k);
  *out = k;
  return KCG_OK;
}

static int checkDims(const uint32_t grid[3], const uint32_t block[3]) {
  if (!grid || !block) return KCG_ERR_INVALID_ARGUMENT;
  for (int i = 0; i < 3; ++i)
    if (grid[i] == 0 || block[i] == 0) return KCG_ERR_INVALID_ARGUMENT;
  if ((uint64_t)block[0] * block[1] * block[2] > 1024) return KCG_ERR_INVALID_ARGUMENT;
  return KCG_OK;
}

int kcg_hip_launch(kcg_kernel_t kernel, const uint32_t grid[3], const uint32_t block[3],
                   uint32_t lds_bytes, void *stream, void **args) {
  if (!kernel) return KCG_ERR_INVALID_ARGUMENT;
  int rc = checkDims(grid, block);
  if (rc) return rc;
  return hipErr(hipModuleLaunchKernel(kernel->fn, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                      lds_bytes, (hipStream_t)stream, args, nullptr));
}

int kcg_hip_time_launches(kcg_kernel_t kernel, const uint32_t grid[3], const uint32_t block[3],
                          uint32_t lds_bytes, void *stream, void **args,
                          int warmup, int iters, float *avg_ms) {
  if (!kernel || !avg_ms || iters <= 0 || warmup < 0) return KCG_ERR_INVALID_ARGUMENT;
  int rc = checkDims(grid, block);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  hipEvent_t t0, t1;
  hipError_t e = hipEventCreate(&t0);
  if (e != hipSuccess) return hipErr(e);
  e = hipEventCreate(&t1);
  if (e != hipSuccess) { (void)hipEventDestroy(t0); return hipErr(e); }
  for (int i = 0; i < warmup && e == hipSuccess; ++i)
    e = hipModuleLaunchKernel(kernel->fn, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                              lds_bytes, s, args, nullptr);
  if (e == hipSuccess) e = hipEventRecord(t0, s);
  for (int i = 0; i < iters && e == hipSuccess; ++i)
    e = hipModuleLaunchKernel(kernel->fn, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                              lds_bytes, s, args, nullptr);
  if (e == hipSuccess) e = hipEventRecord(t1, s);
  if (e == hipSuccess) e = hipEventSynchronize(t1);
  float ms = 0.f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, t0, t1);
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  if (e != hipSuccess) return hipErr(e);
  *avg_ms = ms / (float)iters;
  return KCG_OK;
}

int kcg_hip_time_rotating(kcg_kernel_t kernel, const uint32_t grid[3], const uint32_t block[3],
                          uint32_t lds_bytes, void *stream, void **const *arg_sets, int num_sets,
                          int warmup, float warmup_ms, int runs, int launches_per_run,
                          float *median_ms, float *min_ms) {
  if (!kernel || !arg_sets || num_sets <= 0 || warmup < 0 || runs <= 0 || launches_per_run <= 0 || (!median_ms && !min_ms))
    return KCG_ERR_INVALID_ARGUMENT;
  for (int i = 0; i < num_sets; ++i)
    if (!arg_sets[i]) return KCG_ERR_INVALID_ARGUMENT;
  int rc = checkDims(grid, block);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  hipEvent_t t0, t1;
  hipError_t e = hipEventCreate(&t0);
  if (e != hipSuccess) return hipErr(e);
  e = hipEventCreate(&t1);
  if (e != hipSuccess) { (void)hipEventDestroy(t0); return hipErr(e); }
  int next = 0;
  auto launchGroup = [&](int count, float *ms) {
    hipError_t err = hipEventRecord(t0, s);
    for (int i = 0; i < count && err == hipSuccess; ++i, ++next)
      err = hipModuleLaunchKernel(kernel->fn, grid[0], grid[1], grid[2], block[0], block[1], block[2], lds_bytes, s,
                                  arg_sets[next % num_sets], nullptr);
    if (err == hipSuccess) err = hipEventRecord(t1, s);
    if (err == hipSuccess) err = hipEventSynchronize(t1);
    if (err == hipSuccess) err = hipEventElapsedTime(ms, t0, t1);
    return err;
  };
  // warm-up: at least `warmup` launches and at least `warmup_ms` of device time, in groups of at most 64 launches
  float spent = 0.0f;
  int done = 0;
  while (e == hipSuccess && (done < warmup || spent < warmup_ms) && done < 100000) {
    const int group = std::max(1, std::min(64, std::max(warmup - done, done)));
    float ms = 0.0f;
    e = launchGroup(group, &ms);
    spent += ms;
    done += group;
  }
  std::vector<float> per((size_t)runs, 0.0f);
  for (int r = 0; r < runs && e == hipSuccess; ++r) {
    float ms = 0.0f;
    e = launchGroup(launches_per_run, &ms);
    per[(size_t)r] = ms / (float)launches_per_run;
  }
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  if (e != hipSuccess) return hipErr(e);
  std::sort(per.begin(), per.end());
  if (min_ms) *min_ms = per.front();
  if (median_ms) *median_ms = runs % 2 ? per[(size_t)runs / 2] : 0.5f * (per[(size_t)runs / 2 - 1] + per[(size_t)runs / 2]);
  return KCG_OK;
}

int kcg_hip_launch_sequence(kcg_kernel_t kernel, const uint32_t grid[3], const uint32_t block[3],
                            uint32_t lds_bytes, void *stream, void **const *arg_sets, int num_sets,
                            int first, int count) {
  if (!kernel || !arg_sets || num_sets <= 0 || first < 0 || count < 0) return KCG_ERR_INVALID_ARGUMENT;
  for (int i = 0; i < num_sets; ++i)
    if (!arg_sets[i]) return KCG_ERR_INVALID_ARGUMENT;
  int rc = checkDims(grid, block);
  if (rc) return rc;
  for (int i = 0; i < count; ++i) {
    hipError_t e = hipModuleLaunchKernel(kernel->fn, grid[0], grid[1], grid[2], block[0], block[1], block[2], lds_bytes,
                                         (hipStream_t)stream, arg_sets[(first + i) % num_sets], nullptr);
    if (e != hipSuccess) return hipErr(e);
  }
  return KCG_OK;
}

int kcg_hip_module_destroy(kcg_module_t module) {
  if (!module) return KCG_ERR_INVALID_ARGUMENT;
  hipError_t e = hipModuleUnload(module->mod);
  for (kcg_kernel_s *k : module->kernels) delete k;
  delete module;
  return hipErr(e);
}

const char *kcg_hip_strerror(int code) {
  if (code == KCG_OK) return "success";
  if (code & KCG_ERR_DOMAIN_HIPRTC)
    return rtc().ok ? rtc().getErrorString((hiprtcResult)(code & 0xFFFF)) : "hiprtc error";
  if (code & KCG_ERR_DOMAIN_HIP) return hipGetErrorString((hipError_t)(code & 0xFFFF));
  switch (code) {
    case KCG_ERR_INVALID_ARGUMENT: return "kcg: invalid argument";
    case KCG_ERR_NO_DEVICE: return "kcg: no such HIP device";
    case KCG_ERR_NO_COMPILER: return "kcg: libhiprtc could not be loaded";
    case KCG_ERR_OUT_OF_HOST_MEMORY: return "kcg: out of host memory";
    case KCG_ERR_LOG_TRUNCATED: return "kcg: log truncated";
    case KCG_ERR_SCRATCH_TOO_LARGE: return "kcg: the kernel's workspace is larger than the library's scratch array (KCG_SCRATCH_MAX_BYTES)";
    default: return "kcg: unknown error";
  }
}

int kcg_hip_malloc(void **dptr, size_t bytes) {
  if (!dptr) return KCG_ERR_INVALID_ARGUMENT;
  return hipErr(hipMalloc(dptr, bytes));
}
int kcg_hip_free(void *dptr) { return hipErr(hipFree(dptr)); }
int kcg_hip_memcpy_h2d(void *dst, const void *src, size_t bytes) {
  return hipErr(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
}
int kcg_hip_memcpy_d2h(void *dst, const void *src, size_t bytes) {
  return hipErr(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
}
int kcg_hip_memcpy_d2d(void *dst, const void *src, size_t bytes) {
  return hipErr(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToDevice));
}
int kcg_hip_memset(void *dst, int value, size_t bytes) { return hipErr(hipMemset(dst, value, bytes)); }
int kcg_hip_stream_synchronize(void *stream) { return hipErr(hipStreamSynchronize((hipStream_t)stream)); }
int kcg_hip_device_synchronize(void) { return hipErr(hipDeviceSynchronize()); }

int kcg_hip_stream_create(void **stream) {
  if (!stream) return KCG_ERR_INVALID_ARGUMENT;
  hipStream_t s = nullptr;
  hipError_t rc = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);      // default priority
  *stream = (void *)s;
  return hipErr(rc);
}
int kcg_hip_stream_destroy(void *stream) {
  if (!stream) return KCG_ERR_INVALID_ARGUMENT;
  return hipErr(hipStreamDestroy((hipStream_t)stream));
}

int kcg_hip_graph_begin_capture(void *stream) {
  if (!stream) return KCG_ERR_INVALID_ARGUMENT;      // the null stream cannot be captured
  // thread-local: other threads of the process (an allocator, a data loader) may go on calling HIP meanwhile
  return hipErr(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
}
int kcg_hip_graph_end_capture(void *stream, kcg_graph_t *out) {
  if (!stream || !out) return KCG_ERR_INVALID_ARGUMENT;
  *out = nullptr;
  hipGraph_t graph = nullptr;
  hipError_t rc = hipStreamEndCapture((hipStream_t)stream, &graph);
  if (rc != hipSuccess) return hipErr(rc);
  if (!graph) return KCG_ERR_INVALID_ARGUMENT;
  kcg_graph_s *g = new (std::nothrow) kcg_graph_s;
  if (!g) { (void)hipGraphDestroy(graph); return KCG_ERR_OUT_OF_HOST_MEMORY; }
  g->exec = nullptr;
  g->nodes = 0;
  (void)hipGraphGetNodes(graph, nullptr, &g->nodes);      // a count for the caller to look at; 0 if it cannot be had
  rc = hipGraphInstantiate(&g->exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (rc != hipSuccess) { delete g; return hipErr(rc); }
  *out = g;
  return KCG_OK;
}
int kcg_hip_graph_launch(kcg_graph_t graph, void *stream) {
  if (!graph || !graph->exec) return KCG_ERR_INVALID_ARGUMENT;
  return hipErr(hipGraphLaunch(graph->exec, (hipStream_t)stream));
}
int kcg_hip_graph_num_nodes(kcg_graph_t graph, size_t *count) {
  if (!graph || !count) return KCG_ERR_INVALID_ARGUMENT;
  *count = graph->nodes;
  return KCG_OK;
}
int kcg_hip_graph_destroy(kcg_graph_t graph) {
  if (!graph) return KCG_ERR_INVALID_ARGUMENT;
  hipError_t rc = graph->exec ? hipGraphExecDestroy(graph->exec) : hipSuccess;
  delete graph;
  return hipErr(rc);
}

int kcg_hip_event_create(kcg_event_t *ev) {
  if (!ev) return KCG_ERR_INVALID_ARGUMENT;
  *ev = nullptr;
  kcg_event_s *e = new (std::nothrow) kcg_event_s;
  if (!e) return KCG_ERR_OUT_OF_HOST_MEMORY;
  hipError_t rc = hipEventCreate(&e->ev);
  if (rc != hipSuccess) { delete e; return hipErr(rc); }
  *ev = e;
  return KCG_OK;
}
int kcg_hip_event_record(kcg_event_t ev, void *stream) {
  if (!ev) return KCG_ERR_INVALID_ARGUMENT;
  return hipErr(hipEventRecord(ev->ev, (hipStream_t)stream));
}
int kcg_hip_event_synchronize(kcg_event_t ev) {
  if (!ev) return KCG_ERR_INVALID_ARGUMENT;
  return hipErr(hipEventSynchronize(ev->ev));
}
int kcg_hip_event_elapsed_ms(kcg_event_t start, kcg_event_t stop, float *ms) {
  if (!start || !stop || !ms) return KCG_ERR_INVALID_ARGUMENT;
  return hipErr(hipEventElapsedTime(ms, start->ev, stop->ev));
}
int kcg_hip_event_destroy(kcg_event_t ev) {
  if (!ev) return KCG_ERR_INVALID_ARGUMENT;
  hipError_t rc = hipEventDestroy(ev->ev);
  delete ev;
  return hipErr(rc);
}

}  // extern "C"
