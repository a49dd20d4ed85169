/*
 * kcg_hip.h -- C ABI of libkcg_hip.so: compile, load and launch the gfx950
 * kernels that the HIP backend emits.
 *
 * The reference stops at a source string: KernelCodeGenerator::codegen()
 * (include/KernelCodeGen.h:138-142) returns CUDA text, save() (:99-115) writes
 * it to disk and an out-of-tree harness feeds it to nvcc (test/test.cc:69-77).
 * evaluate() (:134-136) is a stub that returns 0.  These entry points are what
 * that missing device boundary binds on one MI355X: hipRTC turns the emitted
 * source into a code object, hipModule loads it, hipModuleLaunchKernel runs it.
 *
 * Conventions
 *   - plain C, pointers and sizes only; no C++ or torch types cross the ABI.
 *   - every function returns 0 on success.  A non-zero code is either
 *     KCG_ERR_* below, a hipError_t tagged with KCG_ERR_DOMAIN_HIP, or a
 *     hiprtcResult tagged with KCG_ERR_DOMAIN_HIPRTC; kcg_hip_strerror()
 *     decodes all three.  Nothing throws or aborts across the boundary.
 *   - the caller owns device buffers and streams; the library owns module and
 *     kernel handles until kcg_hip_module_destroy().
 *   - functions are re-entrant on distinct handles; there is no internal lock.
 *   - gfx950 only: "--offload-arch=gfx950" is always passed to hipRTC.
 */
#ifndef KCG_HIP_H
#define KCG_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KCG_OK 0
#define KCG_ERR_INVALID_ARGUMENT 1
#define KCG_ERR_NO_DEVICE 2
#define KCG_ERR_OUT_OF_HOST_MEMORY 3
#define KCG_ERR_LOG_TRUNCATED 4
#define KCG_ERR_NO_COMPILER 5
#define KCG_ERR_SCRATCH_TOO_LARGE 6
#define KCG_ERR_DOMAIN_HIP 0x10000    /* code = KCG_ERR_DOMAIN_HIP    | hipError_t   */
#define KCG_ERR_DOMAIN_HIPRTC 0x20000 /* code = KCG_ERR_DOMAIN_HIPRTC | hiprtcResult */

typedef struct kcg_module_s *kcg_module_t;
typedef struct kcg_kernel_s *kcg_kernel_t;
typedef struct kcg_event_s *kcg_event_t;

/* Machine-readable form of the "// grid dims:(..), block dims:(..)" comment
 * that the reference prints above each kernel (src/Backend/CUDA.cc:1031-1036).
 * Dims are stored x, y, z (the comment lists them outer to inner = z, y, x). */
typedef struct kcg_launch_info {
  char name[64];          /* extern "C" symbol, "kernel0", "kernel1", ...      */
  uint32_t grid[3];       /* x, y, z                                           */
  uint32_t block[3];      /* x, y, z                                           */
  uint32_t lds_bytes;     /* dynamic LDS; static LDS is declared in the source */
  uint32_t num_args;      /* device pointers: function inputs, then outputs, then the workspace if there is one;
                             then the scalars                                  */
  uint32_t num_scalars;   /* trailing fp32 scalars (per-tensor scales), 0..2   */
  uint64_t workspace_bytes; /* > 0: the kernel takes one more pointer behind the outputs, a scratch buffer of this
                             size that it shares between its workgroups.  Its first 4096 bytes must be zero before
                             the first launch; every launch leaves them zero, so one buffer serves all launches of
                             the kernel that do not overlap in time.                                              */
  double flops;           /* algorithmic flops of one launch                   */
  double bytes;           /* algorithmic HBM bytes of one launch               */
} kcg_launch_info;

/* Select the device (ordinal 0 on the one-GPU box) and create its context. */
int kcg_hip_init(int device);
int kcg_hip_device_count(int *count);
int kcg_hip_device_name(int device, char *name, size_t cap);

/* Source -> gfx950 code object with hipRTC.  Needs no GPU.  `opts` are extra
 * compiler options.  On a compile error the log is copied to `log` (always
 * NUL terminated when log_cap > 0) and the hiprtc error is returned.  The code
 * object is malloc'ed; release it with kcg_hip_free_code(). */
int kcg_hip_compile_to_code(const char *src, const char *const *opts, int nopts,
                            void **code, size_t *code_size, char *log, size_t log_cap);
void kcg_hip_free_code(void *code);

/* kcg_hip_compile_to_code through an on-disk cache of code objects.  A code object is stored under the
 * first 32 hex digits of SHA-256(compiler text, NUL, source, then NUL + option for every option) + ".hsaco"
 * in the directory the environment variable KCG_CACHE_DIR names, or else in "_cache" beside this library.
 * `refresh` != 0 compiles even when the object is there and rewrites it.  A cache that cannot be read or
 * written is not an error: the call then compiles.  The directory is bounded: a write that takes its ".hsaco"
 * files over KCG_CACHE_MAX_MB megabytes (environment, default 1024; 0 or less: no bound) removes the oldest of them
 * until nine tenths of the bound are left.  No counterpart in the reference (it stops at text). */
int kcg_hip_compile_to_code_cached(const char *src, const char *const *opts, int nopts, int refresh,
                                   void **code, size_t *code_size, char *log, size_t log_cap);
/* kcg_hip_compile_to_code_cached + kcg_hip_load_code. */
int kcg_hip_compile_cached(const char *src, const char *const *opts, int nopts,
                           kcg_module_t *out, char *log, size_t log_cap);
/* The directory kcg_hip_compile_to_code_cached uses. */
int kcg_hip_cache_dir(char *path, size_t cap);

/* Which hipRTC compiles the kernels: "hipRTC <major>.<minor> from <file> (<how it was loaded>)".  The shim
 * loads the ROCm installation's libhiprtc ($ROCM_PATH/lib, or the file KCG_HIPRTC_LIBRARY names) into a
 * link-map namespace of its own, so that a host program's bundled copy under the same soname is not used
 * in its place; the text is part of the key of an on-disk code-object cache.  No counterpart in the
 * reference, which stops at kernel text (include/KernelCodeGen.h:138-142). */
int kcg_hip_compiler_info(char *text, size_t cap);

/* Code object -> loaded module on the current device. */
int kcg_hip_load_code(const void *code, size_t code_size, kcg_module_t *out);

/* kcg_hip_compile_to_code + kcg_hip_load_code. */
int kcg_hip_compile(const char *src, const char *const *opts, int nopts,
                    kcg_module_t *out, char *log, size_t log_cap);

int kcg_hip_get_kernel(kcg_module_t module, const char *name, kcg_kernel_t *out);

/* Launch.  `args` is an array of pointers to the argument values, as
 * hipModuleLaunchKernel takes it.  `stream` is a hipStream_t (NULL = default). */
int kcg_hip_launch(kcg_kernel_t kernel, const uint32_t grid[3], const uint32_t block[3],
                   uint32_t lds_bytes, void *stream, void **args);

/* Average duration of `iters` back-to-back launches after `warmup` untimed
 * ones, measured with HIP events recorded on `stream`. */
int kcg_hip_time_launches(kcg_kernel_t kernel, const uint32_t grid[3], const uint32_t block[3],
                          uint32_t lds_bytes, void *stream, void **args,
                          int warmup, int iters, float *avg_ms);

/* Launch duration with the operands out of the caches: launch i uses arg_sets[i % num_sets] (each an `args`
 * array as kcg_hip_launch takes it; give it three or more sets of buffers that together exceed the 256 MB
 * last-level cache).  After `warmup` untimed launches (at least enough to run for `warmup_ms` milliseconds:
 * the first launches of a process run at idle clocks), `runs` groups of `launches_per_run` launches are timed,
 * each between its own pair of HIP events on `stream`; *median_ms and *min_ms (either may be NULL) receive the
 * median and the minimum of the per-launch averages of the groups. */
int kcg_hip_time_rotating(kcg_kernel_t kernel, const uint32_t grid[3], const uint32_t block[3],
                          uint32_t lds_bytes, void *stream, void **const *arg_sets, int num_sets,
                          int warmup, float warmup_ms, int runs, int launches_per_run,
                          float *median_ms, float *min_ms);

/* kcg_hip_launch for a kernel that takes a workspace (kcg_launch_info.workspace_bytes > 0), for callers that
 * cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference, which launches nothing.  The workspace is a scratch
 * array of KCG_SCRATCH_MAX_BYTES inside the library's own device image (every GPU the library runs on holds
 * one copy until the process ends); the call allocates and frees nothing.  `args` has `num_args` (at most 16)
 * entries as kcg_hip_launch takes them; entry `scratch_arg`, the workspace pointer, is ignored and replaced.
 * A workspace beyond KCG_SCRATCH_MAX_BYTES is refused with KCG_ERR_SCRATCH_TOO_LARGE (use kcg_hip_launch with a
 * buffer of the caller's then).  The counters at the start of the array are cleared by a small kernel in front
 * of every launch, on `stream`.  All calls on one GPU share that GPU's array: calls that overlap in time (two
 * streams, two threads) race on it and give wrong results. */
#define KCG_SCRATCH_MAX_BYTES (32u << 20)
int kcg_hip_launch_scratch(kcg_kernel_t kernel, const uint32_t grid[3], const uint32_t block[3],
                           uint32_t lds_bytes, void *stream, void **args, int num_args, int scratch_arg,
                           size_t scratch_bytes);

/* `count` launches in a row without returning to the caller in between: launch i uses
 * arg_sets[(first + i) % num_sets].  For timed loops whose host side must not be the bottleneck. */
int kcg_hip_launch_sequence(kcg_kernel_t kernel, const uint32_t grid[3], const uint32_t block[3],
                            uint32_t lds_bytes, void *stream, void **const *arg_sets, int num_sets,
                            int first, int count);

int kcg_hip_module_destroy(kcg_module_t module);

const char *kcg_hip_strerror(int code);

/* Thin wrappers for hosts that have no HIP binding of their own. */
int kcg_hip_malloc(void **dptr, size_t bytes);
int kcg_hip_free(void *dptr);
int kcg_hip_memcpy_h2d(void *dst, const void *src, size_t bytes);
int kcg_hip_memcpy_d2h(void *dst, const void *src, size_t bytes);
int kcg_hip_memcpy_d2d(void *dst, const void *src, size_t bytes);
int kcg_hip_memset(void *dst, int value, size_t bytes);
int kcg_hip_stream_synchronize(void *stream);
int kcg_hip_device_synchronize(void);
/* Streams and HIP graphs, for a caller that runs the same sequence of kernels again and again (the kernels of an
 * imported graph, doc/Plan.md:4-8 in the reference's roadmap; the reference itself stops at kernel text): record the
 * sequence once between begin_capture and end_capture on a stream of the caller's (kcg_hip_launch on that stream
 * records instead of running), then replay it with one call.  Streams have the default priority.  Only kernel
 * launches may be recorded: no memset or copy of this library is captured, and a kernel that takes a workspace keeps
 * using the buffer it was recorded with.  The arguments' VALUES (the device pointers) are fixed at capture. */
typedef struct kcg_graph_s *kcg_graph_t;
int kcg_hip_stream_create(void **stream);
int kcg_hip_stream_destroy(void *stream);
int kcg_hip_graph_begin_capture(void *stream);
int kcg_hip_graph_end_capture(void *stream, kcg_graph_t *out);
int kcg_hip_graph_launch(kcg_graph_t graph, void *stream);
int kcg_hip_graph_num_nodes(kcg_graph_t graph, size_t *count);
int kcg_hip_graph_destroy(kcg_graph_t graph);
int kcg_hip_event_create(kcg_event_t *ev);
int kcg_hip_event_record(kcg_event_t ev, void *stream);
int kcg_hip_event_synchronize(kcg_event_t ev);
int kcg_hip_event_elapsed_ms(kcg_event_t start, kcg_event_t stop, float *ms);
int kcg_hip_event_destroy(kcg_event_t ev);

/* ---- synthetic operands on the host -------------------------------------------------------------------
 * The seeded generator that the timed config search (KernelCodeGenerator::evaluate), the generated host
 * adaptor and the benchmark fill kernel operands with, and the narrow-float codecs that go with it.  The
 * reference has neither (its harness is out of tree, test/test.cc:69-104).
 * Element i of stream s under seed z is drawn from splitmix64(z + (s << 40) + i): any element can be made
 * independently.  Uniform: the top 24 bits / 2^24 in [0,1), then p0 + (p1 - p0) * u in fp32.  Normal:
 * Box-Muller in fp64 on the 53-bit uniforms of elements 2j and 2j+1, mean p0, deviation p1, cast to fp32.
 * The fp32 value is multiplied by `scale`, then rounded to the element type: bf16 and f16 to nearest even,
 * e4m3fn to nearest even saturating at +-448, integers truncated toward zero. */
#define KCG_DT_F32 0
#define KCG_DT_BF16 1
#define KCG_DT_F8E4M3 2
#define KCG_DT_F16 3
#define KCG_DT_F64 4
#define KCG_DT_I32 5
#define KCG_DT_I64 6
#define KCG_DT_I16 7
#define KCG_DT_I8 8          /* also the one-byte form of i1 results */
#define KCG_DIST_UNIFORM 0
#define KCG_DIST_NORMAL 1
/* Bytes per element; 0 for an unknown type. */
size_t kcg_dtype_size(int dtype);
int kcg_host_fill(void *dst, size_t count, int dtype, int dist, uint64_t seed, uint64_t stream,
                  float p0, float p1, float scale);
/* Element type -> fp32 (exact for every type but f64 / i64 / i32 beyond 24 bits). */
int kcg_host_to_f32(const void *src, float *dst, size_t count, int dtype);
/* fp32 * scale -> element type, rounding as above. */
int kcg_host_from_f32(const float *src, void *dst, size_t count, int dtype, float scale);

#ifdef __cplusplus
}
#endif
#endif /* KCG_HIP_H */
