/*
 * kcg_codegen.h -- C ABI over the code generator in libkcg_hip.so, for hosts
 * that cannot include the C++ headers (KernelCodeGen.h and friends).
 *
 * The reference has no foreign-function interface: its users link the C++
 * library kcg_runtime and call KernelCodeGenerator directly (test/test.cc:8-49).
 * Each entry point below names the C++ member it forwards to.
 */
#ifndef KCG_CODEGEN_H
#define KCG_CODEGEN_H

#include <stddef.h>
#include <stdint.h>

#include "kcg_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Source text every emitted translation unit starts with.  Static storage. */
const char *kcg_prelude(void);

/* One kernel of a gfx950 kernel family ("layernorm", "elementwise",
 * "gemm_f32", "gemm_bf16", "gemm_fp8", "fmha_bf16") from explicit parameters: the layer
 * HIPGen() sits on (it replaces the per-op printers of src/Backend/CUDA.cc:386-1149).
 * Integer, floating and string parameters are passed as parallel key/value
 * arrays, like the reference's std::map<std::string,int> config tables
 * (include/KernelCodeGen.h:35-58).  On success *src_out is a malloc'ed string
 * (kernel text without the prelude; free with kcg_free_string) and *info is
 * filled.  On failure returns non-zero and copies a message to err. */
int kcg_emit_kernel(const char *family, const char *name,
                    const char *const *ikeys, const int64_t *ivals, int ni,
                    const char *const *fkeys, const double *fvals, int nf,
                    const char *const *skeys, const char *const *svals, int ns,
                    char **src_out, kcg_launch_info *info, char *err, size_t err_cap);

void kcg_free_string(char *s);

/* ---- the generator: graph -> schedule -> source ---------------------------
 * A kcg_generator_t wraps one KernelCodeGen::KernelCodeGenerator
 * (include/KernelCodeGen.h).  Graph values are small non-negative integers;
 * a negative return value is an error whose text kcg_generator_error() returns
 * (the C++ builders print the same text to stderr and return a null Value). */
typedef struct kcg_generator_s *kcg_generator_t;

/* KernelCodeGenerator(platform); createGraph(name) */
kcg_generator_t kcg_generator_create(const char *platform);
void kcg_generator_destroy(kcg_generator_t g);
int kcg_generator_create_graph(kcg_generator_t g, const char *name);
const char *kcg_generator_error(kcg_generator_t g);
/* setLogMode(Log): 0 = Debug, 1 = Release */
void kcg_generator_set_log_mode(kcg_generator_t g, int level);

/* graph.create<Op>(...) -- memory_space / layout take the values of
 * KernelCodeGen::MemorySpace / Layout (include/enum.h); dtype "" inherits. */
int kcg_placeholder(kcg_generator_t g, const int64_t *shape, int rank, const char *dtype);
int kcg_matmul(kcg_generator_t g, int a, int b, const char *dtype);
int kcg_batched_matmul(kcg_generator_t g, int a, int layout_a, int b, int layout_b, const char *dtype);
/* the same products with one fp32 scale per tensor as graph values (placeholders of one float32 element):
 * (scale_a[0] * scale_b[0]) * a * b */
int kcg_matmul_scaled(kcg_generator_t g, int a, int b, int scale_a, int scale_b, const char *dtype);
int kcg_batched_matmul_scaled(kcg_generator_t g, int a, int layout_a, int b, int layout_b, int scale_a, int scale_b,
                              const char *dtype);
int kcg_softmax(kcg_generator_t g, int x, int axis, int memory_space, const char *dtype);
int kcg_relu(kcg_generator_t g, int x, int memory_space, const char *dtype);
int kcg_elementwise(kcg_generator_t g, int x, const char *operation, int memory_space, const char *dtype);
int kcg_binary(kcg_generator_t g, int a, int b, const char *operation, int memory_space, const char *dtype);
int kcg_layernorm(kcg_generator_t g, int x, int scale, int bias, int64_t axis, float eps, int memory_space, const char *dtype);
/* graph.create<Gather>(input, indices, axis, dtype): indices is a placeholder of dtype "index"
 * (reference: include/Frontend/Operators.h Gather, src/Frontend/Operators.cc:1253-1352). */
int kcg_gather(kcg_generator_t g, int x, int indices, int64_t axis, const char *dtype);

/* generator.opts.push_back(std::make_unique<XOptimizer>()): name is "Matmul",
 * "BatchMatmul", "ElementWise", "LayerNorm", "FMHA", "Binary", "Gather" or "Softmax". */
int kcg_add_optimizer(kcg_generator_t g, const char *name);
/* Replace the configuration candidates of one optimizer: `count` maps, map i
 * has sizes[i] entries taken in order from keys/values. */
int kcg_set_configs(kcg_generator_t g, const char *optimizer, int count, const int *sizes,
                    const char *const *keys, const int *values);

/* The configuration candidates of one optimizer as text, one candidate per line, "KEY=value" entries separated by
 * blanks (keys in alphabetical order).  The string belongs to the generator and stays valid until the next call;
 * NULL for an unknown optimizer. */
const char *kcg_get_configs(kcg_generator_t g, const char *optimizer);

/* optimize(graph): 0 on success. */
int kcg_optimize(kcg_generator_t g);
/* codegen(module) on the optimized module; NULL on error.  The string belongs
 * to the generator and stays valid until the next codegen or destroy. */
const char *kcg_codegen(kcg_generator_t g);
/* Which lowering kcg_codegen uses: "families" (default: a recognised operator becomes one of the gfx950 kernel
 * families, sized by its schedule) or "schedule" (the scheduled function body itself, one statement per operation,
 * as the reference's backend prints it, src/Backend/CUDA.cc:61-1184).  A function without an operator tag always
 * takes the second, and so does, with "families", one that its family refuses (a warning on stderr unless the
 * family simply has no form for the element type); "families-only" makes such a refusal an error of kcg_codegen.
 * 0 on success. */
int kcg_set_lowering(kcg_generator_t g, const char *mode);
/* generator.adaptor(kernel_file): C host program that compiles the saved kernel source and launches and
 * times every kernel of the last kcg_codegen (stands in for the reference's adaptor + out-of-tree harness,
 * test/test.cc:69-104).  The string belongs to the generator; NULL on error. */
const char *kcg_adaptor(kcg_generator_t g, const char *kernel_file);
int kcg_num_kernels(kcg_generator_t g);
int kcg_kernel_info(kcg_generator_t g, int index, kcg_launch_info *info);
/* IR function a kernel implements, and the byte size of each pointer argument. */
const char *kcg_kernel_function(kcg_generator_t g, int index);
/* How kernel `index` was lowered: "family <name>", or "schedule" (the function body printed statement by
 * statement), followed in brackets by the reason when a kernel family knows the operator but refused this function. */
const char *kcg_kernel_lowering(kcg_generator_t g, int index);
int kcg_kernel_arg_bytes(kcg_generator_t g, int index, int64_t *bytes, int cap);

/* Element type (KCG_DT_* of kcg_hip.h) of each pointer argument; returns their number. */
int kcg_kernel_arg_types(kcg_generator_t g, int index, int *types, int cap);
/* Operators that the graph calls but that no optimizer has scheduled: the last kcg_codegen emitted no kernel
 * for them (generator.skippedFunctions()). */
int kcg_num_skipped(kcg_generator_t g);
const char *kcg_skipped_function(kcg_generator_t g, int index);

/* The candidates the last kcg_optimize tried (generator.evaluations()): the optimizer, the index of the
 * configuration in its list, the number of kernels the candidate emitted, its latency in ms (FLT_MAX when it
 * failed; 0 without a GPU), whether it is the one kept, and a note (why it failed, or which called operators it
 * leaves unscheduled).  The reference's loop has no such record: its evaluate() is a stub
 * (include/KernelCodeGen.h:134-136, src/KernelCodeGen.cc:23-27). */
int kcg_num_evaluations(kcg_generator_t g);
int kcg_evaluation(kcg_generator_t g, int index, const char **optimizer, int *config_index, int *kernels,
                   float *latency_ms, int *kept, const char **note);
/* Value of `key` in that candidate's configuration map; -1 when the key is absent. */
int kcg_evaluation_config(kcg_generator_t g, int index, const char *key);
/* generator.evaluate(optimized module): latency in ms as above; negative on error. */
float kcg_evaluate(kcg_generator_t g);

/* The calls of the module body in order, with the buffers they read and write, as JSON text (owned by the
 * generator, valid until the next call):
 *   {"buffers": [{"id": 0, "shape": [..], "dtype": "float32", "bytes": n, "input": 0}, ...,  {"id": 7, "alias": 6}],
 *    "calls":   [{"callee": "Matmul_m..", "operands": [ids], "result": id, "scheduled": true}, ...]}
 * "input" is the number of the kcg_placeholder call that made the buffer (0, 1, ... in creation order), or -1
 * for a buffer that an operator builder, a fusion or a call's result allocates; a call's result is a new buffer
 * id, or the id of the operand it returns when the operator works in place (later users name it through an
 * "alias" entry).  What a host needs to run the generated kernels as a graph;
 * the reference leaves that to its out-of-tree harness (test/test.cc:69-104). */
const char *kcg_module_plan(kcg_generator_t g, int which);

/* Text of the graph module (which = 0) or of the optimized module (which = 1);
 * owned by the generator, valid until the next call. */
const char *kcg_dump(kcg_generator_t g, int which);
/* mlir::verify on that module: 0 when it holds. */
int kcg_verify(kcg_generator_t g, int which);
/* func.state of a function of that module ("cpu", "gpu", "" if absent). */
const char *kcg_function_state(kcg_generator_t g, int which, const char *function);

/* Host interpreter (include/IR/Interpreter.h): runs the module-level graph on
 * fp32 host data.  inputs[i] is bound to the i-th placeholder (sizes in
 * elements); the result of the last call is copied to `out` (out_cap elements).
 * Values of narrower element types are rounded to them on the way in.
 * The interpreter runs the threads of a workgroup in lock-step, so it also
 * audits what lock-step hides: shared memory that one thread writes and another
 * reads or overwrites with no gpu.barrier between is an error here.
 * Returns the number of elements written, negative on error. */
int64_t kcg_interpret(kcg_generator_t g, int which, const float *const *inputs, const int64_t *sizes, int num_inputs,
                      float *out, int64_t out_cap);

/* FMHAOptimizer::getAffineMap(name) (reference: src/Optimizer/Optimizer.cc:2201-2437) under the configuration that the
 * last kcg_optimize with the FMHA optimizer left in force, evaluated at `inputs`.  Writes the results to `out` and
 * returns how many there are; -1 for an unknown name, -2 when num_inputs is not the map's input count, -3 when `out`
 * is too small. */
int kcg_fmha_map_evaluate(const char *name, const int64_t *inputs, int num_inputs, int64_t *out, int out_cap);

#ifdef __cplusplus
}
#endif
#endif /* KCG_CODEGEN_H */
