"""The benchmark workloads (operator instances at their full sizes) as kernel
family parameters.  bench.py runs them; build.prebuild_kernels() compiles them
ahead of time so that a GPU box starts from code objects."""

WORKLOADS = {
    # fp32 GEMM, full-precision MFMA
    "gemm_f32_1024": ("gemm_f32", dict(M=1024, N=1024, K=1024)),
    "gemm_f32_4096": ("gemm_f32", dict(M=4096, N=4096, K=4096)),
    "bgemm_f32_16x1024": ("gemm_f32", dict(M=1024, N=1024, K=1024, BATCH=16)),
    # fp64 GEMM on the fp64 MFMA
    "gemm_f64_4096": ("gemm_f64", dict(M=4096, N=4096, K=4096)),
    # LayerNorm 16384 x 4096 fp32 with the GELU fused into the store
    "layernorm_gelu_16384x4096": ("layernorm", dict(ROWS=16384, N=4096, NG=4096, NB=4096, EPS=1e-5, GELU=1)),
    "layernorm_16384x4096": ("layernorm", dict(ROWS=16384, N=4096, NG=4096, NB=4096, EPS=1e-5, GELU=0)),
    # a plain copy of the same tensor (a value-preserving Cast): what a read-once, write-once stream reaches
    "copy_f32_16384x4096": ("elementwise", dict(N=16384 * 4096, OP="Cast", INPLACE=0, IN_T="float", OUT_T="float")),
    "gelu_16384x4096": ("elementwise", dict(N=16384 * 4096, OP="Gelu", INPLACE=0, IN_T="float", OUT_T="float")),
    # quantised-inference GEMM, bf16 operands: 4096 tokens through a linear layer with 11008 outputs and 4096 inputs.
    # The weights as the layer holds them, [N][K] (k-contiguous, like the activations) ...
    "gemm_bf16_nk_4096x11008x4096": ("gemm_bf16", dict(M=4096, N=11008, K=4096, TA=0, TB=1, OUT_BF16=0)),
    # ... and as a row-major [K][N] matrix (transposed in registers on the way into LDS)
    "gemm_bf16_4096x11008x4096": ("gemm_bf16", dict(M=4096, N=11008, K=4096, OUT_BF16=0)),
    # ... with the result rounded to bf16 (half the store), as the vendor library's bf16 GEMM returns it
    "gemm_bf16_4096x11008x4096_bf16out": ("gemm_bf16", dict(M=4096, N=11008, K=4096, OUT_BF16=1)),
    # the same GEMM with fp8 e4m3 operands (B stored [N][K]) and one fp32 scale per tensor
    "gemm_fp8_4096x11008x4096": ("gemm_fp8", dict(M=4096, N=11008, K=4096, TA=0, TB=1, OUT_BF16=0)),
    # ... and with the weights as a row-major [K][N] matrix (byte-transposed on the way into LDS)
    "gemm_fp8_nn_4096x11008x4096": ("gemm_fp8", dict(M=4096, N=11008, K=4096, TA=0, TB=0, OUT_BF16=0)),
    # fused attention forward, bf16, softmax scale 1/sqrt(D)
    "fmha_bf16_b8h32s2048d128": ("fmha_bf16", dict(B=8, H=32, S=2048, D=128, CAUSAL=0, OUT_BF16=1,
                                                   SCALE=128 ** -0.5)),
    "fmha_bf16_b8h32s2048d128_causal": ("fmha_bf16", dict(B=8, H=32, S=2048, D=128, CAUSAL=1, OUT_BF16=1,
                                                          SCALE=128 ** -0.5)),
    # the reference's own attention graph (its test/test.cc:107-147: fp32, no scale, no mask, head dim 64) on the fp32 MFMA,
    # and the benchmark's shape and semantics (head dim 128, 1/sqrt(D), causal) in fp32
    "fmha_f32_b8h32s2048d64": ("fmha_f32", dict(B=8, H=32, S=2048, D=64, CAUSAL=0, SCALE=1.0)),
    "fmha_f32_b8h32s2048d128_causal": ("fmha_f32", dict(B=8, H=32, S=2048, D=128, CAUSAL=1, SCALE=128 ** -0.5)),
    # broadcast bias add over a 16384 x 4096 fp32 activation
    "add_bias_f32_16384x4096": ("binary", dict(OP="Add", DIMS="16384,4096", SA="4096,1", SB="0,1")),
    # embedding lookup: 16384 token rows out of a 32000 x 4096 bf16 table
    "gather_bf16_32000x4096_16384": ("gather", dict(OUTER=1, AXIS=32000, NIDX=16384, INNER=4096, ESIZE=2)),
    # standalone softmax, the LayerNorm workload's shape (256 MB in, 256 MB out)
    "softmax_f32_16384x4096": ("softmax", dict(ROWS=16384, N=4096, INPLACE=0)),
    # ... and in place over rows the size of an attention score row: 512 MB read and written
    "softmax_f32_65536x2048": ("softmax", dict(ROWS=65536, N=2048, INPLACE=1)),
    # The optimizers' own schedules printed statement by statement (LOWERING = "schedule") instead of a kernel family:
    # the reference's 128 x 128 x 16 fp32 GEMM schedule with 8 x 8 results per thread, its three-pass LayerNorm, its
    # elementwise map.  Same operands, same checks, same algorithmic work as the workloads above.
    "gemm_f32_4096_schedule": ("gemm_f32", dict(M=4096, N=4096, K=4096, LOWERING="schedule")),
    "layernorm_16384x4096_schedule": ("layernorm", dict(ROWS=16384, N=4096, NG=4096, NB=4096, EPS=1e-5, GELU=0,
                                                        LOWERING="schedule")),
    "gelu_16384x4096_schedule": ("elementwise", dict(N=16384 * 4096, OP="Gelu", INPLACE=0, IN_T="float", OUT_T="float",
                                                     LOWERING="schedule")),
}


def workload_source(name, overrides=None):
    """(full source text, launch info, family, parameters) of a workload's kernel `kernel0`.  A kernel family is
    instantiated directly; a workload with LOWERING = "schedule" goes through the generator (graph, optimize,
    codegen with the schedule lowering) and takes the algorithmic flops and bytes of its family's launch info.
    `overrides`: family parameters that replace or add to the workload's (a kernel variant on the same operands)."""
    from . import runtime as R
    family, params = WORKLOADS[name]
    if overrides:
        params = dict(params, **overrides)
    fam_params = {k: v for k, v in params.items() if k != "LOWERING"}
    text, info = R.emit_kernel(family, "kernel0", **fam_params)
    if params.get("LOWERING") != "schedule":
        return R.prelude() + text, info, family, params
    from .generator import KernelCodeGenerator, MemorySpace
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph(name)
    if family == "gemm_f32":
        gen.setConfigs("Matmul", [{"BLOCK_SIZE_M": 128, "BLOCK_SIZE_N": 128, "BLOCK_SIZE_K": 16, "THREAD_SIZE_M": 8,
                                   "THREAD_SIZE_N": 8, "VECTORIZE_WIDTH": 4, "WARP_SIZE": 64}])
        gen.opts.append("Matmul")
        a = g.create("PlaceHolder", [params["M"], params["K"]], "float32")
        b = g.create("PlaceHolder", [params["K"], params["N"]], "float32")
        g.create("Matmul", a, b)
    elif family == "layernorm":
        # half a row per team of 512 threads, and the reference's tree over the threads' partial sums (shared memory
        # down to one wavefront, shuffles inside it) in place of the serial sum the default schedule keeps for its
        # bit-for-bit agreement with the naive nest: 0.15 ms against 0.94 ms at 16384 x 4096
        gen.setConfigs("LayerNorm", [{"BLOCK_SIZE": 2048, "THREAD_SIZE": 4, "VECTORIZE_WIDTH": 4, "FUSE_GELU": 0,
                                      "TREE_REDUCE": 1}])
        gen.opts.append("LayerNorm")
        x = g.create("PlaceHolder", [params["ROWS"], params["N"]], "float32")
        s = g.create("PlaceHolder", [params["NG"]], "float32")
        b = g.create("PlaceHolder", [params["NB"]], "float32")
        g.create("LayerNorm", x, s, b, 1, params["EPS"])
    elif family == "elementwise":
        gen.opts.append("ElementWise")
        x = g.create("PlaceHolder", [16384, params["N"] // 16384], "float32")
        g.create("ElementWise", x, params["OP"], MemorySpace.global_)
    else:
        raise ValueError("no schedule workload for family %s" % family)
    gen.optimize(g)
    gen.setLowering("schedule")
    source = gen.codegen()
    (sched,) = gen.launchInfos()
    if sched["num_args"] != info["num_args"]:
        raise RuntimeError("the schedule's kernel takes %d arguments, the family's %d" % (sched["num_args"], info["num_args"]))
    sched["flops"], sched["bytes"] = info["flops"], info["bytes"]
    return source, sched, family, params
