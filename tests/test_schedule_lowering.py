"""The statement-by-statement lowering on the CPU: every optimizer's schedule prints as a kernel that hipRTC compiles
for gfx950, with the launch geometry of its two affine.parallel levels, LDS arrays for its shared buffers, per-lane arrays
for its register buffers and a workgroup barrier for every gpu.barrier.  What the kernels compute is checked on the
device (tests/test_gpu_schedule_lowering.py); here: that the text is what the body says, and that constructs without a
lowering are refused with a reason instead of printed wrongly."""
import re

import numpy as np
import pytest

import oracle_lib as O
import kernelcodegen_amd as K
from kernelcodegen_amd.generator import GeneratorError, KernelCodeGenerator, Layout, MemorySpace


def schedule_source(gen, graph):
    module = gen.optimize(graph)
    ok, msg = gen.verify(1)
    assert ok, msg
    gen.setLowering("schedule")
    src = gen.codegen(module)
    infos = gen.launchInfos()
    body = src[src.index("KCG_SCHEDULE_HELPERS"):]
    assert len(K.compile_to_code(src)) > 1000
    return body, infos, gen._dump(1)


def test_matmul_schedule_prints_what_the_body_says():
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("mm")
    gen.opts.append("Matmul")
    A = g.create("PlaceHolder", [256, 128], "float32")
    B = g.create("PlaceHolder", [128, 512], "float32")
    g.create("Matmul", A, B)
    body, (info,), ir = schedule_source(gen, g)
    assert info["name"] == "kernel0" and info["function"] == "Matmul_m256n512k128"
    # grid (2, 4) and workgroup (16, 16) of the schedule, last dimension fastest
    assert info["grid"] == [4, 2, 1] and info["block"] == [16, 16, 1] and info["num_args"] == 3
    assert info["arg_bytes"] == [256 * 128 * 4, 128 * 512 * 4, 256 * 512 * 4]
    assert "__launch_bounds__(256) kernel0(float* __restrict__ arg0, float* __restrict__ arg1, float* __restrict__ out0)" in body
    assert "#pragma clang fp contract(off)" in body
    # one LDS array per shared buffer of the body, one per-lane array per register buffer, one barrier per gpu.barrier
    assert body.count("__shared__") == len(re.findall(r"memref.alloc\(\) : memref<[^>]*, 2>", ir)) == 2
    assert len(re.findall(r"^\s+float reg\d+\[\d+\];", body, re.M)) == len(re.findall(r"memref.alloc\(\) : memref<[^>]*, 3>", ir)) == 5
    assert body.count("__syncthreads();") == ir.count("gpu.barrier") == 2
    assert "float lds2[4096]" in body and "reg21[64]" in body           # 2x16x128 tiles, the 8x8 accumulator
    # vector accesses of global and shared memory are 16-byte accesses; register arrays are accessed by element
    assert "*(const kcg_v4_float*)(arg0 + " in body and "*(kcg_v4_float*)(out0 + " in body
    # the double-buffer selector of the pipelined loop over k and its guard
    assert re.search(r"if \(-i\d+ \+ 96 >= 0\)", body) and re.search(r"\(i\d+ / 16 \+ 1\) % 2", body)
    # indices that are never negative divide and take remainders with the plain operators
    assert "kcg_floordiv(" not in body.split("#endif")[1]


def test_every_operator_schedule_compiles():
    cases = []

    def ln(g):
        X = g.create("PlaceHolder", [6, 256], "float32")
        S = g.create("PlaceHolder", [256], "float32")
        B = g.create("PlaceHolder", [256], "float32")
        g.create("LayerNorm", X, S, B, 1, 1e-5)
    cases.append(("LayerNorm", ln, 4, ["sqrtf(", "__syncthreads();", "__shared__"]))

    def ew(g):
        X = g.create("PlaceHolder", [2, 48, 64], "float32")
        g.create("ElementWise", X, "Gelu", MemorySpace.global_)
    cases.append(("ElementWise", ew, 2, ["tanhf(", "kcg_v4_float"]))

    def sm(g):
        X = g.create("PlaceHolder", [3, 100], "float32")
        g.create("Softmax", X, -1, MemorySpace.inplace)
    cases.append(("Softmax", sm, 1, ["expf(", "__syncthreads();"]))

    def cmp_(g):
        X = g.create("PlaceHolder", [4, 8], "float32")
        Y = g.create("PlaceHolder", [8], "float32")
        g.create("Binary", X, Y, "Greater")
    cases.append(("Binary", cmp_, 3, ["unsigned char* __restrict__ out0", "(unsigned char)"]))

    def gather(g):
        X = g.create("PlaceHolder", [16, 24], "bfloat16")
        I = g.create("PlaceHolder", [4, 2], "index")
        g.create("Gather", X, I, 0)
    cases.append(("Gather", gather, 3, ["__bf16* __restrict__ arg0", "long* __restrict__ arg1"]))

    def bmm(g):
        A = g.create("PlaceHolder", [2, 64, 128], "float32")
        B = g.create("PlaceHolder", [2, 128, 64], "float32")
        g.create("BatchedMatmul", A, Layout.colMajor, B, Layout.colMajor)
    cases.append(("BatchMatmul", bmm, 3, ["blockIdx.z", "__shared__"]))

    for opt, build, nargs, needles in cases:
        gen = KernelCodeGenerator("ROCm")
        g = gen.createGraph("one")
        gen.opts.append(opt)
        build(g)
        body, (info,), _ = schedule_source(gen, g)
        assert info["num_args"] == nargs, opt
        for needle in needles:
            assert needle in body, (opt, needle)


def test_families_stay_the_default_and_the_switch_goes_both_ways():
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("mm")
    gen.opts.append("Matmul")
    A = g.create("PlaceHolder", [128, 64], "float32")
    B = g.create("PlaceHolder", [64, 128], "float32")
    g.create("Matmul", A, B)
    m = gen.optimize(g)
    assert "mfma_f32_32x32x2f32" in gen.codegen(m)
    assert gen.launchInfos()[0]["lowering"] == "family gemm_f32"
    gen.setLowering("schedule")
    assert "KCG_SCHEDULE_HELPERS" in gen.codegen(m)
    assert gen.launchInfos()[0]["lowering"] == "schedule"
    gen.setLowering("families")
    src = gen.codegen(m)
    assert "mfma_f32_32x32x2f32" in src and "KCG_SCHEDULE_HELPERS" not in src
    with pytest.raises(GeneratorError, match="families"):
        gen.setLowering("cuda")


def test_float64_falls_back_to_the_schedule_by_itself():
    """No LayerNorm family has an f64 form: codegen prints the schedule instead of refusing the operator, and says why."""
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("ln64")
    gen.opts.append("LayerNorm")
    X = g.create("PlaceHolder", [64, 256], "float64")
    S = g.create("PlaceHolder", [256], "float64")
    B = g.create("PlaceHolder", [256], "float64")
    g.create("LayerNorm", X, S, B, 1, 1e-5)
    m = gen.optimize(g)
    src = gen.codegen(m)
    (info,) = gen.launchInfos()
    assert gen.skippedFunctions() == [] and info["arg_bytes"] == [64 * 256 * 8, 256 * 8, 256 * 8, 64 * 256 * 8]
    assert "KCG_SCHEDULE_HELPERS" in src and "double* __restrict__ arg0" in src and "double reg" in src
    assert info["lowering"].startswith("schedule (") and "neither f32, f16 nor bf16" in info["lowering"]   # says why
    assert len(K.compile_to_code(src)) > 1000


def test_float64_matmul_gets_the_f64_mfma_family_and_its_schedule_on_request():
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("mm64")
    gen.opts.append("Matmul")
    A = g.create("PlaceHolder", [128, 64], "float64")
    B = g.create("PlaceHolder", [64, 128], "float64")
    g.create("Matmul", A, B)
    m = gen.optimize(g)
    assert gen.skippedFunctions() == [] and "kcg.cfg.VECTORIZE_WIDTH = 2" in gen._dump(1)
    src = gen.codegen(m)
    (info,) = gen.launchInfos()
    assert info["lowering"] == "family gemm_f64" and "__builtin_amdgcn_mfma_f64_16x16x4f64" in src
    assert info["arg_bytes"] == [128 * 64 * 8, 64 * 128 * 8, 128 * 128 * 8] and info["block"] == [256, 1, 1]
    assert len(K.compile_to_code(src)) > 1000
    gen.setLowering("schedule")
    src = gen.codegen(m)
    (info,) = gen.launchInfos()
    assert info["grid"] == [2, 2, 1] and info["block"] == [16, 16, 1]
    assert "KCG_SCHEDULE_HELPERS" in src and "kcg_v2_double" in src and "double reg" in src
    assert len(K.compile_to_code(src)) > 1000
    a, b = O.uniform((128, 64), 1), O.uniform((64, 128), 2)
    assert O.rel_frobenius(gen.interpret([a, b], (128, 128), which=1), O.matmul_f64(a, b)) <= 1e-7   # fp32 at the boundary of interpret()


def test_tree_reduction_option_builds_the_reference_tree():
    """TREE_REDUCE=1: halving steps, shuffles in the last wavefront, one shared cell (reference
    src/Optimizer/Optimizer.cc:1623-1749); the interpreter's barrier audit passes and the result is the oracle's."""
    shape = (6, 1024)
    x, gamma, beta = O.normal(shape, 305), O.uniform((1024,), 306, 0.5, 1.5), O.uniform((1024,), 307, -0.1, 0.1)
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("LayerNorm", [{"BLOCK_SIZE": 1024, "THREAD_SIZE": 4, "VECTORIZE_WIDTH": 4, "TREE_REDUCE": 1}])
    g = gen.createGraph("ln")
    gen.opts.append("LayerNorm")
    X = g.create("PlaceHolder", list(shape), "float32")
    S = g.create("PlaceHolder", [1024], "float32")
    B = g.create("PlaceHolder", [1024], "float32")
    g.create("LayerNorm", X, S, B, 1, 1e-5)
    body, (info,), ir = schedule_source(gen, g)
    assert ir.count("gpu.shuffle") == 12 and ir.count("memref<1xf32, 2>") >= 2 and "kcg.cfg.TREE_REDUCE = 1" in ir
    assert body.count("__shfl_down(") == 12 and body.count("__syncthreads();") == ir.count("gpu.barrier") == 8
    out = gen.interpret([x, gamma, beta], shape, which=1)          # raises if the schedule would race on the GPU
    assert O.rel_frobenius(out, O.layernorm_f64(x, gamma, beta, 1, 1e-5)) <= 1e-6
    # the kernel family still takes the function: the option changes the schedule, not the operator
    gen.setLowering("families")
    assert "KCG_SCHEDULE_HELPERS" not in gen.codegen()


@pytest.mark.parametrize("shape", [[23, 55], [11, 245], [1, 1021]])
def test_elementwise_schedule_keeps_its_workgroup_within_1024_threads(shape):
    """Extents with few divisors leave the elementwise schedule thread tiles of one element; its block tile must then
    shrink until the workgroup has at most 1024 threads (23 x 55 used to give one of 1265, which no lowering can launch)."""
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("e")
    gen.opts.append("ElementWise")
    x = g.create("PlaceHolder", shape, "float32")
    g.create("ElementWise", x, "Tanh", MemorySpace.global_)
    gen.optimize(g)
    ok, msg = gen.verify(1)
    assert ok, msg
    data = O.normal(tuple(shape), 7)
    assert np.array_equal(gen.interpret([data], tuple(shape), which=1), gen.interpret([data], tuple(shape), which=0))
    gen.setLowering("schedule")
    src = gen.codegen()
    (info,) = gen.launchInfos()
    assert info["block"][0] * info["block"][1] * info["block"][2] <= 1024
    assert info["grid"][0] * info["grid"][1] * info["block"][0] * info["block"][1] >= shape[0] * shape[1] // 16
    assert len(K.compile_to_code(src)) > 500


def test_families_only_turns_a_refusal_into_an_error():
    """A function whose kernel family has no form for it (here: attention with a head dim of 8) is lowered from its
    schedule under "families", and is an error of codegen() under "families-only", for callers that must not get the
    statement-by-statement kernel unnoticed."""
    from kernelcodegen_amd.generator import GeneratorError, KernelCodeGenerator, Layout, MemorySpace
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("FMHA", [{"BLOCK_SIZE": 16, "CAUSAL": 0, "SCALE_RSQRT_D": 1}])
    g = gen.createGraph("attn")
    gen.opts.append("FMHA")
    Q, K, V = (g.create("PlaceHolder", [1, 2, 32, 8], "float32") for _ in range(3))
    S = g.create("BatchedMatmul", Q, Layout.rowMajor, K, Layout.colMajor)
    P = g.create("Softmax", S, -1, MemorySpace.inplace)
    g.create("BatchedMatmul", P, Layout.rowMajor, V, Layout.rowMajor)
    m = gen.optimize(g)
    gen.setLowering("families")
    gen.codegen(m)
    (info,) = gen.launchInfos()
    assert info["lowering"].startswith("schedule (") and "head dims" in info["lowering"]
    gen.setLowering("families-only")
    with pytest.raises(GeneratorError) as err:
        gen.codegen(m)
    assert "head dims" in str(err.value)
    with pytest.raises(GeneratorError):
        gen.setLowering("fast")
