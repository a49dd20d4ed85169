"""Optimizer schedules and the HIP backend, end to end on the CPU:
graph -> optimize -> (host interpreter == oracle) -> codegen -> hipRTC compile.
The scheduled function runs on the interpreter with all threads of a workgroup
in lock-step, so a wrong index map, a missing barrier-side copy or a
double-buffer slip shows up as a numerical difference or an out-of-bounds trap."""
import re

import numpy as np
import pytest

import oracle_lib as O
import kernelcodegen_amd as K
from kernelcodegen_amd.generator import GeneratorError, KernelCodeGenerator, Layout, MemorySpace

SMALL_GEMM = [{"BLOCK_SIZE_M": 32, "BLOCK_SIZE_N": 32, "BLOCK_SIZE_K": 8, "THREAD_SIZE_M": 4, "THREAD_SIZE_N": 4,
               "VECTORIZE_WIDTH": 4, "WARP_SIZE": 64}]



def _gemm_f32_define(src, name, value):
    """A parameter of the fp32 GEMM family in emitted source: of the general kernel (GM_) or of the kernel that loads
    whole tiles of two row-major operands straight into LDS (GL_)."""
    return any("#define %s_%s %s" % (pre, name, value) in src for pre in ("GM", "GL"))


def test_matmul_schedule_is_bit_exact_and_emits_an_mfma_kernel():
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("mm")
    gen.opts.append("Matmul")
    a, b = O.uniform((128, 64), 1), O.uniform((64, 256), 2)
    A = g.create("PlaceHolder", [128, 64], "float32")
    B = g.create("PlaceHolder", [64, 256], "float32")
    g.create("Matmul", A, B)
    m = gen.optimize(g)
    ok, msg = gen.verify(1)
    assert ok, msg
    assert gen.functionState("Matmul_m128n256k64") == "gpu"
    assert np.array_equal(gen.interpret([a, b], (128, 256), which=1), O.matmul(a, b))
    src = gen.codegen(m)
    (info,) = gen.launchInfos()
    assert info["name"] == "kernel0" and info["function"] == "Matmul_m128n256k64"
    assert info["grid"] == [2, 1, 1] and info["block"] == [256, 1, 1]      # 128x128 tiles, 4 wavefronts
    assert info["num_args"] == 3 and info["arg_bytes"] == [128 * 64 * 4, 64 * 256 * 4, 128 * 256 * 4]
    assert "__builtin_amdgcn_mfma_f32_32x32x2f32" in src and _gemm_f32_define(src, "BK", 16)
    assert "// grid dims:(1, 1, 2, ), block dims:(1, 1, 256, )" in src
    assert len(K.compile_to_code(src)) > 1000


@pytest.mark.parametrize("warp", [32, 64])
def test_matmul_schedule_small_tiles_both_wave_widths(warp):
    gen = KernelCodeGenerator("ROCm")
    cfg = dict(SMALL_GEMM[0], WARP_SIZE=warp)
    gen.setConfigs("Matmul", [cfg])
    g = gen.createGraph("mm")
    gen.opts.append("Matmul")
    a, b = O.uniform((64, 48), 3), O.uniform((48, 96), 4)
    A = g.create("PlaceHolder", [64, 48], "float32")
    B = g.create("PlaceHolder", [48, 96], "float32")
    g.create("Matmul", A, B)
    gen.optimize(g)
    assert gen.functionState("Matmul_m64n96k48") == "gpu"
    assert np.array_equal(gen.interpret([a, b], (64, 96), which=1), O.matmul(a, b))
    text = gen._dump(1)
    assert "memref<2x8x32xf32, 2>" in text and "memref<4x4xf32, 3>" in text and "gpu.barrier" in text
    assert "affine_set<(d0) : (-d0 + 32 >= 0)>" in text          # K - 2*BK = 48 - 16


@pytest.mark.parametrize("m,n,k,cfg", [(100, 77, 33, None), (45, 70, 9, SMALL_GEMM[0]), (64, 96, 17, SMALL_GEMM[0])])
def test_matmul_not_divisible_gets_the_guarded_schedule(m, n, k, cfg):
    """Extents that are no multiples of the tile (the reference's optimizer refuses them): loops rounded up, the body
    under `if (m < M && n < N)`, tiled over workgroups and threads without shared tiles.  Bit-exact on the interpreter;
    the GEMM family takes the function (it guards its own edges) and so does the statement-by-statement lowering."""
    gen = KernelCodeGenerator("ROCm")
    if cfg:
        gen.setConfigs("Matmul", [cfg])
    g = gen.createGraph("mm")
    gen.opts.append("Matmul")
    a, b = O.uniform((m, k), 21), O.uniform((k, n), 22)
    A = g.create("PlaceHolder", [m, k], "float32")
    B = g.create("PlaceHolder", [k, n], "float32")
    g.create("Matmul", A, B)
    mod = gen.optimize(g)
    name = "Matmul_m%dn%dk%d" % (m, n, k)
    assert gen.functionState(name) == "gpu" and gen.skippedFunctions() == []
    ok, msg = gen.verify(1)
    assert ok, msg
    text = gen._dump(1)
    assert "kcg.ragged = 1" in text and "affine_set<(d0, d1) : (-d0 + %d >= 0, -d1 + %d >= 0)>" % (m - 1, n - 1) in text
    assert np.array_equal(gen.interpret([a, b], (m, n), which=1), O.matmul(a, b))
    bm = cfg["BLOCK_SIZE_M"] if cfg else 128
    src = gen.codegen(mod)
    (info,) = gen.launchInfos()
    assert info["lowering"] == "family gemm_f32" and info["grid"][0] == -(-m // bm) * -(-n // bm)
    assert _gemm_f32_define(src, "M", m) and len(K.compile_to_code(src)) > 1000
    gen.setLowering("schedule")
    src = gen.codegen(mod)
    (info,) = gen.launchInfos()
    assert info["grid"] == [-(-n // bm), -(-m // bm), 1] and len(K.compile_to_code(src)) > 1000


def test_batched_matmul_not_divisible_gets_the_guarded_schedule():
    batch, m, n, k = (2, 2), 33, 40, 12
    a, b = O.uniform(batch + (k, m), 23), O.uniform(batch + (n, k), 24)          # both operands column-major
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("BatchMatmul", SMALL_GEMM)
    g = gen.createGraph("bmm")
    gen.opts.append("BatchMatmul")
    A = g.create("PlaceHolder", list(a.shape), "float32")
    B = g.create("PlaceHolder", list(b.shape), "float32")
    g.create("BatchedMatmul", A, Layout.colMajor, B, Layout.colMajor)
    mod = gen.optimize(g)
    ok, msg = gen.verify(1)
    assert ok, msg
    text = gen._dump(1)
    assert "kcg.ragged = 1" in text and "= (0, 0, 0) to (4, 2, 2)" in text            # batch 2 x 2 as one grid dimension
    want = np.matmul(np.swapaxes(a, -1, -2).astype(np.float64), np.swapaxes(b, -1, -2).astype(np.float64))
    assert O.rel_frobenius(gen.interpret([a, b], batch + (m, n), which=1), want) <= 1e-6
    src = gen.codegen(mod)
    (info,) = gen.launchInfos()
    assert info["lowering"] == "family gemm_f32" and gen.skippedFunctions() == [] and len(K.compile_to_code(src)) > 1000


def test_matmul_not_divisible_is_left_unscheduled_on_request():
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("Matmul", [dict(SMALL_GEMM[0], RAGGED=0)])
    g = gen.createGraph("mm")
    gen.opts.append("Matmul")
    A = g.create("PlaceHolder", [100, 64], "float32")
    B = g.create("PlaceHolder", [64, 128], "float32")
    g.create("Matmul", A, B)
    m = gen.optimize(g)
    assert gen.functionState("Matmul_m100n128k64") == "cpu"
    assert gen.codegen(m).count("__global__") == 0 and gen.launchInfos() == []
    assert gen.skippedFunctions() == ["Matmul_m100n128k64"]


def test_batched_matmul_schedule():
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("BatchMatmul", SMALL_GEMM)
    g = gen.createGraph("bmm")
    gen.opts.append("BatchMatmul")
    a, b = O.uniform((3, 64, 16), 5), O.uniform((3, 16, 32), 6)
    A = g.create("PlaceHolder", [3, 64, 16], "float32")
    B = g.create("PlaceHolder", [3, 16, 32], "float32")
    g.create("BatchedMatmul", A, Layout.rowMajor, B, Layout.rowMajor)
    m = gen.optimize(g)
    name = "BatchMatmul_3_m64_n32_k16_NN"
    assert gen.functionState(name) == "gpu"
    assert np.array_equal(gen.interpret([a, b], (3, 64, 32), which=1), O.batched_matmul(a, b))
    assert "affine.parallel (%arg3, %arg4, %arg5) = (0, 0, 0) to (3, 2, 1)" in gen._dump(1)   # grid (batch, M/32, N/32)
    src = gen.codegen(m)
    (info,) = gen.launchInfos()
    assert info["grid"] == [2, 3, 1] and _gemm_f32_define(src, "BATCH", 3)
    assert len(K.compile_to_code(src)) > 1000


def test_bf16_matmul_picks_the_16_bit_config_and_kernel():
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("mm16")
    gen.opts.append("Matmul")
    A = g.create("PlaceHolder", [512, 256], "bfloat16")
    B = g.create("PlaceHolder", [256, 512], "bfloat16")
    g.create("Matmul", A, B, "float32")
    m = gen.optimize(g)
    assert gen.functionState("Matmul_m512n512k256") == "gpu"
    src = gen.codegen(m)
    (info,) = gen.launchInfos()
    assert "__builtin_amdgcn_mfma_f32_32x32x16_bf16" in src
    assert "#define GB_BM 256" in src and "#define GB_BK 64" in src and info["block"] == [512, 1, 1]
    assert info["arg_bytes"] == [512 * 256 * 2, 256 * 512 * 2, 512 * 512 * 4]
    assert len(K.compile_to_code(src)) > 1000


@pytest.mark.parametrize("shape", [(2, 48, 64), (6, 10), (3, 5, 7)])
@pytest.mark.parametrize("op,ms", [("Gelu", MemorySpace.global_), ("Relu", MemorySpace.inplace), ("Tanh", MemorySpace.global_)])
def test_elementwise_schedule(shape, op, ms):
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("ew")
    gen.opts.append("ElementWise")
    x = O.normal(shape, 7)
    X = g.create("PlaceHolder", list(shape), "float32")
    g.create("ElementWise", X, op, ms)
    m = gen.optimize(g)
    name = "%s_Elementwise_%s" % (op, "_".join(map(str, shape)))
    assert gen.functionState(name) == "gpu"
    ok, msg = gen.verify(1)
    assert ok, msg
    assert np.array_equal(gen.interpret([x], shape, which=1), O.elementwise(x, op))
    src = gen.codegen(m)
    (info,) = gen.launchInfos()
    assert info["num_args"] == (1 if ms == MemorySpace.inplace else 2)
    assert len(K.compile_to_code(src)) > 1000


@pytest.mark.parametrize("shape,axis,gshape,tpr", [((6, 256), 1, (256,), 64), ((3, 2, 16, 32), 2, (16, 32), 128),
                                                   ((4, 100), 1, (100,), 4)])
def test_layernorm_schedule(shape, axis, gshape, tpr):
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("LayerNorm", [{"BLOCK_SIZE": tpr * 4, "THREAD_SIZE": 4, "VECTORIZE_WIDTH": 4}])
    g = gen.createGraph("ln")
    gen.opts.append("LayerNorm")
    x = O.normal(shape, 8)
    s, b = O.uniform(gshape, 9, 0.5, 1.5), O.uniform(gshape, 10, -0.1, 0.1)
    X = g.create("PlaceHolder", list(shape), "float32")
    S = g.create("PlaceHolder", list(gshape), "float32")
    Bv = g.create("PlaceHolder", list(gshape), "float32")
    g.create("LayerNorm", X, S, Bv, axis, 1e-5)
    m = gen.optimize(g)
    ok, msg = gen.verify(1)
    assert ok, msg
    out = gen.interpret([x, s, b], shape, which=1)
    # the cross-thread reduction changes the summation order: compare to fp64 truth and to the nest
    assert O.rel_frobenius(out, O.layernorm_f64(x, s, b, axis)) <= 1e-6
    assert np.allclose(out, O.layernorm(x, s, b, axis), rtol=0, atol=3e-6)
    text = gen._dump(1)
    assert "gpu.barrier" in text and ", 2>" in text        # partial sums go through shared memory
    src = gen.codegen(m)
    (info,) = gen.launchInfos()
    rows = int(np.prod(shape[:axis]))
    assert info["num_args"] == 4 and "#define LN_ROWS %d" % rows in src and "#define LN_EPS 0x1.4f8b58p-17f" in src
    assert len(K.compile_to_code(src)) > 1000


def test_fmha_fusion_matches_the_unfused_graph_and_the_oracle():
    shp = (2, 2, 32, 8)
    q, k, v = O.normal(shp, 11), O.normal(shp, 12), O.normal(shp, 13)
    for causal, scaled in [(0, 0), (1, 0), (0, 1), (1, 1)]:
        gen = KernelCodeGenerator("ROCm")
        gen.setConfigs("FMHA", [{"BLOCK_SIZE": 16, "CAUSAL": causal, "SCALE_RSQRT_D": scaled}])
        g = gen.createGraph("attn")
        gen.opts.append("FMHA")
        Q = g.create("PlaceHolder", list(shp), "float32")
        Kv = g.create("PlaceHolder", list(shp), "float32")
        V = g.create("PlaceHolder", list(shp), "float32")
        S = g.create("BatchedMatmul", Q, Layout.rowMajor, Kv, Layout.colMajor)
        P = g.create("Softmax", S, -1, MemorySpace.inplace)
        g.create("BatchedMatmul", P, Layout.rowMajor, V, Layout.rowMajor)
        gen.optimize(g)
        ok, msg = gen.verify(1)
        assert ok, msg
        text = gen._dump(1)
        assert text.count("func.call") == 1 and "func.call @Fused_Multi_Head_Attention_2_2_SL32_HD8" in text
        out = gen.interpret([q, k, v], shp, which=1)
        scale = 1.0 / np.sqrt(8.0) if scaled else 1.0
        truth = O.fmha_f64(q, k, v, scale=scale, causal=bool(causal))
        assert O.rel_frobenius(out, truth) <= 2e-6, (causal, scaled)
        if not causal and not scaled:
            assert np.allclose(out, gen.interpret([q, k, v], shp, which=0), atol=3e-6)   # the three unfused nests


def test_fmha_fusion_stages_key_and_value_tiles_in_shared_memory():
    """The fused attention function walks the keys in tiles that the workgroup copies into shared memory, with a
    barrier after the copy and one after the tile's last use (the interpreter's barrier audit runs on it), under
    every combination of mask and tile length; a tile length the threads cannot share out evenly falls back to
    reading the keys from global memory."""
    shp = [2, 3, 64, 32]
    q, k, v = (O.normal(tuple(shp), stream=s) for s in (171, 172, 173))
    for causal in (0, 1):
        for bc, tiles in ((16, True), (0, True), (8, True), (12, False)):
            gen = KernelCodeGenerator("ROCm")
            cfg = {"BLOCK_SIZE": 16, "CAUSAL": causal, "SCALE_RSQRT_D": 1}
            if bc:
                cfg["BLOCK_SIZE_KV"] = bc
            gen.setConfigs("FMHA", [cfg])
            g = gen.createGraph("attn")
            gen.opts.append("FMHA")
            Q, K, V = (g.create("PlaceHolder", shp, "float32") for _ in range(3))
            S = g.create("BatchedMatmul", Q, Layout.rowMajor, K, Layout.colMajor)
            P = g.create("Softmax", S, -1, MemorySpace.inplace)
            g.create("BatchedMatmul", P, Layout.rowMajor, V, Layout.rowMajor)
            gen.optimize(g)
            text = gen._dump(1)
            fused = text[text.index("func.func @Fused_Multi_Head_Attention"):]
            if tiles:
                rows = bc or 64
                assert fused.count("gpu.barrier") == 2
                assert fused.count("memref.alloc() : memref<%dx32xf32, 2>" % rows) == 2
                assert "kcg.cfg.BLOCK_SIZE_KV = %d" % rows in fused
            else:
                assert "gpu.barrier" not in fused and "kcg.cfg.BLOCK_SIZE_KV = 0" in fused
            out = gen.interpret([q, k, v], tuple(shp), which=1)
            truth = O.fmha_f64(q, k, v, scale=32 ** -0.5, causal=bool(causal))
            assert O.rel_frobenius(out, truth) <= 1e-6


def test_fmha_fusion_takes_a_sequence_length_its_block_does_not_divide():
    """50 queries in workgroups of 16: a fourth, partly filled workgroup whose surplus threads do nothing (their whole
    body sits under `row < 50`), keys read from global memory (no barrier under a condition that differs between
    threads).  On the interpreter against the oracle, masked and not; both lowerings give a kernel that compiles;
    RAGGED = 0 leaves the graph unfused."""
    shp = (2, 2, 50, 8)
    q, k, v = O.normal(shp, 21), O.normal(shp, 22), O.normal(shp, 23)
    for causal in (0, 1):
        gen = KernelCodeGenerator("ROCm")
        gen.setConfigs("FMHA", [{"BLOCK_SIZE": 16, "CAUSAL": causal, "SCALE_RSQRT_D": 1}])
        g = gen.createGraph("attn")
        gen.opts.append("FMHA")
        Q, Kv, V = (g.create("PlaceHolder", list(shp), "float32") for _ in range(3))
        S = g.create("BatchedMatmul", Q, Layout.rowMajor, Kv, Layout.colMajor)
        P = g.create("Softmax", S, -1, MemorySpace.inplace)
        g.create("BatchedMatmul", P, Layout.rowMajor, V, Layout.rowMajor)
        m = gen.optimize(g)
        ok, msg = gen.verify(1)
        assert ok, msg
        text = gen._dump(1)
        fused = text[text.index("func.func @Fused_Multi_Head_Attention_2_2_SL50_HD8"):]
        assert "(2, 2, 4)" in fused and "affine.if" in fused and "gpu.barrier" not in fused
        out = gen.interpret([q, k, v], shp, which=1)
        assert O.rel_frobenius(out, O.fmha_f64(q, k, v, scale=8 ** -0.5, causal=bool(causal))) <= 2e-6
        src = gen.codegen(m)          # a head dim of 8: no attention family takes it, the schedule as written
        (info,) = gen.launchInfos()
        assert info["lowering"].startswith("schedule") and info["grid"] == [4, 2, 2] and info["block"] == [16, 1, 1]
        assert len(K.compile_to_code(src)) > 1000
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("FMHA", [{"BLOCK_SIZE": 16, "CAUSAL": 0, "SCALE_RSQRT_D": 1, "RAGGED": 0}])
    g = gen.createGraph("attn")
    gen.opts.append("FMHA")
    Q, Kv, V = (g.create("PlaceHolder", list(shp), "float32") for _ in range(3))
    S = g.create("BatchedMatmul", Q, Layout.rowMajor, Kv, Layout.colMajor)
    P = g.create("Softmax", S, -1, MemorySpace.inplace)
    g.create("BatchedMatmul", P, Layout.rowMajor, V, Layout.rowMajor)
    gen.optimize(g)
    assert "Fused_Multi_Head_Attention" not in gen._dump(1)


@pytest.mark.parametrize("dtype", ["bfloat16", "float16"])
def test_fmha_bf16_codegen(dtype):
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("FMHA", [{"BLOCK_SIZE": 128, "CAUSAL": 1, "SCALE_RSQRT_D": 1}])
    g = gen.createGraph("attn")
    gen.opts.append("FMHA")
    shp = [2, 4, 256, 128]
    Q = g.create("PlaceHolder", shp, dtype)
    Kv = g.create("PlaceHolder", shp, dtype)
    V = g.create("PlaceHolder", shp, dtype)
    S = g.create("BatchedMatmul", Q, Layout.rowMajor, Kv, Layout.colMajor, "float32")
    P = g.create("Softmax", S, -1, MemorySpace.inplace)
    g.create("BatchedMatmul", P, Layout.rowMajor, V, Layout.rowMajor, dtype)
    m = gen.optimize(g)
    src = gen.codegen(m)
    assert ("#define FA_F16 1" in src) == (dtype == "float16")          # one family for both 16-bit float types
    (info,) = gen.launchInfos()
    assert info["function"].startswith("Fused_Multi_Head_Attention_2_4_SL256_HD128") and info["num_args"] == 4
    assert "mfma" in src
    assert len(K.compile_to_code(src)) > 1000


def test_several_operators_in_one_module_get_numbered_kernels():
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("demo")
    for name in ("Matmul", "ElementWise", "LayerNorm"):
        gen.opts.append(name)
    A = g.create("PlaceHolder", [128, 128], "float32")
    B = g.create("PlaceHolder", [128, 128], "float32")
    Cv = g.create("Matmul", A, B)
    g.create("Relu", Cv, MemorySpace.inplace)
    X = g.create("PlaceHolder", [64, 1024], "float32")
    S = g.create("PlaceHolder", [1024], "float32")
    Bv = g.create("PlaceHolder", [1024], "float32")
    Y = g.create("LayerNorm", X, S, Bv, 1, 1e-5)
    g.create("ElementWise", Y, "Gelu", MemorySpace.global_)
    m = gen.optimize(g)
    src = gen.codegen(m)
    infos = gen.launchInfos()
    # the Matmul absorbs its Relu; the GELU was scheduled (ElementWise runs before LayerNorm here)
    # before the LayerNorm could absorb it, so it stays a kernel of its own
    assert [i["name"] for i in infos] == ["kernel0", "kernel1", "kernel2"]
    assert sorted(i["function"].split("_")[0] for i in infos) == ["Gelu", "LayerNorm", "Matmul"]
    assert src.count('extern "C" __global__') == 3 and _gemm_f32_define(src, "RELU", 1)
    assert len(K.compile_to_code(src)) > 1000


def test_unknown_platform_is_an_error_not_undefined_behaviour():
    gen = KernelCodeGenerator("CUDA")
    g = gen.createGraph("x")
    gen.opts.append("ElementWise")
    X = g.create("PlaceHolder", [8, 8], "float32")
    g.create("ElementWise", X, "Relu", MemorySpace.global_)
    m = gen.optimize(g)
    with pytest.raises(GeneratorError, match="not supported"):
        gen.codegen(m)


def _pass_md():
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "pass_md_structure.json")) as f:
        return json.load(f)


def test_matmul_schedule_reproduces_the_reference_dump_structure():
    """The reference's own optimized-Matmul dump (doc/pass.md:3-132, 2048x2048x1024 with its A100
    config) fixes buffer shapes, the prefetch guard and the launch shape; the same config through this
    schedule must give the same structure."""
    fx = _pass_md()["matmul_2048x2048x1024"]
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("mm")
    gen.opts.append("Matmul")
    gen.setConfigs("Matmul", [fx["config"]])
    A = g.create("PlaceHolder", [2048, 1024], "float32")
    B = g.create("PlaceHolder", [1024, 2048], "float32")
    g.create("Matmul", A, B)
    gen.optimize(g)
    ok, msg = gen.verify(1)
    assert ok, msg
    text = gen._dump(1)
    for shape in fx["shared_buffers"]:
        assert "memref<%sxf32, 2>" % "x".join(map(str, shape)) in text
    assert text.count("memref.alloc() : memref<2x8x128xf32, 2>") == 2
    assert text.count("memref.alloc() : memref<2x8xf32, 3>") == 2
    assert "memref.alloc() : memref<8x8xf32, 3>" in text
    assert "(%s)" % fx["prefetch_guard_set"] in text
    assert "affine.parallel" in text and "(16, 16)" in text


TILED_FMHA = {"BLOCK_SIZE": 128, "HdxBr": 128 * 64, "BrxBc": 128 * 64, "WarpX_O": 2, "Slice": 8, "BrTileS": 8, "BcTileS": 8,
              "BrTileO": 8, "HdTileO": 8, "Width": 4, "WARP_SIZE": 64}


def _attention_graph(shp, cfg, dtype="float32"):
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("FMHA", [cfg])
    g = gen.createGraph("attn")
    gen.opts.append("FMHA")
    Q, K, V = (g.create("PlaceHolder", list(shp), dtype) for _ in range(3))
    S = g.create("BatchedMatmul", Q, Layout.rowMajor, K, Layout.colMajor)
    P = g.create("Softmax", S, -1, MemorySpace.inplace)
    g.create("BatchedMatmul", P, Layout.rowMajor, V, Layout.rowMajor)
    m = gen.optimize(g)
    ok, msg = gen.verify(1)
    assert ok, msg
    text = gen._dump(1)
    fused = text[text.index("func.func @Fused_Multi_Head_Attention"):]
    return gen, m, fused[:fused.index("return %arg3")]


def test_tiled_attention_schedule_reproduces_the_reference_dump_structure():
    """The reference's own fused-attention dump (doc/pass.md:136-405: B8 H32 S2048 D64 fp32 under the config of
    include/KernelCodeGen.h:51-54) fixes the launch shape, every buffer, the loops, the barriers, the two integer
    sets and the shuffles; the same config through FMHAOptimizer must give the same structure.  Where the dump shows
    one of the reference's slips, the fixture says what the dump does and this schedule must differ in exactly that:
    the probability tile is allocated as it is indexed (64 x 128), the result store takes threadIdx.x for its thread id."""
    from kernelcodegen_amd.generator import fmha_map
    fx = _pass_md()["fmha_8_32_2048_64"]
    gen, m, fused = _attention_graph((8, 32, 2048, 64), dict(fx["config"], CAUSAL=0, SCALE_RSQRT_D=0))
    assert fused.startswith("func.func @%s(" % fx["function"])
    assert fused.count("memref<%sxf32, 1>" % fx["argument"]) >= 5       # Q, K, V, O and the result type
    assert "affine.parallel (%%arg4, %%arg5, %%arg6) = (0, 0, 0) to (%d, %d, %d)" % tuple(fx["grid"]) in fused
    assert "affine.parallel (%%arg7) = (0) to (%d)" % fx["block"][0] in fused
    allocs = re.findall(r"memref\.alloc\(\) : memref<([0-9x]+)xf32, (\d)>", fused)
    shape = lambda a: [int(t) for t in a[0].split("x")]
    head = allocs[:len(fx["workgroup_allocs"])]
    for got, want in zip(head, fx["workgroup_allocs"]):
        assert shape(got) == want.get("indexed_as", want["shape"]) and int(got[1]) == want["space"], (got, want)
    rest = [shape(a) for a in allocs[len(head):] if a[1] == "3"]
    # per key tile: Q and K staging registers and the score tile (in either order), two fragments per product,
    # row maximum / sum, the factor, the V staging registers; after the loop the sums
    for want in fx["key_tile_allocs"] + fx["fragment_allocs"]:
        assert want in rest, (want, rest)
    assert all(a[1] in "23" for a in allocs)                             # nothing in global memory
    for lo, hi, step in fx["loops"].values():
        assert ("= %d to %d step %d {" % (lo, hi, step)) in fused, (lo, hi, step)
    assert fused.count("gpu.barrier") == fx["barriers"]
    sets = [re.sub(r"\s", "", t) for t in re.findall(r"affine_set<\([^)]*\) : \((.*?)\)>\(", fused)]
    canon = lambda t: sorted(re.sub(r"\s", "", t).replace(">=0", "").replace("==0", "").replace("-", "+-").split("+"))
    assert any(canon(t) == canon(fx["statistics_init_set"]) and t.endswith(">=0") for t in sets), sets
    assert any(canon(t) == canon(fx["first_lane_set"]) and t.endswith("==0") for t in sets), sets
    assert fx["lowest"].lower() in fused.lower()
    sh = fx["shuffles"]
    assert fused.count("gpu.shuffle  down") + fused.count("gpu.shuffle down") == sh["down_count"]
    assert fused.count("gpu.shuffle  idx") + fused.count("gpu.shuffle idx") == sh["idx_count"]
    # the index maps at the fixture's sampled points (the dump's own access expressions, evaluated by hand there)
    pt, t = fx["sampled_points"], fx["sampled_points"]["tid"]
    q = pt["load_q_row_col"]
    assert fmha_map("loadTileQ", 1, 2, q["block"], t, q["hd_outer"], q["iv"]) == [1, 2] + q["value"]
    assert fmha_map("storeTileQ", t, q["iv"], 3) == [q["value"][1] - q["hd_outer"] + 3, q["value"][0] - q["block"] * 128]
    assert fmha_map("loadFragQ", t, 5, pt["frag_q_col"]["iv"]) == [5, pt["frag_q_col"]["value"]]
    assert fmha_map("loadFragK", t, 5, pt["frag_k_col"]["iv"]) == [5, pt["frag_k_col"]["value"]]
    assert fmha_map("brIdxS", t, pt["statistics_row"]["br"]) == [pt["statistics_row"]["value"]]
    assert fmha_map("storeTileP", t, pt["store_p"]["bc"], pt["store_p"]["br"]) == pt["store_p"]["value"]
    assert fmha_map("loadFactor", t, pt["factor_col"]["iv"]) == [pt["factor_col"]["value"]]
    assert fmha_map("brIdxO", t, pt["factor_col"]["iv"]) == [pt["factor_col"]["value"]]
    v = pt["load_v_row_col"]
    assert fmha_map("loadTileV", 1, 2, t, v["kv"], v["bc_outer"], v["iv"]) == [1, 2] + v["value"]
    assert fmha_map("storeTileV", t, v["iv"]) == [v["value"][0] - v["kv"] - v["bc_outer"], v["value"][1]]
    p = pt["frag_p"]
    assert fmha_map("loadFragP", t, p["bc_outer"], p["bc_inner"], p["iv"]) == p["value"]
    assert fmha_map("loadFragV", t, 3, pt["frag_v_col"]["iv"]) == [3, pt["frag_v_col"]["value"]]
    o = pt["store_o_row_col"]
    assert fmha_map("storeTileO", 1, 2, o["block"], t, o["br"], o["hd"]) == [1, 2] + o["value"]
    with pytest.raises(Exception):
        fmha_map("noSuchMap", 0)
    # and the function gets a kernel from the schedule lowering: grid (x, y, z) = (16, 32, 8), 128 threads
    gen.setLowering("schedule")
    src = gen.codegen(m)
    (info,) = gen.launchInfos()
    assert info["grid"] == [16, 32, 8] and info["block"] == [128, 1, 1] and info["lowering"] == "schedule"
    assert src.count("__syncthreads()") == fx["barriers"] and "__shfl_down" in src
    assert len(K.compile_to_code(src)) > 1000


def test_naive_attention_functions_match_the_reference_fixture():
    """The three unfused functions of the reference's attention graph as its dump shows them (doc/pass.md:406-467):
    names, argument shapes, loop extents, the two loads of each product."""
    fx = _pass_md()["naive_batch_matmul_softmax"]
    shp = fx["shape"]
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("attn")
    Q, K, V = (g.create("PlaceHolder", shp, "float32") for _ in range(3))
    S = g.create("BatchedMatmul", Q, Layout.rowMajor, K, Layout.colMajor)
    P = g.create("Softmax", S, -1, MemorySpace.inplace)
    g.create("BatchedMatmul", P, Layout.rowMajor, V, Layout.rowMajor)
    text = gen._dump(0)
    for name, want in fx["functions"].items():
        assert "func.func @%s(" % name in text, name
        body = text[text.index("func.func @%s(" % name):]
        body = body[:body.index("return")]
        head = body[:body.index("\n")]
        for i, a in enumerate(want["args"]):
            assert "%%arg%d: memref<%sxf32, 1>" % (i, a) in head
        assert 'func.state = "cpu"' in head
        extents = [int(t) for t in re.findall(r"affine\.for %arg\d+ = 0 to (\d+)", body)]
        assert extents == want["loops"], (name, extents)
        for load in want.get("loads", []):
            assert "affine.load " + load in body, (name, load)
        if "exp" in want:
            assert body.count("math.exp") == want["exp"] and body.count("arith.divf") == want["divf"]


@pytest.mark.parametrize("shp,warp,causal,scaled", [((1, 2, 256, 64), 32, 0, 0), ((1, 2, 256, 64), 64, 1, 1),
                                                    ((1, 1, 384, 128), 64, 0, 1), ((2, 1, 256, 128), 32, 1, 0)])
def test_tiled_attention_schedule_matches_the_oracle(shp, warp, causal, scaled):
    """The tiled schedule on the host interpreter (lock-step threads, so with its audit of barriers and with the
    shuffles between the threads that share a query) against fp64 attention: the reference's semantics (no scale, no
    mask) and with both, head dims 64 (Br 128, Bc 64) and 128 (Br 64, Bc 128), 32- and 64-thread layout units."""
    gen, m, fused = _attention_graph(shp, dict(TILED_FMHA, WARP_SIZE=warp, CAUSAL=causal, SCALE_RSQRT_D=scaled))
    assert "kcg.cfg.TILED = 1" in fused and "gpu.shuffle" in fused and fused.count("gpu.barrier") == 5
    q, k, v = (O.normal(shp, stream=s) for s in (271, 272, 273))
    out = gen.interpret([q, k, v], shp, which=1)
    truth = O.fmha_f64(q, k, v, scale=(shp[3] ** -0.5 if scaled else 1.0), causal=bool(causal))
    assert O.rel_frobenius(out, truth) <= 2e-6
    if not causal and not scaled:
        assert np.allclose(out, gen.interpret([q, k, v], shp, which=0), atol=3e-6)        # the three unfused nests


def test_attention_shapes_outside_the_tiled_layout_take_the_row_schedule():
    """A sequence length that Br does not divide, a head dim that HdxBr is no multiple of, or 16-bit operands: the
    fusion still happens, with one query row per thread."""
    for shp, dtype in (((1, 2, 200, 64), "float32"), ((1, 1, 256, 96), "float32"), ((1, 1, 256, 64), "bfloat16")):
        gen, m, fused = _attention_graph(shp, dict(TILED_FMHA, CAUSAL=0, SCALE_RSQRT_D=1), dtype)
        assert "kcg.cfg.TILED = 0" in fused and "gpu.shuffle" not in fused
        if dtype == "float32" and shp[2] <= 200:
            q, k, v = (O.normal(shp, stream=s) for s in (281, 282, 283))
            out = gen.interpret([q, k, v], shp, which=1)
            assert O.rel_frobenius(out, O.fmha_f64(q, k, v, scale=shp[3] ** -0.5)) <= 2e-6


@pytest.mark.parametrize("batched", [False, True])
def test_quantised_product_carries_its_scales_through_the_schedule(batched):
    """fp8 operands with their per-tensor fp32 scales as graph values: the naive nest and the scheduled function both
    compute (scale_a * scale_b) * A B on the interpreter, the kernel the function gets takes five pointers (no scalar
    arguments), and the plan lists the scales among the graph's inputs."""
    m, n, k = 128, 128, 64
    a, b = O.normal((m, k), 221), O.normal((k, n), 222, std=0.02)
    sa, sb = float(np.abs(a).max()) / 448.0, float(np.abs(b).max()) / 448.0
    aq, bq = O.from_fp8_bits(O.to_fp8_bits(a, 1.0 / sa)), O.from_fp8_bits(O.to_fp8_bits(b, 1.0 / sb))
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("mm8")
    gen.opts.append("BatchMatmul" if batched else "Matmul")
    A = g.create("PlaceHolder", [m, k], "float8_e4m3")
    B = g.create("PlaceHolder", [n, k] if batched else [k, n], "float8_e4m3")
    SA, SB = g.create("PlaceHolder", [1], "float32"), g.create("PlaceHolder", [1], "float32")
    if batched:
        g.create("BatchedMatmul", A, Layout.rowMajor, B, Layout.colMajor, SA, SB, "float32")
    else:
        g.create("Matmul", A, B, SA, SB, "float32")
    ins = [aq, np.ascontiguousarray(bq.T) if batched else bq, np.array([sa], np.float32), np.array([sb], np.float32)]
    truth = O.matmul_f64(aq, bq) * (np.float32(sa) * np.float32(sb))
    assert O.rel_frobenius(gen.interpret(ins, (m, n), which=0), truth) <= 1e-6
    module = gen.optimize(g)
    ok, msg = gen.verify(1)
    assert ok, msg
    assert O.rel_frobenius(gen.interpret(ins, (m, n), which=1), truth) <= 1e-6
    src = gen.codegen(module)
    (info,) = gen.launchInfos()
    assert info["function"].endswith("_scaled") and info["lowering"] == "family gemm_fp8"
    assert info["num_args"] == 5 and info["num_scalars"] == 0
    assert ("#define GF_SCALE_PTR %d" % (1 if batched else 2)) in src and len(K.compile_to_code(src)) > 1000
    plan = gen.plan(1)
    assert [bf["input"] for bf in plan["buffers"] if bf.get("shape") == [1]] == [2, 3]
    # a scale that is not one float32 element is refused
    with pytest.raises(GeneratorError):
        g.create("Matmul", A, B, A, SB, "float32")


def test_naive_layernorm_dump_matches_reference_fixture():
    fx = _pass_md()["layernorm_2_768_768_axis_1"]
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("ln")
    X = g.create("PlaceHolder", [2, 768, 768], "float32")
    S = g.create("PlaceHolder", [768, 768], "float32")
    Bv = g.create("PlaceHolder", [768, 768], "float32")
    g.create("LayerNorm", X, S, Bv, 1, 1e-5)
    text = g.dump()
    fn = text[text.index("func.func @%s(" % fx["function"]):]
    assert "arith.constant %s : f32" % fx["group_size_constant"] in fn
    assert fn.count("iter_args(") == fx["iter_args_loops"]
    assert fn.count("arith.divf") == fx["divf"] and fn.count("math.sqrt") == fx["sqrt"]


def test_layernorm_absorbs_a_following_gelu():
    shape = (8, 1024)
    x = O.normal(shape, 31)
    s, b = O.uniform((1024,), 32, 0.5, 1.5), O.uniform((1024,), 33, -0.1, 0.1)
    for fuse in (1, 0):
        gen = KernelCodeGenerator("ROCm")
        g = gen.createGraph("ln_gelu")
        gen.opts.append("LayerNorm")
        gen.opts.append("ElementWise")
        gen.setConfigs("LayerNorm", [{"BLOCK_SIZE": 1024, "THREAD_SIZE": 4, "VECTORIZE_WIDTH": 4, "FUSE_GELU": fuse}])
        X = g.create("PlaceHolder", list(shape), "float32")
        S = g.create("PlaceHolder", [1024], "float32")
        Bv = g.create("PlaceHolder", [1024], "float32")
        Y = g.create("LayerNorm", X, S, Bv, 1, 1e-5)
        g.create("ElementWise", Y, "Gelu", MemorySpace.global_)
        m = gen.optimize(g)
        ok, msg = gen.verify(1)
        assert ok, msg
        out = gen.interpret([x, s, b], shape, which=1)
        assert O.rel_frobenius(out, O.elementwise(O.layernorm(x, s, b, 1), "Gelu")) <= 1e-6
        src = gen.codegen(m)
        infos = gen.launchInfos()
        text = gen._dump(1)
        if fuse:
            assert len(infos) == 1 and "#define LN_GELU 1" in src
            assert "func.call @Gelu_Elementwise" not in text and "math.tanh" in text
        else:
            assert len(infos) == 2 and "#define LN_GELU 0" in src
            assert "func.call @Gelu_Elementwise_8_1024" in text


def test_gelu_with_another_consumer_is_not_fused():
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("ln_two_users")
    gen.opts.append("LayerNorm")
    X = g.create("PlaceHolder", [8, 256], "float32")
    S = g.create("PlaceHolder", [256], "float32")
    Bv = g.create("PlaceHolder", [256], "float32")
    Y = g.create("LayerNorm", X, S, Bv, 1, 1e-5)
    g.create("ElementWise", Y, "Gelu", MemorySpace.global_)
    g.create("ElementWise", Y, "Tanh", MemorySpace.global_)
    gen.optimize(g)
    text = gen._dump(1)
    assert "func.call @Gelu_Elementwise_8_256" in text and "kcg.fused_gelu" not in text


@pytest.mark.parametrize("batch", [(3,), (2, 3)])
@pytest.mark.parametrize("la,lb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_batched_matmul_schedule_layouts_and_batch_dims(batch, la, lb):
    """Every operand layout and several batch dims (collapsed into one grid dimension): the
    scheduled function on the lock-step interpreter equals the oracle bit for bit."""
    m, n, k = 64, 32, 16
    a = O.uniform(batch + ((k, m) if la else (m, k)), 5)
    b = O.uniform(batch + ((n, k) if lb else (k, n)), 6)
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("BatchMatmul", SMALL_GEMM)
    g = gen.createGraph("bmm")
    gen.opts.append("BatchMatmul")
    A = g.create("PlaceHolder", list(a.shape), "float32")
    B = g.create("PlaceHolder", list(b.shape), "float32")
    g.create("BatchedMatmul", A, la, B, lb)
    mod = gen.optimize(g)
    ok, msg = gen.verify(1)
    assert ok, msg
    name = "BatchMatmul_%s_m64_n32_k16_%s%s" % ("_".join(map(str, batch)), "NT"[la], "NT"[lb])
    assert gen.functionState(name) == "gpu"
    assert np.array_equal(gen.interpret([a, b], batch + (m, n), which=1), O.batched_matmul(a, b, bool(la), bool(lb)))
    src = gen.codegen(mod)
    (info,) = gen.launchInfos()
    assert info["grid"] == [2, int(np.prod(batch)), 1]
    if la or lb:
        assert "#define GM_TA %d" % la in src and "#define GM_TB %d" % lb in src
    else:                                             # two row-major operands: either kernel, and the direct-load one has no such switch
        assert "#define GL_NAME" in src or ("#define GM_TA 0" in src and "#define GM_TB 0" in src)


def test_matmul_absorbs_a_following_relu():
    a, b = O.uniform((128, 64), 41), O.uniform((64, 256), 42)
    for fuse in (1, 0):
        gen = KernelCodeGenerator("ROCm")
        g = gen.createGraph("mm_relu")
        gen.opts.append("Matmul")
        cfgs = gen.getConfigs("Matmul") if hasattr(gen, "getConfigs") else None
        if not fuse:
            gen.setConfigs("Matmul", [{"BLOCK_SIZE_M": 128, "BLOCK_SIZE_N": 128, "BLOCK_SIZE_K": 16, "GROUP_SIZE_M": 8,
                                       "THREAD_SIZE_M": 8, "THREAD_SIZE_N": 8, "VECTORIZE_WIDTH": 4, "WARP_SIZE": 64,
                                       "DTYPE_BITS": 32, "FUSE_RELU": 0}])
        A = g.create("PlaceHolder", [128, 64], "float32")
        B = g.create("PlaceHolder", [64, 256], "float32")
        C = g.create("Matmul", A, B)
        g.create("Relu", C, MemorySpace.inplace)
        m = gen.optimize(g)
        ok, msg = gen.verify(1)
        assert ok, msg
        out = gen.interpret([a, b], (128, 256), which=1)
        assert np.array_equal(out, np.maximum(O.matmul(a, b), 0))
        src = gen.codegen(m)
        text = gen._dump(1)
        assert _gemm_f32_define(src, "RELU", 1) == bool(fuse)
        assert ("func.call @Relu_Elementwise" in text) == (not fuse)


@pytest.mark.parametrize("sa,sb,op", [((16, 1, 1, 64), (1, 8, 64), "Add"), ((4, 6), (6,), "Mul"), ((3, 5, 7), (3, 5, 7), "Sub"),
                                      ((8, 12), (8, 1), "Div")])
def test_binary_schedule(sa, sb, op):
    x, y = O.uniform(sa, 51, 0.5, 2.0), O.uniform(sb, 52, 0.5, 2.0)
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("bin")
    gen.opts.append("Binary")
    X = g.create("PlaceHolder", list(sa), "float32")
    Y = g.create("PlaceHolder", list(sb), "float32")
    g.create("Binary", X, Y, op)
    m = gen.optimize(g)
    ok, msg = gen.verify(1)
    assert ok, msg
    ref = {"Add": x + y, "Mul": x * y, "Sub": x - y, "Div": x / y}[op].astype(np.float32)
    assert np.array_equal(gen.interpret([x, y], ref.shape, which=1), ref)
    src = gen.codegen(m)
    (info,) = gen.launchInfos()
    assert info["num_args"] == 3 and "#define BN_OP" in src
    assert len(K.compile_to_code(src)) > 1000


@pytest.mark.parametrize("op", ["Equal", "Greater"])
def test_binary_comparisons_give_one_byte_per_element(op):
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("cmp")
    gen.opts.append("Binary")
    X = g.create("PlaceHolder", [4, 8], "float32")
    Y = g.create("PlaceHolder", [8], "float32")
    g.create("Binary", X, Y, op)
    m = gen.optimize(g)
    ok, msg = gen.verify(1)
    assert ok, msg
    x, y = np.round(O.normal((4, 8), 53)), np.round(O.normal((8,), 54))     # small integers: equal pairs occur
    ref = (x == y) if op == "Equal" else (x > y)
    assert ref.any() and not ref.all()
    assert np.array_equal(gen.interpret([x, y], (4, 8), which=1).astype(bool), ref)
    src = gen.codegen(m)
    (info,) = gen.launchInfos()
    assert info["arg_bytes"] == [128, 32, 32] and "#define BN_OP %d" % (5 if op == "Equal" else 6) in src
    assert len(K.compile_to_code(src)) > 1000


@pytest.mark.parametrize("shape,ishape,axis,dtype", [((2, 5, 8), (2, 3), 1, "float32"), ((64, 32), (48,), 0, "float32"),
                                                      ((3, 7), (5,), 1, "float32"), ((4, 5, 6), (1,), 1, "float32"),
                                                      ((16, 24), (4, 2), 0, "bfloat16")])
def test_gather_schedule(shape, ishape, axis, dtype):
    x = O.normal(shape, stream=71)
    if dtype == "bfloat16":
        x = O.round_bf16(x)
    idx = np.random.RandomState(11).randint(0, shape[axis], size=ishape)
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("gather")
    gen.opts.append("Gather")
    X = g.create("PlaceHolder", list(shape), dtype)
    I = g.create("PlaceHolder", list(ishape), "index")
    g.create("Gather", X, I, axis)
    m = gen.optimize(g)
    ok, msg = gen.verify(1)
    assert ok, msg
    ref = O.gather(x, idx, axis)
    assert np.array_equal(gen.interpret([x, idx.astype(np.float32)], ref.shape, which=1), ref)
    src = gen.codegen(m)
    (info,) = gen.launchInfos()
    assert info["num_args"] == 3 and "#define GA_AXIS %d" % shape[axis] in src
    assert info["arg_bytes"][1] == 8 * idx.size
    assert len(K.compile_to_code(src)) > 1000


@pytest.mark.parametrize("shape", [(4, 6, 512), (3, 100), (2, 2, 8, 2048), (5, 1001)])
def test_standalone_softmax_schedule(shape):
    x = O.normal(shape, stream=81, std=2.0)
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("softmax")
    gen.opts.append("Softmax")
    X = g.create("PlaceHolder", list(shape), "float32")
    g.create("Softmax", X, -1, MemorySpace.inplace)
    m = gen.optimize(g)
    ok, msg = gen.verify(1)
    assert ok, msg
    ref = O.softmax(x.copy())
    # the team adds its partial sums in another order than the row loop does
    assert O.rel_frobenius(gen.interpret([x], shape, which=1), ref.astype(np.float64)) <= 1e-6
    src = gen.codegen(m)
    (info,) = gen.launchInfos()
    assert info["num_args"] == 1 and "#define SM_N %d" % shape[-1] in src
    assert len(K.compile_to_code(src)) > 1000


def test_softmax_inside_attention_is_left_to_the_fusion():
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("FMHA", [{"BLOCK_SIZE": 64, "CAUSAL": 0, "SCALE_RSQRT_D": 1}])
    g = gen.createGraph("attn")
    gen.opts.append("FMHA")
    gen.opts.append("Softmax")
    Q, Kk, V = (g.create("PlaceHolder", [1, 2, 128, 64], "float32") for _ in range(3))
    S = g.create("BatchedMatmul", Q, Layout.rowMajor, Kk, Layout.colMajor)
    P = g.create("Softmax", S, -1, MemorySpace.inplace)
    g.create("BatchedMatmul", P, Layout.rowMajor, V, Layout.rowMajor)
    m = gen.optimize(g)
    text = m.dump()
    assert "Fused_Multi_Head_Attention" in text
    assert 'kcg.op = "Softmax"' not in text


def test_imported_graph_runs_through_the_whole_generator():
    """kernelcodegen_amd.importer: a graph written as data with ONNX operator names goes through the Frontend
    builders, the optimizers (with their fusions) and the backend."""
    from kernelcodegen_amd.importer import import_graph
    desc = {"name": "block",
            "inputs": [{"name": "tok", "shape": [128], "dtype": "index"}, {"name": "table", "shape": [100, 64]},
                       {"name": "w", "shape": [64, 128]}, {"name": "g", "shape": [128]}, {"name": "b", "shape": [128]}],
            "nodes": [{"op": "Gather", "inputs": ["table", "tok"], "output": "x", "axis": 0},
                      {"op": "MatMul", "inputs": ["x", "w"], "output": "h"},
                      {"op": "Relu", "inputs": ["h"], "output": "h"},
                      {"op": "LayerNormalization", "inputs": ["h", "g", "b"], "output": "y", "axis": -1, "epsilon": 1e-5},
                      {"op": "Gelu", "inputs": ["y"], "output": "z"}]}
    import json
    gen, g, values = import_graph(json.dumps(desc))
    assert list(gen.opts) == ["Matmul", "LayerNorm", "Gather", "ElementWise"] and set(values) == {"tok", "table", "w", "g", "b", "x", "h", "y", "z"}
    gen.setConfigs("Matmul", SMALL_GEMM)
    m = gen.optimize(g)
    ok, msg = gen.verify(1)
    assert ok, msg
    tok = np.random.RandomState(0).randint(0, 100, size=128)
    table, w = O.normal((100, 64), 91), O.uniform((64, 128), 92)
    gm, bt = O.uniform((128,), 93, 0.5, 1.5), O.uniform((128,), 94, -0.1, 0.1)
    ref = O.elementwise(O.layernorm(np.maximum(O.matmul(O.gather(table, tok, 0), w), 0), gm, bt, 1), "Gelu")
    out = gen.interpret([tok.astype(np.float32), table, w, gm, bt], ref.shape, which=1)
    assert O.rel_frobenius(out, ref.astype(np.float64)) <= 1e-6
    src = gen.codegen(m)
    functions = sorted(i["function"] for i in gen.launchInfos())
    # Relu went into the Matmul kernel and Gelu into the LayerNorm kernel
    assert functions == ["Gather_100_64_indices_128_axis_0", "LayerNorm_128_128_axis_1", "Matmul_m128n128k64"]
    assert _gemm_f32_define(src, "RELU", 1) and "#define LN_GELU 1" in src
    assert len(K.compile_to_code(src)) > 1000
    with pytest.raises(GeneratorError, match="not supported by the importer"):
        import_graph({"inputs": [{"name": "x", "shape": [4]}], "nodes": [{"op": "Conv", "inputs": ["x"], "output": "y"}]})



def test_operators_over_a_single_row_are_scheduled():
    """Softmax of a vector, LayerNorm over the whole tensor (axis 0) and a Gather with one index along an inner axis
    have no loop over rows / take the loop index as a plain value; random graphs found all three unscheduled or
    aborting.  Each is scheduled now (a loop of one trip stands for the loop over the rows; `split` hands a plain-value
    user the sum of the new indices through an affine.apply), computes on the interpreter what the naive nest
    computes, and gets a kernel from both lowerings."""
    def finish(gen, g, inputs, shape, want, tol):
        gen.optimize(g)
        ok, msg = gen.verify(1)
        assert ok, msg
        assert O.rel_frobenius(gen.interpret(inputs, shape, which=1), want) <= tol
        for lowering in ("families", "schedule"):
            gen.setLowering(lowering)
            src = gen.codegen()
            assert gen.skippedFunctions() == [] and len(gen.launchInfos()) == 1
            assert len(K.compile_to_code(src)) > 500
    x = O.normal((37,), 5)
    gen = KernelCodeGenerator("ROCm"); g = gen.createGraph("g"); gen.opts.append("Softmax")
    g.create("Softmax", g.create("PlaceHolder", [37], "float32"), -1, MemorySpace.inplace)
    finish(gen, g, [x], (37,), O.softmax_f64(x), 2e-6)
    x, gm, bt = O.normal((16, 12), 6), O.uniform((16, 12), 7, 0.5, 1.5), O.uniform((16, 12), 8, -0.1, 0.1)
    gen = KernelCodeGenerator("ROCm"); g = gen.createGraph("g"); gen.opts.append("LayerNorm")
    X, S, B = (g.create("PlaceHolder", [16, 12], "float32") for _ in range(3))
    g.create("LayerNorm", X, S, B, 0, 1e-5)
    finish(gen, g, [x, gm, bt], (16, 12), O.layernorm(x, gm, bt, 0), 2e-6)
    x, idx = O.normal((4, 8), 9), np.array([5], dtype=np.int64)
    gen = KernelCodeGenerator("ROCm"); g = gen.createGraph("g"); gen.opts.append("Gather")
    g.create("Gather", g.create("PlaceHolder", [4, 8], "float32"), g.create("PlaceHolder", [1], "index"), 1)
    finish(gen, g, [x, idx], (4,), x[:, 5], 0.0)
