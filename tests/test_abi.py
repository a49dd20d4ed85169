"""The C-ABI library without a GPU: it loads, exports every function the two
public headers declare, compiles emitted kernels for gfx950 (hipRTC needs no
device) and reports errors through return codes and caller buffers."""
import ctypes as C
import os

import numpy as np
import re
import subprocess

import pytest

import kernelcodegen_amd as K
from kernelcodegen_amd import _lib, runtime as R

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    return sorted(set(re.findall(r"\b(kcg_[a-z0-9_]+)\s*\(", text)))


@pytest.mark.parametrize("header", ["kcg_hip.h", "kcg_codegen.h"])
def test_library_exports_every_declared_function(header):
    names = declared_functions(header)
    assert len(names) >= 10
    lib = _lib.lib()
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_signatures_carry_no_framework_types():
    for header in ("kcg_hip.h", "kcg_codegen.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        assert 'extern "C"' in text
        code = re.sub(r"//[^\n]*", "", re.sub(r"/\*.*?\*/", "", text, flags=re.S))
        assert "torch" not in code and "std::" not in code and "at::" not in code and "#include <string>" not in code


def test_compile_error_is_a_return_code_and_a_log():
    code, size = C.c_void_p(), C.c_size_t()
    log = C.create_string_buffer(4096)
    rc = _lib.lib().kcg_hip_compile_to_code(b'extern "C" __global__ void k(float* p) { p[0] = undeclared_name; }',
                                            None, 0, C.byref(code), C.byref(size), log, len(log))
    assert rc != 0 and (rc & 0x20000)                     # hipRTC error domain
    assert b"undeclared_name" in log.value
    assert b"HIPRTC" in _lib.lib().kcg_hip_strerror(rc)
    with pytest.raises(_lib.KcgError, match="undeclared_name"):
        R.compile_to_code('extern "C" __global__ void k(float* p) { p[0] = undeclared_name; }', use_cache=False)


def test_small_log_buffer_is_truncated_not_overrun():
    code, size = C.c_void_p(), C.c_size_t()
    log = C.create_string_buffer(b"\xAA" * 64, 64)
    rc = _lib.lib().kcg_hip_compile_to_code(b"this is not HIP", None, 0, C.byref(code), C.byref(size), log, 16)
    assert rc != 0
    assert log.raw[15:16] == b"\0" and log.raw[16:] == b"\xAA" * 48


def test_null_arguments_are_rejected():
    lib = _lib.lib()
    assert lib.kcg_hip_compile_to_code(None, None, 0, None, None, None, 0) == 1
    assert lib.kcg_hip_get_kernel(None, b"k", None) == 1
    grid = (C.c_uint32 * 3)(1, 1, 1)
    assert lib.kcg_hip_launch(None, grid, grid, 0, None, None) == 1
    assert lib.kcg_hip_module_destroy(None) in (0, 1)
    assert b"invalid argument" in lib.kcg_hip_strerror(1)
    # streams and graphs: the null stream cannot be captured, a null graph cannot be launched or destroyed
    assert lib.kcg_hip_stream_create(None) == 1 and lib.kcg_hip_stream_destroy(None) == 1
    assert lib.kcg_hip_graph_begin_capture(None) == 1
    assert lib.kcg_hip_graph_end_capture(None, None) == 1
    assert lib.kcg_hip_graph_launch(None, None) == 1
    assert lib.kcg_hip_graph_num_nodes(None, None) == 1
    assert lib.kcg_hip_graph_destroy(None) == 1


def test_emitter_reports_bad_parameters():
    with pytest.raises(_lib.KcgError, match="unknown kernel family"):
        R.emit_kernel("conv2d", "kernel0", N=1)
    with pytest.raises(_lib.KcgError, match="needs parameter"):
        R.emit_kernel("gemm_f32", "kernel0", M=64, N=64)
    with pytest.raises(_lib.KcgError, match="C identifier"):
        R.emit_kernel("gemm_f32", "kernel-0", M=64, N=64, K=64)
    with pytest.raises(_lib.KcgError, match="head dim must be a multiple of 32"):
        R.emit_kernel("fmha_bf16", "kernel0", B=1, H=1, S=128, D=80)
    # a sequence length that no tile divides is taken: one workgroup per (partly filled) query tile, never persistent
    text, info = R.emit_kernel("fmha_bf16", "kernel0", B=1, H=2, S=100, D=64)
    assert info["grid"] == [2, 1, 1] and info["block"] == [256, 1, 1] and "#define FA_PERSIST 0" in text
    with pytest.raises(_lib.KcgError, match="positive"):
        R.emit_kernel("fmha_bf16", "kernel0", B=1, H=1, S=128, D=64, SCALE=-1.0)
    with pytest.raises(_lib.KcgError, match="QW must be 1 or 2"):
        R.emit_kernel("fmha_bf16", "kernel0", B=1, H=1, S=128, D=64, BR=32, QW=2)
    with pytest.raises(_lib.KcgError, match="odd number of bytes"):
        R.emit_kernel("gather", "kernel0", OUTER=1, AXIS=4, NIDX=2, INNER=3, ESIZE=1)


def test_fmha_f32_pairs_query_tiles_under_the_mask_on_large_grids():
    """fmha_f32 with a causal mask: a workgroup takes two query tiles of a head (the longest with the shortest) once the
    halved grid still has two workgroups for each of the 256 CUs; PAIR overrides it where a pairing exists (the mask, an
    even number of query tiles) and is refused elsewhere."""
    text, info = R.emit_kernel("fmha_f32", "kernel0", B=8, H=32, S=2048, D=128, CAUSAL=1)
    assert "#define FF_PAIR 1" in text and info["grid"] == [8 * 32 * 8, 1, 1]
    text, info = R.emit_kernel("fmha_f32", "kernel0", B=8, H=32, S=2048, D=64, CAUSAL=0)
    assert "#define FF_PAIR 0" in text and info["grid"] == [8 * 32 * 16, 1, 1]
    text, info = R.emit_kernel("fmha_f32", "kernel0", B=1, H=8, S=1024, D=64, CAUSAL=1)
    assert "#define FF_PAIR 0" in text and info["grid"] == [64, 1, 1]
    text, info = R.emit_kernel("fmha_f32", "kernel0", B=1, H=8, S=1024, D=64, CAUSAL=1, PAIR=1)
    assert "#define FF_PAIR 1" in text and info["grid"] == [32, 1, 1]
    text, info = R.emit_kernel("fmha_f32", "kernel0", B=8, H=32, S=2048, D=128, CAUSAL=1, PAIR=0)
    assert "#define FF_PAIR 0" in text and info["grid"] == [8 * 32 * 16, 1, 1]
    text, info = R.emit_kernel("fmha_f32", "kernel0", B=1, H=1, S=200, D=64, CAUSAL=1, PAIR=1)     # a partly filled last tile
    assert "#define FF_PAIR 1" in text and info["grid"] == [1, 1, 1]
    for bad in (dict(S=384, CAUSAL=1), dict(S=256, CAUSAL=0), dict(S=300, CAUSAL=1)):
        with pytest.raises(_lib.KcgError, match="PAIR needs the causal mask"):
            R.emit_kernel("fmha_f32", "kernel0", B=1, H=1, D=64, PAIR=1, **bad)


def test_gemm_f32_small_launches_split_the_k_tile_between_two_wavefront_groups():
    """gemm_f32 with whole 64 x 64 x 32 tiles on a launch of at most 256 workgroups: two groups of four wavefronts (WK = 2)
    and three LDS buffers (NBUF = 3) by default; larger launches and larger tiles keep one group and two buffers; the
    parameters are refused where the kernel has no such form."""
    text, info = R.emit_kernel("gemm_f32", "kernel0", M=1024, N=1024, K=1024)
    assert "#define GL_WK 2" in text and "#define GL_NBUF 3" in text and info["block"] == [512, 1, 1] and info["grid"][0] == 256
    text, info = R.emit_kernel("gemm_f32", "kernel0", M=1024, N=1024, K=1024, WK=1)
    assert "#define GL_WK 1" in text and "#define GL_NBUF 2" in text and info["block"] == [256, 1, 1]
    text, info = R.emit_kernel("gemm_f32", "kernel0", M=1536, N=1536, K=1536)
    assert "#define GL_WK 1" in text and "#define GL_NBUF 2" in text and info["grid"][0] == 576
    text, info = R.emit_kernel("gemm_f32", "kernel0", M=4096, N=4096, K=4096)
    assert "#define GL_WK 1" in text and "#define GL_NBUF 2" in text and info["block"] == [1024, 1, 1]
    with pytest.raises(_lib.KcgError, match="WK is 1 or 2"):
        R.emit_kernel("gemm_f32", "kernel0", M=4096, N=4096, K=4096, WK=2)          # k-tiles of 16
    with pytest.raises(_lib.KcgError, match="WK is 1 or 2"):
        R.emit_kernel("gemm_f32", "kernel0", M=100, N=64, K=64, WK=2)               # no whole tiles
    with pytest.raises(_lib.KcgError, match="NBUF is 2"):
        R.emit_kernel("gemm_f32", "kernel0", M=1024, N=1024, K=1024, NBUF=5)
    with pytest.raises(_lib.KcgError, match="NBUF is 2"):
        R.emit_kernel("gemm_f32", "kernel0", M=1024, N=1024, K=1024, TB=1, NBUF=3)  # the kernel with register staging


def test_fp8_direct_load_kernel_strip_height():
    """The strips of tile rows that the fp8 kernel for full tiles walks: the rows of one XCD's run of tiles when that
    is one to four whole rows, four otherwise; a GROUP_M that the caller names is kept."""
    def strip(**kw):
        text = R.emit_kernel("gemm_fp8", "kernel0", TB=1, **kw)[0]
        assert "global_load_lds_dwordx4" in text
        return int(text.split("#define G8_GROUP_M ")[1].split()[0])
    assert strip(M=4096, N=11008, K=4096) == 2        # 16 x 43 tiles, 86 per XCD
    assert strip(M=4096, N=4096, K=4096) == 2         # 16 x 16 tiles, 32 per XCD
    assert strip(M=8192, N=8192, K=4096) == 4         # 32 x 32 tiles, 128 per XCD
    assert strip(M=16384, N=4096, K=4096) == 4        # 64 x 16 tiles, 128 per XCD: eight rows, more than four
    assert strip(M=3072, N=8192, K=4096) == 4         # 12 x 32 tiles, 48 per XCD: one row and a half
    assert strip(M=768, N=768, K=256, BM=256, BN=256) == 4    # 9 tiles: no multiple of the 8 XCDs
    assert strip(M=4096, N=11008, K=4096, GROUP_M=8) == 8


@pytest.mark.parametrize("family,params,nargs", [
    ("layernorm", dict(ROWS=8, N=1000, NG=1000, NB=1000, EPS=1e-5, GELU=1), 4),
    ("layernorm", dict(ROWS=2, N=589824, NG=589824, NB=589824, EPS=1e-5), 4),
    ("softmax", dict(ROWS=4, N=151936, INPLACE=0), 2),              # a row too long for registers: the streamed kernel
    ("softmax", dict(ROWS=3, N=33369, INPLACE=1, F16=1), 1),
    ("elementwise", dict(N=1001, OP="Gelu", INPLACE=0, IN_T="float", OUT_T="float"), 2),
    ("binary", dict(OP="Add", DIMS="16,1,128,256", SA="256,0,0,1", SB="0,0,256,1"), 3),
    ("softmax", dict(ROWS=48, N=2048, INPLACE=1), 1),
    ("softmax", dict(ROWS=7, N=1001, INPLACE=0), 2),
    ("gather", dict(OUTER=4, AXIS=100, NIDX=7, INNER=33, ESIZE=4), 3),
    ("gather", dict(OUTER=1, AXIS=32000, NIDX=128, INNER=4096, ESIZE=2), 3),
    ("gemm_f32", dict(M=100, N=77, K=33), 3),
    ("gemm_f64", dict(M=100, N=77, K=33), 3),
    ("gemm_f64", dict(M=4096, N=4096, K=4096, TA=1, TB=1), 3),
    ("gemm_bf16", dict(M=512, N=512, K=256, TA=1, TB=0, OUT_BF16=1), 3),
    ("gemm_bf16", dict(M=256, N=256, K=64, WM=2, WN=2, STAGES=2), 3),
    ("gemm_fp8", dict(M=256, N=256, K=256, TA=0, TB=1), 5),
    ("gemm_fp8", dict(M=100, N=77, K=200, TA=1, TB=0), 5),
    ("fmha_bf16", dict(B=2, H=2, S=256, D=64, CAUSAL=1, SCALE=0.125), 4),
    ("fmha_bf16", dict(B=1, H=2, S=512, D=128, CAUSAL=0, SCALE=0.0884, BR=256, QW=2), 4),
])
def test_every_family_compiles_for_gfx950_without_a_gpu(family, params, nargs):
    text, info = R.emit_kernel(family, "kernel0", **params)
    assert info["name"] == "kernel0" and info["num_args"] == nargs
    assert 'extern "C" __global__' in text
    blob = R.compile_to_code(R.prelude() + text, use_cache=False)
    assert blob[:4] == b"\x7fELF" and len(blob) > 1000


def _adaptor_for_matmul(tmp_path):
    from kernelcodegen_amd.generator import KernelCodeGenerator
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("mm")
    gen.opts.append("Matmul")
    A = g.create("PlaceHolder", [512, 256], "float32")
    B = g.create("PlaceHolder", [256, 512], "float32")
    C1 = g.create("Matmul", A, B)
    gen.opts.append("ElementWise")
    g.create("ElementWise", C1, "Gelu", 1)
    src = gen.codegen(gen.optimize(g))
    kfile = tmp_path / "kernels.hip"
    kfile.write_text(src)
    text = gen.adaptor(kfile)
    cfile = tmp_path / "adaptor.c"
    cfile.write_text(text)
    exe = tmp_path / "adaptor"
    libdir = os.path.dirname(_lib.LIB_PATH)
    r = subprocess.run(["gcc", "-Wall", "-Wextra", "-Werror", str(cfile), "-I", os.path.join(ROOT, "include"), "-L", libdir,
                        "-lkcg_hip", "-lm", "-Wl,-rpath," + libdir, "-o", str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    return gen, text, exe


def test_adaptor_is_a_self_contained_c_program(tmp_path):
    """generator.adaptor(): the host program that stands in for the reference's adaptor + harness
    (test/test.cc:69-104) names every kernel with its launch shape and buffer sizes and builds with a C compiler."""
    gen, text, exe = _adaptor_for_matmul(tmp_path)
    infos = gen.launchInfos()
    assert len(infos) == 2
    for info in infos:
        check = {"Matmul_m512n512k256": "gemm", "Gelu_Elementwise_512_512": "elementwise"}[info["function"]]
        assert '{"%s", "%s", "%s", {%d, %d, %d}' % ((info["name"], info["function"], check) + tuple(info["grid"])) in text
    assert '#include "kcg_hip.h"' in text and "hip/hip_runtime" not in text
    assert os.path.exists(exe)


@pytest.mark.gpu
def test_adaptor_runs_and_reports_every_kernel(tmp_path):
    gen, text, exe = _adaptor_for_matmul(tmp_path)
    print("adaptor", exe, flush=True)
    r = subprocess.run([str(exe), "5"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    lines = [l for l in r.stdout.splitlines() if "Latency" in l]
    # kernels are numbered in module order, not call order
    assert len(lines) == 2 and sorted(l.split(" Latency")[0].split(" ", 1)[1] for l in lines) == [
        "(Gelu_Elementwise_512_512)", "(Matmul_m512n512k256)"]
    assert sorted(l.split(" ")[0] for l in lines) == ["kernel0", "kernel1"]
    for l in lines:
        assert 0.0 < float(l.split("Latency = ")[1].split(" ms")[0]) < 10.0
        # the generated program checks a sample of each result against a plain C evaluation of the operator
        assert "correctness: Done" in l and float(l.split("max rel err = ")[1].split(" ")[0]) <= 1e-4


@pytest.mark.gpu
def test_adaptor_reports_a_wrong_kernel(tmp_path):
    """The same program run on a kernel file whose product kernel is replaced by one that writes something else
    (same name, same arguments) says FAILED for that kernel and exits with a non-zero status."""
    gen, text, exe = _adaptor_for_matmul(tmp_path)
    kfile = tmp_path / "kernels.hip"
    name = [i["name"] for i in gen.launchInfos() if i["function"] == "Matmul_m512n512k256"][0]
    src = kfile.read_text()
    start = src.index('extern "C" __global__', src.index("// Matmul_m512n512k256"))
    end = src.index("// Gelu_Elementwise_512_512") if src.index("// Gelu_Elementwise_512_512") > start else len(src)
    bogus = ('extern "C" __global__ void %s(const float* A, const float* B, float* C) {\n'
             '  C[blockIdx.x * blockDim.x + threadIdx.x] = 0.25f * A[0] + B[0];\n}\n' % name)
    kfile.write_text(src[:start] + bogus + src[end:])
    r = subprocess.run([str(exe), "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2, r.stderr
    line = [l for l in r.stdout.splitlines() if "(Matmul_m512n512k256)" in l][0]
    assert "correctness: FAILED" in line
    assert "correctness: Done" in [l for l in r.stdout.splitlines() if "(Gelu_Elementwise_512_512)" in l][0]



def test_kernels_are_compiled_by_the_installations_hiprtc_whatever_the_process_loaded(tmp_path):
    """The shim opens the ROCm installation's libhiprtc in a namespace of its own: the code object of one
    source text is the same bytes in a process that loaded torch (whose wheel bundles another hipRTC under
    the same soname) first and in one that did not."""
    info = R.compiler_info()
    assert info.startswith("hipRTC ") and "libhiprtc.so.7 (own namespace)" in info
    script = tmp_path / "hash.py"
    script.write_text(
        "import sys, hashlib\n"
        "if sys.argv[1] == 'torch':\n"
        "    import torch\n"
        "sys.path.insert(0, %r)\n"
        "from kernelcodegen_amd import runtime as R\n"
        "text, info = R.emit_kernel('elementwise', 'kernel0', N=4096, OP='Relu', INPLACE=0, IN_T='float', OUT_T='float')\n"
        "blob = R.compile_to_code(R.prelude() + text, use_cache=False)\n"
        "print(R.compiler_info(), hashlib.sha256(blob).hexdigest())\n" % os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    outs = [subprocess.run(["python", str(script), mode], capture_output=True, text=True, timeout=300)
            for mode in ("plain", "torch")]
    for o in outs:
        assert o.returncode == 0, o.stderr[-500:]
    assert outs[0].stdout.strip().splitlines()[-1] == outs[1].stdout.strip().splitlines()[-1]


def test_code_object_cache_on_disk(tmp_path, monkeypatch):
    """The library keeps code objects under SHA-256(compiler, NUL, source, NUL + option ...)[:32] + '.hsaco' in
    KCG_CACHE_DIR, the options being the whole vector the compiler sees: the library's own (target, -O3, packed fp32
    operations off) and then the caller's; a second request is served from the file, `refresh` compiles again and
    rewrites it."""
    import hashlib
    monkeypatch.setenv("KCG_CACHE_DIR", str(tmp_path / "objects"))
    assert R.cache_dir() == str(tmp_path / "objects")
    text, _ = R.emit_kernel("elementwise", "kernel0", N=1024, OP="Tanh", INPLACE=0, IN_T="float", OUT_T="float")
    src = R.prelude() + text
    blob = R.compile_to_code(src, opts=("-DKCG_TEST_OPTION=1",))
    builtin = ["--offload-arch=gfx950", "-O3", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
    key = hashlib.sha256(R.compiler_info().encode() + b"\0" + src.encode() +
                         b"".join(b"\0" + o.encode() for o in builtin + ["-DKCG_TEST_OPTION=1"])).hexdigest()[:32]
    path = tmp_path / "objects" / (key + ".hsaco")
    assert path.read_bytes() == blob and blob[:4] == b"\x7fELF"
    path.write_bytes(b"served from the cache")
    assert R.compile_to_code(src, opts=("-DKCG_TEST_OPTION=1",)) == b"served from the cache"
    assert R.compile_to_code(src, opts=("-DKCG_TEST_OPTION=1",), refresh=True) == blob and path.read_bytes() == blob
    assert R.compile_to_code(src, opts=("-DKCG_TEST_OPTION=1",), use_cache=False) == blob
    assert sorted(f.name for f in (tmp_path / "objects").iterdir()) == [key + ".hsaco"]


def test_code_object_cache_is_bounded(tmp_path, monkeypatch):
    """KCG_CACHE_MAX_MB bounds the cache directory: when a newly written object takes the *.hsaco files over the bound,
    the oldest ones go until nine tenths of it are left; the new object and other files stay."""
    import os
    objects = tmp_path / "objects"
    objects.mkdir()
    monkeypatch.setenv("KCG_CACHE_DIR", str(objects))
    monkeypatch.setenv("KCG_CACHE_MAX_MB", "1")
    for i, age in enumerate((400, 300, 200, 100)):           # four objects of 300 KiB, the first the oldest
        f = objects / ("%032x.hsaco" % i)
        f.write_bytes(b"x" * (300 * 1024))
        os.utime(f, (1_700_000_000 - age, 1_700_000_000 - age))
    (objects / "notes.txt").write_bytes(b"y" * (2 * 1024 * 1024))
    text, _ = R.emit_kernel("elementwise", "kernel0", N=1024, OP="Relu", INPLACE=0, IN_T="float", OUT_T="float")
    blob = R.compile_to_code(R.prelude() + text, opts=("-DKCG_BOUND_TEST=1",))
    left = sorted(f.name for f in objects.iterdir())
    new = [n for n in left if n.endswith(".hsaco") and not n.startswith("0" * 28)]
    assert len(new) == 1 and (objects / new[0]).read_bytes() == blob
    # 1200 KiB + the new object exceed 1 MiB: the oldest go, one by one, until at most 0.9 MiB are left
    total, expect = 4 * 300 * 1024 + len(blob), [0, 1, 2, 3]
    while total > (1 << 20) // 10 * 9:
        total -= 300 * 1024
        expect.pop(0)
    assert 1 <= len(expect) <= 3
    assert [n for n in left if n.startswith("0" * 28)] == ["%032x.hsaco" % i for i in expect], left
    assert "notes.txt" in left
    monkeypatch.setenv("KCG_CACHE_MAX_MB", "0")               # no bound
    for i in range(4, 8):
        (objects / ("%032x.hsaco" % i)).write_bytes(b"x" * (300 * 1024))
    R.compile_to_code(R.prelude() + text, opts=("-DKCG_BOUND_TEST=2",))
    assert len([f for f in objects.iterdir() if f.name.endswith(".hsaco")]) == len(expect) + 1 + 4 + 1


def test_host_generator_and_codecs_agree_with_the_oracle():
    """The library's seeded generator and narrow-float codecs (used by evaluate(), the generated adaptor and the
    benchmark) against the oracle's, which is pinned on its own: same bits for every element type."""
    import ctypes as C
    import oracle_lib as O
    L = _lib.lib()
    n = 100001
    out = np.empty(n, dtype=np.float32)
    assert L.kcg_host_fill(out.ctypes.data, n, 0, 0, O.SEED, 7, -1.0, 1.0, 1.0) == 0
    assert np.array_equal(out, O.uniform((n,), stream=7))
    assert L.kcg_host_fill(out.ctypes.data, n, 0, 1, O.SEED, 9, 0.5, 2.0, 1.0) == 0
    ref = O.normal((n,), stream=9, mean=0.5, std=2.0)
    assert np.array_equal(out, ref)
    h = np.empty(n, dtype=np.uint16)
    assert L.kcg_host_fill(h.ctypes.data, n, 1, 1, O.SEED, 9, 0.5, 2.0, 1.0) == 0
    assert np.array_equal(h, O.to_bf16_bits(ref))
    b = np.empty(n, dtype=np.uint8)
    assert L.kcg_host_fill(b.ctypes.data, n, 2, 1, O.SEED, 9, 0.5, 2.0, 37.5) == 0
    assert np.array_equal(b, O.to_fp8_bits(ref, 37.5))
    # every e4m3 code decodes alike; values across the whole range, ties included, encode alike
    codes = np.arange(256, dtype=np.uint8)
    dec = np.empty(256, dtype=np.float32)
    assert L.kcg_host_to_f32(codes.ctypes.data, dec.ctypes.data_as(C.POINTER(C.c_float)), 256, 2) == 0
    want = O.from_fp8_bits(codes)
    assert np.array_equal(np.isnan(dec), np.isnan(want)) and np.array_equal(dec[~np.isnan(want)], want[~np.isnan(want)])
    finite = want[~np.isnan(want)]
    probes = np.concatenate([finite, (finite[:-1] + finite[1:]) / 2, finite * 1.03, finite * 0.97,
                             np.array([1e-4, 2.0 ** -10, 2.0 ** -9 * 1.5, 447.9, 448.0, 464.0, 1e6, -1e6, np.inf], dtype=np.float32),
                             O.normal((20000,), stream=11, std=100.0)]).astype(np.float32)
    enc = np.empty(probes.size, dtype=np.uint8)
    assert L.kcg_host_from_f32(probes.ctypes.data_as(C.POINTER(C.c_float)), enc.ctypes.data, probes.size, 2, 1.0) == 0
    assert np.array_equal(enc & 0x7F, O.to_fp8_bits(probes) & 0x7F)          # the sign of a zero result aside
    nz = (enc & 0x7F) != 0
    assert np.array_equal(enc[nz], O.to_fp8_bits(probes)[nz])
    # IEEE half against numpy's conversion, subnormals, ties and overflow included
    vals = np.concatenate([O.normal((50000,), stream=12, std=30.0), O.normal((50000,), stream=13, std=1e-5),
                           np.array([65504.0, 65519.9, 65520.0, 1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 0.0, -0.0,
                                     2.0 ** -14, 2.0 ** -14 * (1 - 2.0 ** -12)], dtype=np.float32)]).astype(np.float32)
    f16 = np.empty(vals.size, dtype=np.uint16)
    assert L.kcg_host_from_f32(vals.ctypes.data_as(C.POINTER(C.c_float)), f16.ctypes.data, vals.size, 3, 1.0) == 0
    assert np.array_equal(f16, vals.astype(np.float16).view(np.uint16))
    back = np.empty(vals.size, dtype=np.float32)
    assert L.kcg_host_to_f32(f16.ctypes.data, back.ctypes.data_as(C.POINTER(C.c_float)), vals.size, 3) == 0
    assert np.array_equal(back, f16.view(np.float16).astype(np.float32))
    assert L.kcg_host_fill(out.ctypes.data, n, 99, 0, 1, 1, 0.0, 1.0, 1.0) == 1 and L.kcg_dtype_size(99) == 0


def test_compiler_info_rejects_null():
    assert _lib.lib().kcg_hip_compiler_info(None, 0) == 1
