"""The C-ABI library without a GPU: it loads, exports every function the two
public headers declare, compiles emitted kernels for gfx950 (hipRTC needs no
device) and reports errors through return codes and caller buffers."""
import ctypes as C
import os
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


def test_emitter_reports_bad_parameters():
    with pytest.raises(_lib.KcgError, match="unknown kernel family"):
        R.emit_kernel("conv2d", "kernel0", N=1)
    with pytest.raises(_lib.KcgError, match="needs parameter"):
        R.emit_kernel("gemm_f32", "kernel0", M=64, N=64)
    with pytest.raises(_lib.KcgError, match="C identifier"):
        R.emit_kernel("gemm_f32", "kernel-0", M=64, N=64, K=64)
    with pytest.raises(_lib.KcgError, match="multiple of BR and BC"):
        R.emit_kernel("fmha_bf16", "kernel0", B=1, H=1, S=100, D=64)
    with pytest.raises(_lib.KcgError, match="positive"):
        R.emit_kernel("fmha_bf16", "kernel0", B=1, H=1, S=128, D=64, SCALE=-1.0)
    with pytest.raises(_lib.KcgError, match="QW must be 1 or 2"):
        R.emit_kernel("fmha_bf16", "kernel0", B=1, H=1, S=128, D=64, BR=32, QW=2)
    with pytest.raises(_lib.KcgError, match="odd number of bytes"):
        R.emit_kernel("gather", "kernel0", OUTER=1, AXIS=4, NIDX=2, INNER=3, ESIZE=1)


@pytest.mark.parametrize("family,params,nargs", [
    ("layernorm", dict(ROWS=8, N=1000, NG=1000, NB=1000, EPS=1e-5, GELU=1), 4),
    ("layernorm", dict(ROWS=2, N=589824, NG=589824, NB=589824, EPS=1e-5), 4),
    ("elementwise", dict(N=1001, OP="Gelu", INPLACE=0, IN_T="float", OUT_T="float"), 2),
    ("binary", dict(OP="Add", DIMS="16,1,128,256", SA="256,0,0,1", SB="0,0,256,1"), 3),
    ("softmax", dict(ROWS=48, N=2048, INPLACE=1), 1),
    ("softmax", dict(ROWS=7, N=1001, INPLACE=0), 2),
    ("gather", dict(OUTER=4, AXIS=100, NIDX=7, INNER=33, ESIZE=4), 3),
    ("gather", dict(OUTER=1, AXIS=32000, NIDX=128, INNER=4096, ESIZE=2), 3),
    ("gemm_f32", dict(M=100, N=77, K=33), 3),
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
                        "-lkcg_hip", "-Wl,-rpath," + libdir, "-o", str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    return gen, text, exe


def test_adaptor_is_a_self_contained_c_program(tmp_path):
    """generator.adaptor(): the host program that stands in for the reference's adaptor + harness
    (test/test.cc:69-104) names every kernel with its launch shape and buffer sizes and builds with a C compiler."""
    gen, text, exe = _adaptor_for_matmul(tmp_path)
    infos = gen.launchInfos()
    assert len(infos) == 2
    for info in infos:
        assert '{"%s", "%s", {%d, %d, %d}' % ((info["name"], info["function"]) + tuple(info["grid"])) in text
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
    assert R._cache_path("x", ()) != R._cache_path("y", ())


def test_compiler_info_rejects_null():
    assert _lib.lib().kcg_hip_compiler_info(None, 0) == 1
