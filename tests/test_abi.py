"""The C-ABI library without a GPU: it loads, exports every function the two
public headers declare, compiles emitted kernels for gfx950 (hipRTC needs no
device) and reports errors through return codes and caller buffers."""
import ctypes as C
import os
import re

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
