"""Builds and runs the C++ unit checks of the IR, the Analyzer and the Rewriter
primitives (tests/cpp/test_rewriter.cc): once against the shipped library, once
as a whole-source AddressSanitizer + UBSan build (host code only)."""
import glob
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "kernelcodegen_amd")
OUT = os.path.join(ROOT, "tests", "cpp", "_build")
SRC = os.path.join(ROOT, "tests", "cpp", "test_rewriter.cc")
EXPECTED = ["every_operator_both_lowerings", "affine_algebra", "ir_basics_and_analyzer", "identify_batch_matmul", "split", "reorder_and_bufferize",
            "parallel", "read_write_vectorize_cache", "if_simplification_and_unroll", "matmul_schedule_pipeline",
            "hand_scripted_schedule_lowering", "swap_constant_loop_grid_to_block", "collapse_and_helpers", "irregular_and_block_helpers", "usage_contract", "optimizer_helper_members", "fmha_tiled_maps"]


def _check(output):
    lines = output.splitlines()
    for name in EXPECTED:
        assert "ok " + name in lines, output[-3000:]
    assert "ALL OK" in lines, output[-3000:]


def test_cpp_checks_against_the_library():
    from kernelcodegen_amd import build as B
    B.build()
    os.makedirs(OUT, exist_ok=True)
    exe = os.path.join(OUT, "test_rewriter")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-I", os.path.join(ROOT, "include"), SRC, "-o", exe,
                           "-L", PKG, "-lkcg_hip", "-Wl,-rpath," + PKG])
    res = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout[-3000:] + res.stderr[-3000:]
    _check(res.stdout)


def test_cpp_checks_under_address_and_ub_sanitizers():
    from kernelcodegen_amd import build as B
    B.gen_templates()
    os.makedirs(OUT, exist_ok=True)
    exe = os.path.join(OUT, "test_rewriter_asan")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    from kernelcodegen_amd import build as B2
    B2.build()
    # host code under the sanitizers; the library's one device translation unit as the object the build made
    srcs = sorted(glob.glob(os.path.join(PKG, "csrc", "*", "*.cc"))) + [os.path.join(PKG, "csrc", "runtime", "kcg_scratch.o")]
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
                           "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(ROOT, "include"), "-I", os.path.join(PKG, "csrc"),
                           "-I", os.path.join(rocm, "include"), SRC] + srcs +
                          ["-o", exe, "-L", os.path.join(rocm, "lib"), "-lamdhip64", "-lhiprtc",
                           "-Wl,-rpath," + os.path.join(rocm, "lib")])
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")
    res = subprocess.run([exe], capture_output=True, text=True, timeout=600, env=env)
    assert res.returncode == 0, res.stdout[-3000:] + res.stderr[-3000:]
    assert "runtime error" not in res.stderr and "AddressSanitizer" not in res.stderr, res.stderr[-3000:]
    _check(res.stdout)


def test_reference_style_program_against_the_library():
    """tests/cpp/test_api.cc: the call sequences of the reference's test/test.cc on platform "ROCm"."""
    from kernelcodegen_amd import build as B
    B.build()
    os.makedirs(OUT, exist_ok=True)
    exe = os.path.join(OUT, "test_api")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-I", os.path.join(ROOT, "include"),
                           os.path.join(ROOT, "tests", "cpp", "test_api.cc"), "-o", exe,
                           "-L", PKG, "-lkcg_hip", "-Wl,-rpath," + PKG])
    res = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout[-3000:] + res.stderr[-3000:]
    lines = res.stdout.splitlines()
    for name in ("public_optimizer_members", "elementwise_cast", "layernorm", "matmul_and_save", "batched_matmul", "flash_attention", "other_platform",
                 "binary_gather_softmax_adaptor"):
        assert "ok " + name in lines, res.stdout[-3000:]
    assert "ALL OK" in lines


def test_cmake_target_kcg_runtime(tmp_path):
    """The reference's users link `kcg_runtime` (its src/CMakeLists.txt:16-73): a consumer project that adds this
    repository as a subdirectory and links that target must build and run the reference-style program."""
    import shutil
    if not shutil.which("cmake") or not shutil.which("ninja"):
        pytest.skip("cmake / ninja not on PATH")
    consumer = tmp_path / "consumer"
    consumer.mkdir()
    (consumer / "CMakeLists.txt").write_text(
        "cmake_minimum_required(VERSION 3.16)\nproject(consumer LANGUAGES CXX)\n"
        "set(KCG_BUILD_API_TEST OFF CACHE BOOL \"\" FORCE)\n"
        "add_subdirectory(%s kcg)\n"
        "add_executable(demo %s)\n"
        "target_link_libraries(demo PRIVATE kcg_runtime)\n" % (ROOT, os.path.join(ROOT, "tests", "cpp", "test_api.cc")))
    build = tmp_path / "build"
    subprocess.check_call(["cmake", "-S", str(consumer), "-B", str(build), "-G", "Ninja"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["cmake", "--build", str(build), "-j8"], stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    assert (build / "kcg" / "libkcg_runtime.so").exists()
    res = subprocess.run([str(build / "demo")], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout[-3000:] + res.stderr[-3000:]
    assert "ALL OK" in res.stdout.splitlines()
    # the C ABI is in the same library
    import ctypes
    lib = ctypes.CDLL(str(build / "kcg" / "libkcg_runtime.so"))
    for sym in ("kcg_hip_compile", "kcg_hip_launch", "kcg_generator_create", "kcg_codegen"):
        assert hasattr(lib, sym), sym
