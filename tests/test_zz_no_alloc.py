"""kcg_hip_launch_scratch, the entry point that allocates nothing: a kernel with a workspace (the bf16 GEMM with
its last tiles split along k) launched through the C ABI on the library's own scratch array must give the very
bits that kcg_hip_launch gives on a workspace of the caller's -- on two calls in a row, the second on a smaller
problem, which finds the array as the first left it."""
import ctypes as C

import numpy as np
import pytest

import oracle_lib as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rt():
    from kernelcodegen_amd import runtime as R
    from kernelcodegen_amd._lib import lib, check
    check(lib().kcg_hip_init(0), "kcg_hip_init")
    return R


def _case(rt, m, n, k, tile, full, units, seed):
    text, info = rt.emit_kernel("gemm_bf16", "kernel0", M=m, N=n, K=k, BM=tile, BN=tile, SK_FULL=full, SK_UNITS=units)
    assert info["workspace_bytes"] > 0 and info["num_args"] == 4
    kern = rt.compile_source(rt.prelude() + text, [info]).kernel("kernel0")
    a = O.round_bf16(O.normal((m, k), stream=seed))
    b = O.round_bf16(O.normal((k, n), stream=seed + 1, std=0.02))
    ad = torch.from_numpy(a).cuda().to(torch.bfloat16)
    bd = torch.from_numpy(b).cuda().to(torch.bfloat16)
    return kern, info, a, b, ad, bd


def _launch_both(rt, kern, info, ad, bd, m, n):
    """(result through kcg_hip_launch on a caller's workspace, result through kcg_hip_launch_scratch)."""
    from kernelcodegen_amd._lib import lib, check
    L = lib()
    grid, block = (C.c_uint32 * 3)(*info["grid"]), (C.c_uint32 * 3)(*info["block"])
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    c_ref = torch.full((m, n), float("nan"), device="cuda")
    c_new = torch.full((m, n), float("nan"), device="cuda")
    workspace = torch.zeros(int(info["workspace_bytes"]), dtype=torch.uint8, device="cuda")

    def args(*tensors):
        holders = [C.c_void_p(t.data_ptr() if t is not None else 0) for t in tensors]
        return holders, (C.c_void_p * len(holders))(*[C.cast(C.pointer(h), C.c_void_p) for h in holders])

    h1, a1 = args(ad, bd, c_ref, workspace)
    check(L.kcg_hip_launch(kern.handle, grid, block, info["lds_bytes"], stream, a1), "kcg_hip_launch")
    h2, a2 = args(ad, bd, c_new, None)              # the workspace slot is ignored and replaced
    check(L.kcg_hip_launch_scratch(kern.handle, grid, block, info["lds_bytes"], stream, a2, 4, 3,
                                   int(info["workspace_bytes"])), "kcg_hip_launch_scratch")
    torch.cuda.synchronize()
    return c_ref, c_new


def test_launch_on_the_librarys_scratch_array_matches_launch_on_a_callers_workspace(rt):
    # first call: 40 tiles of 128 x 128, 24 of them split over 32 units (4 MiB of workspace)
    m, n, k = 640, 1024, 512
    kern, info, a, b, ad, bd = _case(rt, m, n, k, 128, 16, 32, 461)
    print("scratch launch", m, n, k, info["workspace_bytes"], flush=True)
    c_ref, c_new = _launch_both(rt, kern, info, ad, bd, m, n)
    assert torch.equal(c_ref, c_new)
    assert O.rel_frobenius(c_new.cpu().numpy(), O.matmul_f64(a, b)) <= 1e-5
    # second call, right behind it: a smaller problem (36 tiles, 4 split over 16 units) on the array as the first left it
    m2, n2, k2 = 768, 768, 256
    kern2, info2, a2, b2, ad2, bd2 = _case(rt, m2, n2, k2, 128, 32, 16, 463)
    assert info2["workspace_bytes"] < info["workspace_bytes"]
    print("scratch launch", m2, n2, k2, info2["workspace_bytes"], flush=True)
    c_ref2, c_new2 = _launch_both(rt, kern2, info2, ad2, bd2, m2, n2)
    assert torch.equal(c_ref2, c_new2)
    assert O.rel_frobenius(c_new2.cpu().numpy(), O.matmul_f64(a2, b2)) <= 1e-5
    # and the first problem once more through the Python wrapper, several times
    for _ in range(3):
        c = torch.full((m, n), float("nan"), device="cuda")
        kern.launch_scratch(ad, bd, c)
        torch.cuda.synchronize()
        assert torch.equal(c, c_ref)


def test_scratch_launch_refuses_what_does_not_fit(rt):
    from kernelcodegen_amd._lib import lib, strerror
    L = lib()
    # the benchmark shape split over 256 units of 256 x 256 needs 128 MiB: beyond the 32 MiB array
    text, info = rt.emit_kernel("gemm_bf16", "kernel0", M=4096, N=11008, K=4096, SK_UNITS=256)
    assert info["workspace_bytes"] > (32 << 20)
    kern = rt.compile_source(rt.prelude() + text, [info]).kernel("kernel0")
    grid, block = (C.c_uint32 * 3)(*info["grid"]), (C.c_uint32 * 3)(*info["block"])
    slots = (C.c_void_p * 4)()
    rc = L.kcg_hip_launch_scratch(kern.handle, grid, block, 0, None, slots, 4, 3, int(info["workspace_bytes"]))
    assert rc == 6 and "scratch" in strerror(rc)
    assert L.kcg_hip_launch_scratch(kern.handle, grid, block, 0, None, slots, 4, 4, 4096) == 1      # argument index out of range
    assert L.kcg_hip_launch_scratch(kern.handle, grid, block, 0, None, slots, 17, 3, 4096) == 1     # more than 16 arguments
    assert L.kcg_hip_launch_scratch(None, grid, block, 0, None, slots, 4, 3, 4096) == 1
