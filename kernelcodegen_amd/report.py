"""Latency of the emitted kernels next to the vendor libraries' routines for the same operation, in the
style of the reference's performance/output.log ("My Matmul Latency", "cublas Latency(NN)", "cublas Ratio",
produced there by an out-of-tree harness, test/test.cc:69-104):

    python -m kernelcodegen_amd.report [--workloads NAME ...] [--iters N]

The vendor side goes through torch (matmul -> hipBLASLt / rocBLAS, scaled_dot_product_attention, layer_norm,
softmax, gelu, add, index_select, _scaled_mm for fp8) and is a yardstick only: nothing in the library calls it.  Ratio = vendor
latency / own latency, as in the reference's log (100 % = parity, above = faster than the vendor routine).  Both sides
run on three operand sets in turn (results included), so that neither finds its operands in the last-level cache.
"""
import argparse
import sys


SETS = 3        # operand sets launched in turn, so that no launch finds its operands in the last-level cache


def _time(torch, fn, warmup, iters):
    """Best of three runs of `iters` calls fn(i); the callee picks operand set i % SETS."""
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(3):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(iters):
            fn(i)
        b.record()
        torch.cuda.synchronize()
        best = min(best, a.elapsed_time(b) / iters)
    return best


def vendor_routine(torch, family, p, args):
    """(label, callable) of the library routine that computes what the workload's kernel computes, or None."""
    F = torch.nn.functional
    if family in ("gemm_f32", "gemm_f64", "gemm_bf16"):
        a, b = args[0], args[1]
        ta, tb = p.get("TA", 0), p.get("TB", 0)
        lhs = a.transpose(-1, -2) if ta else a
        rhs = b.transpose(-1, -2) if tb else b
        out_dtype = torch.float32 if family != "gemm_bf16" or not p.get("OUT_BF16", 0) else torch.bfloat16
        if family == "gemm_bf16" and out_dtype == torch.float32:
            # the library's bf16 GEMM returns bf16; the fp32 result of this workload costs it a conversion pass
            return "hipBLASLt bf16 (bf16 result)", lambda: torch.matmul(lhs, rhs)
        return ("rocBLAS/hipBLASLt " + {"gemm_f32": "fp32", "gemm_f64": "fp64"}.get(family, "bf16")), lambda: torch.matmul(lhs, rhs)
    if family == "gemm_fp8" and hasattr(torch, "_scaled_mm") and not p.get("TA", 0) and p.get("BATCH", 1) == 1:
        a, w, _, sa, sw = args
        lhs = a[0]
        rhs = w[0].transpose(0, 1) if p.get("TB", 0) else w[0]
        if not p.get("TB", 0):
            return None       # the library wants the second operand column-major
        scale_a, scale_b = torch.tensor(sa, device=a.device), torch.tensor(sw, device=a.device)
        out_dtype = torch.bfloat16 if p.get("OUT_BF16", 0) else torch.float32
        return "hipBLASLt fp8 (torch._scaled_mm)", lambda: torch._scaled_mm(lhs, rhs, scale_a=scale_a, scale_b=scale_b,
                                                                           out_dtype=out_dtype)
    if family == "fmha_bf16":
        q, k, v = args[:3]
        causal, scale = bool(p.get("CAUSAL", 0)), float(p.get("SCALE", 1.0))
        return "torch SDPA", lambda: F.scaled_dot_product_attention(q, k, v, is_causal=causal, scale=scale)
    if family == "layernorm":
        x, g, b = args[:3]
        n, eps = p["N"], float(p.get("EPS", 1e-5))
        if p.get("GELU"):
            return "torch layer_norm + gelu(tanh)", lambda: F.gelu(F.layer_norm(x, (n,), g, b, eps), approximate="tanh")
        return "torch layer_norm", lambda: F.layer_norm(x, (n,), g, b, eps)
    if family == "elementwise" and p.get("OP") == "Gelu":
        x = args[0]
        return "torch gelu(tanh)", lambda: F.gelu(x, approximate="tanh")
    if family == "softmax":
        x = args[0]
        return "torch softmax", lambda: torch.softmax(x, dim=-1)
    if family == "binary" and p.get("OP") == "Add":
        x, y = args[:2]
        return "torch add", lambda: torch.add(x, y)
    if family == "gather":
        table, idx = args[:2]
        return "torch index_select", lambda: torch.index_select(table, 1, idx)
    return None


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--workloads", nargs="*", default=None)
    ap.add_argument("--iters", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    opts = ap.parse_args(argv)
    import os
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import torch
    if not torch.cuda.is_available():
        print("report: no GPU visible", file=sys.stderr)
        return 1
    import bench
    from . import runtime as R
    from ._lib import lib, check
    from .configs import WORKLOADS, workload_source
    check(lib().kcg_hip_init(0), "kcg_hip_init")
    print("Find the device successfully: %s" % torch.cuda.get_device_name(0))
    for name in (opts.workloads or list(WORKLOADS)):
        source, info, family, params = workload_source(name)
        mod = R.compile_source(source, [info])
        kern = mod.kernel("kernel0")
        operands = bench.Operands(torch, R, family, params)
        sets = [operands.make() for _ in range(SETS)]
        mine = _time(torch, lambda i: kern.launch(*sets[i % SETS]), opts.warmup, opts.iters)
        print("%s : %s" % (name, ", ".join("%s=%s" % kv for kv in sorted(params.items()))))
        print("My %s Latency = %g ms" % (family, mine))
        vend = vendor_routine(torch, family, params, sets[0])
        if vend is not None:
            label = vend[0]
            fns = [vendor_routine(torch, family, params, s)[1] for s in sets]
            held = [None] * SETS      # the last results stay alive, so the allocator hands out SETS result buffers in turn

            def theirs_once(i):
                held[i % SETS] = fns[i % SETS]()
            try:
                theirs = _time(torch, theirs_once, opts.warmup, opts.iters)
            except Exception as e:      # a routine the installed library does not offer for this type or shape
                print("%s not available: %s" % (label, str(e).splitlines()[0][:120]))
                vend = None
        if vend is not None:
            print("%s Latency = %g ms" % (label, theirs))
            print("%s Ratio = %g%%" % (label, 100.0 * theirs / mine))
        print("", flush=True)
        mod.destroy()
        del sets, vend, operands
        fns = held = None
        torch.cuda.empty_cache()
    return 0


if __name__ == "__main__":
    sys.exit(main())
