"""Operator-level convenience wrappers: emit the gfx950 kernel for one
operator instance, compile it once, launch it on torch device tensors.
Shapes are static (baked into the kernel), like every kernel the generator
emits."""
import math

import torch

from . import runtime as R


def _need_cuda(*ts):
    for t in ts:
        if not (t.is_cuda and t.is_contiguous()):
            raise ValueError("operands must be contiguous device tensors")


# storage type of the row kernels (their arithmetic is fp32 throughout): the kernels' F16 parameter
_STORAGE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def layernorm(x, gamma, beta, axis, eps=1e-5, gelu=False, out=None, **cfg):
    _need_cuda(x, gamma, beta)
    axis = axis + x.dim() if axis < 0 else axis
    rows = int(math.prod(x.shape[:axis])) if axis > 0 else 1
    n = x.numel() // rows
    if x.dtype not in _STORAGE or gamma.dtype != x.dtype or beta.dtype != x.dtype:
        raise ValueError("the LayerNorm kernel takes fp32, IEEE half or bfloat16 tensors of one type")
    k = R.get_kernel("layernorm", ROWS=rows, N=n, NG=gamma.numel(), NB=beta.numel(), EPS=float(eps),
                     GELU=int(gelu), F16=_STORAGE[x.dtype], **cfg)
    y = torch.empty_like(x) if out is None else out
    k.launch(x, gamma, beta, y)
    return y


def elementwise(x, op, inplace=False, out_dtype=None, **cfg):
    _need_cuda(x)
    ctype = {torch.float32: "float", torch.int32: "int", torch.float16: "_Float16", torch.bfloat16: "__bf16"}
    out_dtype = out_dtype or x.dtype
    k = R.get_kernel("elementwise", N=x.numel(), OP=op, INPLACE=int(inplace), IN_T=ctype[x.dtype],
                     OUT_T=ctype[out_dtype], **cfg)
    if inplace:
        k.launch(x)
        return x.view(out_dtype)
    y = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    k.launch(x, y)
    return y


_FAMILY = {torch.float32: "gemm_f32", torch.float64: "gemm_f64", torch.bfloat16: "gemm_bf16", torch.float16: "gemm_bf16"}


def batched_matmul(a, b, trans_a=False, trans_b=False, out_dtype=None, **cfg):
    """a: [..., m, k] (or [..., k, m] when trans_a), b: [..., k, n] (or [..., n, k]).  out_dtype None: fp64 for fp64
    operands, fp32 for all others; a type the operands' kernel family does not write raises."""
    _need_cuda(a, b)
    if a.dtype != b.dtype or a.dtype not in _FAMILY:
        raise ValueError("unsupported operand dtypes")
    batch = int(math.prod(a.shape[:-2])) if a.dim() > 2 else 1
    m, k = (a.shape[-1], a.shape[-2]) if trans_a else (a.shape[-2], a.shape[-1])
    n, k2 = (b.shape[-2], b.shape[-1]) if trans_b else (b.shape[-1], b.shape[-2])
    if k != k2:
        raise ValueError("incompatible K dimensions")
    extra = {}
    if out_dtype is None:
        out_dtype = torch.float64 if a.dtype == torch.float64 else torch.float32
    if a.dtype in (torch.bfloat16, torch.float16):
        if out_dtype not in (torch.float32, a.dtype):
            raise ValueError("a 16-bit GEMM writes fp32 or its operands' type")
        extra["OUT_BF16"] = int(out_dtype == a.dtype)       # a 16-bit result, of the operands' type
        if a.dtype == torch.float16:
            extra["F16"] = 1
    elif a.dtype == torch.float64:
        if out_dtype != torch.float64:
            raise ValueError("fp64 GEMM writes fp64")
    elif out_dtype != torch.float32:
        raise ValueError("fp32 GEMM writes fp32")
    kern = R.get_kernel(_FAMILY[a.dtype], M=m, N=n, K=k, BATCH=batch, TA=int(trans_a), TB=int(trans_b),
                        **extra, **cfg)
    c = torch.empty(tuple(a.shape[:-2]) + (m, n), dtype=out_dtype, device=a.device)
    kern.launch(a, b, c)
    return c


def matmul_fp8(a, b, scale_a, scale_b, trans_a=False, trans_b=True, out_dtype=torch.float32, **cfg):
    """(scale_a * op(a)) (scale_b * op(b)) with fp8 e4m3 operands, one fp32 scale per tensor and fp32
    accumulation.  a: [..., m, k] (or [..., k, m] when trans_a), b: [..., k, n] (or [..., n, k] when
    trans_b, the default: both operands k-contiguous, no transposition on the way into LDS)."""
    _need_cuda(a, b)
    if a.dtype != torch.float8_e4m3fn or b.dtype != torch.float8_e4m3fn:
        raise ValueError("operands must be float8_e4m3fn")
    if out_dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("output must be fp32 or bf16")
    batch = int(math.prod(a.shape[:-2])) if a.dim() > 2 else 1
    m, k = (a.shape[-1], a.shape[-2]) if trans_a else (a.shape[-2], a.shape[-1])
    n, k2 = (b.shape[-2], b.shape[-1]) if trans_b else (b.shape[-1], b.shape[-2])
    if k != k2:
        raise ValueError("incompatible K dimensions")
    kern = R.get_kernel("gemm_fp8", M=m, N=n, K=k, BATCH=batch, TA=int(trans_a), TB=int(trans_b),
                        OUT_BF16=int(out_dtype == torch.bfloat16), **cfg)
    c = torch.empty(tuple(a.shape[:-2]) + (m, n), dtype=out_dtype, device=a.device)
    kern.launch(a, b, c, float(scale_a), float(scale_b))
    return c


def matmul(a, b, **cfg):
    return batched_matmul(a, b, **cfg)


def fmha(q, k, v, scale=None, causal=False, out_dtype=None, **cfg):
    """softmax(scale * q k^T [+ causal mask]) v over [B, H, S, D] operands, all fp32, all bf16 or all IEEE half; the
    result has their type (default) or is fp32.  fp32 operands run both products on the fp32 MFMA (fmha_f32)."""
    _need_cuda(q, k, v)
    if q.dim() != 4 or q.shape != k.shape or q.shape != v.shape:
        raise ValueError("q, k, v must share one [B, H, S, D] shape")
    if not (q.dtype == k.dtype == v.dtype and q.dtype in (torch.float32, torch.bfloat16, torch.float16)):
        raise ValueError("the fused attention kernels take fp32, bf16 or IEEE half operands")
    out_dtype = q.dtype if out_dtype is None else out_dtype
    if out_dtype not in (q.dtype, torch.float32):
        raise ValueError("output must have the operands' type or be fp32")
    b, h, s, d = q.shape
    scale = d ** -0.5 if scale is None else float(scale)
    if q.dtype == torch.float32:
        kern = R.get_kernel("fmha_f32", B=b, H=h, S=s, D=d, CAUSAL=int(causal), SCALE=scale, **cfg)
        o = torch.empty(q.shape, dtype=torch.float32, device=q.device)
        kern.launch(q, k, v, o)
        return o
    kern = R.get_kernel("fmha_bf16", B=b, H=h, S=s, D=d, CAUSAL=int(causal), SCALE=scale,
                        OUT_BF16=int(out_dtype == q.dtype), F16=int(q.dtype == torch.float16), **cfg)
    o = torch.empty(q.shape, dtype=out_dtype, device=q.device)
    kern.launch(q, k, v, o)
    return o


def binary(x, y, op, inplace=False, **cfg):
    """x op y (Add, Sub, Mul, Div, Pow; Equal and Greater give a bool tensor) on two fp32 or two IEEE half tensors
    with numpy-style broadcasting."""
    _need_cuda(x, y)
    if x.dtype not in (torch.float32, torch.float16) or y.dtype != x.dtype:
        raise ValueError("the binary kernel takes two fp32 or two IEEE half operands")
    shape = torch.broadcast_shapes(x.shape, y.shape)

    def strides(t):
        out, run = [0] * len(shape), 1
        for i in range(t.dim()):
            extent = t.shape[t.dim() - 1 - i]
            if extent != 1:
                out[len(shape) - 1 - i] = run
            run *= extent
        return ",".join(map(str, out))

    k = R.get_kernel("binary", OP=op, DIMS=",".join(map(str, shape)), SA=strides(x), SB=strides(y), INPLACE=int(inplace),
                     F16=int(x.dtype == torch.float16), **cfg)
    if inplace:
        k.launch(x, y)
        return x
    z = torch.empty(shape, dtype=torch.bool if op in ("Equal", "Greater") else x.dtype, device=x.device)
    k.launch(x, y, z)
    return z


def gather(x, indices, axis=0, **cfg):
    """out[o.., i.., r..] = x[o.., indices[i..], r..]: dimension `axis` of x is replaced by the dimensions of
    `indices` (int64; a single index, shape (1,), drops the dimension).  Indices outside the axis are clamped.
    `cfg` overrides kernel parameters (BLOCK, UNROLL)."""
    _need_cuda(x, indices)
    if indices.dtype != torch.int64:
        raise ValueError("gather indices must be int64")
    if not -x.dim() <= axis < x.dim():
        raise ValueError("axis out of range")
    axis %= x.dim()
    x, indices = x.contiguous(), indices.contiguous()
    outer = 1
    for d in x.shape[:axis]:
        outer *= d
    inner = 1
    for d in x.shape[axis + 1:]:
        inner *= d
    single = tuple(indices.shape) == (1,)
    shape = tuple(x.shape[:axis]) + (() if single else tuple(indices.shape)) + tuple(x.shape[axis + 1:])
    kern = R.get_kernel("gather", OUTER=outer, AXIS=x.shape[axis], NIDX=indices.numel(), INNER=inner, ESIZE=x.element_size(), **cfg)
    out = torch.empty(shape, dtype=x.dtype, device=x.device)
    kern.launch(x, indices, out)
    return out


def softmax(x, inplace=False):
    """softmax over the last axis of an fp32, IEEE half or bfloat16 tensor (fp32 arithmetic)."""
    _need_cuda(x)
    if x.dtype not in _STORAGE:
        raise ValueError("the softmax kernel takes fp32, IEEE half or bfloat16 operands")
    x = x if inplace else x.contiguous()
    if not x.is_contiguous():
        raise ValueError("an in-place softmax needs a contiguous tensor")
    n = x.shape[-1]
    kern = R.get_kernel("softmax", ROWS=x.numel() // n, N=n, INPLACE=int(inplace), F16=_STORAGE[x.dtype])
    if inplace:
        kern.launch(x)
        return x
    y = torch.empty_like(x)
    kern.launch(x, y)
    return y

