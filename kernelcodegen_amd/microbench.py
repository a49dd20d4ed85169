"""Ceilings of the part that the GEMM and attention kernels are designed against,
measured with a few tiny probe kernels compiled and launched through the C ABI (on one MI355X):

    python -m kernelcodegen_amd.microbench                    # parts 1-3
    python -m kernelcodegen_amd.microbench attention-power     # part 4
    python -m kernelcodegen_amd.microbench gemm-power          # part 4 for the GEMM workloads
    rocprofv3 --pmc SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE -d OUT -o pmc --output-format csv -- \
        python3 -m kernelcodegen_amd.microbench lds-groups      # part 5 (read OUT/pmc_counter_collection.csv)

1. v_mfma_f32_32x32x16_bf16 issue rate from registers only, on all-zero and on
   N(0,1) operands (the difference is the power limit of the part);
2. the same loop with the GEMM's LDS fragment reads (ds_read_b128, padded rows);
   1b / 2b: both for v_mfma_f32_32x32x64_f8f6f4 on e4m3 operands;
   1c / 2c: both shapes against their 16-row siblings v_mfma_f32_16x16x32_bf16 and v_mfma_f32_16x16x128_f8f6f4 (the
   same products per wavefront, 4 x 8 tiles instead of 2 x 4; reads from unpadded, swizzled 128-byte rows), 200 launches
   in a row: the deeper, smaller shape touches the fp32 accumulators half as often per result;
3. MFMA next to ordinary VALU work: interleaved in one wavefront's instruction
   stream, or placed in the other wavefront of the same SIMD.
4. the attention kernel (or the GEMM kernels) of the benchmark workloads on their generated operands and on
   all-zero operands: the same instruction stream, so the difference is what the data costs in power.
5. which lanes of a wavefront an LDS access serves in the same pass: dispatch j of the probe has only
   lanes 0 and j active, at different addresses in the same banks; under the bank-conflict counter
   the dispatches whose lane shares a pass with lane 0 show conflict cycles (dispatch 0: lane 0 alone).
   Kernel probe_read uses ds_read_b128, probe_write ds_write_b32.
"""
import sys

MFMA_SRC = r'''
#define ITERS 2048
extern "C" __global__ __launch_bounds__(NT) void kname(float* out, const unsigned short* in) {
  __shared__ __attribute__((aligned(16))) char smem[65536];
  const int tid = threadIdx.x, lane = tid & 63;
  for (int i = tid; i < 65536 / 16; i += NT) ((kcg_u32x4*)smem)[i] = ((const kcg_u32x4*)in)[i & 255];
  __syncthreads();
  kcg_f32x16 acc[TM][TN];
  for (int i = 0; i < TM; ++i) for (int j = 0; j < TN; ++j) for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  const char* cA = smem + (lane & 31) * 144 + (lane >> 5) * 16 + (tid >> 6) * 1024;
  kcg_bf16x8 fa[TM], fb[TN];
  for (int i = 0; i < TM; ++i) fa[i] = *(const kcg_bf16x8*)(cA + i * 32 * 144);
  for (int j = 0; j < TN; ++j) fb[j] = *(const kcg_bf16x8*)(cA + j * 32 * 144 + 64);
#pragma unroll 1
  for (int it = 0; it < ITERS; ++it) {
    asm volatile("" ::: "memory");
#if READS
    const int off = (it & 3) * 32;
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[i] = *(const kcg_bf16x8*)(cA + i * 32 * 144 + off);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[j] = *(const kcg_bf16x8*)(cA + j * 32 * 144 + off + 4096);
#endif
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
  }
  float s = 0.f;
  for (int i = 0; i < TM; ++i) for (int j = 0; j < TN; ++j) for (int v = 0; v < 16; ++v) s += acc[i][j][v];
  out[blockIdx.x * NT + tid] = s;
}
'''

MFMA8_SRC = r'''
#define ITERS 2048
extern "C" __global__ __launch_bounds__(NT) void kname(float* out, const unsigned char* in) {
  __shared__ __attribute__((aligned(16))) char smem[65536];
  const int tid = threadIdx.x, lane = tid & 63;
  for (int i = tid; i < 65536 / 16; i += NT) ((kcg_u32x4*)smem)[i] = ((const kcg_u32x4*)in)[i & 255];
  __syncthreads();
  kcg_f32x16 acc[TM][TN];
  for (int i = 0; i < TM; ++i) for (int j = 0; j < TN; ++j) for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  // rows of 128 + 16 bytes: a lane's 32 bytes of k are two 16-byte reads
  const char* cA = smem + (lane & 31) * 144 + (lane >> 5) * 32 + (tid >> 6) * 512;
  kcg_i32x8 fa[TM], fb[TN];
  auto frag = [&](const char* p) {
    const kcg_i32x4 lo = *(const kcg_i32x4*)p, hi = *(const kcg_i32x4*)(p + 16);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  for (int i = 0; i < TM; ++i) fa[i] = frag(cA + i * 32 * 144);
  for (int j = 0; j < TN; ++j) fb[j] = frag(cA + j * 32 * 144 + 64);
#pragma unroll 1
  for (int it = 0; it < ITERS; ++it) {
    asm volatile("" ::: "memory");
#if READS
    const int off = (it & 1) * 64;
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[i] = frag(cA + i * 32 * 144 + off);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[j] = frag(cA + j * 32 * 144 + off + 8192);
#endif
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], acc[i][j], 0, 0, 0, 0, 0, 0);
  }
  float s = 0.f;
  for (int i = 0; i < TM; ++i) for (int j = 0; j < TN; ++j) for (int v = 0; v < 16; ++v) s += acc[i][j][v];
  out[blockIdx.x * NT + tid] = s;
}
'''

MFMA16_SRC = r'''
#define ITERS 2048
extern "C" __global__ __launch_bounds__(NT) void kname(float* out, const unsigned short* in) {
  __shared__ __attribute__((aligned(16))) char smem[65536];
  const int tid = threadIdx.x, lane = tid & 63;
  for (int i = tid; i < 65536 / 16; i += NT) ((kcg_u32x4*)smem)[i] = ((const kcg_u32x4*)in)[i & 255];
  __syncthreads();
  kcg_f32x4 acc[TM][TN];
  for (int i = 0; i < TM; ++i) for (int j = 0; j < TN; ++j) for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;
  // lane l: row l % 16, chunk l / 16 (+ 4 per k-step) at position chunk ^ ((row / 2) % 8) of a 128-byte row
  const int sw = (lane & 15) >> 1;
  const char* cA = smem + (lane & 15) * 128 + (tid >> 6) * 2048;
#if FP8
  kcg_i32x8 fa[TM], fb[TN];
  auto frag = [&](const char* row, int it) {
    const int c = (lane >> 4);                        // chunks c and c + 4: 32 bytes of k per lane
    const kcg_i32x4 lo = *(const kcg_i32x4*)(row + ((c ^ sw) * 16) + (it & 1) * 32768), hi = *(const kcg_i32x4*)(row + (((c + 4) ^ sw) * 16) + (it & 1) * 32768);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
#else
  kcg_bf16x8 fa[TM], fb[TN];
  auto frag = [&](const char* row, int it) { return *(const kcg_bf16x8*)(row + ((((lane >> 4) + 4 * (it & 1)) ^ sw) * 16)); };
#endif
  for (int i = 0; i < TM; ++i) fa[i] = frag(cA + i * 16 * 128, 0);
  for (int j = 0; j < TN; ++j) fb[j] = frag(cA + j * 16 * 128 + 16384, 1);
#pragma unroll 1
  for (int it = 0; it < ITERS; ++it) {
    asm volatile("" ::: "memory");
#if READS
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[i] = frag(cA + i * 16 * 128, it);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[j] = frag(cA + j * 16 * 128 + 16384, it);
#endif
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#if FP8
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fa[i], fb[j], acc[i][j], 0, 0, 0, 0, 0, 0);
#else
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
#endif
  }
  float s = 0.f;
  for (int i = 0; i < TM; ++i) for (int j = 0; j < TN; ++j) for (int v = 0; v < 4; ++v) s += acc[i][j][v];
  out[blockIdx.x * NT + tid] = s;
}
'''

COEXEC_SRC = r'''
#define ITERS 4096
extern "C" __global__ __launch_bounds__(NT) void kname(float* out, const float* in) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  kcg_f32x16 acc[4];
  for (int i = 0; i < 4; ++i) for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
  kcg_bf16x8 fa, fb;
  for (int j = 0; j < 8; ++j) { fa[j] = (__bf16)in[lane + j]; fb[j] = (__bf16)in[lane + 8 + j]; }
  float x[NV];
  for (int j = 0; j < NV; ++j) x[j] = in[tid + j];
  const bool do_mfma = MODE == 0 || MODE == 2 || (MODE == 3 && wave < NT / 128);
  const bool do_valu = MODE == 1 || MODE == 2 || (MODE == 3 && wave >= NT / 128);
#pragma unroll 1
  for (int it = 0; it < ITERS; ++it) {
    asm volatile("" ::: "memory");
    if (do_mfma) {
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb, acc[i], 0, 0, 0);
    }
    if (do_valu) {
#pragma unroll
      for (int j = 0; j < NV; ++j) x[j] = __builtin_fmaf(x[j], 1.0001f, 0.5f);
    }
#if MODE == 2
#pragma unroll
    for (int i = 0; i < 4; ++i) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x002, NV / 4, 0); }
#endif
  }
  float s = 0.f;
  for (int i = 0; i < 4; ++i) for (int v = 0; v < 16; ++v) s += acc[i][v];
  for (int j = 0; j < NV; ++j) s += x[j];
  out[blockIdx.x * NT + tid] = s;
}
'''


LDS_PROBE_SRC = r'''
extern "C" __global__ __launch_bounds__(64) void probe_read(const int* __restrict__ offs, unsigned* __restrict__ out) {
  __shared__ __attribute__((aligned(16))) char smem[32768];
  const int lane = threadIdx.x;
  for (int i = lane; i < 32768 / 4; i += 64) ((unsigned*)smem)[i] = i;
  __syncthreads();
  const int a = offs[lane];
  kcg_u32x4 acc = {0, 0, 0, 0};
  if (a >= 0) {
#pragma unroll 1
    for (int it = 0; it < 2048; ++it) acc += *(const volatile kcg_u32x4*)(smem + a);
  }
  out[blockIdx.x * 64 + lane] = acc[0] + acc[1] + acc[2] + acc[3];
}
extern "C" __global__ __launch_bounds__(64) void probe_write(const int* __restrict__ offs, unsigned* __restrict__ out) {
  __shared__ __attribute__((aligned(16))) char smem[32768];
  const int lane = threadIdx.x;
  ((unsigned*)smem)[lane] = 0;
  const int a = offs[lane];
  if (a >= 0) {
#pragma unroll 1
    for (int it = 0; it < 2048; ++it) *(volatile unsigned*)(smem + a) = it;
  }
  __syncthreads();
  out[blockIdx.x * 64 + lane] = ((unsigned*)smem)[lane];
}
'''


def lds_groups(torch, R):
    infos = [dict(name=n, grid=[256, 1, 1], block=[64, 1, 1], lds_bytes=0, num_args=2, num_scalars=0, flops=0, bytes=0)
             for n in ("probe_read", "probe_write")]
    mod = R.compile_source(R.prelude() + LDS_PROBE_SRC, infos)
    out = torch.zeros(256 * 64, dtype=torch.int32, device="cuda")
    for name in ("probe_read", "probe_write"):
        k = mod.kernel(name)
        for j in range(64):
            offs = [-1] * 64
            offs[0] = 0
            if j:
                offs[j] = 4096          # other address, same banks as lane 0
            k.launch(torch.tensor(offs, dtype=torch.int32, device="cuda"), out)
        torch.cuda.synchronize()
    mod.destroy()
    print("launched 64 dispatches of probe_read and of probe_write; dispatch j (from 0) pairs lane 0 with lane j")
    return 0


def attention_power(torch, R, names=("fmha_bf16_b8h32s2048d128", "fmha_bf16_b8h32s2048d128_causal")):
    import os
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench
    from .configs import WORKLOADS
    print("%-36s %-18s %10s %10s" % ("workload", "operands", "ms", "TFLOP/s"))
    for name in names:
        family, params = WORKLOADS[name]
        text, info = R.emit_kernel(family, "kernel0", **params)
        mod = R.compile_source(R.prelude() + text, [info])
        k = mod.kernel("kernel0")
        args = bench.Operands(torch, R, family, params).make()
        nin = 2 if family.startswith("gemm") else 3          # operands in front, then the result (and scalars)
        for label, scale in (("as generated", 1.0), ("zeros", 0.0), ("as generated, again", 1.0)):
            a = [(x.float() * scale).to(x.dtype) if scale != 1.0 else x for x in args[:nin]] + list(args[nin:])
            ms = k.time(*a, warmup=10, iters=60)
            print("%-36s %-18s %10.4f %10.1f" % (name, label, ms, info["flops"] / ms / 1e9), flush=True)
        mod.destroy()
    return 0


def _kernel(R, body, name, defines, nt, blocks):
    src = R.prelude() + "".join("#define %s %d\n" % kv for kv in defines.items()) + body.replace("kname", name)
    info = dict(name=name, grid=[blocks, 1, 1], block=[nt, 1, 1], lds_bytes=0, num_args=2, num_scalars=0, flops=0, bytes=0)
    mod = R.compile_source(src, [info])
    return mod, mod.kernel(name)


def main():
    import torch
    from . import runtime as R
    from ._lib import lib, check
    check(lib().kcg_hip_init(0), "kcg_hip_init")
    if len(sys.argv) > 1 and sys.argv[1] == "lds-groups":
        return lds_groups(torch, R)
    if len(sys.argv) > 1 and sys.argv[1] == "attention-power":
        return attention_power(torch, R)
    if len(sys.argv) > 1 and sys.argv[1] == "gemm-power":
        return attention_power(torch, R, ("gemm_bf16_nk_4096x11008x4096", "gemm_bf16_4096x11008x4096",
                                          "gemm_fp8_4096x11008x4096", "gemm_f32_4096"))
    print("1/2. v_mfma_f32_32x32x16_bf16 rate, 256 workgroups (one per CU)")
    print("%-10s %-8s %-7s %-22s %10s %10s" % ("operands", "threads", "tile", "LDS fragment reads", "ms", "TFLOP/s"))
    for std in (0.0, 1.0):
        for nt, tm, tn in ((256, 2, 4), (512, 2, 4)):
            for reads in (0, 1):
                name = "m_%d_%d_%d_%d" % (nt, tm, tn, reads)
                mod, k = _kernel(R, MFMA_SRC, name, dict(NT=nt, TM=tm, TN=tn, READS=reads), nt, 256)
                out = torch.zeros(256 * nt, device="cuda")
                inp = (torch.randn(65536, device="cuda") * std).bfloat16().view(torch.int16)
                ms = k.time(out, inp, warmup=2, iters=10)
                flops = 256 * (nt // 64) * 2048 * tm * tn * 32 * 32 * 16 * 2
                print("%-10s %-8d %dx%-5d %-22s %10.3f %10.1f" % ("zeros" if std == 0 else "N(0,1)", nt, tm, tn,
                                                                   "yes" if reads else "no", ms, flops / ms / 1e9), flush=True)
                mod.destroy()
    print("1b/2b. v_mfma_f32_32x32x64_f8f6f4 (e4m3 operands) rate, 256 workgroups (one per CU)")
    print("%-10s %-8s %-7s %-22s %10s %10s" % ("operands", "threads", "tile", "LDS fragment reads", "ms", "TFLOP/s"))
    for std in (0.0, 1.0):
        for nt, tm, tn in ((256, 2, 4), (512, 2, 4)):
            for reads in (0, 1):
                name = "m8_%d_%d_%d_%d" % (nt, tm, tn, reads)
                mod, k = _kernel(R, MFMA8_SRC, name, dict(NT=nt, TM=tm, TN=tn, READS=reads), nt, 256)
                out = torch.zeros(256 * nt, device="cuda")
                inp = (torch.randn(65536, device="cuda") * std * 64.0).to(torch.float8_e4m3fn).view(torch.uint8)
                ms = k.time(out, inp, warmup=2, iters=10)
                flops = 256 * (nt // 64) * 2048 * tm * tn * 32 * 32 * 64 * 2
                print("%-10s %-8d %dx%-5d %-22s %10.3f %10.1f" % ("zeros" if std == 0 else "N(0,64)", nt, tm, tn,
                                                                   "yes" if reads else "no", ms, flops / ms / 1e9), flush=True)
                mod.destroy()
    print("1c/2c. 32-row against 16-row MFMA shapes, 512 lanes, 256 workgroups, best of three runs of 200 launches")
    print("%-10s %-28s %-22s %10s %10s" % ("operands", "instruction", "LDS fragment reads", "ms", "TFLOP/s"))
    for fp8 in (0, 1):
        for std in (0.0, 1.0):
            for reads in (0, 1):
                for small in (0, 1):
                    name = "s_%d_%d_%d" % (fp8, reads, small)
                    if small:
                        tm, tn, per = 4, 8, 16 * 16 * (128 if fp8 else 32) * 2
                        mod, k = _kernel(R, MFMA16_SRC, name, dict(NT=512, TM=tm, TN=tn, READS=reads, FP8=fp8), 512, 256)
                    else:
                        tm, tn, per = 2, 4, 32 * 32 * (64 if fp8 else 16) * 2
                        mod, k = _kernel(R, MFMA8_SRC if fp8 else MFMA_SRC, name, dict(NT=512, TM=tm, TN=tn, READS=reads), 512, 256)
                    out = torch.zeros(256 * 512, device="cuda")
                    rnd = torch.randn(65536, device="cuda") * std
                    inp = (rnd * 64.0).to(torch.float8_e4m3fn).view(torch.uint8) if fp8 else rnd.bfloat16().view(torch.int16)
                    ms = min(k.time(out, inp, warmup=5, iters=200) for _ in range(3))
                    flops = 256 * 8 * 2048 * tm * tn * per
                    what = ("v_mfma_f32_16x16x128_f8f6f4" if small else "v_mfma_f32_32x32x64_f8f6f4") if fp8 else ("v_mfma_f32_16x16x32_bf16" if small else "v_mfma_f32_32x32x16_bf16")
                    print("%-10s %-28s %-22s %10.3f %10.1f" % ("zeros" if std == 0 else "random", what, "yes" if reads else "no", ms, flops / ms / 1e9), flush=True)
                    mod.destroy()
    print("3. four MFMAs and NV fp32 FMAs per iteration; ms for 4096 iterations, 256 workgroups")
    modes = {0: "MFMA only", 1: "VALU only", 2: "one wavefront, interleaved", 3: "MFMA in waves 0..n/2, VALU in the rest"}
    print("%-8s %-4s %-42s %10s" % ("threads", "NV", "what runs", "ms"))
    for nv in (16, 28):
        for nt in (256, 512):
            for mode in (0, 1, 2, 3):
                name = "c_%d_%d_%d" % (nt, nv, mode)
                mod, k = _kernel(R, COEXEC_SRC, name, dict(NT=nt, NV=nv, MODE=mode), nt, 256)
                out = torch.zeros(256 * nt, device="cuda")
                inp = torch.randn(4096, device="cuda")
                ms = k.time(out, inp, warmup=2, iters=10)
                print("%-8d %-4d %-42s %10.3f" % (nt, nv, modes[mode], ms), flush=True)
                mod.destroy()
    return 0


if __name__ == "__main__":
    sys.exit(main())
