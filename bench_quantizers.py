#!/usr/bin/env python3
"""Throughput of the HBM-bound quantizer kernels on the shapes of the RTN / AWQ / FP8+pack configurations.

Every line is one kernel launched through the C ABI on preallocated, rotating buffers (large enough in total to
defeat the 256 MB Infinity Cache), timed with device events over back-to-back launches after a warm-up.
`GB/s` counts ALGORITHMIC bytes: each input element read once, each output element written once, plus the per-row
parameters.  Prints one JSON object per line.

    python bench_quantizers.py
"""
import json

import torch

from lightcompress_amd import _lib as L


def main():
    if not torch.cuda.is_available():
        raise SystemExit('bench_quantizers.py needs a GPU')
    dev = torch.device('cuda:0')
    lib, st = L.lib(), L.stream()
    bf, f32 = torch.bfloat16, torch.float32

    def rot(shape, dtype, scale, total=1.3e9):
        n = max(3, int(total / (shape[0] * shape[1] * torch.tensor([], dtype=dtype).element_size())))
        return [(torch.randn(*shape, device=dev) * scale).to(dtype) for _ in range(n)]

    def timeit(fn, n=60, warm=25):
        for i in range(warm):
            fn(i)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(n):
            fn(i)
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e-3 / n

    def report(name, kernel, nbytes, t):
        print(json.dumps({'case': name, 'kernel': kernel, 'us': round(t * 1e6, 2), 'algorithmic_MB': round(nbytes / 1e6, 1),
                          'GB/s': round(nbytes / t / 1e9, 1), 'frac_of_8TBps': round(nbytes / t / 8e12, 4)}), flush=True)

    def quant_int(xs, rows, cols, qmin, qmax, flags, dq=None, codes=None, cd=L.CODE_NONE, sdt=None):
        dt = xs[0].dtype
        sc = torch.empty(rows, dtype=dt, device=dev)
        zr = torch.empty(rows, dtype=dt, device=dev)
        def fn(i):
            k = i % len(xs)
            L.check(lib.lcq_quant_int(L.ptr(xs[k]), L.i32(L.dtype_code(dt)), L.i64(rows), L.i64(cols), L.f32(qmin), L.f32(qmax),
                                      L.i32(flags), L.f32(1), L.ptr(dq[k] if dq else None), L.ptr(codes[k] if codes else None),
                                      L.i32(cd), L.ptr(sc), L.ptr(zr), st), 'lcq_quant_int')
        return fn

    def quant_fp(xs, rows, cols, dq=None, codes=None, cd=L.CODE_NONE):
        sc = torch.empty(rows, dtype=xs[0].dtype, device=dev)
        def fn(i):
            k = i % len(xs)
            L.check(lib.lcq_quant_fp(L.ptr(xs[k]), L.i32(L.dtype_code(xs[0].dtype)), L.i64(rows), L.i64(cols), L.i32(4), L.i32(3),
                                     L.f32(448.0), L.i32(0), L.ptr(dq[k] if dq else None), L.ptr(codes[k] if codes else None),
                                     L.i32(cd), L.ptr(sc), st), 'lcq_quant_fp')
        return fn

    # warm the clocks
    a = torch.randn(8192, 8192, device=dev)
    for _ in range(40):
        a @ a
    torch.cuda.synchronize()
    del a

    # RTN config: fp32 [4096, 4096], INT4 asym g128: dq + uint8 codes + scales / zeros
    xs = rot((4096, 4096), f32, 0.02)
    dq = [torch.empty_like(x) for x in xs]
    cds = [torch.empty(4096, 4096, dtype=torch.uint8, device=dev) for _ in xs]
    n, g = 4096 * 4096, 128
    t = timeit(quant_int(xs, n // g, g, 0, 15, 0, dq, cds, L.CODE_U8))
    report('RTN int4 asym g128, fp32 4096x4096 -> dq + u8 codes', 'row_team_kernel<IntOp<f32>>', n * 9 + n // g * 8, t)
    t = timeit(quant_int(xs, n // g, g, 0, 15, 0, dq))
    report('RTN int4 asym g128 fake quant, fp32 4096x4096', 'row_team_kernel<IntOp<f32>>', n * 8 + n // g * 8, t)
    del xs, dq, cds

    # AWQ config: bf16 [11008, 4096] fake quant, int4 asym g128
    xs = rot((11008, 4096), bf, 0.02)
    dq = [torch.empty_like(x) for x in xs]
    n = 11008 * 4096
    t = timeit(quant_int(xs, n // g, g, 0, 15, 0, dq))
    report('int4 asym g128 fake quant, bf16 11008x4096', 'row_team_kernel<IntOp<bf16>>', n * 4 + n // g * 4, t)
    del xs, dq

    # FP8 + pack config: 16 experts [2048, 7168] bf16 at once, and one expert alone
    for ne in (16, 1):
        R, K = ne * 2048, 7168
        xs = rot((R, K), bf, 0.006, total=3e9 if ne > 1 else 1.3e9)
        n = R * K
        cds = [torch.empty(R, K, dtype=torch.uint8, device=dev) for _ in xs]
        t = timeit(quant_fp(xs, R, K, None, cds, L.CODE_FP8), n=30 if ne > 1 else 60)
        report(f'fp8 e4m3 per-channel real quant, bf16 {ne}x[2048,7168]', 'row_block_kernel<FpOp<bf16>>', n * 3 + R * 2, t)
        pk = [torch.empty(R, K // 8, dtype=torch.int32, device=dev) for _ in xs]
        t = timeit(quant_int(xs, n // g, g, -8, 7, L.FLAG_SYM, None, pk, L.CODE_CT4), n=30 if ne > 1 else 60)
        report(f'int4 sym g128 quantize + compressed-tensors pack, bf16 {ne}x[2048,7168]', 'row_team_kernel<IntOp<bf16, CT4>>',
               n * 2.5 + n // g * 2, t)
        del xs, cds, pk
    # per-token dynamic fp8 fake quant of activations [8192, 7168]
    xs = rot((8192, 7168), bf, 1.0)
    dq = [torch.empty_like(x) for x in xs]
    n = 8192 * 7168
    t = timeit(quant_fp(xs, 8192, 7168, dq))
    report('fp8 e4m3 per-token fake quant, bf16 8192x7168', 'row_block_kernel<FpOp<bf16>>', n * 4 + 8192 * 2, t)


if __name__ == '__main__':
    main()
