#!/usr/bin/env python3
"""Benchmark of the layer-wise quantization hot path on one MI355X.

One "step" = GPTQ (w4 asym g128, act_order, damp 0.01, blocksize 128) of one
Llama-3-8B-shape decoder layer: for each of the four activation streams
(attention input, o_proj input, MLP input with K=4096; down_proj input with
K=14336) 128 calibration batches of 2048 tokens go through GPTQ.add_batch of
every Linear that sees them (q,k,v / o / gate,up / down; Linears that are
handed the identical tensor share one Hessian, `seconds_separate_hessians`
is the run with one Hessian per Linear as the reference keeps them), then
every Linear runs the damped Cholesky chain and the lazy-batch column loop.
Inputs are synthetic (lognormal per-channel scaled Gaussians, random-init
weights) and resident in HBM before the timed region.

Prints ONE JSON line.  `roofline` describes the dominant kernel (the bf16 MFMA
Hessian at K=14336); `roofline_quantizer` the fused RTN quantizer on the RTN
configuration; `cpu_baseline` the CPU oracle timed on a bounded sample of the
same workload; `configs` the wall times of the other configurations of the
baseline (one GPTQ Linear, the 20-point AWQ search, the 256-expert FP8 + int4
pack sweep) each next to its own CPU-oracle sample; `quantizers` the HBM-bound
kernels one by one, with `hbm_copy` (a plain device copy on the same box) as
the ceiling they can be held against.

    python bench.py                      # everything (a few minutes, most of it the CPU legs)
    python bench.py --only layer         # the headline only        (also: hessian, quantizers, c2, c3, c5)
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

LINEARS = [  # name, out_features, in_features, activation stream
    ('q_proj', 4096, 4096, 'attn_in'), ('k_proj', 1024, 4096, 'attn_in'), ('v_proj', 1024, 4096, 'attn_in'),
    ('o_proj', 4096, 4096, 'o_in'),
    ('gate_proj', 14336, 4096, 'mlp_in'), ('up_proj', 14336, 4096, 'mlp_in'),
    ('down_proj', 4096, 14336, 'down_in'),
]
SUBSETS = [['q_proj', 'k_proj', 'v_proj'], ['o_proj'], ['gate_proj', 'up_proj'], ['down_proj']]
STREAM_K = {'attn_in': 4096, 'o_in': 4096, 'mlp_in': 4096, 'down_in': 14336}
NB, TOK = 128, 2048
CFG = {'weight': dict(bit=4, symmetric=False, granularity='per_group', group_size=128),
       'special': dict(actorder=True, static_groups=False, percdamp=0.01, blocksize=128, true_sequential=True)}


def _sha16(path):
    import hashlib
    try:
        with open(os.path.join(ROOT, path), 'rb') as f:
            return hashlib.sha256(f.read()).hexdigest()[:16]
    except OSError:
        return None


def traffic_bytes(key, launch_us=None):
    """HBM-side bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script, kept in
    profiles/traffic.json next to the summaries that derive them (counters cannot be read inside the timed process).
    The entry carries the launch duration of the run it was taken at and a hash of the kernel's source file:
    -> (bytes, stale) with stale = True when the source has changed since, or when this run's launch duration
    differs from the recorded one by more than 10 %."""
    try:
        with open(os.path.join(ROOT, 'profiles', 'traffic.json')) as f:
            e = json.load(f).get(key, {})
    except (OSError, ValueError):
        return None, None
    if 'bytes' not in e:
        return None, None
    stale = False
    if e.get('source') and e.get('source_sha256_16') and _sha16(e['source']) != e['source_sha256_16']:
        stale = True
    if launch_us and e.get('launch_us') and abs(launch_us - e['launch_us']) > 0.1 * e['launch_us']:
        stale = True
    if not e.get('launch_us') or not e.get('source_sha256_16'):
        stale = True                                      # an entry without its stamp cannot be tied to this kernel
    return e['bytes'], stale


class Layer:
    def __init__(self, w):
        self.weight = w


def ev():
    import torch
    return torch.cuda.Event(enable_timing=True)


def timeit(fn, n, warm):
    import torch
    for i in range(warm):
        fn(i)
    a, b = ev(), ev()
    a.record()
    for i in range(n):
        fn(i)
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e-3 / n


def cpu_threads():
    import torch
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get('OMP_NUM_THREADS', cores)))
    torch.set_num_threads(cores)
    return cores


# ---------------------------------------------------------------------------------------------------------------
# headline: GPTQ of a full Llama-3-8B-shape layer
# ---------------------------------------------------------------------------------------------------------------
def bench_layer(args, out):
    import torch
    from lightcompress_amd.gptq import GPTQ
    dev = torch.device('cuda:0')
    weights = {n: (torch.randn(r, k, device=dev) * 0.02).bfloat16() for n, r, k, _ in LINEARS}
    streams = {}
    for sname, K in STREAM_K.items():
        sigma = torch.exp(torch.randn(K, device=dev))
        x = torch.empty(NB, TOK, K, dtype=torch.bfloat16, device=dev)
        for b in range(NB):
            x[b] = (torch.randn(TOK, K, device=dev) * sigma).bfloat16()
        streams[sname] = x
    phases = {'hessian_ms': 0.0, 'chain_ms': 0.0, 'loop_ms': 0.0}

    def one_layer(share, record=None, check=None):
        gp = GPTQ({'weight': CFG['weight'], 'special': dict(CFG['special'], auto_share=share)})
        layers = {n: Layer(torch.nn.Parameter(weights[n].clone(), requires_grad=False)) for n, *_ in LINEARS}
        marks = []
        for subset in SUBSETS:
            sub = {'layers': {n: layers[n] for n in subset}}
            gp.subset_init(sub)
            x = streams[[s for n, _, _, s in LINEARS if n == subset[0]][0]]
            e0 = ev(); e0.record()
            for b in range(NB):
                xb = x[b:b + 1]
                for n in subset:                       # every Linear's hook fires on every batch
                    gp.add_batch(layers[n], n, xb, None)
            e1 = ev(); e1.record()
            if record is None and check is None:
                gp.subset_transform(sub)               # the reference's driver of a subset (gptq.py:96-112)
            elif check is not None:                    # untimed: the same driver, keeping each Linear's summed loss
                gp.subset_transform(sub)
                for n in subset:
                    check[n] = gp.last_errors[n]
            else:                                      # same work one Linear at a time, with events between the phases
                for n in subset:
                    gp.initialize_qparams_and_prepare_weights(layers[n], n)
                    a = ev(); a.record()
                    W, U = gp.process_hessian_and_weights(layers[n], n, for_loop=True)
                    b_ = ev(); b_.record()
                    gp.update_layer_with_transformed_weights(layers[n], W, U, n)
                    c = ev(); c.record()
                    gp.free(n)
                    marks.append(('chain_ms', a, b_)); marks.append(('loop_ms', b_, c))
            marks.append(('hessian_ms', e0, e1))
        torch.cuda.synchronize()
        if record is not None:
            for k, a, b_ in marks:
                record[k] += a.elapsed_time(b_)
        return layers

    # Default path: Linears that receive the very same tensor on every call (q/k/v, gate/up) share one Hessian and
    # one Cholesky chain (detected by add_batch; results bit-identical to separate Hessians).
    for _ in range(args.warmup):
        one_layer(True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        one_layer(True)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    # the outputs of one more (untimed) pass must be sane: finite weights and qparams, a positive finite loss
    losses = {}
    checked = one_layer(True, check=losses)
    last_error = {}
    for n, *_ in LINEARS:
        lay = checked[n]
        ok = bool(torch.isfinite(lay.weight.data).all()) and bool(torch.isfinite(lay.buf_scales).all()) \
            and bool((lay.buf_scales > 0).all()) and bool(torch.isfinite(lay.buf_zeros).all())
        le = float(losses[n])
        if not ok or not (le > 0 and le == le and le != float('inf')):
            print(f'bench.py: {n}: non-finite outputs or loss {le}', file=sys.stderr)
            sys.exit(1)
        last_error[n] = round(le, 3)
    del checked
    # where the time goes: one more pass, one Linear at a time with events between the phases (untimed; the chains of
    # a subset run one after the other here, in the timed pass subset_transform starts them side by side)
    one_layer(True, phases)
    for k in phases:
        phases[k] = round(phases[k], 3)
    # the reference's behaviour: one Hessian and one chain per Linear, also where the inputs are identical
    one_layer(False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        one_layer(False)
    torch.cuda.synchronize()
    dt_separate = (time.perf_counter() - t0) / args.steps
    out.update({'value': round(dt, 4), 'ms_per_step': round(dt * 1e3, 2),
                'value_is': 'seconds_shared_hessians: Linears handed the identical tensor (q/k/v, gate/up) accumulate ONE Hessian '
                            '(4 accumulations and 4 Cholesky chains per layer, every shared call verified bit for bit on the device); '
                            'results are bit-identical to separate accumulation',
                'seconds_shared_hessians': round(dt, 4),
                'seconds_separate_hessians': round(dt_separate, 4),
                'seconds_separate_hessians_is': 'like for like with the reference: 7 Hessian accumulations and 7 chains per layer '
                                                '(special.auto_share: False); compare THIS figure with a reference run',
                'last_error': last_error, 'breakdown_ms': phases})
    return streams['down_in']


# ---------------------------------------------------------------------------------------------------------------
# dominant kernel: bf16 MFMA Hessian at K=14336, live HIP-event timing on the launch stream
# ---------------------------------------------------------------------------------------------------------------
def bench_hessian(args, out, x=None):
    import torch
    from lightcompress_amd import _lib as L
    from lightcompress_amd.gptq import GPTQ
    dev = torch.device('cuda:0')
    K = 14336
    FOLD = GPTQ(CFG).hessian_fold(K)                      # add_batch calls per launch, as the layer run issues them
    TL = FOLD * TOK
    if x is None:
        x = (torch.randn(3 * FOLD, TOK, K, device=dev) * torch.exp(torch.randn(K, device=dev))).bfloat16()
    nb = x.shape[0]
    H = torch.zeros(K, K, device=dev)
    lib, st = L.lib(), L.stream()
    # the launch add_batch issues: lcq_hessian_accum_balanced (the tiles of the last round of workgroups cut into token
    # ranges; the small launch that folds their partial sums into H is part of the timed call)
    ws_bytes = lib.lcq_hessian_balanced_workspace_bytes(L.i64(K), L.i64(TL))
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)

    def hess(b):
        b = (b * FOLD) % (nb - FOLD + 1)
        L.check(lib.lcq_hessian_accum_balanced(L.ptr(H), L.i64(K), L.ptr(x[b]), L.ptr(x[b]), L.i32(L.BF16), L.i64(TL), L.i64(K),
                                               L.f32(0.5), L.f32(0.01), L.ptr(ws), L.i64(ws_bytes), st), 'hessian')
    t_h = timeit(hess, 32, 16)
    # the vendor library on the same operands, for scale: the full product X^T X as one bf16 GEMM through torch
    # (hipBLASLt; bf16 output, no accumulation into H), same token-major layout of both operands
    xl = [x[b * FOLD:(b + 1) * FOLD].reshape(TL, K) for b in range(nb // FOLD)]
    t_lib = timeit(lambda i: torch.matmul(xl[i % len(xl)].t(), xl[i % len(xl)]), 8, 3)
    alg_flops = 2.0 * TL * K * K
    tiles = sum(K // 128 - 2 * ti for ti in range(K // 256))          # 256x128 tiles that reach the upper triangle
    exe_flops = 2.0 * TL * tiles * 256 * 128
    traffic, stale = traffic_bytes('hessian_kernel_K14336_T8192', t_h * 1e6) if FOLD == 4 else (None, None)
    out['roofline'] = {
        'kernel': f'hessian_kernel<bf16> K=14336 T={TL} (+ tail_fold_kernel)', 'bound': 'mfma', 'achieved': round(exe_flops / t_h / 1e12, 2),
        'peak': 2500.0, 'unit': 'TFLOP/s', 'frac': round(exe_flops / t_h / 2.5e15, 4),
        'traffic': traffic, 'traffic_stale': stale,
        'launch_us': round(t_h * 1e6, 2), 'flop_executed_per_launch': exe_flops,
        'algorithmic_tflops': round(alg_flops / t_h / 1e12, 2), 'frac_algorithmic': round(alg_flops / t_h / 2.5e15, 4),
        'library_gemm': {'what': 'torch.matmul(X.t(), X), bf16, the whole K x K product on the same tokens (hipBLASLt)',
                         'us': round(t_lib * 1e6, 1), 'tflops': round(alg_flops / t_lib / 1e12, 1),
                         'frac': round(alg_flops / t_lib / 2.5e15, 4)},
        'note': 'achieved / frac count the flops the matrix pipes execute (the 256x128 tiles that reach the upper '
                'triangle of the symmetric H: matrix-pipe utilisation against the 2.4 GHz peak); the algorithmic figure '
                '2*T*K^2 of the full product X^T X per launch is in algorithmic_tflops / frac_algorithmic.  rocprofv3 '
                'counters (profiles/) show the pipes busy for 3/4 of the cycles at a shader clock the chip holds near '
                '1.4 GHz under this kernel'}


# ---------------------------------------------------------------------------------------------------------------
# HBM-bound quantizer kernels one by one (algorithmic bytes: every input element read once, every output once)
# ---------------------------------------------------------------------------------------------------------------
def bench_quantizers(args, out):
    import torch
    from lightcompress_amd import _lib as L
    dev = torch.device('cuda:0')
    lib, st = L.lib(), L.stream()
    bf, f32 = torch.bfloat16, torch.float32
    rows_out = []

    def rot(shape, dtype, scale, total=1.3e9):
        n = max(3, int(total / (shape[0] * shape[1] * torch.tensor([], dtype=dtype).element_size())))
        return [(torch.randn(*shape, device=dev) * scale).to(dtype) for _ in range(n)]

    def report(name, kernel, rbytes, wbytes, t):
        nbytes = rbytes + wbytes
        mix = min((1, 2, 4, 8), key=lambda m: abs(math.log(rbytes / wbytes / m)))    # nearest probed read:write ratio
        rows_out.append({'case': name, 'kernel': kernel, 'us': round(t * 1e6, 2), 'MB': round(nbytes / 1e6, 1),
                         'GB/s': round(nbytes / t / 1e9, 1), 'frac': round(nbytes / t / 8e12, 4), 'read:write': f'{mix}:1'})
        return rows_out[-1]

    def quant_int(xs, rows, cols, qmin, qmax, flags, dq=None, codes=None, cd=L.CODE_NONE):
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

    # a plain device copy on this box: the ceiling an HBM-bound kernel can be held against
    src = [torch.empty(64 << 20, dtype=torch.float32, device=dev).normal_() for _ in range(3)]
    dst = [torch.empty_like(s) for s in src]
    t = timeit(lambda i: dst[i % 3].copy_(src[i % 3]), 30, 10)
    nb_copy = 2 * src[0].numel() * 4
    ones = torch.ones(8192, dtype=f32, device=dev)
    def own_copy(i):                                         # x / 1 through this library's own load / store path
        L.check(lib.lcq_div_cols(L.ptr(src[i % 3]), L.i32(L.F32), L.i64(src[0].numel() // 8192), L.i64(8192), L.ptr(ones),
                                 L.ptr(dst[i % 3]), st), 'lcq_div_cols')
    t2 = timeit(own_copy, 30, 10)
    out['hbm_copy'] = {'GB/s': round(nb_copy / min(t, t2) / 1e9, 1), 'frac': round(nb_copy / min(t, t2) / 8e12, 4),
                       'torch_copy_GB/s': round(nb_copy / t / 1e9, 1), 'lcq_div_cols_by_one_GB/s': round(nb_copy / t2 / 1e9, 1),
                       'what': 'plain streaming copies of 256 MiB fp32 tensors on this box (read + written bytes, three rotating '
                               'pairs): torch copy_ and this library x / 1 kernel; GB/s = the faster one'}
    # the same for other mixes of reads and writes (a quantizer that packs reads four bytes for each one it writes):
    # this library's streaming probe, 512 MiB read per launch
    big = torch.cat([x.view(-1) for x in src[:2]])
    room = torch.empty_like(big)
    mixes = {}
    for m in (0, 1, 2, 4, 8):
        tm = timeit(lambda i: L.check(lib.lcq_stream_probe(L.ptr(big), L.ptr(room), L.i64(big.numel() * 4), L.i64(room.numel() * 4),
                                                           L.i32(m), st), 'lcq_stream_probe'), 20, 5)
        mixes['read only' if m == 0 else f'{m}:1'] = round(big.numel() * 4 * (1 + (1 / m if m else 0)) / tm / 1e9, 1)
    out['hbm_stream_mix'] = {'GB/s': mixes, 'what': 'read + written bytes per second of a kernel that only streams (xor of m 16-byte '
                             'chunks read -> one chunk written), by its ratio of bytes read to bytes written; 512 MiB read per launch'}
    del src, dst, big, room

    # RTN config: fp32 [4096, 4096], INT4 asym g128: dq + uint8 codes + scales / zeros
    xs = rot((4096, 4096), f32, 0.02)
    dq = [torch.empty_like(x) for x in xs]
    cds = [torch.empty(4096, 4096, dtype=torch.uint8, device=dev) for _ in xs]
    n, g = 4096 * 4096, 128
    t = timeit(quant_int(xs, n // g, g, 0, 15, 0, dq, cds, L.CODE_U8), 60, 25)
    r = report('RTN int4 asym g128, fp32 4096x4096 -> dq + u8 codes + scales/zeros', 'row_team_kernel<IntOp<f32>>', n * 4, n * 5 + n // g * 8, t)
    traffic, stale = traffic_bytes('rtn_quant_int4_g128_4096x4096_f32', r['us'])
    out['roofline_quantizer'] = {'kernel': 'row_team_kernel<IntOp<f32>> 4096x4096 g128 dq+u8', 'bound': 'hbm', 'achieved': r['GB/s'],
                                 'peak': 8000.0, 'unit': 'GB/s', 'frac': r['frac'],
                                 'traffic': traffic, 'traffic_stale': stale, 'launch_us': r['us']}
    t = timeit(quant_int(xs, n // g, g, 0, 15, 0, dq), 60, 25)
    report('RTN int4 asym g128 fake quant, fp32 4096x4096', 'row_team_kernel<IntOp<f32>>', n * 4, n * 4 + n // g * 8, t)
    del xs, dq, cds
    # AWQ config: bf16 [11008, 4096] fake quant, int4 asym g128
    xs = rot((11008, 4096), bf, 0.02)
    dq = [torch.empty_like(x) for x in xs]
    n = 11008 * 4096
    t = timeit(quant_int(xs, n // g, g, 0, 15, 0, dq), 60, 25)
    report('int4 asym g128 fake quant, bf16 11008x4096', 'row_team_kernel<IntOp<bf16>>', n * 2, n * 2 + n // g * 4, t)
    del xs, dq
    # FP8 + pack config: 16 experts [2048, 7168] bf16 at once, and one expert alone
    for ne in (16, 1):
        R, K = ne * 2048, 7168
        xs = rot((R, K), bf, 0.006, total=3e9 if ne > 1 else 1.3e9)
        n = R * K
        cds = [torch.empty(R, K, dtype=torch.uint8, device=dev) for _ in xs]
        t = timeit(quant_fp(xs, R, K, None, cds, L.CODE_FP8), 30 if ne > 1 else 60, 12 if ne > 1 else 25)
        report(f'fp8 e4m3 per-channel real quant, bf16 {ne}x[2048,7168]', 'row_block_kernel<FpOp<bf16>>', n * 2, n + R * 2, t)
        pk = [torch.empty(R, K // 8, dtype=torch.int32, device=dev) for _ in xs]
        t = timeit(quant_int(xs, n // g, g, -8, 7, L.FLAG_SYM, None, pk, L.CODE_CT4), 30 if ne > 1 else 60, 12 if ne > 1 else 25)
        report(f'int4 sym g128 quantize + compressed-tensors pack, bf16 {ne}x[2048,7168]', 'row_team_kernel<IntOp<bf16, CT4>>',
               n * 2, n * 0.5 + n // g * 2, t)
        del xs, cds, pk
    # per-token dynamic fp8 fake quant of activations [8192, 7168]
    xs = rot((8192, 7168), bf, 1.0)
    dq = [torch.empty_like(x) for x in xs]
    n = 8192 * 7168
    t = timeit(quant_fp(xs, 8192, 7168, dq), 60, 25)
    report('fp8 e4m3 per-token fake quant, bf16 8192x7168', 'row_block_kernel<FpOp<bf16>>', n * 2, n * 2 + 8192 * 2, t)
    for r in rows_out:
        r['frac_of_copy'] = round(r['GB/s'] / out['hbm_copy']['GB/s'], 3)
        r['frac_of_stream_mix'] = round(r['GB/s'] / mixes[r['read:write']], 3)
    out['quantizers'] = rows_out


# ---------------------------------------------------------------------------------------------------------------
# the other configurations of the baseline: wall time on the GPU next to a CPU-oracle sample
# ---------------------------------------------------------------------------------------------------------------
def bench_c1(args):
    """RTN fake + real quant of one fp32 4096x4096 weight through the class API; CPU oracle at full size."""
    import torch
    from lightcompress_amd import IntegerQuantizer
    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(0)
    w = torch.randn(4096, 4096, generator=g) * 0.02
    idx = torch.randperm(w.numel(), generator=g)[:int(0.001 * w.numel())]
    w.view(-1)[idx] *= 20
    q = IntegerQuantizer(4, False, 'per_group', group_size=128)
    wd = w.to(dev)
    def run(i):
        q.fake_quant_weight_dynamic(wd)
        q.real_quant_weight_dynamic(wd)
    t = timeit(run, 20, 5)
    res = {'workload': 'RTN INT4 asym g128, fp32 4096x4096: fake_quant_weight_dynamic + real_quant_weight_dynamic (class API, '
                       'weight served from cache)', 'gpu_s': round(t, 6)}
    if not args.no_cpu:
        from oracle import quant_ref as Q
        cores = cpu_threads()
        spec = Q.IntSpec(4, False, 'per_group', group_size=128)
        t0 = time.perf_counter()
        Q.int_fake_quant_dynamic(spec, w)
        Q.int_real_quant_dynamic(spec, w)
        res['cpu_baseline'] = {'value': round(time.perf_counter() - t0, 4), 'unit': 's', 'cores': cores, 'kind': 'port',
                               'sample': 'full size'}
    return res


def bench_c2(args):
    """GPTQ of a single 4096 -> 4096 Linear, 128 x 2048 calibration tokens, act_order off."""
    import torch
    from lightcompress_amd.gptq import GPTQ
    dev = torch.device('cuda:0')
    K = R = 4096
    w = (torch.randn(R, K, device=dev) * 0.02).bfloat16()
    sigma = torch.exp(torch.randn(K, device=dev))
    x = torch.empty(NB, TOK, K, dtype=torch.bfloat16, device=dev)
    for b in range(NB):
        x[b] = (torch.randn(TOK, K, device=dev) * sigma).bfloat16()
    cfg = {'weight': CFG['weight'], 'special': dict(CFG['special'], actorder=False)}
    def run(i):
        gp = GPTQ(cfg)
        layer = Layer(torch.nn.Parameter(w.clone(), requires_grad=False))
        sub = {'layers': {'fc': layer}}
        gp.subset_init(sub)
        for b in range(NB):
            gp.add_batch(layer, 'fc', x[b:b + 1], None)
        gp.subset_transform(sub)
        return gp, layer
    run(0)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(3):
        gp, layer = run(i)
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / 3
    assert bool(torch.isfinite(layer.weight.data).all()) and float(gp.last_error) > 0
    return {'workload': 'GPTQ w4 asym g128, one Linear 4096->4096 bf16, 128x2048 calib tokens, act_order off', 'gpu_s': round(t, 5),
            'last_error': round(float(gp.last_error), 3)}


def bench_c3(args):
    """AWQ 20-point scale search on a SwiGLU MLP 4096 / 11008 with 128 x 512 calibration tokens."""
    import torch
    from lightcompress_amd.awq import Awq
    dev = torch.device('cuda:0')
    Hd, I = 4096, 11008
    mk = lambda r, c: (torch.randn(r, c, device=dev) * 0.02).bfloat16()
    class Fc:
        def __init__(self, w):
            self.weight = Layer(w)
            self.weight.data = w
    gate, up, down = Fc(mk(I, Hd)), Fc(mk(I, Hd)), mk(Hd, I)
    x = (torch.randn(128, 512, Hd, device=dev) * torch.exp(torch.randn(Hd, device=dev))).bfloat16()
    F = torch.nn.functional
    def mlp(xx):
        return (F.silu(xx @ gate.weight.data.t()) * (xx @ up.weight.data.t())) @ down.t()
    awq = Awq({'weight': CFG['weight'], 'special': {}})
    layers = {'gate': gate, 'up': up}
    awq.search_scale_subset(None, layers, [x], mlp, False, {})
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    best = awq.search_scale_subset(None, layers, [x], mlp, False, {})
    torch.cuda.synchronize()
    t = time.perf_counter() - t0
    losses = awq.search_losses.clone()
    # this library's share: the same search with the inspect module replaced by a stored output (no GEMMs)
    y = mlp(x)
    awq.search_scale_subset(None, layers, [x], lambda xx: y, False, {})
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    awq.search_scale_subset(None, layers, [x], lambda xx: y, False, {})
    torch.cuda.synchronize()
    t_own = time.perf_counter() - t0
    t_gemm = t - t_own
    assert bool(torch.isfinite(losses).all()) and bool(torch.isfinite(best).all())
    res = {'workload': 'AWQ 20-point scale search, SwiGLU MLP 4096/11008 bf16, 128x512 calib tokens, w4 asym g128, trans v2',
           'gpu_s': round(t, 4), 'own_kernels_s': round(t_own, 4), 'library_gemm_s': round(t_gemm, 4),
           'best_grid_point': int(torch.argmin(losses)),
           'note': 'own_kernels_s = the search with the inspect module replaced by a stored output (W*s -> fake quant, x/s, '
                   'loss, mean|x|: this library); library_gemm_s = the rest, i.e. the 21 forwards of the inspect module '
                   '(hipBLASLt through torch)'}
    if not args.no_cpu:
        from oracle import awq_ref as A, quant_ref as Q
        cores = cpu_threads()
        spec = Q.IntSpec(4, False, 'per_group', group_size=128)
        ns = 8                                                   # 8 of 128 sequences, 1 of 20 grid points
        xc = x[:ns].cpu()
        wc = {'gate': gate.weight.data.cpu(), 'up': up.weight.data.cpu()}
        dc = down.cpu()
        fwd = lambda xx, ww: (F.silu(xx @ ww['gate'].t()) * (xx @ ww['up'].t())) @ dc.t()
        t0 = time.perf_counter()
        org = fwd(xc, wc)
        t_org = time.perf_counter() - t0
        t0 = time.perf_counter()
        s = A.get_scales(xc, None, 0.5)
        wq = {k: A.scale_and_fake_quant(v, s, spec) for k, v in wc.items()}
        t_w = time.perf_counter() - t0
        t0 = time.perf_counter()
        o = fwd(A.scaling_input(xc, s), wq)
        A.loss(org, o)
        t_x = time.perf_counter() - t0
        total = t_org * (128 / ns) + 20 * (t_w + t_x * (128 / ns))
        res['cpu_baseline'] = {'value': round(total, 1), 'unit': 's', 'cores': cores, 'kind': 'port',
                               'sample': f'oracle on {ns} of 128 sequences and 1 of 20 grid points (weight scaling + fake quant at '
                                         'full size), token-dependent parts scaled by 16, the grid by 20'}
    return res


def bench_c5(args):
    """FP8 E4M3 per-channel real quant and INT4 g128 quant + pack of 256 experts (gate/up 2048x7168, down 7168x2048),
    plus per-token FP8 fake quant of 8192 x 7168 activations, through the class API."""
    import torch
    from lightcompress_amd import FloatQuantizer, IntegerQuantizer
    dev = torch.device('cuda:0')
    E = 256
    gate_up = (torch.randn(E * 2, 2048, 7168, device=dev) * 0.006).bfloat16()       # gate and up of every expert
    down = (torch.randn(E, 7168, 2048, device=dev) * 0.006).bfloat16()
    act = (torch.randn(8192, 7168, device=dev) * torch.exp(torch.randn(7168, device=dev))).bfloat16()
    fq = FloatQuantizer('e4m3', True, 'per_channel', use_qtorch=True)
    iq = IntegerQuantizer(4, True, 'per_group', group_size=128)
    aq = FloatQuantizer('e4m3', True, 'per_token', use_qtorch=True)
    # experts are independent and per-channel / per-group rows do not care which expert they belong to: 16 experts per call
    def sweep(fn):
        for i in range(0, E * 2, 32):
            fn(gate_up[i:i + 32].reshape(-1, 7168))
        for i in range(0, E, 16):
            fn(down[i:i + 16].reshape(-1, 2048))
    def timed(fn):
        sweep(fn); torch.cuda.synchronize()
        t0 = time.perf_counter()
        sweep(fn); torch.cuda.synchronize()
        return time.perf_counter() - t0
    t_fp8 = timed(lambda w: fq.real_quant_weight_dynamic(w))
    t_int4 = timed(lambda w: iq.real_quant_pack_dynamic(w))
    t_act = timeit(lambda i: aq.fake_quant_act_dynamic(act), 20, 5)
    n = E * 3 * 2048 * 7168
    res = {'workload': '256 experts x (gate, up 2048x7168; down 7168x2048) bf16: FP8 E4M3 per-channel real quant; INT4 sym g128 '
                       'quantize + compressed-tensors pack; per-token FP8 fake quant of 8192x7168 activations',
           'fp8_weights_s': round(t_fp8, 5), 'fp8_weights_GB/s': round((n * 3 + E * 3 * 2048 * 2) / t_fp8 / 1e9, 1),
           'int4_pack_s': round(t_int4, 5), 'int4_pack_GB/s': round((n * 2.5 + n // 128 * 2) / t_int4 / 1e9, 1),
           'act_fp8_s': round(t_act, 6), 'act_fp8_GB/s': round(8192 * 7168 * 4 / t_act / 1e9, 1),
           'gpu_s': round(t_fp8 + t_int4 + t_act, 5)}
    if not args.no_cpu:
        from oracle import pack_ref, quant_ref as Q
        cores = cpu_threads()
        ws = [gate_up[0].cpu(), gate_up[1].cpu(), down[0].cpu()]                      # one expert of 256
        fs, isp = Q.FloatSpec('e4m3', 'per_channel'), Q.IntSpec(4, True, 'per_group', group_size=128)
        t0 = time.perf_counter()
        for w in ws:
            Q.float_real_quant_dynamic(fs, w)
        t_f = time.perf_counter() - t0
        t0 = time.perf_counter()
        for w in ws:
            c, s, _ = Q.int_real_quant_dynamic(isp, w)
            pack_ref.pack_ct(c, s, 4)
        t_i = time.perf_counter() - t0
        t0 = time.perf_counter()
        Q.float_fake_quant_dynamic(Q.FloatSpec('e4m3', 'per_token'), act.cpu())
        t_a = time.perf_counter() - t0
        res['cpu_baseline'] = {'value': round(E * (t_f + t_i) + t_a, 1), 'unit': 's', 'cores': cores, 'kind': 'port',
                               'sample': 'oracle on 1 of 256 experts (3 matrices) for FP8 and INT4 + pack, scaled by 256; the '
                                         'activation tensor at full size',
                               'parts_s': {'fp8_weights': round(E * t_f, 1), 'int4_pack': round(E * t_i, 1), 'act_fp8': round(t_a, 2)}}
    return res


def cpu_baseline_layer():
    """The CPU oracle (a port of the reference's torch op sequence) on a bounded sample of the layer."""
    import torch
    from oracle import gptq_ref as G, quant_ref as Q
    cores = cpu_threads()
    g = torch.Generator().manual_seed(0)
    t = {}
    # Hessian, K=4096: 2 of 128 batches
    K = 4096
    x = (torch.randn(2, TOK, K, generator=g)).bfloat16()
    H, n = torch.zeros(K, K), 0
    t0 = time.perf_counter()
    for b in range(2):
        n = G.add_batch(H, n, x[b:b + 1])
    t['hess4096_per_batch'] = (time.perf_counter() - t0) / 2
    # Hessian, K=14336: 1 of 128 batches
    K2 = 14336
    x2 = torch.randn(1, TOK, K2, generator=g).bfloat16()
    H2 = torch.zeros(K2, K2)
    t0 = time.perf_counter()
    G.add_batch(H2, 0, x2)
    t['hess14336_per_batch'] = time.perf_counter() - t0
    del H2, x2
    # Cholesky chain, K=4096 (K=14336 extrapolated cubically)
    H += 0.01 * torch.mean(torch.diag(H)) * torch.eye(K)
    W = torch.randn(4096, K, generator=g) * 0.02
    t0 = time.perf_counter()
    Wp, U, _ = G.process_hessian_and_weights(W, H, 0.01, None)
    t['chain4096'] = time.perf_counter() - t0
    # column loop: first 2 of 32 blocks of a 4096x4096 Linear
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    t0 = time.perf_counter()
    G.weight_transform(Wp[:, :256].contiguous(), U[:256, :256].contiguous(), spec)
    t['loop_per_block_R4096'] = (time.perf_counter() - t0) / 2
    hess = 6 * NB * t['hess4096_per_batch'] + NB * t['hess14336_per_batch']
    chain = 6 * t['chain4096'] + t['chain4096'] * (14336 / 4096) ** 3
    # blocks x rows: q,o 32 blocks x 4096 rows; k,v 32 x 1024; gate,up 32 x 14336; down 112 x 4096
    loop = t['loop_per_block_R4096'] * (2 * 32 + 2 * 32 * 0.25 + 2 * 32 * 3.5 + 112)
    total = hess + chain + loop
    c2 = NB * t['hess4096_per_batch'] + t['chain4096'] + 32 * t['loop_per_block_R4096']
    return ({'value': round(total, 1), 'unit': 's', 'cores': cores, 'kind': 'port',
             'sample': 'oracle timed on 2/128 Hessian batches at K=4096, 1/128 at K=14336, the Cholesky chain at K=4096 '
                       '(K=14336 extrapolated by K^3), 2 column-loop blocks at R=4096 (in-block part only, scaled by rows '
                       'and blocks); extrapolated linearly to the full layer (one Hessian per Linear, as the reference keeps them)',
             'parts_s': {'hessian': round(hess, 1), 'chain': round(chain, 1), 'loop': round(loop, 1)}},
            {'value': round(c2, 1), 'unit': 's', 'cores': cores, 'kind': 'port',
             'sample': 'the same oracle timings: 128 x the per-batch Hessian at K=4096, one chain, 32 x the per-block loop time'})


def gpu_main(args):
    import torch
    from lightcompress_amd import _lib as L
    dev = torch.device('cuda:0')
    torch.cuda.set_device(dev)
    L.lib()
    torch.manual_seed(0)
    only = args.only
    out = {
        'metric': 'gptq_w4g128_seconds_per_llama3_8b_layer', 'value': None, 'unit': 's',
        'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': None,
        'higher_is_better': False, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'bf16 in / fp32 accumulate',
        'data': 'synthetic',
        'config': {'workload': 'GPTQ w4 asym g128 act_order, full Llama-3-8B-shape decoder layer (q,o 4096x4096; k,v 1024x4096; '
                               'gate,up 14336x4096; down 4096x14336), 128x2048 calib tokens per stream, add_batch per Linear per '
                               'batch; Linears fed the identical tensor (q,k,v / gate,up) share one Hessian '
                               '(seconds_separate_hessians: one per Linear)',
                   'blocksize': 128, 'percdamp': 0.01},
    }
    x_down = None
    if only in ('all', 'layer'):
        x_down = bench_layer(args, out)
    if only in ('all', 'layer', 'hessian'):
        bench_hessian(args, out, x_down)
    del x_down
    torch.cuda.empty_cache()
    if only in ('all', 'quantizers'):
        bench_quantizers(args, out)
    configs = {}
    if only in ('all', 'c1'):
        configs['C1_rtn'] = bench_c1(args)
    if only in ('all', 'c2'):
        configs['C2_gptq_linear'] = bench_c2(args)
        torch.cuda.empty_cache()
    if only in ('all', 'c3'):
        configs['C3_awq_search'] = bench_c3(args)
        torch.cuda.empty_cache()
    if only in ('all', 'c5'):
        configs['C5_fp8_int4_experts'] = bench_c5(args)
        torch.cuda.empty_cache()
    if not args.no_cpu and only in ('all', 'layer', 'c2'):
        layer_cpu, c2_cpu = cpu_baseline_layer()
        if only != 'c2':
            out['cpu_baseline'] = layer_cpu
        if 'C2_gptq_linear' in configs:
            configs['C2_gptq_linear']['cpu_baseline'] = c2_cpu
    if configs:
        out['configs'] = configs
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=2)
    ap.add_argument('--warmup', type=int, default=1)
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline legs')
    ap.add_argument('--only', default='all', choices=['all', 'layer', 'hessian', 'quantizers', 'c1', 'c2', 'c3', 'c5'],
                    help='run one part (profiling); the default runs everything')
    args = ap.parse_args()
    if args.gpus != 1:
        print('bench.py: this build runs on ONE GPU (one process, no collectives); --gpus must be 1', file=sys.stderr)
        sys.exit(2)
    gpu_main(args)


if __name__ == '__main__':
    main()
