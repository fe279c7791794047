#!/usr/bin/env python3
"""Benchmark of the layer-wise quantization hot path on one MI355X.

One "step" = GPTQ (w4 asym g128, act_order, damp 0.01, blocksize 128) of one
Llama-3-8B-shape decoder layer: for each of the four activation streams
(attention input, o_proj input, MLP input with K=4096; down_proj input with
K=14336) 128 calibration batches of 2048 tokens go through GPTQ.add_batch of
every Linear that sees them (q,k,v / o / gate,up / down; Linears that are
handed the identical tensor share one Hessian, `seconds_separate_hessians`
is the run with one Hessian per Linear as the reference keeps them), then
every Linear runs the damped Cholesky chain and the lazy-batch column loop.  Inputs are synthetic (lognormal
per-channel scaled Gaussians, random-init weights) and resident in HBM before
the timed region.

Prints ONE JSON line (see the keys below).  `roofline` describes the dominant
kernel (the bf16 MFMA Hessian at K=14336); `roofline_quantizer` the fused RTN
quantizer on BASELINE config 1; `cpu_baseline` the CPU oracle timed on a
bounded sample of the same workload.
"""
import argparse
import json
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
# HBM-side bytes per launch of the two roofline kernels: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this script,
# scaled by the same counters' reading for a copy kernel of known size (profiles/hessian_kernel_K14336_T8192.md,
# profiles/rtn_quant_int4_g128_4096x4096_f32.md).  Counters cannot be read from inside the timed process.
HESSIAN_TRAFFIC_BYTES = 6.890e9
RTN_TRAFFIC_BYTES = 1.501e8
CFG = {'weight': dict(bit=4, symmetric=False, granularity='per_group', group_size=128),
       'special': dict(actorder=True, static_groups=False, percdamp=0.01, blocksize=128, true_sequential=True)}


class Layer:
    def __init__(self, w):
        self.weight = w


def gpu_main(args):
    import torch
    from lightcompress_amd import IntegerQuantizer, _lib as L
    from lightcompress_amd.gptq import GPTQ

    dev = torch.device('cuda:0')
    torch.cuda.set_device(dev)
    L.lib()
    torch.manual_seed(0)

    # ---- synthetic inputs, resident before timing -------------------------------------
    weights = {n: (torch.randn(r, k, device=dev) * 0.02).bfloat16() for n, r, k, _ in LINEARS}
    streams = {}
    for sname, K in STREAM_K.items():
        sigma = torch.exp(torch.randn(K, device=dev))
        x = torch.empty(NB, TOK, K, dtype=torch.bfloat16, device=dev)
        for b in range(NB):
            x[b] = (torch.randn(TOK, K, device=dev) * sigma).bfloat16()
        streams[sname] = x

    def ev():
        return torch.cuda.Event(enable_timing=True)

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
                gp._chains_ahead(sub['layers'])
                for n in subset:
                    gp.layer_transform(layers[n], n)
                    gp.free(n)
                    check[n] = gp.last_error
            else:                                      # same work one Linear at a time, with events between the phases
                for n in subset:
                    gp.initialize_qparams_and_prepare_weights(layers[n], n)
                    a = ev(); a.record()
                    W, U = gp.process_hessian_and_weights(layers[n], n)
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

    # ---- dominant kernel: bf16 MFMA Hessian at K=14336, live HIP-event timing ------------------
    K = 14336
    H = torch.zeros(K, K, device=dev)
    x = streams['down_in']
    lib, st = L.lib(), L.stream()
    FOLD = GPTQ(CFG).hessian_fold(14336)                      # add_batch calls per launch, as the layer run above issues them
    TL = FOLD * TOK
    def hess(b):
        b = (b * FOLD) % (NB - FOLD + 1)
        L.check(lib.lcq_hessian_accum(L.ptr(H), L.i64(K), L.ptr(x[b]), L.i32(L.BF16), L.i64(TL), L.i64(K), L.f32(0.5),
                                      L.f32(0.01), st), 'hessian')
    for b in range(16):
        hess(b)
    n_launch = 32
    a, b_ = ev(), ev()
    a.record()
    for b in range(n_launch):
        hess(b)
    b_.record(); torch.cuda.synchronize()
    t_h = a.elapsed_time(b_) * 1e-3 / n_launch
    alg_flops = 2.0 * TL * K * K
    tiles = sum(K // 128 - 2 * ti for ti in range(K // 256))          # 256x128 tiles that reach the upper triangle
    exe_flops = 2.0 * TL * tiles * 256 * 128
    roofline = {'kernel': f'hessian_kernel<bf16> K=14336 T={TL}', 'bound': 'mfma', 'achieved': round(alg_flops / t_h / 1e12, 2),
                'peak': 2500.0, 'unit': 'TFLOP/s', 'frac': round(alg_flops / t_h / 2.5e15, 4),
                'traffic': HESSIAN_TRAFFIC_BYTES if FOLD == 4 else None,
                'launch_us': round(t_h * 1e6, 2), 'executed_tflops': round(exe_flops / t_h / 1e12, 2),
                'frac_executed': round(exe_flops / t_h / 2.5e15, 4),
                'note': 'achieved counts the full 2*T*K^2 product; only tiles on/above the diagonal are executed'}
    del H

    # ---- quantizer: BASELINE config 1 (fp32 4096x4096, INT4 asym g128: dq + u8 codes + scales/zeros) ----
    nbuf = 6
    ws = [torch.randn(4096, 4096, device=dev) * 0.02 for _ in range(nbuf)]
    dq = [torch.empty_like(w) for w in ws]
    codes = [torch.empty(4096, 4096, dtype=torch.uint8, device=dev) for _ in range(nbuf)]
    rows = 4096 * 4096 // 128
    sc, zr = torch.empty(rows, 1, device=dev), torch.empty(rows, 1, device=dev)
    def rtn(i):
        L.check(lib.lcq_quant_int(L.ptr(ws[i % nbuf]), L.i32(L.F32), L.i64(rows), L.i64(128), L.f32(0), L.f32(15),
                                  L.i32(0), L.f32(1), L.ptr(dq[i % nbuf]), L.ptr(codes[i % nbuf]), L.i32(L.CODE_U8), L.ptr(sc),
                                  L.ptr(zr), st), 'quant')
    for i in range(6):
        rtn(i)
    a, b_ = ev(), ev()
    a.record()
    for i in range(60):
        rtn(i)
    b_.record(); torch.cuda.synchronize()
    t_q = a.elapsed_time(b_) * 1e-3 / 60
    q_bytes = 4096 * 4096 * (4 + 4 + 1) + rows * 8
    roofline_q = {'kernel': 'row_team_kernel<IntOp<f32>> 4096x4096 g128 dq+u8', 'bound': 'hbm',
                  'achieved': round(q_bytes / t_q / 1e9, 1), 'peak': 8000.0, 'unit': 'GB/s',
                  'frac': round(q_bytes / t_q / 8e12, 4), 'traffic': RTN_TRAFFIC_BYTES, 'launch_us': round(t_q * 1e6, 2)}

    out = {
        'metric': 'gptq_w4g128_seconds_per_llama3_8b_layer', 'value': round(dt, 4), 'unit': 's',
        'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': round(dt * 1e3, 2),
        'higher_is_better': False, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'bf16 in / fp32 accumulate',
        'data': 'synthetic',
        'config': {'workload': 'GPTQ w4 asym g128 act_order, full Llama-3-8B-shape decoder layer (q,o 4096x4096; k,v 1024x4096; '
                               'gate,up 14336x4096; down 4096x14336), 128x2048 calib tokens per stream, add_batch per Linear per batch; '
                               'Linears fed the identical tensor (q,k,v / gate,up) share one Hessian (seconds_separate_hessians: '
                               'one per Linear)',
                   'blocksize': 128, 'percdamp': 0.01},
        'seconds_separate_hessians': round(dt_separate, 4),
        'last_error': last_error,
        'breakdown_ms': phases,
        'roofline': roofline, 'roofline_quantizer': roofline_q,
    }
    if not args.no_cpu:
        out['cpu_baseline'] = cpu_baseline()
    print(json.dumps(out))


def cpu_baseline():
    """The CPU oracle (a port of the reference's torch op sequence) on a bounded sample of the layer."""
    import torch
    from oracle import gptq_ref as G, quant_ref as Q
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get('OMP_NUM_THREADS', cores)))
    torch.set_num_threads(cores)
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
    return {'value': round(total, 1), 'unit': 's', 'cores': cores, 'kind': 'port',
            'sample': 'oracle timed on 2/128 Hessian batches at K=4096, 1/128 at K=14336, the Cholesky chain at K=4096 '
                      '(K=14336 extrapolated by K^3), 2 column-loop blocks at R=4096 (in-block part only, scaled by rows '
                      'and blocks); extrapolated linearly to the full layer',
            'parts_s': {'hessian': round(hess, 1), 'chain': round(chain, 1), 'loop': round(loop, 1)}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=2)
    ap.add_argument('--warmup', type=int, default=1)
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg')
    args = ap.parse_args()
    if args.gpus != 1:
        print('bench.py: this build runs on ONE GPU (one process, no collectives); --gpus must be 1', file=sys.stderr)
        sys.exit(2)
    gpu_main(args)


if __name__ == '__main__':
    main()
