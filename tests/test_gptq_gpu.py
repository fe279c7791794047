"""GPU parity of the GPTQ path (Hessian, Cholesky chain, column loop) against the CPU oracle.

Tolerances (from the task's north star): Hessian within 1e-5 relative (fp32);
integer codes agree on >= 99.9 % of entries; reconstruction loss
||(W - What) X||^2 within 1 % of the oracle's.
"""
import types

import pytest
import torch

from oracle import gptq_ref as G, quant_ref as Q
from tests.helpers import assert_bit_equal, gen
from tests.test_oracle_gptq import calib_batches

pytestmark = pytest.mark.gpu

CFG = {'weight': dict(bit=4, symmetric=False, granularity='per_group', group_size=128),
       'special': dict(actorder=False, static_groups=False, percdamp=0.01, blocksize=128, true_sequential=True)}


def make_gptq(**special):
    from lightcompress_amd.gptq import GPTQ
    cfg = {'weight': dict(CFG['weight']), 'special': dict(CFG['special'], **special)}
    if 'weight' in special:
        cfg['weight'] = special.pop('weight')
        cfg['special'].pop('weight')
    return GPTQ(cfg)


def linear(W):
    return types.SimpleNamespace(weight=types.SimpleNamespace(data=W, shape=W.shape))


class Layer:
    def __init__(self, W):
        self.weight = torch.nn.Parameter(W, requires_grad=False)


@pytest.mark.parametrize('K,T,nb', [(256, 64, 3), (512, 100, 4), (384, 2048, 2), (1000, 33, 2), (4096, 256, 2)])
def test_hessian_within_1e5(dev, K, T, nb):
    batches = calib_batches(nb, T, K, seed=1000)
    g = make_gptq()
    layer = Layer(torch.zeros(8, K, device=dev))
    g.layers_cache['l'] = {}
    g.layer_init(layer, 'l')
    Ho = torch.zeros(K, K)
    n = 0
    for b in batches:
        g.add_batch(layer, 'l', b.unsqueeze(0).to(dev), None)
        n = G.add_batch(Ho, n, b.unsqueeze(0))
    H = g.hessian('l').cpu()
    assert g.layers_cache['l']['nsamples'] == n
    ref64 = G.hessian_closed_form(batches)
    scale = float(ref64.abs().max())
    assert float((H.double() - ref64).abs().max()) / scale < 1e-5          # vs the fp64 closed form
    assert float((H - Ho).abs().max()) / scale < 1e-5                       # vs the fp32 oracle
    assert float((H.double() - ref64).norm() / ref64.norm()) < 1e-5
    assert torch.equal(H, H.t())


@pytest.mark.parametrize('K,T,slices', [(512, 1000, 3), (1000, 333, 5), (256, 40, 8), (4096, 416, 3)])
def test_hessian_token_shares_sum_to_the_single_accumulator(dev, K, T, slices):
    """lcq_hessian_accum_sliced: the tokens of a launch in `slices` shares with an accumulator each, two launches with
    the recurrence's alpha / beta, then lcq_hessian_gather_slices: the sum equals what one accumulator holds (up to
    the order of fp32 additions) and the closed form in fp64; the other accumulators come back zeroed.  (256, 40, 8)
    leaves six shares without tokens: they only scale."""
    from lightcompress_amd import _lib as L
    lib = L.lib()
    xs = [(torch.randn(T, K, generator=gen(1300 + i)) * (1 + i)).bfloat16() for i in range(2)]
    xd = [x.to(dev) for x in xs]
    one = torch.zeros(K, K, device=dev)
    acc = torch.zeros(slices, K, K, device=dev)
    for i, (al, be) in enumerate(((0.0, 2.0), (0.5, 1.0))):
        L.check(lib.lcq_hessian_accum(L.ptr(one), L.i64(K), L.ptr(xd[i]), L.i32(L.BF16), L.i64(T), L.i64(K), L.f32(al), L.f32(be),
                                      L.stream()), 'one')
        L.check(lib.lcq_hessian_accum_sliced(L.ptr(acc), L.i64(K), L.ptr(xd[i]), L.ptr(xd[i]), L.i32(L.BF16), L.i64(T), L.i64(K),
                                             L.f32(al), L.f32(be), L.i32(slices), L.i64(K * K), L.stream()), 'sliced')
    assert int((acc[1:] != 0).any(dim=2).any(dim=1).sum()) >= min(slices - 1, (T + 31) // 32 - 1)    # shares really used
    L.check(lib.lcq_hessian_gather_slices(L.ptr(acc), L.i64(K), L.i32(slices), L.i64(K * K), L.stream()), 'gather')
    assert not bool(acc[1:].any())
    up = torch.triu(torch.ones(K, K, dtype=torch.bool))
    got, want = acc[0].cpu(), one.cpu()
    ref = 0.5 * 2.0 * xs[0].double().t() @ xs[0].double() + xs[1].double().t() @ xs[1].double()
    scale = float(ref.abs().max())
    assert float((got - want)[up].abs().max()) / scale < 2e-6
    assert float((got.double() - ref)[up].abs().max()) / scale < 1e-5
    # refused: a stride that lets the accumulators overlap, a share count out of range
    assert lib.lcq_hessian_accum_sliced(L.ptr(acc), L.i64(K), L.ptr(xd[0]), L.ptr(xd[0]), L.i32(L.BF16), L.i64(T), L.i64(K),
                                        L.f32(0.0), L.f32(1.0), L.i32(slices), L.i64(K * K - 8), L.stream()) != 0
    assert lib.lcq_hessian_accum_sliced(L.ptr(acc), L.i64(K), L.ptr(xd[0]), L.ptr(xd[0]), L.i32(L.BF16), L.i64(T), L.i64(K),
                                        L.f32(0.0), L.f32(1.0), L.i32(65), L.i64(K * K), L.stream()) != 0


@pytest.mark.parametrize('K,T', [(8192, 2048), (14336, 4096)])
def test_hessian_with_the_last_round_split(dev, K, T):
    """lcq_hessian_accum_balanced: the tiles of the last, partly filled round of workgroups are cut into token ranges
    whose partial sums meet in a workspace.  Same H as the plain launch up to the order of fp32 additions, the closed
    form in fp64 within 1e-5, the same bits from run to run; where no split pays the call needs no workspace."""
    from lightcompress_amd import _lib as L
    lib = L.lib()
    g = torch.Generator(device=dev)
    g.manual_seed(K + T)
    xs = [(torch.randn(T, K, device=dev, generator=g) * torch.exp(0.5 * torch.randn(K, device=dev, generator=g))).bfloat16() for _ in range(2)]
    nbytes = lib.lcq_hessian_balanced_workspace_bytes(L.i64(K), L.i64(T))
    assert nbytes > 0 and nbytes % (256 * 128 * 4) == 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    ws.fill_(0x7f)                                              # whatever the workspace held must not matter
    outs = []
    for rep in range(2):
        Hb = torch.ones(K, K, device=dev)
        for x, (al, be) in zip(xs, ((0.0, 2.0), (0.5, 1.0))):
            L.check(lib.lcq_hessian_accum_balanced(L.ptr(Hb), L.i64(K), L.ptr(x), L.ptr(x), L.i32(L.BF16), L.i64(T), L.i64(K), L.f32(al),
                                                   L.f32(be), L.ptr(ws), L.i64(nbytes), L.stream()), 'balanced')
        outs.append(Hb)
    assert torch.equal(outs[0], outs[1])
    Hp = torch.ones(K, K, device=dev)
    for x, (al, be) in zip(xs, ((0.0, 2.0), (0.5, 1.0))):
        L.check(lib.lcq_hessian_accum(L.ptr(Hp), L.i64(K), L.ptr(x), L.i32(L.BF16), L.i64(T), L.i64(K), L.f32(al), L.f32(be), L.stream()), 'plain')
    up = torch.triu(torch.ones(K, K, dtype=torch.bool, device=dev))
    scale = float(Hp[up].abs().max())
    assert float((outs[0] - Hp)[up].abs().max()) / scale < 2e-6
    assert int((outs[0] != Hp)[up].sum()) > 0                    # the split really happened: another order of additions
    ref = xs[0].double().t() @ xs[0].double() + xs[1].double().t() @ xs[1].double()
    assert float((outs[0].double() - ref)[up].abs().max()) / scale < 1e-5
    del ref
    assert lib.lcq_hessian_accum_balanced(L.ptr(Hp), L.i64(K), L.ptr(xs[0]), L.ptr(xs[0]), L.i32(L.BF16), L.i64(T), L.i64(K), L.f32(0.0),
                                          L.f32(1.0), L.ptr(ws), L.i64(nbytes - 16), L.stream()) == -5
    # no split: fewer than two rounds of tiles, ragged sizes
    for K2, T2 in ((4096, 2048), (1000, 64), (8192, 2040)):
        assert lib.lcq_hessian_balanced_workspace_bytes(L.i64(K2), L.i64(T2)) == 0
    K2, T2 = 1000, 64
    x = torch.randn(T2, K2, device=dev).bfloat16()
    a, b = torch.zeros(K2, K2, device=dev), torch.zeros(K2, K2, device=dev)
    L.check(lib.lcq_hessian_accum_balanced(L.ptr(a), L.i64(K2), L.ptr(x), L.ptr(x), L.i32(L.BF16), L.i64(T2), L.i64(K2), L.f32(0.0), L.f32(1.0),
                                           L.ptr(None), L.i64(0), L.stream()), 'no workspace')
    L.check(lib.lcq_hessian_accum(L.ptr(b), L.i64(K2), L.ptr(x), L.i32(L.BF16), L.i64(T2), L.i64(K2), L.f32(0.0), L.f32(1.0), L.stream()), 'plain')
    assert torch.equal(a, b)


@pytest.mark.parametrize('slices', [1, 3, 'auto'])
def test_hessian_shares_through_add_batch_and_reads_in_between(dev, slices):
    """`special.hessian_slices`: whatever the number of accumulators, reading H in the middle of the calibration
    (which sums the shares and clears all but the first) and going on afterwards ends at the closed form."""
    K, T = 512, 160
    batches = calib_batches(7, T, K, seed=1400)
    g = make_gptq(hessian_slices=slices, hessian_defer=3)
    layer = Layer(torch.zeros(8, K, device=dev))
    g.layers_cache['l'] = {}
    g.layer_init(layer, 'l')
    assert (g.layers_cache['l']['H_shares'] is None) == (slices == 1)
    for i, b in enumerate(batches):
        g.add_batch(layer, 'l', b.unsqueeze(0).to(dev), None)
        if i in (1, 4):
            part = g.hessian('l').cpu().double()
            ref = G.hessian_closed_form(batches[:i + 1])
            assert float((part - ref).abs().max() / ref.abs().max()) < 1e-5
            sh = g.layers_cache['l']['H_shares']
            assert sh is None or not bool(sh[1:].any())
    H = g.hessian('l').cpu()
    ref = G.hessian_closed_form(batches)
    assert float((H.double() - ref).abs().max() / ref.abs().max()) < 1e-5
    assert torch.equal(H, H.t())


def test_hessian_batched_call_and_fp16(dev):
    K = 256
    batches = calib_batches(4, 48, K, seed=1100, dtype=torch.float16)
    g = make_gptq()
    layer = Layer(torch.zeros(8, K, device=dev))
    g.layers_cache['l'] = {}
    g.layer_init(layer, 'l')
    g.add_batch(layer, 'l', torch.stack(batches).to(dev), None)              # [4, 48, K]: counts 4 batches
    assert g.layers_cache['l']['nsamples'] == 4
    ref = G.hessian_closed_form(batches)
    H = g.hessian('l').cpu().double()
    assert float((H - ref).abs().max() / ref.abs().max()) < 1e-5


@pytest.mark.parametrize('defer', [1, 3, 4, 'auto'])
def test_hessian_deferred_launches(dev, defer):
    """Folding several add_batch calls into one launch leaves H and nsamples as per-call updates do,
    for ragged token counts and for inputs the caller overwrites right after the call."""
    K = 320
    shapes = [(1, 96), (2, 96), (1, 96), (1, 40), (1, 96), (3, 64), (1, 96), (1, 700), (1, 96)]
    g = make_gptq(hessian_defer=defer)
    layer = Layer(torch.zeros(8, K, device=dev))
    g.layers_cache['l'] = {}
    g.layer_init(layer, 'l')
    Ho = torch.zeros(K, K)
    n = 0
    flat = []
    for i, (b, T) in enumerate(shapes):
        x = calib_batches(b, T, K, seed=1200 + i)
        xb = torch.stack(x)
        xd = xb.to(dev)
        g.add_batch(layer, 'l', xd, None)
        xd.zero_()                                  # the staged copy must not alias the caller's tensor
        n = G.add_batch(Ho, n, xb)
        flat.append(xb)
        assert g.layers_cache['l']['nsamples'] == n
    H = g.hessian('l').cpu()
    scale = float(Ho.abs().max())
    assert float((H - Ho).abs().max()) / scale < 1e-5
    assert torch.equal(H, H.t())
    # closed form: (2 / n) * sum_i X_i^T X_i over every token
    X = torch.cat([f.reshape(-1, K) for f in flat]).double()
    ref = (2.0 / n) * X.t() @ X
    assert float((H.double() - ref).abs().max() / ref.abs().max()) < 1e-5


def _chain_inputs(K, seed, dead=()):
    H = G.hessian_closed_form(calib_batches(4, max(64, K // 4), K, seed=seed)).float()
    for j in dead:
        H[:, j] = 0; H[j, :] = 0
    return H


@pytest.mark.parametrize('K,actorder,dead', [(128, False, ()), (256, True, (5,)), (384, False, ()), (1000, True, (0, 999)),
                                             (2048, True, ()), (3000, False, (7,))])
def test_cholesky_chain(dev, K, actorder, dead):
    from lightcompress_amd import _lib as L
    H = _chain_inputs(K, 4000 + K, dead)
    W = torch.randn(16, K, generator=gen(9))
    perm = G.act_order(H) if actorder else None
    Wo, Uo, _ = G.process_hessian_and_weights(W, H, 0.01, perm, dtype=torch.float64)
    Hd, Wd = torch.triu(H).to(dev).contiguous(), W.to(dev).contiguous()     # only the upper triangle is read
    permd = perm.to(dev) if perm is not None else None
    nbytes = L.lib().lcq_chol_inv_upper_workspace_bytes(L.i64(K))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    status = torch.ones(1, dtype=torch.int32, device=dev)
    U = torch.empty(K, K, device=dev)
    L.check(L.lib().lcq_chol_inv_upper(L.ptr(Hd), L.i64(K), L.ptr(permd), L.f32(0.01), L.ptr(Wd), L.i64(16), L.ptr(U),
                                       L.ptr(ws), L.i64(nbytes), L.ptr(status), L.stream()), 'chain')
    U = U.cpu()
    assert int(status.item()) == 0
    assert torch.equal(torch.triu(U), U) and bool((torch.diag(U) > 0).all())
    rel = float((U.double() - Uo).abs().max() / Uo.abs().max())
    assert rel < 2e-5, rel
    # dead columns are zeroed in the caller's (un-permuted) weights
    Wexp = W.clone(); Wexp[:, list(dead)] = 0
    assert torch.equal(Wd.cpu(), Wexp)
    # defining property in fp64: U^T U (H + damp I) = I
    Hp = H.double().clone()
    for j in dead:
        Hp[j, j] = 1
    if perm is not None:
        Hp = Hp[perm][:, perm]
    Hp += 0.01 * torch.mean(torch.diag(Hp)) * torch.eye(K, dtype=torch.float64)
    res = (U.double().t() @ U.double() @ Hp - torch.eye(K, dtype=torch.float64)).abs().max()
    assert float(res) < 5e-3, float(res)


@pytest.mark.parametrize('K,actorder,dead', [(128, False, ()), (256, True, (5,)), (1024, True, (0, 1023)), (2048, False, ())])
def test_block_factor_against_fp64(dev, K, actorder, dead):
    """lcq_chol_block_factor: P[b, b] = U[b, b] and P[p, b] = M[p, b] U[b, b] (p < b) with M = U^-1, 128-column blocks,
    against the reference chain in fp64; and the identity that makes the loop run on it: with D = W0 - Q and the
    reference's errors E (E U = D), sum_{p<b} D[:, p] P[p, b] = - sum_{p<b} E[:, p] U[p, b] for every block b."""
    from lightcompress_amd import _lib as L
    H = _chain_inputs(K, 4100 + K, dead)
    perm = G.act_order(H) if actorder else None
    _, Uo, _ = G.process_hessian_and_weights(torch.zeros(1, K), H, 0.01, perm, dtype=torch.float64)
    Mo = torch.linalg.solve_triangular(Uo, torch.eye(K, dtype=torch.float64), upper=True)
    Po = torch.zeros_like(Uo)
    for b in range(K // 128):
        sl = slice(128 * b, 128 * b + 128)
        Po[sl, sl] = Uo[sl, sl]
        Po[:128 * b, sl] = Mo[:128 * b, sl] @ Uo[sl, sl]
    Hd = torch.triu(H).to(dev).contiguous()
    permd = perm.to(dev) if perm is not None else None
    nbytes = L.lib().lcq_chol_inv_upper_workspace_bytes(L.i64(K))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    status = torch.ones(1, dtype=torch.int32, device=dev)
    P = torch.empty(K, K, device=dev)
    L.check(L.lib().lcq_chol_block_factor(L.ptr(Hd), L.i64(K), L.ptr(permd), L.f32(0.01), L.ptr(None), L.i64(0), L.ptr(P),
                                          L.ptr(ws), L.i64(nbytes), L.ptr(status), L.stream()), 'block factor')
    P = P.cpu()
    assert int(status.item()) == 0
    assert torch.equal(torch.triu(P), P)
    rel = float((P.double() - Po).abs().max() / Po.abs().max())
    assert rel < 2e-5, rel
    # the loop's identity, in fp64 on the device result: errors E of the reference recurrence satisfy E U = D, and the
    # weights the loop finds at block b are W0[:, b] - sum_{p<b} E[:, p] U[p, b] = W0[:, b] + sum_{p<b} D[:, p] P[p, b]
    D = torch.randn(8, K, generator=gen(77), dtype=torch.float64)
    E = torch.linalg.solve_triangular(Uo, D, upper=True, left=False)
    for b in range(1, K // 128):
        sl = slice(128 * b, 128 * b + 128)
        want = -(E[:, :128 * b] @ Uo[:128 * b, sl])
        got = D[:, :128 * b] @ P.double()[:128 * b, sl]
        assert float((got - want).abs().max()) <= 1e-3 * float(want.abs().max()) + 1e-9, b
    # K must be whole blocks
    assert L.lib().lcq_chol_block_factor(L.ptr(Hd), L.i64(K - 8), L.ptr(None), L.f32(0.01), L.ptr(None), L.i64(0), L.ptr(P.to(dev)),
                                         L.ptr(ws), L.i64(nbytes), L.ptr(status), L.stream()) != 0


def test_cholesky_reports_indefinite_matrix(dev):
    from lightcompress_amd import _lib as L
    K = 128
    H = -torch.eye(K)
    Hd = H.to(dev)
    nbytes = L.lib().lcq_chol_inv_upper_workspace_bytes(L.i64(K))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    U = torch.empty(K, K, device=dev)
    L.check(L.lib().lcq_chol_inv_upper(L.ptr(Hd), L.i64(K), L.ptr(None), L.f32(0.01), L.ptr(None), L.i64(0), L.ptr(U),
                                       L.ptr(ws), L.i64(nbytes), L.ptr(status), L.stream()), 'chain')
    assert int(status.item()) == 1
    assert L.lib().lcq_chol_inv_upper(L.ptr(Hd), L.i64(K), L.ptr(None), L.f32(0.01), L.ptr(None), L.i64(0), L.ptr(U),
                                      L.ptr(ws), L.i64(16), L.ptr(status), L.stream()) == -5   # workspace too small


def _loop_case(R, K, g, blocksize, sym, seed):
    H = G.hessian_closed_form(calib_batches(6, max(64, K // 2), K, seed=seed)).float()
    W0 = torch.randn(R, K, generator=gen(seed + 1)) * 0.02
    spec = Q.IntSpec(4, sym, 'per_group', group_size=g)
    W, U, _ = G.process_hessian_and_weights(W0, H, 0.01, None)
    return spec, W0, W, U


@pytest.mark.parametrize('R,K,g,bs,sym', [(64, 512, 128, 128, False), (40, 512, 128, 128, True), (32, 512, 64, 128, False),
                                           (32, 512, 256, 128, False), (48, 384, 128, 64, False), (16, 328, 128, 128, False),
                                           (32, 400, 100, 128, False),      # groups that open inside an octet / a block
                                           (32, 512, 128, 256, False), (24, 768, 64, 256, True), (16, 640, 128, 384, False),
                                           (16, 512, 256, 256, False), (16, 1280, 128, 512, False)])   # blocks wider than a kernel pass
def test_column_loop_against_oracle(dev, R, K, g, bs, sym):
    spec, W0, W, U = _loop_case(R, K, g, bs, sym, 5000 + K + g)
    tmp_o, Loss_o, groups = G.weight_transform(W.clone(), U, spec, blocksize=bs)
    so, zo = G.merge_groups(groups)
    gp = make_gptq(blocksize=bs, weight=dict(bit=4, symmetric=sym, granularity='per_group', group_size=g))
    gp.n_nonout = gp.columns = K
    gp._setup_groups(None, R, K)
    Wd = W.clone().to(dev)
    tmp, Losses = torch.zeros_like(Wd), torch.zeros_like(Wd)
    gp.weight_transform(Wd, U.to(dev).contiguous(), Losses, tmp)
    tmp, Losses = tmp.cpu(), Losses.cpu()
    assert torch.equal(tmp[:, 0], W[:, 0])
    assert float((tmp - tmp_o).abs().max()) < 1e-4 * float(tmp_o.abs().max())
    G_ = so.numel() // R
    s, z = gp._scales.cpu(), (None if sym else gp._zeros.cpu())
    assert torch.allclose(s.reshape(-1, 1), so, rtol=1e-4)
    codes_o = G.codes_from(tmp_o, so, zo, spec)
    codes = G.codes_from(tmp, s.reshape(-1, 1), None if sym else z.reshape(-1, 1), spec)
    agree = float((codes == codes_o).float().mean())
    assert agree >= 0.999, agree
    assert abs(float(Losses.sum()) - float(Loss_o.sum())) <= 1e-3 * float(Loss_o.sum())


@pytest.mark.parametrize('R,K,g,sym,variant', [(64, 512, 128, False, 'minmax'), (40, 640, 64, True, 'minmax'), (32, 512, 32, False, 'minmax'),
                                               (40, 512, 128, False, 'round_zp_off'), (32, 512, 128, False, 'mse'),
                                               (32, 384, 0, False, 'per_channel')])
def test_column_loop_on_the_block_factor(dev, R, K, g, sym, variant):
    """weight_transform handed the block factor P (and the weights as they were before the loop) instead of U: the
    compensated weights, group parameters and losses of the reference loop on U, for dynamic groups inside a block,
    un-rounded zero points, a calibrator that runs on the host side at every group opening, and given parameters."""
    spec, W0, W, U = _loop_case(R, K, g if g else 128, 128, sym, 5600 + K + g)
    wcfg = dict(bit=4, symmetric=sym, granularity='per_group', group_size=g)
    kw, layer, fn = {}, None, None
    if variant == 'round_zp_off':
        spec.round_zp = False
        wcfg['round_zp'] = False
    if variant == 'mse':
        wcfg['calib_algo'] = 'mse'
    if variant == 'per_channel':
        spec = Q.IntSpec(4, sym, 'per_channel')
        wcfg = dict(bit=4, symmetric=sym, granularity='per_channel')
        _, s0, z0, _, _ = Q.int_tensor_qparams(spec, W0)
        kw['static_qparams'] = (s0, z0)
        layer = types.SimpleNamespace(buf_scales=s0.to(dev), buf_zeros=z0.to(dev))
    if variant == 'mse':                                  # against this library's loop on U: the same search kernel
        tmp_o, Loss_o, s_u, _ = _run_loop(dev, make_gptq(weight=wcfg), W, U, R, K)
    else:
        tmp_o, Loss_o, groups = G.weight_transform(W.clone(), U, spec, qparams_fn=fn, **kw)
    P = G.block_factor(U.double()).float()
    gp = make_gptq(weight=wcfg)
    assert gp._block_factor_ok(K)
    gp.n_nonout = gp.columns = K
    gp._setup_groups(layer, R, K)
    Wd, Pd = W.clone().to(dev), P.to(dev).contiguous()
    gp._loop_factor, gp._loop_W0 = (Pd.data_ptr(), True), Wd.clone()
    tmp, Losses = torch.zeros_like(Wd), torch.zeros_like(Wd)
    gp.weight_transform(Wd, Pd, Losses, tmp)
    tmp, Losses = tmp.cpu(), Losses.cpu()
    s, z = gp._scales.cpu(), (None if sym else gp._zeros.cpu())
    if variant == 'mse':                                  # a shrink search may tie between neighbouring steps
        same = torch.isclose(s, s_u, rtol=1e-4).all(dim=1)
        assert float(same.float().mean()) >= 0.8
        assert float((tmp - tmp_o)[same].abs().max()) < 1e-4 * float(tmp_o.abs().max())
        assert abs(float(Losses.sum()) - float(Loss_o.sum())) <= 0.02 * float(Loss_o.sum())
    else:
        assert float((tmp - tmp_o).abs().max()) < 1e-4 * float(tmp_o.abs().max())
        assert abs(float(Losses.sum()) - float(Loss_o.sum())) <= 1e-3 * float(Loss_o.sum())
    if variant not in ('per_channel', 'mse'):
        so, zo = G.merge_groups(groups)
        assert torch.allclose(s.reshape(-1, 1), so, rtol=1e-4)
        codes_o = G.codes_from(tmp_o, so, zo, spec)
        codes = G.codes_from(tmp, s.reshape(-1, 1), None if sym else z.reshape(-1, 1), spec)
        assert float((codes == codes_o).float().mean()) >= 0.999
    # without the weights before the loop the call is refused, and U given as U still takes the reference's path
    gp._loop_W0 = None
    with pytest.raises(Exception):
        gp.weight_transform(W.clone().to(dev), Pd, torch.zeros_like(Wd), torch.zeros_like(Wd))


def test_per_channel_static_loop(dev):
    R, K = 32, 256
    spec = Q.IntSpec(4, False, 'per_channel')
    H = G.hessian_closed_form(calib_batches(4, 128, K, seed=6000)).float()
    W0 = torch.randn(R, K, generator=gen(6001)) * 0.02
    _, s0, z0, _, _ = Q.int_tensor_qparams(spec, W0)
    W, U, _ = G.process_hessian_and_weights(W0, H, 0.01, None)
    tmp_o, Loss_o, _ = G.weight_transform(W.clone(), U, spec, static_qparams=(s0, z0))
    gp = make_gptq(weight=dict(bit=4, symmetric=False, granularity='per_channel'))
    gp.n_nonout = gp.columns = K
    layer = types.SimpleNamespace(buf_scales=s0.to(dev), buf_zeros=z0.to(dev))
    gp._setup_groups(layer, R, K)
    Wd = W.clone().to(dev)
    tmp, Losses = torch.zeros_like(Wd), torch.zeros_like(Wd)
    gp.weight_transform(Wd, U.to(dev).contiguous(), Losses, tmp)
    assert float((tmp.cpu() - tmp_o).abs().max()) < 1e-4 * float(tmp_o.abs().max())


@pytest.mark.parametrize('actorder', [False, True])
@pytest.mark.parametrize('sym', [False, True])
def test_static_groups_loop(dev, actorder, sym):
    """static_groups: True (gptq.py:143-148, 224-227): the loop takes the RTN group parameters of the original
    column order, found through the act-order permutation, and refreshes nothing."""
    R, K, g = 48, 512, 64
    H = G.hessian_closed_form(calib_batches(6, 256, K, seed=9100)).float()
    W0 = torch.randn(R, K, generator=gen(9101)) * 0.02
    spec = Q.IntSpec(4, sym, 'per_group', group_size=g)
    _, s0, z0, _, _ = Q.int_tensor_qparams(spec, W0)
    perm = G.act_order(H) if actorder else None
    W, U, _ = G.process_hessian_and_weights(W0, H, 0.01, perm)
    sg = s0.reshape(R, K // g)
    zg = None if sym else z0.reshape(R, K // g)
    tmp_o, Loss_o, _ = G.weight_transform(W.clone(), U, spec, static_groups=(sg, zg, perm))
    gp = make_gptq(actorder=actorder, static_groups=True, weight=dict(bit=4, symmetric=sym, granularity='per_group', group_size=g))
    gp.n_nonout = gp.columns = K
    if actorder:
        gp.perm = perm.to(dev)
    layer = types.SimpleNamespace(buf_scales=s0.to(dev), buf_zeros=None if sym else z0.to(dev))
    gp._setup_groups(layer, R, K)
    Wd = W.clone().to(dev)
    tmp, Losses = torch.zeros_like(Wd), torch.zeros_like(Wd)
    gp.weight_transform(Wd, U.to(dev).contiguous(), Losses, tmp)
    tmp, Losses = tmp.cpu(), Losses.cpu()
    assert float((tmp - tmp_o).abs().max()) < 1e-4 * float(tmp_o.abs().max())
    cols = perm if actorder else torch.arange(K)
    s_col = sg[:, cols // g]
    z_col = torch.zeros_like(s_col) if sym else zg[:, cols // g]
    code = lambda t: torch.clamp(torch.round(t / s_col) + z_col, spec.qmin, spec.qmax)
    agree = float((code(tmp) == code(tmp_o)).float().mean())
    assert agree >= 0.999, agree
    assert abs(float(Losses.sum()) - float(Loss_o.sum())) <= 1e-3 * float(Loss_o.sum())


@pytest.mark.parametrize('actorder', [False, True])
def test_layer_end_to_end(dev, actorder):
    """add_batch x N -> layer_transform, against the fp32 oracle: codes and reconstruction loss."""
    R, K, nb, T = 96, 1024, 8, 256
    batches = calib_batches(nb, T, K, seed=7000)
    W0 = (torch.randn(R, K, generator=gen(7001)) * 0.02).bfloat16()
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    Ho = torch.zeros(K, K); n = 0
    for b in batches:
        n = G.add_batch(Ho, n, b.unsqueeze(0))
    ref = G.gptq_layer(W0, Ho, spec, actorder=actorder)

    gp = make_gptq(actorder=actorder)
    layer = Layer(W0.to(dev))
    gp.subset_init({'layers': {'fc': layer}})
    for b in batches:
        gp.add_batch(layer, 'fc', b.unsqueeze(0).to(dev), None)
    if actorder:                                   # same permutation on both sides (argsort ties are unordered)
        gp.hessian_sorting('fc')
        assert torch.equal(torch.sort(gp.perm.cpu()).values, torch.arange(K))
        d = torch.diag(Ho)[gp.perm.cpu()]
        assert bool((d[:-1] >= d[1:] * (1 - 1e-5)).all())
    gp.layer_transform(layer, 'fc')
    Wq = layer.weight.data.cpu()
    assert Wq.dtype == torch.float32 and Wq.shape == (R, K)
    s = layer.buf_scales.cpu(); z = layer.buf_zeros.cpu()
    assert s.shape == (R * K // 128, 1)
    perm = gp.perm.cpu() if actorder else torch.arange(K)
    if actorder:
        ref = G.gptq_layer(W0, Ho, spec, actorder=False) if False else ref
    tmp_perm = Wq[:, perm]
    codes = G.codes_from(tmp_perm, s, z, spec)
    if (not actorder) or torch.equal(perm, ref['perm']):
        codes_o = G.codes_from(ref['tmp_perm'], ref['scales'], ref['zeros'], spec)
        agree = float((codes == codes_o).float().mean())
        assert agree >= 0.999, agree
    X = torch.cat(batches).float()
    invp = torch.argsort(perm)
    What = Q.int_dequant(codes.reshape(-1, 128), s, z).reshape(R, K)[:, invp]
    ro = ref['perm'] if actorder else torch.arange(K)
    codes_ref = G.codes_from(ref['tmp_perm'], ref['scales'], ref['zeros'], spec)
    What_o = Q.int_dequant(codes_ref.reshape(-1, 128), ref['scales'], ref['zeros']).reshape(R, K)[:, torch.argsort(ro)]
    l, lo = G.recon_loss(W0.float(), What, X), G.recon_loss(W0.float(), What_o, X)
    assert abs(l - lo) <= 0.01 * lo, (l, lo)
    assert abs(float(gp.last_error) - ref['loss']) <= 0.01 * ref['loss']
    # deploy-time partials reproduce the codes
    wq = gp.wquantizer
    layer.buf_qmax, layer.buf_qmin = wq.qmax, wq.qmin
    fq = gp.w_qdq(layer, wq)
    assert fq.dtype == torch.bfloat16 and fq.shape == (R, K)


def test_shared_hessian_matches_separate(dev):
    R, K = 32, 512
    batches = calib_batches(4, 128, K, seed=8000)
    Wa = (torch.randn(R, K, generator=gen(8001)) * 0.02).bfloat16()
    Wb = (torch.randn(R // 2, K, generator=gen(8002)) * 0.02).bfloat16()
    outs = []
    for share in (False, True):
        gp = make_gptq(actorder=True)
        la, lb = Layer(Wa.to(dev)), Layer(Wb.to(dev))
        gp.subset_init({'layers': {'a': la, 'b': lb}})
        if share:
            gp.share_input(['a', 'b'])
        for x in batches:
            gp.add_batch(la, 'a', x.unsqueeze(0).to(dev)); gp.add_batch(lb, 'b', x.unsqueeze(0).to(dev))
        gp.subset_transform({'layers': {'a': la, 'b': lb}})
        outs.append((la.weight.data.cpu(), lb.weight.data.cpu(), lb.buf_scales.cpu()))
    for x, y in zip(*outs):
        assert torch.equal(x, y)


@pytest.mark.parametrize('actorder', [False, True])
def test_chains_side_by_side_match_one_by_one(dev, actorder):
    """subset_transform starts the Cholesky chains of a subset on separate streams (chain_overlap, the default); the
    weights, scales and losses must be those of the one-by-one order, bit for bit, also with a dead column and with
    Linears of different input widths in one subset."""
    R = 48
    Ks = {'a': 1536, 'b': 1536, 'c': 640}
    xs = {K: calib_batches(4, 96, K, seed=8100 + K) for K in set(Ks.values())}
    for K in xs:
        for x in xs[K]:
            x[:, 7] = 0                                           # a dead column
    Ws = {n: (torch.randn(R, K, generator=gen(8200 + i)) * 0.02).bfloat16() for i, (n, K) in enumerate(Ks.items())}
    outs = []
    for overlap in (False, True):
        gp = make_gptq(actorder=actorder, chain_overlap=overlap)
        layers = {n: Layer(Ws[n].to(dev)) for n in Ks}
        gp.subset_init({'layers': layers})
        for j in range(4):
            for n, K in Ks.items():
                gp.add_batch(layers[n], n, xs[K][j].unsqueeze(0).bfloat16().to(dev))
        gp.subset_transform({'layers': layers})
        torch.cuda.synchronize()
        assert gp._shared == {}
        outs.append([t for n in Ks for t in (layers[n].weight.data.cpu(), layers[n].buf_scales.cpu(), layers[n].buf_zeros.cpu())]
                    + [gp.last_error.cpu()])
    for x, y in zip(*outs):
        assert torch.equal(x, y)


@pytest.mark.parametrize('bit,sym,g,bs,R,K,wdtype', [
    (3, False, 128, 128, 40, 768, torch.bfloat16),      # R not a multiple of the 16 rows of a workgroup
    (8, True, 64, 128, 64, 640, torch.float16),         # fp16 weights, symmetric 8 bit
    (2, False, 32, 64, 24, 512, torch.float32),         # 2 bit, small groups, half-size blocks
    (4, False, 256, 128, 32, 1280, torch.bfloat16),     # groups wider than a block
    (4, True, 128, 128, 130, 1152, torch.bfloat16),     # odd row count, K = 9 blocks
    (4, False, 128, 256, 40, 1024, torch.bfloat16),     # blocks of 256 columns: two kernel passes each
])
@pytest.mark.parametrize('block_factor', [True, False])
def test_layer_configurations(dev, bit, sym, g, bs, R, K, wdtype, block_factor):
    """layer_transform over bit widths, symmetry, group / block sizes and weight dtypes against the fp32 oracle:
    codes >= 99.9 % equal, summed loss within 0.1 %.  block_factor False is the reference's chain (cholesky, inverse,
    cholesky) and is held to that bar as it stands.  block_factor True (the default) skips the triangular inverse where
    the quantizer's groups allow it; it is closer to exact arithmetic than the fp32 chain, and at 8 bit the fp32 oracle
    itself is further than 0.1 % from the fp64 one, so a run that misses the bar against the fp32 oracle has to meet it
    against the fp64 oracle."""
    batches = calib_batches(6, 160, K, seed=9300 + K + bit)
    W0 = (torch.randn(R, K, generator=gen(9301 + bit)) * 0.02).to(wdtype)
    spec = Q.IntSpec(bit, sym, 'per_group', group_size=g)
    Ho = torch.zeros(K, K); n = 0
    for b in batches:
        n = G.add_batch(Ho, n, b.unsqueeze(0))
    ref = G.gptq_layer(W0, Ho, spec, blocksize=bs)
    gp = make_gptq(blocksize=bs, block_factor=block_factor,
                   weight=dict(bit=bit, symmetric=sym, granularity='per_group', group_size=g))
    assert gp._block_factor_ok(K) == (block_factor and bs == 128 and K % 128 == 0 and 128 % g == 0)
    layer = Layer(W0.to(dev))
    gp.subset_init({'layers': {'fc': layer}})
    for b in batches:
        gp.add_batch(layer, 'fc', b.unsqueeze(0).to(dev), None)
    gp.subset_transform({'layers': {'fc': layer}})
    Wq = layer.weight.data.cpu()
    s = layer.buf_scales.cpu()
    z = None if sym else layer.buf_zeros.cpu()
    assert torch.allclose(s, ref['scales'], rtol=1e-3)
    codes = G.codes_from(Wq, s, z, spec)
    codes_o = G.codes_from(ref['tmp_perm'], ref['scales'], ref['zeros'], spec)
    agree = float((codes == codes_o).float().mean())
    loss_ref = ref['loss']
    if agree < 0.999 and gp._block_factor_ok(K):
        H64 = torch.zeros(K, K, dtype=torch.float64); n = 0
        for b in batches:
            n = G.add_batch(H64, n, b.unsqueeze(0))
        ref64 = G.gptq_layer(W0, H64, spec, blocksize=bs, dtype=torch.float64)
        codes64 = G.codes_from(ref64['tmp_perm'].float(), ref64['scales'].float(), None if sym else ref64['zeros'].float(), spec)
        assert float((codes_o == codes64).float().mean()) < 0.999       # the fp32 oracle misses the fp64 one by as much
        agree = float((codes == codes64).float().mean())
        loss_ref = ref64['loss']
    assert agree >= 0.999, agree
    assert abs(float(gp.last_error) - loss_ref) <= 1e-3 * loss_ref


def _run_loop(dev, gp, W, U, R, K):
    gp.n_nonout = gp.columns = K
    gp._setup_groups(None, R, K)
    Wd = W.clone().to(dev)
    tmp, Losses = torch.zeros_like(Wd), torch.zeros_like(Wd)
    gp.weight_transform(Wd, U.to(dev).contiguous(), Losses, tmp)
    return tmp.cpu(), Losses.cpu(), gp._scales.cpu(), (None if gp.wquantizer.sym else gp._zeros.cpu())


@pytest.mark.parametrize('R,K,g,bs', [(32, 1200, 100, 128),      # the group opened at 1000 runs past the 1024-column window
                                      (32, 1100, 128, 100),      # window of 800 columns: the group at 768 crosses it
                                      (24, 2304, 384, 128)])     # groups wider than a block that straddle windows
def test_groups_that_cross_the_update_window(dev, R, K, g, bs):
    """The deferred update reaches far-away columns once per 8 blocks; a group that opens inside such a window and
    ends behind it must still see every earlier block's update in all of its columns (gptq.py:216-222, 244)."""
    spec, W0, W, U = _loop_case(R, K, g, bs, False, 5100 + K + g)
    tmp_o, Loss_o, groups = G.weight_transform(W.clone(), U, spec, blocksize=bs)
    so, zo = G.merge_groups(groups)
    gp = make_gptq(blocksize=bs, weight=dict(bit=4, symmetric=False, granularity='per_group', group_size=g))
    tmp, Losses, s, z = _run_loop(dev, gp, W, U, R, K)
    assert torch.allclose(s.reshape(-1, 1), so, rtol=1e-4)
    assert torch.allclose(z.reshape(-1, 1), zo, atol=0.5)
    assert float((z.reshape(-1, 1) != zo).float().mean()) < 2e-3
    assert float((tmp - tmp_o).abs().max()) < 1e-4 * float(tmp_o.abs().max())
    codes_o = G.codes_from(tmp_o, so, zo, spec)
    codes = G.codes_from(tmp, s.reshape(-1, 1), z.reshape(-1, 1), spec)
    assert float((codes == codes_o).float().mean()) >= 0.999
    assert abs(float(Losses.sum()) - float(Loss_o.sum())) <= 1e-3 * float(Loss_o.sum())


@pytest.mark.parametrize('g,bs,K', [(128, 128, 512), (64, 128, 384), (256, 128, 1280)])
def test_loop_with_unrounded_zero_points(dev, g, bs, K):
    """round_zp: False reaches the loop through wquantizer.get_tensor_qparams / quant_dequant (gptq.py:229, 358-366):
    zero = qmin - min/scale un-rounded, code = clamp(round(w / max(scale, 1e-9) + zero))."""
    R = 40
    spec, W0, W, U = _loop_case(R, K, g, bs, False, 5300 + K + g)
    spec.round_zp = False
    tmp_o, Loss_o, groups = G.weight_transform(W.clone(), U, spec, blocksize=bs)
    so, zo = G.merge_groups(groups)
    assert float((zo != torch.round(zo)).float().mean()) > 0.9             # the zero points really are fractional
    gp = make_gptq(blocksize=bs, weight=dict(bit=4, symmetric=False, granularity='per_group', group_size=g, round_zp=False))
    tmp, Losses, s, z = _run_loop(dev, gp, W, U, R, K)
    assert torch.allclose(s.reshape(-1, 1), so, rtol=1e-4)
    assert torch.allclose(z.reshape(-1, 1), zo, rtol=1e-3, atol=1e-3)
    assert float((tmp - tmp_o).abs().max()) < 1e-4 * float(tmp_o.abs().max())
    codes_o = G.codes_from(tmp_o, so, zo, spec)
    codes = G.codes_from(tmp, s.reshape(-1, 1), z.reshape(-1, 1), spec)
    assert float((codes == codes_o).float().mean()) >= 0.999
    assert abs(float(Losses.sum()) - float(Loss_o.sum())) <= 1e-3 * float(Loss_o.sum())
    # and it differs from the rounded-zero-point loop, i.e. the flag is not ignored
    gp2 = make_gptq(blocksize=bs, weight=dict(bit=4, symmetric=False, granularity='per_group', group_size=g))
    _, _, _, z2 = _run_loop(dev, gp2, W, U, R, K)
    assert not torch.equal(z2, z)


@pytest.mark.parametrize('g,bs,K', [(128, 128, 512), (64, 128, 256), (256, 128, 1280)])
def test_loop_with_mse_calibrated_groups(dev, g, bs, K):
    """calib_algo: mse (the GPTQ recipe offers it) reaches the loop through search_column_qparams ->
    wquantizer.get_tensor_qparams (gptq.py:358-366): every group's range is the shrunken one of get_mse_range."""
    R = 32
    spec, W0, W, U = _loop_case(R, K, g, bs, False, 5500 + K + g)
    tmp_o, Loss_o, groups = G.weight_transform(W.clone(), U, spec, blocksize=bs, qparams_fn=G.mse_tensor_qparams)
    so, zo = G.merge_groups(groups)
    _, _, groups_mm = G.weight_transform(W.clone(), U, spec, blocksize=bs)
    assert not torch.equal(G.merge_groups(groups_mm)[0], so)               # mse ranges differ from min/max ranges
    gp = make_gptq(blocksize=bs, weight=dict(bit=4, symmetric=False, granularity='per_group', group_size=g, calib_algo='mse'))
    tmp, Losses, s, z = _run_loop(dev, gp, W, U, R, K)
    # the shrink search picks between steps whose errors can tie to within fp32 summation noise: nearly all rows
    # choose the oracle's step, the others an adjacent one
    same = torch.isclose(s.reshape(-1, 1), so, rtol=1e-4)
    assert float(same.float().mean()) >= 0.98, float(same.float().mean())
    rows_ok = same.reshape(R, -1).all(dim=1)
    assert float(rows_ok.float().mean()) >= 0.8
    codes_o = G.codes_from(tmp_o, so, zo, spec)
    codes = G.codes_from(tmp, s.reshape(-1, 1), z.reshape(-1, 1), spec)
    agree = (codes == codes_o)[rows_ok]
    assert float(agree.float().mean()) >= 0.999                             # rows with the same ranges: same codes
    assert abs(float(Losses.sum()) - float(Loss_o.sum())) <= 0.02 * float(Loss_o.sum())


def test_learnable_calibration_without_factors_is_minmax(dev):
    """search_column_qparams passes no factors (gptq.py:358-366), so calib_algo='learnable' falls through to the
    plain min/max range (quant.py:207-221): same weights, losses and qparams as the default calibrator."""
    spec, W0, W, U = _loop_case(16, 256, 128, 128, False, 5700)
    outs = []
    for algo in ('learnable', 'minmax'):
        gp = make_gptq(weight=dict(bit=4, symmetric=False, granularity='per_group', group_size=128, calib_algo=algo))
        outs.append(_run_loop(dev, gp, W, U, 16, 256))
    for a, b in zip(*outs):
        assert torch.equal(a, b)


@pytest.mark.parametrize('actorder', [False, True])
@pytest.mark.parametrize('sym', [False, True])
def test_deploy_partials_w_q_and_w_qdq(dev, actorder, sym):
    """w_qdq / w_q (gptq.py:411-452) on a transformed layer: static fake / real quantization of the compensated
    weights with the loop's qparams - in processing order and un-permuted again when groups follow act-order; w_q
    rounds the scales to the model dtype first."""
    R, K, g = 64, 768, 128
    batches = calib_batches(4, 256, K, seed=9500)
    W0 = (torch.randn(R, K, generator=gen(9501)) * 0.02).bfloat16()
    spec = Q.IntSpec(4, sym, 'per_group', group_size=g)
    gp = make_gptq(actorder=actorder, weight=dict(bit=4, symmetric=sym, granularity='per_group', group_size=g))
    layer = Layer(W0.to(dev))
    gp.subset_init({'layers': {'fc': layer}})
    for b in batches:
        gp.add_batch(layer, 'fc', b.unsqueeze(0).to(dev), None)
    gp.layer_transform(layer, 'fc')
    wq = gp.wquantizer
    layer.buf_qmax, layer.buf_qmin = wq.qmax, wq.qmin
    Wt = layer.weight.data.cpu()
    s = layer.buf_scales.cpu()
    z = None if sym else layer.buf_zeros.cpu()
    zz = torch.tensor(0.0) if sym else z
    if sym and hasattr(layer, 'buf_zeros'):
        del layer.buf_zeros
    fq = gp.w_qdq(layer, wq)
    src = Wt
    if actorder:
        assert gp.need_perm
        src = Wt[:, layer.buf_perm.cpu()]
    want = Q.int_fake_quant_static(spec, src, s, zz, spec.qmax, spec.qmin).to(torch.bfloat16)
    if actorder:
        want = want[:, layer.buf_invperm.cpu()]
    assert_bit_equal(fq, want, 'w_qdq')
    # fake-quantised values sit on the loop's grid: they reproduce the loop's codes
    codes_loop = G.codes_from(src, s, z, spec)
    back = Q.int_quant(spec, Q.int_fake_quant_static(spec, src, s, zz, spec.qmax, spec.qmin).reshape(-1, g), s, zz, spec.qmax,
                       spec.qmin).reshape(R, K)
    assert torch.equal(back, codes_loop)
    if not actorder:                                    # real-quant export needs groups in the original order (gptq.py:455-457)
        if sym:
            layer.buf_zeros = torch.tensor(0.0)
        codes, s_out, z_out = gp.w_q(layer, wq)
        oc, os_, oz = Q.int_real_quant_static(spec, Wt, s.to(torch.bfloat16), zz, spec.qmax, spec.qmin)
        assert_bit_equal(codes, oc, 'w_q codes')
        assert_bit_equal(s_out, os_, 'w_q scales')
        if sym:
            assert z_out is None
        else:
            assert_bit_equal(z_out, oz, 'w_q zeros')


def _subset_run(dev, Ws, feeds, **special):
    """feeds: list over calls of {name: tensor}; returns per layer (weight, scales, zeros) and the GPTQ object state."""
    gp = make_gptq(actorder=True, **special)
    layers = {n: Layer(w.to(dev)) for n, w in Ws.items()}
    gp.subset_init({'layers': layers})
    followed = {}
    for call in feeds:
        for n, x in call.items():
            gp.add_batch(layers[n], n, x.data, None)               # hooks pass `inp[0].data`: a fresh alias every call
        followed = {n: gp.layers_cache[n].get('leader', n) for n in layers}
    Hs = {n: gp.hessian(n).clone() for n in layers}
    gp.subset_transform({'layers': layers})
    torch.cuda.synchronize()
    out = {n: (layers[n].weight.data.cpu(), layers[n].buf_scales.cpu(), layers[n].buf_zeros.cpu(), Hs[n].cpu()) for n in layers}
    return out, followed


def test_identical_inputs_share_one_hessian_automatically(dev):
    """q/k/v-style hooks hand the same tensor to every Linear of the subset: one Hessian accumulates, the others
    follow, and every result is bit-identical to separate accumulation."""
    K = 640
    Ws = {'q': (torch.randn(64, K, generator=gen(1)) * 0.02).bfloat16(), 'k': (torch.randn(32, K, generator=gen(2)) * 0.02).bfloat16(),
          'v': (torch.randn(32, K, generator=gen(3)) * 0.02).bfloat16(), 'other': (torch.randn(48, K, generator=gen(4)) * 0.02).bfloat16()}
    xs = [b.to(dev) for b in calib_batches(11, 96, K, seed=8300)]
    ys = [b.to(dev) for b in calib_batches(11, 96, K, seed=8400)]
    feeds = [{'q': x, 'k': x, 'v': x, 'other': y} for x, y in zip(xs, ys)]
    shared, followed = _subset_run(dev, Ws, feeds, hessian_defer=4)
    assert followed == {'q': 'q', 'k': 'q', 'v': 'q', 'other': 'other'}
    separate, followed2 = _subset_run(dev, Ws, feeds, hessian_defer=4, auto_share=False)
    assert followed2 == {n: n for n in Ws}
    for n in Ws:
        for a, b in zip(shared[n], separate[n]):
            assert torch.equal(a, b), n


@pytest.mark.parametrize('actorder,static_groups', [(True, False), (False, False), (True, True)])
def test_stacked_column_loop_matches_per_linear_loops(dev, actorder, static_groups):
    """Linears that share a chain run through the column loop stacked into one matrix (special.fuse_loops, default on).
    Rows are independent, so each Linear gets what its own loop gives: the same weights, scales, zero points and summed
    loss (to the rounding of the update GEMM, whose kernel may change with the row count; bit for bit at this size)."""
    K = 1024
    Ws = {'q': (torch.randn(256, K, generator=gen(11)) * 0.02).bfloat16(), 'k': (torch.randn(64, K, generator=gen(12)) * 0.02).bfloat16(),
          'v': (torch.randn(72, K, generator=gen(13)) * 0.02).bfloat16()}
    xs = [b.to(dev) for b in calib_batches(6, 256, K, seed=8700)]
    runs = []
    for fuse in (True, False):
        gp = make_gptq(actorder=actorder, static_groups=static_groups, fuse_loops=fuse)
        layers = {n: Layer(w.to(dev)) for n, w in Ws.items()}
        gp.subset_init({'layers': layers})
        if static_groups:
            for lay in layers.values():
                gp.collect_layer_qparams(lay)
        for x in xs:
            for n in Ws:
                gp.add_batch(layers[n], n, x.data, None)
        assert {gp.layers_cache[n].get('leader', n) for n in Ws} == {'q'}
        gp.subset_transform({'layers': layers})
        torch.cuda.synchronize()
        assert gp._shared == {} and gp.layers_cache == {}
        for n in Ws:                                      # every Linear owns its storage (no views of the stacked matrix)
            assert layers[n].weight.data.untyped_storage().nbytes() == Ws[n].numel() * 4
        errs = {n: float(gp.last_errors[n]) for n in Ws} if fuse else None
        runs.append(({n: (layers[n].weight.data.cpu(), layers[n].buf_scales.cpu(), layers[n].buf_zeros.cpu()) for n in Ws}, errs))
    (fused, errs), (alone, _) = runs
    for n in Ws:
        assert fused[n][0].shape == Ws[n].shape
        for a, b in zip(fused[n], alone[n]):
            assert torch.equal(a, b), n
    # the per-Linear losses of the stacked run are those of separate runs
    for n in Ws:
        gp = make_gptq(actorder=actorder, static_groups=static_groups, fuse_loops=False)
        lay = Layer(Ws[n].to(dev))
        gp.subset_init({'layers': {n: lay}})
        if static_groups:
            gp.collect_layer_qparams(lay)
        for x in xs:
            gp.add_batch(lay, n, x.data, None)
        gp.layer_transform(lay, n)
        assert abs(float(gp.last_error) - errs[n]) <= 1e-6 * abs(errs[n]), n


@pytest.mark.parametrize('split_at', [1, 4, 5, 8])
def test_sharing_falls_back_when_an_input_differs(dev, split_at):
    """The moment one call brings a different tensor the follower continues with its own Hessian - a copy of the
    shared state as it was before that call - and the final results equal separate accumulation bit for bit."""
    K = 384
    Ws = {'a': (torch.randn(32, K, generator=gen(5)) * 0.02).bfloat16(), 'b': (torch.randn(48, K, generator=gen(6)) * 0.02).bfloat16()}
    xs = [b.to(dev) for b in calib_batches(10, 64, K, seed=8500)]
    other = calib_batches(1, 64, K, seed=8600)[0].to(dev)
    feeds = [{'a': x, 'b': (other if i == split_at else x)} for i, x in enumerate(xs)]
    shared, followed = _subset_run(dev, Ws, feeds, hessian_defer=4)
    assert followed == {'a': 'a', 'b': 'b'}
    separate, _ = _subset_run(dev, Ws, feeds, hessian_defer=4, auto_share=False)
    for n in Ws:
        for a, b in zip(shared[n], separate[n]):
            assert torch.equal(a, b), n
    # same memory, same shape, but modified in place between the two hooks: the device comparison reports it
    from lightcompress_amd import _lib as L
    gp = make_gptq(actorder=True)
    layers = {n: Layer(w.to(dev)) for n, w in Ws.items()}
    gp.subset_init({'layers': layers})
    x = xs[0].clone()
    gp.add_batch(layers['a'], 'a', x, None)
    x.mul_(2)
    gp.add_batch(layers['b'], 'b', x, None)
    with pytest.raises(L.LcqError, match='written in place'):
        gp.hessian('b')


@pytest.mark.parametrize('defer', [1, 'auto'])
@pytest.mark.parametrize('K,T,nb', [(512, 100, 5), (1000, 33, 3), (2048, 512, 2)])
def test_hessian_from_fp32_activations(dev, K, T, nb, defer):
    """add_batch upcasts with .float() (gptq.py:289), so fp32 activations count in full precision: the kernel takes
    them as two bf16 halves (four exact products) and must stay within 1e-5 of the fp64 closed form and of the fp32
    oracle - rounding the activations to bf16 first would not."""
    g = gen(8700 + K)
    sigma = torch.exp(torch.randn(K, generator=g))
    batches = [torch.randn(T, K, generator=g) * sigma for _ in range(nb)]
    gp = make_gptq(hessian_defer=defer)
    layer = Layer(torch.zeros(8, K, device=dev))
    gp.layers_cache['l'] = {}
    gp.layer_init(layer, 'l')
    Ho, n = torch.zeros(K, K), 0
    for b in batches:
        gp.add_batch(layer, 'l', b.unsqueeze(0).to(dev), None)
        n = G.add_batch(Ho, n, b.unsqueeze(0))
    H = gp.hessian('l').cpu()
    ref64 = G.hessian_closed_form(batches)
    scale = float(ref64.abs().max())
    assert float((H.double() - ref64).abs().max()) / scale < 1e-5
    assert float((H - Ho).abs().max()) / scale < 1e-5
    assert float((H.double() - ref64).norm() / ref64.norm()) < 1e-5
    assert torch.equal(H, H.t())
    # the bf16-rounded activations are a different matrix at this tolerance
    rounded = G.hessian_closed_form([b.bfloat16() for b in batches])
    assert float((rounded - ref64).abs().max()) / scale > 1e-4


@pytest.mark.parametrize('gran,n_out', [('per_group', 100), ('per_channel', 37), ('per_group', 128)])
def test_owq_layer(dev, gran, n_out):
    """special.owq: outlier-last column order, loop and group ranges over the non-outlier columns only, outlier
    columns written back with the loop's compensation, per_channel qparams from the permuted non-outlier weight,
    w_qdq restoring the kept columns - against the fp32 oracle."""
    R, K, g, nb, T = 64, 768, 128, 6, 200
    batches = calib_batches(nb, T, K, seed=7100)
    W0 = (torch.randn(R, K, generator=gen(7101)) * 0.02).bfloat16()
    spec = Q.IntSpec(4, False, gran, group_size=g)
    Ho = torch.zeros(K, K); n = 0
    for b in batches:
        n = G.add_batch(Ho, n, b.unsqueeze(0))
    ref = G.gptq_layer(W0, Ho, spec, owq_n_out=n_out)
    wcfg = dict(bit=4, symmetric=False, granularity=gran)
    if gran == 'per_group':
        wcfg['group_size'] = g
    gp = make_gptq(weight=wcfg, owq=True, n_outs=[5, n_out], actorder=True)
    assert gp.actorder is False and gp.need_perm
    gp.set_block_linears(['other', 'fc'])
    layer = Layer(W0.to(dev))
    gp.subset_init({'layers': {'fc': layer}})
    if gran == 'per_channel':
        gp.collect_layer_qparams(layer)
    for b in batches:
        gp.add_batch(layer, 'fc', b.unsqueeze(0).to(dev), None)
    gp.layer_transform(layer, 'fc')
    nq = K - n_out
    perm = layer.buf_perm.cpu()
    assert int(layer.buf_n_nonout) == nq and torch.equal(torch.sort(perm[:nq]).values, perm[:nq])
    d = torch.diag(Ho)
    assert float(d[perm[nq:]].min()) >= float(d[perm[:nq]].max()) * (1 - 1e-5)
    Wq = layer.weight.data.cpu()
    tmp = Wq[:, perm]
    if torch.equal(perm, ref['perm']):
        if gran == 'per_group':
            s, z = layer.buf_scales.cpu(), layer.buf_zeros.cpu()
            assert s.shape == ref['scales'].shape
            codes = G.codes_from(tmp[:, :nq], s, z, spec)
            codes_o = G.codes_from(ref['tmp_perm'][:, :nq], ref['scales'], ref['zeros'], spec)
        else:
            s, z = layer.buf_scales.cpu().float(), layer.buf_zeros.cpu().float()
            so, zo = ref['static_qparams']
            assert torch.allclose(s, so, rtol=1e-6) and torch.equal(z, zo)
            codes = Q.int_quant(spec, tmp[:, :nq], s, z, spec.qmax, spec.qmin)
            codes_o = Q.int_quant(spec, ref['tmp_perm'][:, :nq], so, zo, spec.qmax, spec.qmin)
        assert float((codes == codes_o).float().mean()) >= 0.999
        keep, keep_o = tmp[:, nq:], ref['weight'][:, perm][:, nq:]
        assert float((keep - keep_o).abs().max()) <= 1e-3 * float(keep_o.abs().max())
    assert abs(float(gp.last_error) - ref['loss']) <= 0.01 * ref['loss']
    if gran == 'per_channel':
        layer.buf_qmax, layer.buf_qmin = gp.wquantizer.qmax, gp.wquantizer.qmin
        fq = gp.w_qdq(layer, gp.wquantizer).cpu().float()
        assert torch.equal(fq[:, perm][:, nq:], tmp[:, nq:].bfloat16().float())
        want = Q.int_fake_quant_static(spec, tmp, s, z, spec.qmax, spec.qmin)[:, :nq].bfloat16().float()
        assert torch.equal(fq[:, perm][:, :nq], want)


def test_split_gemm_has_fp32_accuracy(dev):
    """The large fp32 products run on the bf16 matrix pipe with three-way split operands (lcq_set_gemm_split, default
    on).  Against an fp64 product: the split path is as close as the fp32 pipe, for both operand layouts ([k][n] through
    lcq_gptq_trailing, [n][k] inside the Cholesky chain), for interior and ragged tiles; and the chain's factor agrees
    between the two settings to fp32 rounding."""
    import ctypes
    from lightcompress_amd import _lib as L
    lib = L.lib()
    lib.lcq_set_gemm_split.restype = ctypes.c_int
    g = gen(9100)
    R, K = 2304, 2400                                   # 18 x 17 tiles, the last column of tiles ragged
    W0 = (torch.randn(R, K, generator=g) * 0.02).to(dev)
    U = torch.triu(torch.randn(K, K, generator=g) * 0.05).to(dev).contiguous()
    Err = (torch.randn(R, 384, generator=g) * torch.exp(torch.randn(384, generator=g))).to(dev).contiguous()
    k1, k2, j1, j2 = 0, 384, 384, K
    want = W0.double()
    want[:, j1:j2] -= Err.double() @ U.double()[k1:k2, j1:j2]
    errs = {}
    try:
        for mode in (0, 1):
            lib.lcq_set_gemm_split(L.i32(mode))
            W = W0.clone()
            L.check(lib.lcq_gptq_trailing(L.ptr(W), L.ptr(Err), L.i64(384), L.ptr(U), L.i64(R), L.i64(K), L.i64(k1), L.i64(k2),
                                          L.i64(j1), L.i64(j2), L.stream()), 'trailing')
            assert torch.equal(W[:, :j1], W0[:, :j1])
            errs[mode] = float((W.double() - want).abs().max() / want.abs().max())
        assert errs[1] <= max(2 * errs[0], 2e-7) and errs[0] < 5e-6, errs
        # the chain: same factor either way, same distance from the fp64 identity
        Kc = 1536
        X = torch.randn(2 * Kc, Kc, generator=g) * torch.exp(0.7 * torch.randn(Kc, generator=g))
        H0 = (X.t() @ X / Kc).to(dev)
        Hd = H0.double() + 0.01 * torch.diag(H0).double().mean() * torch.eye(Kc, device=dev, dtype=torch.float64)
        ws_bytes = lib.lcq_chol_inv_upper_workspace_bytes(L.i64(Kc))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        status = torch.zeros(1, dtype=torch.int32, device=dev)
        Us, res = {}, {}
        for mode in (0, 1):
            lib.lcq_set_gemm_split(L.i32(mode))
            H = H0.clone()
            L.check(lib.lcq_chol_inv_upper(L.ptr(H), L.i64(Kc), None, L.f32(0.01), None, L.i64(0), L.ptr(H), L.ptr(ws),
                                           L.i64(ws_bytes), L.ptr(status), L.stream()), 'chain')
            assert int(status.item()) == 0
            Us[mode] = H.double()
            res[mode] = float((Us[mode].t() @ Us[mode] @ Hd - torch.eye(Kc, device=dev, dtype=torch.float64)).abs().max())
        assert res[1] <= max(2 * res[0], 1e-5) and res[0] < 2e-5, res
        assert float((Us[0] - Us[1]).abs().max() / Us[0].abs().max()) < 1e-5
    finally:
        lib.lcq_set_gemm_split(L.i32(1))


@pytest.mark.parametrize('sym', [False, True])
def test_groups_view_and_ready(dev, sym):
    """`groups` is the reference's list of per-group dicts (gptq.py:358-366, 385-395): entry i holds the [R, 1]
    scale / zero of group i, and stacking them the way update_model_qparams does (:397-409) gives the layer's
    buffers.  `ready` (gptq.py:473-477) is False until something fills `qparams['scale']`."""
    R, K, g = 24, 384, 128
    gp = make_gptq(weight=dict(bit=4, symmetric=sym, granularity='per_group', group_size=g))
    layer = linear((torch.randn(R, K, generator=gen(77)) * 0.02).bfloat16().to(dev))
    gp.collect_layer_qparams(layer)
    gp.layer_init(layer, 'l')
    for b in calib_batches(3, 96, K, seed=78):
        gp.add_batch(layer, 'l', b.bfloat16().to(dev))
    gp.layer_transform(layer, 'l')
    assert gp.ready() is False
    groups = gp.groups
    assert len(groups) == K // g
    for d in groups:
        assert d['scale'].shape == (R, 1) and d['qmax'] == gp.wquantizer.qmax and d['qmin'] == gp.wquantizer.qmin
    stacked = torch.stack([d['scale'] for d in groups], dim=1).reshape(-1, 1)
    assert torch.equal(stacked, layer.buf_scales)
    if sym:
        assert all(float(d['zero']) == 0.0 for d in groups)
    else:
        assert torch.equal(torch.stack([d['zero'] for d in groups], dim=1).reshape(-1, 1), layer.buf_zeros)
    gp.qparams['scale'] = layer.buf_scales
    assert bool(gp.ready()) == bool(torch.all(layer.buf_scales != 0))


@pytest.mark.parametrize('sym', [False, True])
def test_qparam_bookkeeping_methods_by_name(dev, sym):
    """split_qparams / merge_qparams / search_group_qparams / search_column_qparams / search_layer_qparams /
    update_model_qparams (gptq.py:332-409) keep the reference's names and meaning on top of the [R, G] tables."""
    R, K, g = 24, 384, 128
    gp = make_gptq(weight=dict(bit=4, symmetric=sym, granularity='per_group', group_size=g))
    w = (torch.randn(R, K, generator=gen(81)) * 0.02).bfloat16()
    layer = linear(w.to(dev))
    gp.collect_layer_qparams(layer)
    gp.columns = K
    spec = Q.IntSpec(4, sym, 'per_group', group_size=g)
    _, os_, oz, _, _ = Q.int_tensor_qparams(spec, w)                 # [R * G, 1], groups of a row side by side
    parts = gp.split_qparams(layer.buf_scales)
    assert len(parts) == K // g and all(p.shape == (R, 1) for p in parts)
    for gi, p in enumerate(parts):
        assert_bit_equal(p, os_.reshape(R, -1)[:, gi:gi + 1], f'scales of group {gi}')
    assert torch.equal(gp.merge_qparams(parts), layer.buf_scales) and gp.merge_qparams(3) == 3
    gp.search_group_qparams(layer)
    groups = gp.groups
    assert len(groups) == K // g
    for gi, d in enumerate(groups):
        assert torch.equal(d['scale'], parts[gi].float())
        if not sym:
            assert torch.equal(d['zero'], gp.split_qparams(layer.buf_zeros)[gi].float())
    # new parameters for the middle group from other values, as the loop finds them on the compensated weights
    w2 = (torch.randn(R, g, generator=gen(82)) * 0.05).float()
    gp.search_column_qparams(w2.to(dev), g)
    _, s2, z2, _, _ = Q.int_tensor_qparams(spec, w2)
    assert_bit_equal(gp.qparams['scale'], s2, 'current scale')
    assert torch.equal(gp.groups[1]['scale'].cpu(), s2) and torch.equal(gp.groups[0]['scale'], parts[0].float())
    if not sym:
        assert torch.equal(gp.groups[1]['zero'].cpu(), z2)
    gp.update_model_qparams(layer)
    want = os_.reshape(R, -1).float().clone()
    want[:, 1] = s2.reshape(-1)
    assert torch.equal(layer.buf_scales.cpu(), want.reshape(-1, 1))
    # per_channel: the buffers become the current qparams
    gc = make_gptq(weight=dict(bit=4, symmetric=sym, granularity='per_channel'))
    lc = linear(w.to(dev))
    gc.collect_layer_qparams(lc)
    gc.search_layer_qparams(lc)
    assert gc.qparams['scale'] is lc.buf_scales and bool(gc.ready())


def test_indefinite_hessian_raises_unless_the_check_is_off(dev):
    """gptq.py:172: torch.linalg.cholesky raises on a matrix that is not positive-definite; here the chain's status
    word is read before the weights are written back.  `check_positive_definite: False` skips the read."""
    R, K = 16, 256
    for check in (True, False):
        gp = make_gptq(check_positive_definite=check, weight=dict(bit=4, symmetric=False, granularity='per_group', group_size=128))
        W0 = (torch.randn(R, K, generator=gen(79)) * 0.02).bfloat16().to(dev)
        layer = linear(W0.clone())
        gp.collect_layer_qparams(layer)
        gp.layer_init(layer, 'l')
        gp.add_batch(layer, 'l', torch.randn(64, K, generator=gen(80)).bfloat16().to(dev))
        H = gp.hessian('l')
        H.neg_()                                         # negative definite: the first pivot fails
        if check:
            with pytest.raises(torch.linalg.LinAlgError):
                gp.layer_transform(layer, 'l')
            assert torch.equal(layer.weight.data, W0)    # nothing was written back
        else:
            gp.layer_transform(layer, 'l')


@pytest.mark.parametrize('K', [768, 1536, 2304, 3072, 5120, 6144])
def test_hessian_auto_settings_between_the_tuned_widths(dev, K):
    """`hessian_defer: auto` / `hessian_slices: auto` are tables tuned at a handful of widths; whatever they pick at
    the widths in between (folds of 16 / 8 calls, 1 - 8 token shares, with or without the split last round), add_batch
    over a number of calls that leaves a partly filled staging buffer ends at the closed form."""
    T, nb = 96, 21
    gp = make_gptq()
    layer = Layer(torch.zeros(8, K, device=dev))
    gp.layers_cache['l'] = {}
    gp.layer_init(layer, 'l')
    g = torch.Generator(device=dev)
    g.manual_seed(K)
    xs = [(torch.randn(1, T, K, device=dev, generator=g) * (1 + i % 3)).bfloat16() for i in range(nb)]
    for x in xs:
        gp.add_batch(layer, 'l', x, None)
    H = gp.hessian('l')
    ref = torch.zeros(K, K, dtype=torch.float64, device=dev)
    for x in xs:
        xd = x[0].double()
        ref.addmm_(xd.t(), xd)
    ref *= 2.0 / nb
    assert gp.layers_cache['l']['nsamples'] == nb
    assert float((H.double() - ref).abs().max() / ref.abs().max()) < 1e-5
    assert torch.equal(H, H.t())


def test_switch_combinations_give_one_result(dev):
    """The `special` switches that only rearrange work (auto_share, fuse_loops, block_factor, chain_overlap,
    hessian_defer, hessian_slices, share_verify) in all 128 combinations on a subset of three Linears with a common
    input: every combination reproduces the plain one (one Hessian per Linear, one launch per call, the reference's
    chain, one loop per Linear) to >= 99.9 % of the codes and 1e-3 of the loss; combinations that differ only in
    switches with bit-identical semantics (sharing, verification, overlap, stacking) agree bit for bit."""
    import itertools
    K = 512
    Ws = {'q': (torch.randn(96, K, generator=gen(21)) * 0.02).bfloat16(), 'k': (torch.randn(32, K, generator=gen(22)) * 0.02).bfloat16(),
          'v': (torch.randn(48, K, generator=gen(23)) * 0.02).bfloat16()}
    xs = [b.to(dev) for b in calib_batches(7, 128, K, seed=9900)]
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)

    def run(**special):
        gp = make_gptq(actorder=True, **special)
        layers = {n: Layer(w.to(dev)) for n, w in Ws.items()}
        gp.subset_init({'layers': layers})
        for x in xs:
            for n in Ws:
                gp.add_batch(layers[n], n, x.data, None)
        gp.subset_transform({'layers': layers})
        torch.cuda.synchronize()
        return {n: (layers[n].weight.data.cpu(), layers[n].buf_scales.cpu(), layers[n].buf_zeros.cpu(), layers[n].buf_perm.cpu(),
                    float(gp.last_errors[n])) for n in Ws}

    base = run(auto_share=False, fuse_loops=False, block_factor=False, chain_overlap=False, hessian_defer=1, hessian_slices=1)
    seen = {}
    for share, fuse, bf, ov, defer, slices, verify in itertools.product((True, False), (True, False), (True, False), (True, False),
                                                                        (1, 'auto'), (1, 'auto'), (True, False)):
        got = run(auto_share=share, fuse_loops=fuse, block_factor=bf, chain_overlap=ov, hessian_defer=defer, hessian_slices=slices,
                  share_verify=verify)
        for n in Ws:
            w, s_, z_, perm, loss = got[n]
            bw, bs_, bz_, bperm, bloss = base[n]
            assert torch.equal(perm, bperm), (n, share, fuse, bf, ov, defer, slices)
            codes = G.codes_from(w[:, perm], s_, z_, spec)
            bcodes = G.codes_from(bw[:, perm], bs_, bz_, spec)
            assert float((codes == bcodes).float().mean()) >= 0.999, (n, share, fuse, bf, ov, defer, slices)
            assert abs(loss - bloss) <= 1e-3 * bloss
        # the arithmetic depends on the factor (bf) and on how the Hessian was summed (defer, slices) only
        key = (bf, defer, slices)
        if key in seen:
            for n in Ws:
                for a, b in zip(got[n][:4], seen[key][n][:4]):
                    assert torch.equal(a, b), (n, share, fuse, bf, ov, defer, slices, verify)
        else:
            seen[key] = got


@pytest.mark.parametrize('R', [6144, 6151, 9000])
@pytest.mark.parametrize('mode', ['searched', 'searched_sym', 'static', 'block_factor'])
def test_block_kernel_workgroup_shapes_agree(dev, R, mode):
    """lcq_gptq_block takes 32 rows per workgroup from 6144 rows on and 16 below (the kernel every small case above
    runs against the oracle): rows do not interact, so the two shapes must agree bit for bit on every output, also
    with a ragged last workgroup."""
    from lightcompress_amd import _lib as L
    lib = L.lib()
    K, i1, g = 512, 256, 64
    G = K // g
    U = (torch.triu(torch.randn(K, K, generator=gen(1)) * 0.02) + torch.eye(K) * 1.5).to(dev)
    W0 = (torch.randn(R, K, generator=gen(2)) * 0.05).to(dev)
    outs = []
    for extra in (L.FLAG_ROWS16, 0):
        flags = extra | (L.FLAG_SYM if mode == 'searched_sym' else 0) | (L.FLAG_STATIC if mode == 'static' else 0)
        W = W0.clone()
        W[:, i1:] += 0.01                                   # what earlier blocks' updates would have left
        tmp, Lo = torch.zeros_like(W), torch.zeros_like(W)
        Err = torch.zeros(R, 128, device=dev)
        sc = (torch.rand(R, G, generator=gen(3)) * 0.01 + 0.005).to(dev)
        ze = torch.randint(0, 16, (R, G), generator=gen(4)).float().to(dev)
        L.check(lib.lcq_gptq_block(L.ptr(W), L.ptr(tmp), L.ptr(Lo), L.ptr(Err), L.i64(128), L.ptr(U),
                                   L.ptr(W0) if mode == 'block_factor' else None, L.i64(R), L.i64(K), L.i64(K), L.i64(i1),
                                   L.i32(128), L.i32(g), L.f32(0.0), L.f32(15.0), L.i32(flags), L.ptr(sc), L.ptr(ze), None,
                                   L.i64(G), L.stream()), 'lcq_gptq_block')
        torch.cuda.synchronize()
        outs.append((tmp, Lo, Err, sc, ze))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    assert float(outs[0][1].sum()) > 0 and bool(torch.isfinite(outs[0][2]).all())
