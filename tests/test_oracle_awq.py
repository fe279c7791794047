"""Pins the AWQ oracle without a GPU: ratio 0 is plain RTN, the scale
normalisation, and a brute-force fp64 grid search on a tiny SwiGLU MLP."""
import pytest
import torch

from oracle import awq_ref as A, quant_ref as Q
from tests.helpers import gen, weight_like


def swiglu(x, w):
    h = torch.nn.functional.silu(x @ w['gate'].t()) * (x @ w['up'].t())
    return h @ w['down'].t() if 'down' in w else h


def tiny_case(dtype, seed=0, T=64, K=256, I=384):
    g = gen(seed)
    sigma = torch.exp(torch.randn(K, generator=g))
    x = (torch.randn(2, T, K, generator=g) * sigma).to(dtype)
    w = {'gate': (torch.randn(I, K, generator=g) * 0.02).to(dtype), 'up': (torch.randn(I, K, generator=g) * 0.02).to(dtype)}
    down = (torch.randn(K, I, generator=g) * 0.02).to(dtype)
    return x, w, down


def test_ratio_zero_is_plain_rtn_and_scales_are_normalised():
    x, w, down = tiny_case(torch.float32)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    s0 = A.get_scales(x, None, 0.0)
    assert torch.equal(s0, torch.ones_like(s0))
    assert torch.equal(A.scale_and_fake_quant(w['gate'], s0, spec), Q.int_fake_quant_dynamic(spec, w['gate']))
    assert torch.equal(A.scaling_input(x, s0), x)
    for r in (0.25, 0.5, 0.95):
        s = A.get_scales(x, None, r)
        assert abs(float(s.max() * s.min()) - 1.0) < 1e-5
        # scales follow the activation magnitude: the ordering of channels is that of mean|x|
        assert torch.equal(torch.argsort(s), torch.argsort(A.act_scale(x).pow(r).clamp(min=1e-4)))
    # closed form of the activation statistic
    assert torch.allclose(A.act_scale(x), x.abs().reshape(-1, 256).sum(0) / 128, rtol=1e-6)


def test_weight_scale_closed_form():
    _, w, _ = tiny_case(torch.float32, seed=1)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    ws = A.weight_scale([w['gate'], w['up']], spec)
    ref = 0
    for m in (w['gate'], w['up']):
        a = m.abs().reshape(m.shape[0], -1, 128)
        ref = ref + (a / a.amax(-1, keepdim=True)).reshape(m.shape).mean(0)
    assert torch.allclose(ws, ref / 2, rtol=1e-6)
    assert float(ws.max()) <= 1.0


def test_grid_search_matches_bruteforce_fp64():
    x, w, down = tiny_case(torch.float64, seed=2)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    fwd = lambda xx, ww: swiglu(xx, dict(ww, down=down))
    best, losses = A.search_scale(w, x, fwd, spec)
    assert len(losses) == 20
    # independent evaluation of every grid point
    org = fwd(x, w)
    xm = x.abs().reshape(-1, x.shape[-1]).mean(0)
    brute = []
    for n in range(20):
        s = xm.pow(n / 20).clamp(min=1e-4)
        s = s / (s.max() * s.min()).sqrt()
        wq = {k: Q.int_fake_quant_dynamic(spec, v * s) for k, v in w.items()}
        brute.append(float(((org - fwd(x / s, wq)) ** 2).mean()))
    assert torch.allclose(torch.tensor(losses), torch.tensor(brute), rtol=1e-9)
    k = min(range(20), key=lambda i: brute[i])
    s = xm.pow(k / 20).clamp(min=1e-4)
    assert torch.allclose(best, s / (s.max() * s.min()).sqrt())
    # activation-aware scaling beats plain RTN on outlier channels
    assert min(brute) < brute[0]


# ---- AutoClipper (auto_clip.py:83-191) ------------------------------------------------------------
def _clip_objective_fp64(spec, w, x, n_grid=20, n_steps=10, clip_sym=False):
    """The objective in plain fp64 math, written from its definition: for every (row, group, shrink step) the
    mean over tokens of (x_g . (fq(clamp(w_g)) - w_g))^2, with fq evaluated by the oracle quantizer on the clamped
    bf16 group."""
    R, K = w.shape
    g = spec.group_size
    G = K // g
    wg = w.reshape(R, G, g)
    xg = x.reshape(-1, G, g).double()
    out = torch.zeros(R, G, n_steps, dtype=torch.float64)
    for s in range(n_steps):
        hi = (wg.abs().amax(-1, keepdim=True) if clip_sym else wg.amax(-1, keepdim=True)) * (1 - s / n_grid)
        lo = -hi if clip_sym else wg.amin(-1, keepdim=True) * (1 - s / n_grid)
        cw = torch.clamp(wg, lo, hi)
        qw = Q.int_fake_quant_dynamic(spec, cw.reshape(R, K)).reshape(R, G, g)
        d = (qw.double() - wg.double())                                  # [R, G, g]
        e = torch.einsum('tgj,rgj->rtg', xg, d)                          # [R, T, G]
        out[:, :, s] = e.pow(2).mean(dim=1)
    return out


@pytest.mark.parametrize('clip_sym', [False, True])
def test_auto_clip_oracle_tracks_the_fp64_objective(clip_sym):
    R, K, T = 64, 256, 96
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    w = weight_like(R, K, seed=61, dtype=torch.bfloat16)
    x = (torch.randn(T, K, generator=gen(62)) * torch.exp(torch.randn(K, generator=gen(63)))).bfloat16()
    bmax, bmin, errs = A.auto_clip_layer(spec, w, [x.clone()], clip_sym=clip_sym, n_sample_token=T)
    assert bmax.shape == bmin.shape == (R, 2, 1) and errs.shape == (R, 2, 10)
    ref = _clip_objective_fp64(spec, w, x, clip_sym=clip_sym)
    # the bf16 chain (products, sums, difference, square, mean all rounded to 8 bits) follows the exact objective
    rel = (errs.double() - ref).abs() / ref.clamp(min=1e-30)
    assert float(rel.median()) < 0.02 and float(rel.quantile(0.99)) < 0.25
    # the selection is the first minimum of the rounded errors, and the ranges are the shrunken originals
    pick = torch.zeros(R, 2, dtype=torch.long)
    best = torch.full((R, 2), 1e9).bfloat16()
    for s in range(10):
        better = errs[:, :, s] < best
        best[better] = errs[:, :, s][better]
        pick[better] = s
    wg = w.reshape(R, 2, 128)
    org_max = wg.abs().amax(-1) if clip_sym else wg.amax(-1)
    want_max = torch.stack([org_max * (1 - s / 20) for s in range(10)], dim=-1).gather(-1, pick.unsqueeze(-1))
    assert torch.equal(bmax, want_max)
    if clip_sym:
        assert torch.equal(bmin, -bmax)
    # agreement with the exact argmin wherever the exact objective separates the best two steps by > 5 %
    top2 = ref.topk(2, dim=-1, largest=False).values
    clear = top2[..., 1] > 1.05 * top2[..., 0]
    assert float(clear.float().mean()) > 0.3
    assert bool((pick[clear] == ref.argmin(-1)[clear]).all())


def test_auto_clip_oracle_known_optima():
    """An outlier weight whose input channel is silent costs nothing to clip: the search shrinks deep.  When that channel carries all the signal, clipping only hurts: step 0 (no clipping) wins."""
    R, K, T = 64, 128, 64
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    w = (torch.randn(R, K, generator=gen(71)) * 0.02)
    w[:, 5] = 1.0                                      # outlier column, 50 sigma
    w[:, 9] = -1.0
    w = w.bfloat16()
    x = torch.randn(T, K, generator=gen(72))
    x_silent = x.clone(); x_silent[:, 5] = 0; x_silent[:, 9] = 0
    bmax, bmin, errs = A.auto_clip_layer(spec, w, [x_silent.bfloat16()], n_sample_token=T)
    assert float((bmax.flatten().float() / w.float().amax(1)).mean()) < 0.7          # deep steps on average
    assert float(errs[:, 0, 9].float().mean()) < 0.9 * float(errs[:, 0, 0].float().mean())
    x_loud = torch.zeros(T, K); x_loud[:, 5] = x[:, 5]; x_loud[:, 9] = x[:, 9]
    bmax, bmin, errs = A.auto_clip_layer(spec, w, [x_loud.bfloat16()], n_sample_token=T)
    assert bool((bmax.flatten() == w.amax(1)).all()) and bool((bmin.flatten() == w.amin(1)).all())
    # apply_clip: the weight is clamped group-wise into the found range
    cl = A.apply_clip_v1(w, bmin, bmax)
    assert torch.equal(cl, w)


def test_auto_clip_oracle_v2_is_the_range_scaled_quantizer():
    """clip_version v2 (auto_clip.py:263-272): sigmoid(logit(r)) = r, so the learnable range is the shrunken min/max
    range and the weight is quantized UNclamped against it (the code clamp cuts the tails).  Pinned in fp32 by that
    closed form written without logit/sigmoid; step 0 (logit(1) = inf, sigmoid = 1) is plain min/max fake quant; and
    the factors of get_clip_factor map back to the found range."""
    R, K, T = 64, 256, 48
    w = weight_like(R, K, seed=81)
    x = torch.randn(T, K, generator=gen(82)) * torch.exp(0.5 * torch.randn(K, generator=gen(83)))
    for spec, clip_sym in [(Q.IntSpec(4, False, 'per_channel'), False), (Q.IntSpec(8, True, 'per_channel'), True),
                           (Q.IntSpec(4, False, 'per_group', group_size=128), False)]:
        gs = spec.group_size if spec.granularity == 'per_group' else K
        G = K // gs
        bmax, bmin, errs = A.auto_clip_layer(spec, w, [x.clone()], clip_sym=clip_sym, n_sample_token=T, clip_version='v2')
        assert bmax.shape == (R, G, 1) and errs.shape == (R, G, 10)
        wg, xg = w.reshape(R, G, gs), x.reshape(T, G, gs)
        org = torch.einsum('tgj,rgj->rtg', xg.double(), wg.double())
        hi0 = wg.abs().amax(-1, keepdim=True) if clip_sym else wg.amax(-1, keepdim=True)
        lo0 = wg.amin(-1, keepdim=True)
        want = torch.zeros(R, G, 10, dtype=torch.float64)
        for s in range(10):
            hi = hi0 * (1 - s / 20)
            lo = -hi if clip_sym else lo0 * (1 - s / 20)
            if spec.symmetric:                                      # get_learnable_range, sym: +-factor * max(|min|, |max|)
                amax = torch.max(wg.amax(-1, keepdim=True).abs(), lo0.abs()).clamp(min=1e-5)
                hi = (hi / hi0) * amax
                lo = -hi
            sc, z, qmax, qmin = Q.int_qparams(spec, lo, hi)
            q = Q.int_quant_dequant(spec, wg, sc, z, qmax, qmin)
            want[:, :, s] = (torch.einsum('tgj,rgj->rtg', xg.double(), q.double()) - org).pow(2).mean(1)
        rel = (errs.double() - want).abs() / want.clamp(min=1e-30)
        assert float(rel.median()) < 1e-3 and float(rel.quantile(0.99)) < 0.05, (float(rel.median()), float(rel.max()))
        # step 0 is the plain fake quant of the unclipped weight
        e0 = (torch.einsum('tgj,rgj->rtg', xg.double(), Q.int_fake_quant_dynamic(spec, w).reshape(R, G, gs).double()) - org).pow(2).mean(1)
        if not clip_sym or spec.symmetric:
            assert torch.allclose(errs[:, :, 0].double(), e0, rtol=1e-3, atol=1e-12)
        # the stored factors give the found range back through the learnable range
        up, low = A.clip_factor(spec, w, bmin, bmax, clip_sym)
        lo_l, hi_l = A.learnable_range(spec, Q.reshape_rows(spec, w), low, up)
        if spec.symmetric == clip_sym:
            assert torch.allclose(hi_l.reshape(bmax.shape), bmax, rtol=1e-5)
            if not clip_sym:
                assert torch.allclose(lo_l.reshape(bmin.shape), bmin, rtol=1e-5)


def test_auto_clip_oracle_with_activation_quantization():
    """w_only=False: the activations are fake-quantized as [1, T, G, gs], i.e. one range per token and group
    (per_token reshapes nothing, the range reduces the last axis).  Pinned by that per-(token, group) closed form and
    by the 16-bit limit in which activation quantization is the identity."""
    R, K, T = 64, 256, 32
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    w = weight_like(R, K, seed=91)
    x = torch.randn(T, K, generator=gen(92))
    a8 = Q.IntSpec(8, True, 'per_token')
    qx = Q.int_fake_quant_dynamic(a8, x.reshape(1, T, 2, 128))
    rows = x.reshape(T * 2, 128)
    sc = rows.abs().amax(-1, keepdim=True).clamp(min=1e-5) / 127
    assert torch.equal(qx.reshape(T * 2, 128), torch.clamp(torch.round(rows / sc), -128, 127) * sc)
    _, _, e_w = A.auto_clip_layer(spec, w, [x.clone()], n_sample_token=T)
    _, _, e_a16 = A.auto_clip_layer(spec, w, [x.clone()], n_sample_token=T, aspec=Q.IntSpec(16, True, 'per_token'))
    _, _, e_a8 = A.auto_clip_layer(spec, w, [x.clone()], n_sample_token=T, aspec=a8)
    assert torch.allclose(e_a16, e_w, rtol=2e-3)
    # the 8-bit error is the objective evaluated with qx on the quantized side only
    wg = w.reshape(R, 2, 128)
    org = torch.einsum('tgj,rgj->rtg', x.reshape(T, 2, 128).double(), wg.double())
    q0 = Q.int_fake_quant_dynamic(spec, w).reshape(R, 2, 128)
    want0 = (torch.einsum('tgj,rgj->rtg', qx.reshape(T, 2, 128).double(), q0.double()) - org).pow(2).mean(1)
    assert torch.allclose(e_a8[:, :, 0].double(), want0, rtol=1e-3)


def test_gqa_search_reduces_to_the_plain_search_and_repeats_per_group():
    """is_gqa (awq.py:88-93, 104-105; base_blockwise_quantization.py:614-618).
    * The repeated vector indexes the key/value channel of every query channel: column c of o_proj belongs to query
      head c // head_dim, which shares key/value head (c // head_dim) // groups (written out as a loop here).
    * With one query head per key/value head and an identity v_proj the GQA search is the plain v2 search."""
    kvh, hd, groups = 3, 4, 2
    s = torch.arange(kvh * hd, dtype=torch.float32) + 1
    rep = A.repeat_gqa(s, kvh, hd, groups)
    want = [float(s[((c // hd) // groups) * hd + c % hd]) for c in range(kvh * groups * hd)]
    assert rep.tolist() == want

    x, w, down = tiny_case(torch.float32, seed=21, T=32, K=256, I=128)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    fwd = lambda xx, ww: xx @ ww['o'].t()
    weights = {'o': w['gate']}
    best, losses = A.search_scale(weights, x, fwd, spec)
    best_g, losses_g = A.search_scale(weights, x, fwd, spec, gqa=(lambda t: t, 4, 64, 1))
    assert losses == losses_g and torch.equal(best, best_g)
    # genuinely grouped: 2 key/value heads serve 4 query heads; the result has one entry per key/value channel and
    # the search still returns a minimum of its own losses
    v = torch.randn(128, 256, generator=gen(22)) * 0.05
    best_g, losses_g = A.search_scale(weights, x, fwd, spec, gqa=(lambda t: t @ v.t(), 2, 64, 2))
    assert best_g.shape == (128,) and abs(float(best_g.max() * best_g.min()) - 1) < 1e-5
    assert losses_g[0] == losses[0]                               # ratio 0: all-ones scales either way


def test_several_inputs_pick_by_the_first_input_and_return_the_mean_scales():
    """awq.py:245-248 tests `loss_mean < best_error` after EVERY input.  Losses are positive, so a partial sum after
    the second input can never beat the record its own first term set or failed to beat: the chosen grid point is the
    argmin of the first input's weighted loss; `best_scales` aliases `scales_mean`, which the in-place `+=` of the
    later inputs completes to the mean over all inputs.  Shown here on the statement-for-statement restatement."""
    dtype = torch.float32
    x0, w, down = tiny_case(dtype, seed=11, T=48)
    g = gen(12)
    x1 = (torch.randn(4, 48, 256, generator=g) * torch.exp(torch.randn(256, generator=g))).to(dtype)   # other statistics
    x2 = (torch.randn(2, 48, 256, generator=g) * 3).to(dtype)           # sample counts are multiples of the first's
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    fwd = lambda xx, ww: swiglu(xx, dict(ww, down=down))
    inputs = [x0, x1, x2]
    best, trace = A.search_scale_inputs(w, inputs, fwd, spec)
    first = [row[0] for row in trace]
    full = [row[-1] for row in trace]
    k = min(range(20), key=lambda i: first[i])
    n = sum(x.shape[0] for x in inputs)
    want = sum(x.shape[0] / n * A.get_scales(x, None, k / 20) for x in inputs)
    assert torch.allclose(best, want, rtol=1e-6)
    # the single-input search on the first tensor alone picks the same grid point
    _, losses0 = A.search_scale(w, x0, fwd, spec)
    assert min(range(20), key=lambda i: losses0[i]) == k
    # and the quirk is observable: the mean loss over all inputs prefers another point in this case
    assert all(f > a for f, a in zip(full, first))
    assert min(range(20), key=lambda i: full[i]) != k


def test_micro_batches_average_per_batch_statistics():
    """awq_bs: statistics, forward and loss run per micro-batch and are averaged (awq.py:74-85, 110-145); with equal
    micro-batches that is the statistic of the whole tensor up to rounding, so the search result is unchanged."""
    x, w, down = tiny_case(torch.float64, seed=13, T=32)
    x = torch.cat([x, x.flip(0) * 1.5])                       # 4 samples
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    fwd = lambda xx, ww: swiglu(xx, dict(ww, down=down))
    b_all, t_all = A.search_scale_inputs(w, [x], fwd, spec)
    b_two, t_two = A.search_scale_inputs(w, [x], fwd, spec, bs=2)
    assert torch.allclose(b_all, b_two, rtol=1e-12)
    # (scales that differ in the last bit move a few codes across a rounding boundary)
    assert all(abs(a[0] - b[0]) <= 1e-3 * abs(a[0]) for a, b in zip(t_all, t_two))
    # v1 divides by the weight statistic: ratio 0 gives 1 / w_max (normalised), not ones
    b_v1, _ = A.search_scale_inputs(w, [x], fwd, spec, version='v1', n_grid=1)
    wm = A.weight_scale(list(w.values()), spec)
    s = (1 / wm).clamp(min=1e-4)
    assert torch.allclose(b_v1, s / (s.max() * s.min()).sqrt(), rtol=1e-12)
