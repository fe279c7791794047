"""Pins the GPTQ oracle (Hessian, Cholesky chain, column loop) without a GPU:
closed forms, invariants, and an independent textbook recurrence in fp64."""
import numpy as np
import pytest
import scipy.linalg
import torch

from oracle import gptq_ref as G, quant_ref as Q
from tests.helpers import gen


def calib_batches(n, tokens, K, seed=1000, dtype=torch.bfloat16):
    sigma = torch.exp(torch.randn(K, generator=gen(seed - 1)))
    return [(torch.randn(tokens, K, generator=gen(seed + b)) * sigma).to(dtype) for b in range(n)]


def test_hessian_running_mean_equals_closed_form():
    K = 96
    batches = calib_batches(7, 50, K)
    H = torch.zeros(K, K)
    n = 0
    for b in batches:
        n = G.add_batch(H, n, b.unsqueeze(0))
    assert n == 7
    ref = G.hessian_closed_form(batches)                       # fp64
    assert float((H.double() - ref).abs().max() / ref.abs().max()) < 1e-6
    assert torch.equal(H, H.t())
    x = torch.cat(batches).double()
    assert torch.allclose(torch.diag(ref), (2.0 / 7) * (x * x).sum(0), rtol=1e-12)
    # a batched call counts its batch dimension, not its tokens (gptq.py:258, 283-286)
    H2 = torch.zeros(K, K)
    n2 = G.add_batch(H2, 0, torch.stack(batches[:4]))
    assert n2 == 4
    assert torch.allclose(H2.double(), G.hessian_closed_form(batches[:4]), rtol=1e-5, atol=1e-6 * float(ref.abs().max()))
    # chunking the token dimension does not change the sum
    H3 = torch.zeros(K, K)
    G.add_batch(H3, 0, torch.stack(batches[:4]), chunk_num=4)
    assert torch.allclose(H3, H2, rtol=1e-5, atol=1e-6 * float(ref.abs().max()))


def test_cholesky_chain_is_upper_factor_of_damped_inverse():
    K = 64
    H = G.hessian_closed_form(calib_batches(4, 80, K))
    H[:, 5] = 0; H[5, :] = 0                                    # a dead input channel
    W = torch.randn(8, K, generator=gen(3), dtype=torch.float64)
    perm = G.act_order(H)
    Wp, U, invperm = G.process_hessian_and_weights(W, H, 0.01, perm, dtype=torch.float64)
    assert torch.equal(torch.triu(U), U) and bool((torch.diag(U) > 0).all())
    Hd = H.clone(); Hd[5, 5] = 1
    Hd = Hd[perm][:, perm]
    Hd += 0.01 * torch.mean(torch.diag(Hd)) * torch.eye(K, dtype=torch.float64)
    assert float((U.t() @ U @ Hd - torch.eye(K, dtype=torch.float64)).abs().max()) < 1e-9
    ref = scipy.linalg.cholesky(np.linalg.inv(Hd.numpy()), lower=False)
    assert np.allclose(U.numpy(), ref, rtol=1e-9, atol=1e-12)
    assert torch.equal(Wp[:, invperm][:, 5], torch.zeros(8, dtype=torch.float64))       # dead column zeroed
    assert torch.equal(Wp[:, invperm][:, 6], W[:, 6])
    # the equivalent route  J H J = L L^T,  U = J L^-1 J  (what the GPU chain computes)
    J = torch.arange(K - 1, -1, -1)
    Lf = torch.linalg.cholesky(Hd[J][:, J])
    U2 = torch.linalg.inv(Lf)[J][:, J]
    assert float((U2 - U).abs().max() / U.abs().max()) < 1e-12


def _textbook_gptq(W, Hd, spec):
    """Original GPTQ/OBQ recurrence, no Cholesky: eliminate one column of the inverse at a time."""
    W = W.clone().double()
    K = W.shape[1]
    Hinv = torch.linalg.inv(Hd.double())
    Qw = torch.zeros_like(W)
    for i in range(K):
        if i % spec.group_size == 0:
            _, s, z, qmax, qmin = Q.int_tensor_qparams(spec, W[:, i:i + spec.group_size])
        w = W[:, i]
        q = Q.int_quant_dequant(spec, w.unsqueeze(1), s, z, qmax, qmin).squeeze(1)
        Qw[:, i] = q
        err = (w - q) / Hinv[i, i]
        W[:, i:] -= err.unsqueeze(1) * Hinv[i, i:].unsqueeze(0)
        # remove row/column i from the inverse (Gaussian elimination step)
        Hinv[i + 1:, i + 1:] -= torch.outer(Hinv[i + 1:, i], Hinv[i, i + 1:]) / Hinv[i, i]
    return Qw


@pytest.mark.parametrize('blocksize', [128, 64, 256])
def test_column_loop_matches_textbook_recurrence_and_loss_identity(blocksize):
    R, K, g = 4, 256, 128
    spec = Q.IntSpec(4, False, 'per_group', group_size=g)
    H = G.hessian_closed_form(calib_batches(6, 64, K, seed=2000))
    W0 = torch.randn(R, K, generator=gen(5), dtype=torch.float64) * 0.02
    W, U, _ = G.process_hessian_and_weights(W0, H, 0.01, None, dtype=torch.float64)
    Hd = H + 0.01 * torch.mean(torch.diag(H)) * torch.eye(K, dtype=torch.float64)
    tmp, Losses, groups = G.weight_transform(W, U, spec, blocksize=blocksize)
    assert len(groups) == K // g
    scales, zeros = G.merge_groups(groups)
    # dequantised result of the loop = quant_dequant(tmp) with the loop's qparams
    rows = tmp.reshape(-1, g)
    Qloop = Q.int_quant_dequant(spec, rows, scales, zeros, spec.qmax, spec.qmin).reshape(R, K)
    if g % blocksize == 0:
        # the lazy batch is an exact re-association of the textbook algorithm when every group starts
        # at a block start (otherwise the range is read from W, which misses the block-local
        # updates: reference quirk, gptq.py:216-222)
        Qt = _textbook_gptq(W0, Hd, spec)
        assert float((Qt - Qloop).abs().max()) < 1e-9
    # first processed column is untouched
    assert torch.equal(tmp[:, 0], W0[:, 0])
    # sum of the per-column losses equals the quadratic form of the total weight change
    D = W0 - Qloop
    assert abs(float(Losses.sum()) - 0.5 * float(torch.trace(D @ Hd @ D.t()))) < 1e-12 + 1e-9 * float(Losses.sum())


@pytest.mark.parametrize('g,static', [(128, False), (64, False), (32, False), (128, True)])
def test_loop_on_the_block_factor_is_the_reference_loop(g, static):
    """The chain that skips the triangular inverse hands the loop P (P[b,b] = U[b,b], P[p,b] = U^-1[p,b] U[b,b]) and
    every block passes (quantized - original) on instead of its errors.  In fp64 that loop gives the reference loop's
    compensated weights, losses and group parameters whenever a group lies inside one 128-column block, including
    groups that open in the middle of a block (whose ranges the reference reads from the partly updated W)."""
    R, K = 6, 640
    spec = Q.IntSpec(4, False, 'per_group', group_size=g)
    H = G.hessian_closed_form(calib_batches(6, 96, K, seed=2100 + g))
    W0 = torch.randn(R, K, generator=gen(6), dtype=torch.float64) * 0.02
    W, U, _ = G.process_hessian_and_weights(W0, H, 0.01, None, dtype=torch.float64)
    P = G.block_factor(U)
    assert torch.equal(torch.triu(P), P)
    for b in range(K // 128):
        assert torch.equal(P[128 * b:128 * b + 128, 128 * b:128 * b + 128], U[128 * b:128 * b + 128, 128 * b:128 * b + 128])
    sg = None
    if static:                                            # parameters given per group of the original order
        _, s_, z_, _, _ = Q.int_tensor_qparams(spec, W0.float())
        sg = (s_.reshape(R, K // g).double(), z_.reshape(R, K // g).double(), None)
    tmp, Losses, groups = G.weight_transform(W.clone(), U, spec, static_groups=sg)
    tmp_p, Losses_p, groups_p = G.weight_transform(W.clone(), P, spec, static_groups=sg, block_factor_W0=W.clone())
    assert float((tmp - tmp_p).abs().max()) < 1e-12
    assert float((Losses - Losses_p).abs().max()) < 1e-12 * max(1.0, float(Losses.abs().max()))
    assert len(groups) == len(groups_p) == (0 if static else K // g)
    for (s1, z1), (s2, z2) in zip(groups, groups_p):
        assert float((s1 - s2).abs().max()) < 1e-14 and torch.equal(z1, z2)
    # a group wider than a block is outside what P can reproduce: the ranges of its later columns differ
    if not static and g == 128:
        spec2 = Q.IntSpec(4, False, 'per_group', group_size=256)
        t1, _, _ = G.weight_transform(W.clone()[:, :512], U[:512, :512], spec2)
        t2, _, _ = G.weight_transform(W.clone()[:, :512], G.block_factor(U[:512, :512]), spec2, block_factor_W0=W.clone()[:, :512])
        assert float((t1 - t2).abs().max()) > 1e-9


def test_identity_hessian_reduces_to_rtn():
    R, K = 8, 256
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    W0 = torch.randn(R, K, generator=gen(6)) * 0.02
    tmp, Losses, groups = G.weight_transform(W0.clone(), torch.eye(K), spec, blocksize=128)
    assert torch.equal(tmp, W0)                                  # no error feedback reaches later columns
    s, z = G.merge_groups(groups)
    _, s0, z0, _, _ = Q.int_tensor_qparams(spec, W0)
    assert torch.equal(s, s0) and torch.equal(z, z0)
    fq = Q.int_fake_quant_dynamic(spec, W0)
    assert torch.allclose(Losses, (W0 - fq) ** 2 / 2)


def test_static_groups_look_up_the_original_columns_group():
    """static_groups (gptq.py:143-148, 224-227): with an identity Hinv nothing propagates, so column j of the
    permuted loop must be quantized exactly like column perm[j] of plain RTN on the original order - a lookup by the
    permuted position, or a refresh at group boundaries, fails this."""
    R, K, g = 6, 256, 64
    spec = Q.IntSpec(4, False, 'per_group', group_size=g)
    W0 = torch.randn(R, K, generator=gen(16)) * 0.02
    W0[:, 64:128] *= 5                                           # groups with clearly different scales
    _, s0, z0, _, _ = Q.int_tensor_qparams(spec, W0)
    sg, zg = s0.reshape(R, K // g), z0.reshape(R, K // g)
    fq = Q.int_fake_quant_dynamic(spec, W0)
    perm = torch.randperm(K, generator=gen(17))
    for p in (None, perm):
        Wp = W0 if p is None else W0[:, p]
        tmp, Losses, groups = G.weight_transform(Wp.clone(), torch.eye(K), spec, static_groups=(sg, zg, p))
        assert groups == [] and torch.equal(tmp, Wp)
        want = fq if p is None else fq[:, p]
        assert torch.allclose(Losses, (Wp - want) ** 2 / 2, rtol=0, atol=0)


def test_actorder_and_layer_driver_roundtrip():
    R, K = 8, 256
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    batches = calib_batches(4, 64, K, seed=3000)
    H = G.hessian_closed_form(batches).float()
    W0 = (torch.randn(R, K, generator=gen(7)) * 0.02)
    out = G.gptq_layer(W0, H, spec, actorder=True)
    assert torch.equal(torch.sort(out['perm']).values, torch.arange(K))
    # processing order is by decreasing Hessian diagonal
    d = torch.diag(H)[out['perm']]
    assert bool((d[:-1] >= d[1:]).all())
    codes = G.codes_from(out['tmp_perm'], out['scales'], out['zeros'], spec)
    assert codes.min() >= 0 and codes.max() <= 15
    # GPTQ lowers the layer-output error relative to plain RTN on the calibration data
    X = torch.cat(batches).float()
    deq = Q.int_quant_dequant(spec, out['tmp_perm'].reshape(-1, 128), out['scales'], out['zeros'], spec.qmax, spec.qmin)
    What = deq.reshape(R, K)[:, torch.argsort(out['perm'])]
    assert G.recon_loss(W0, What, X) < G.recon_loss(W0, Q.int_fake_quant_dynamic(spec, W0), X)


@pytest.mark.parametrize('gran', ['per_group', 'per_channel'])
def test_owq_keeps_outlier_columns_and_the_loss_identity(gran):
    """OWQ (gptq.py:44-56, 66-83, 158-167, 187-188).  Column order: the n_out largest diagonal entries last, the rest in
    their original order.  The un-quantized columns behave like columns quantized to themselves, so the loss identity
    holds over ALL columns with the outlier columns' compensated values on the quantized side; with n_out = 0 the
    result is plain GPTQ in the original order."""
    R, K, g, n_out = 4, 256, 64, 64
    spec = Q.IntSpec(4, False, gran, group_size=g)
    H = G.hessian_closed_form(calib_batches(6, 64, K, seed=2100))
    perm = G.owq_order(H, n_out)
    top = torch.argsort(torch.diag(H), descending=True)[:n_out]
    assert torch.equal(perm[K - n_out:], top)
    assert torch.equal(perm[:K - n_out], torch.sort(perm[:K - n_out]).values) and torch.equal(torch.sort(perm).values, torch.arange(K))
    W0 = torch.randn(R, K, generator=gen(6), dtype=torch.float64) * 0.02
    out = G.gptq_layer(W0, H, spec, dtype=torch.float64, owq_n_out=n_out)
    Wp = W0[:, perm]
    Hd = (H + 0.01 * torch.mean(torch.diag(H)) * torch.eye(K, dtype=torch.float64))[perm][:, perm]
    tmp = out['weight'][:, perm]                            # processing order again
    nq = K - n_out
    if gran == 'per_group':
        assert out['scales'].shape == (R * (nq // g), 1)
        Qd = Q.int_quant_dequant(spec, tmp[:, :nq].reshape(-1, g), out['scales'], out['zeros'], spec.qmax, spec.qmin).reshape(R, nq)
    else:
        s_, z_ = out['static_qparams']
        want_s, want_z = Q.int_tensor_qparams(spec, Wp[:, :nq])[1:3]
        assert torch.equal(s_, want_s) and torch.equal(z_, want_z)
        Qd = Q.int_quant_dequant(spec, tmp[:, :nq], s_, z_, spec.qmax, spec.qmin)
    full = torch.cat([Qd, tmp[:, nq:]], dim=1)
    D = Wp - full
    assert abs(out['loss'] - 0.5 * float(torch.trace(D @ Hd @ D.t()))) < 1e-12 + 1e-9 * out['loss']
    assert not torch.equal(tmp[:, nq:], Wp[:, nq:])         # the kept columns did take the compensation
    plain = G.gptq_layer(W0, H, spec, dtype=torch.float64, static_qparams=Q.int_tensor_qparams(spec, W0)[1:3])
    zero = G.gptq_layer(W0, H, spec, dtype=torch.float64, owq_n_out=0)
    assert torch.equal(zero['weight'], plain['weight']) and zero['loss'] == plain['loss']
