"""The headline shapes at full size: K = 14336 (down_proj), R = 14336 (gate / up) and the 4096 x 4096 single Linear.

The CPU oracle cannot run a 14336-wide layer in test time, so these cases are checked through properties that do
not depend on the size and that the device can evaluate in fp64 with plain torch ops:
  * Hessian: H == (2 / n) * X^T X computed in fp64 from the same tokens, within 1e-5;
  * Cholesky chain: U upper triangular with a positive diagonal and  U^T U (H_perm + damp I) == I  in fp64;
  * column loop + chain together: sum(Losses) == 1/2 tr((W0 - Q)(H_perm + damp I)(W0 - Q)^T), which holds for ANY
    choice of quantized values Q when U is the exact factor and the error feedback is applied exactly
    (tests/test_oracle_gptq.py shows it on the oracle in fp64);
The 4096 x 4096 Linear is additionally compared with the CPU oracle itself on 8 calibration batches.
"""
import pytest
import torch

from oracle import gptq_ref as G, quant_ref as Q
from tests.helpers import gen
from tests.test_gptq_gpu import Layer, make_gptq

pytestmark = pytest.mark.gpu


def _device_batches(dev, nb, T, K, seed):
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    sigma = torch.exp(torch.randn(K, device=dev, generator=g))
    return [(torch.randn(T, K, device=dev, generator=g) * sigma).bfloat16() for _ in range(nb)]


def _qdq(tmp, s, z, g):
    """quant_dequant of every column with its group's parameters, fp32 torch ops (quant.py:698-716)."""
    R, K = tmp.shape
    t = tmp.reshape(R, K // g, g)
    s, z = s.reshape(R, K // g, 1), z.reshape(R, K // g, 1)
    return ((torch.clamp(torch.round(t / s) + z, 0, 15) - z) * s).reshape(R, K)


@pytest.mark.parametrize('R,K,nb', [(4096, 14336, 8),        # down_proj: 28 super-panels, 14 update windows, 2 Hessian folds
                                    (14336, 4096, 8)])       # gate / up: 14336 rows through the column loop
def test_llama3_8b_shapes_by_fp64_properties(dev, R, K, nb):
    T, g = 2048, 128
    xs = _device_batches(dev, nb, T, K, seed=100 + K)
    gw = torch.Generator(device=dev)
    gw.manual_seed(7 + R)
    W0 = (torch.randn(R, K, device=dev, generator=gw) * 0.02).bfloat16()
    gp = make_gptq(actorder=True)
    layer = Layer(W0.clone())
    gp.subset_init({'layers': {'fc': layer}})
    for x in xs:
        gp.add_batch(layer, 'fc', x.unsqueeze(0), None)
    H = gp.hessian('fc').clone()

    # -- Hessian against fp64 on the same tokens
    H64 = torch.zeros(K, K, dtype=torch.float64, device=dev)
    for x in xs:
        xd = x.double()
        H64.addmm_(xd.t(), xd)
    H64 *= 2.0 / nb
    del xs
    scale = float(H64.abs().max())
    assert float((H.double() - H64).abs().max()) / scale < 1e-5
    assert float((H.double() - H64).norm() / H64.norm()) < 1e-5
    assert torch.equal(H, H.t())

    # -- Cholesky chain
    gp.initialize_qparams_and_prepare_weights(layer, 'fc')
    perm = gp.perm
    d = torch.diag(H)[perm]
    assert bool((d[:-1] >= d[1:]).all()) and torch.equal(torch.sort(perm).values, torch.arange(K, device=dev))
    W, U = gp.process_hessian_and_weights(layer, 'fc')
    assert int(gp._status.item()) == 0
    assert torch.equal(W, W0.float()[:, perm])
    assert torch.equal(torch.triu(U), U) and bool((torch.diag(U) > 0).all()) and bool(torch.isfinite(U).all())
    Hd = H64[perm][:, perm]
    del H64
    Hd.diagonal().add_(0.01 * Hd.diagonal().mean())
    U64 = U.double()
    res = (U64.t() @ U64) @ Hd
    res.diagonal().sub_(1.0)
    resid = float(res.abs().max())
    del res, U64
    print(f'K={K}: chain residual max|U^T U H_d - I| = {resid:.3e}')
    assert resid < 1e-3, resid

    # -- column loop: loss identity, group parameters, un-permutation
    W0p = W.clone()
    gp.update_layer_with_transformed_weights(layer, W, U, 'fc')
    tmp = layer.weight.data[:, perm]
    assert bool(torch.isfinite(tmp).all())
    s, z = layer.buf_scales.reshape(R, K // g), layer.buf_zeros.reshape(R, K // g)
    assert bool((s > 0).all()) and bool((z == torch.round(z)).all()) and float(z.min()) >= 0 and float(z.max()) <= 15
    assert torch.equal(tmp[:, 0], W0p[:, 0])                         # the first processed column is untouched
    Qv = _qdq(tmp, s, z, g)
    Dm = (W0p - Qv).double()
    rhs = 0.5 * float(((Dm @ Hd) * Dm).sum())
    lhs = float(gp.last_error)
    print(f'R={R} K={K}: sum(Losses) = {lhs:.6g}, 1/2 tr((W0-Q) H_d (W0-Q)^T) = {rhs:.6g}')
    assert abs(lhs - rhs) <= 1e-4 * rhs, (lhs, rhs)
    # compensation pays: plain RTN of the original weights loses more under the same metric
    t0 = W0p.reshape(R, K // g, g)
    mn, mx = t0.amin(-1, keepdim=True), t0.amax(-1, keepdim=True)
    s0 = (mx - mn).clamp(min=1e-5) / 15
    z0 = (-torch.round(mn / s0)).clamp(0, 15)
    Dr = (W0p - _qdq(W0p, s0, z0, g)).double()
    assert rhs < 0.9 * 0.5 * float(((Dr @ Hd) * Dr).sum())


def test_gptq_4096_linear_against_cpu_oracle(dev):
    """BASELINE config 2 at its full 4096 x 4096 size (act_order off, w4 asym g128), 8 calibration batches of 2048
    tokens generated on the CPU: codes >= 99.9 % equal, loss within 1 %, Hessian within 1e-5."""
    R = K = 4096
    nb, T = 8, 2048
    sigma = torch.exp(torch.randn(K, generator=gen(0)))
    batches = [(torch.randn(T, K, generator=gen(1000 + b)) * sigma).bfloat16() for b in range(nb)]
    W0 = (torch.randn(R, K, generator=gen(1)) * 0.02).bfloat16()
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    torch.set_num_threads(16)
    Ho, n = torch.zeros(K, K), 0
    for b in batches:
        n = G.add_batch(Ho, n, b.unsqueeze(0))
    ref = G.gptq_layer(W0, Ho, spec, actorder=False)

    gp = make_gptq(actorder=False)
    layer = Layer(W0.to(dev))
    gp.subset_init({'layers': {'fc': layer}})
    for b in batches:
        gp.add_batch(layer, 'fc', b.unsqueeze(0).to(dev), None)
    H = gp.hessian('fc').cpu()
    assert float((H - Ho).abs().max() / Ho.abs().max()) < 1e-5
    gp.layer_transform(layer, 'fc')
    Wq, s, z = layer.weight.data.cpu(), layer.buf_scales.cpu(), layer.buf_zeros.cpu()
    # a code that rounds the other way (fp32 summation order) changes the feedback to every later column of its row,
    # so a few later group ranges of that row move: nearly all scales coincide, not all
    close = torch.isclose(s, ref['scales'], rtol=1e-3).float().mean()
    print(f'4096x4096: scales within 1e-3: {float(close):.6f}')
    assert float(close) > 0.995
    codes = G.codes_from(Wq, s, z, spec)
    codes_o = G.codes_from(ref['tmp_perm'], ref['scales'], ref['zeros'], spec)
    agree = float((codes == codes_o).float().mean())
    print(f'4096x4096: code agreement {agree:.6f}, loss {float(gp.last_error):.6g} vs {ref["loss"]:.6g}')
    assert agree >= 0.999, agree
    assert abs(float(gp.last_error) - ref['loss']) <= 0.01 * ref['loss']
    # reconstruction loss ||(W - What) X||^2 through the Hessian: tr(D H D^T) * n / 2
    Hd = Ho.double()
    def recon(c, sc, zp):
        D = W0.double() - Q.int_dequant(c.reshape(-1, 128), sc, zp).reshape(R, K).double()
        return float(((D @ Hd) * D).sum())
    l, lo = recon(codes, s, z), recon(codes_o, ref['scales'], ref['zeros'])
    assert abs(l - lo) <= 0.01 * lo, (l, lo)


@pytest.mark.parametrize('entry', ['lcq_chol_inv_upper', 'lcq_chol_block_factor'])
def test_chain_lookahead_changes_nothing(dev, entry):
    """Chains of K >= 8192 run the far part of every deep trailing update on a second stream beside the next
    super-panel (lcq_set_chain_lookahead, default on).  The factor is the one-stream factor up to fp32 rounding (a part
    of an update may take the other GEMM kernel than the whole would), it is reproducible bit for bit from run to run
    and from stream to stream (no race between the two streams), and the caller's stream is where it is ready."""
    from lightcompress_amd import _lib as L
    K = 8192
    g = torch.Generator(device=dev)
    g.manual_seed(3)
    X = torch.randn(2 * K, K, device=dev, generator=g) * torch.exp(0.5 * torch.randn(K, device=dev, generator=g))
    H = (X.t() @ X) / K
    del X
    lib = L.lib()
    nbytes = lib.lcq_chol_inv_upper_workspace_bytes(L.i64(K))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    status = torch.ones(1, dtype=torch.int32, device=dev)
    outs = []
    side = torch.cuda.Stream(device=dev)
    try:
        for on, stream in ((0, None), (1, None), (1, side), (1, None)):
            lib.lcq_set_chain_lookahead(L.i32(on))
            Hc, U = H.clone(), torch.empty(K, K, device=dev)
            torch.cuda.synchronize()
            with torch.cuda.stream(stream if stream is not None else torch.cuda.current_stream()):
                L.check(getattr(lib, entry)(L.ptr(Hc), L.i64(K), L.ptr(None), L.f32(0.01), L.ptr(None), L.i64(0), L.ptr(U),
                                            L.ptr(ws), L.i64(nbytes), L.ptr(status), L.stream()), entry)
                total = U.sum()                           # queued behind the call on the same stream: must see all of U
            torch.cuda.synchronize()
            assert int(status.item()) == 0
            assert float(total) == float(U.sum())
            outs.append(U)
    finally:
        assert lib.lcq_set_chain_lookahead(L.i32(1)) in (0, 1)
    assert torch.equal(outs[1], outs[2]) and torch.equal(outs[1], outs[3])
    rel = float((outs[0].double() - outs[1].double()).abs().max() / outs[0].abs().max())
    assert rel < 1e-5, rel
