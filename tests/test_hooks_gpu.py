"""The boundary the way the reference drives it: forward hooks on the Linears of a decoder block.

The reference reaches GPTQ.add_batch only through forward hooks (`cache_input_hook`, gptq.py:246-251, which passes
`inp[0].data`), registered on every Linear of a subset while the block runs over the calibration batches
(base_blockwise_quantization.py:397-440); after a subset is transformed the next subset is hooked and the block runs
again on the weights quantized so far (`rehook_next_subset`, :529-549).  This file builds a small Llama-style block
(RMSNorm, grouped-query attention, SwiGLU; defined here, random weights) and drives lightcompress_amd.gptq.GPTQ through
that sequence, then checks what the hooks bring about: q/k/v and gate/up end up sharing a Hessian and o / down do not,
the results equal a run without sharing, the codes agree with the CPU oracle fed the same captured activations, and a
second run reproduces the first bit for bit.

Also here: the layer kinds add_batch / process_hessian_and_weights tell apart (transformers.Conv1D, nn.Conv2d,
gptq.py:130-133, 190-191, 262-278) and what happens when a hook input is written in place between two hooks.
"""
import functools

import pytest
import torch
from torch import nn

from oracle import gptq_ref as G, quant_ref as Q
from tests.helpers import gen
from tests.test_gptq_gpu import make_gptq

pytestmark = pytest.mark.gpu

HID, HEADS, KV, INTER = 256, 4, 2, 640
SUBSETS = [['q_proj', 'k_proj', 'v_proj'], ['o_proj'], ['gate_proj', 'up_proj'], ['down_proj']]
SPEC = Q.IntSpec(4, False, 'per_group', group_size=128)


class RMSNorm(nn.Module):
    def __init__(self, n):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(n))

    def forward(self, x):
        v = x.float()
        return (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + 1e-6)).to(x.dtype) * self.weight


class Block(nn.Module):
    def __init__(self):
        super().__init__()
        hd = HID // HEADS
        self.q_proj, self.k_proj, self.v_proj = nn.Linear(HID, HID, bias=False), nn.Linear(HID, KV * hd, bias=False), nn.Linear(HID, KV * hd, bias=False)
        self.o_proj = nn.Linear(HID, HID, bias=False)
        self.gate_proj, self.up_proj, self.down_proj = nn.Linear(HID, INTER, bias=False), nn.Linear(HID, INTER, bias=False), nn.Linear(INTER, HID, bias=False)
        self.ln1, self.ln2 = RMSNorm(HID), RMSNorm(HID)

    def forward(self, x):
        B, T, _ = x.shape
        hd = HID // HEADS
        h = self.ln1(x)
        q = self.q_proj(h).view(B, T, HEADS, hd).transpose(1, 2)
        k = self.k_proj(h).view(B, T, KV, hd).transpose(1, 2).repeat_interleave(HEADS // KV, dim=1)
        v = self.v_proj(h).view(B, T, KV, hd).transpose(1, 2).repeat_interleave(HEADS // KV, dim=1)
        a = nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).reshape(B, T, HID)
        x = x + self.o_proj(a)
        h = self.ln2(x)
        return x + self.down_proj(nn.functional.silu(self.gate_proj(h)) * self.up_proj(h))


def _block(dev, seed=0, dtype=torch.bfloat16):
    torch.manual_seed(seed)
    blk = Block()
    for i, p in enumerate(blk.parameters()):
        if p.dim() == 2:
            p.data = torch.randn(p.shape, generator=gen(seed + 10 * i)) * 0.05
    return blk.to(dev).to(dtype)


def _calib(dev, nb=6, B=2, T=48, dtype=torch.bfloat16):
    sigma = torch.exp(0.7 * torch.randn(HID, generator=gen(50)))
    return [(torch.randn(B, T, HID, generator=gen(60 + i)) * sigma).to(dtype).to(dev) for i in range(nb)]


def _drive(dev, blk, data, captured=None, **special):
    """block_transform (base_blockwise_quantization.py:468-527) for GPTQ with true_sequential: per subset, hooks on its
    Linears -> block forward over every calibration batch -> hooks off -> subset_transform; the next subset's forward
    then runs on the fake-quantized weights of this one (w_qdq, what the FakeQuantLinear replacement computes,
    :529-549).  Returns per Linear (compensated fp32 weight, scales, zeros, perm) as subset_transform left them."""
    gp = make_gptq(actorder=True, **special)
    named = dict(blk.named_modules())
    gp.model_dtype = next(blk.parameters()).dtype
    leaders, errors, state = {}, {}, {}
    for names in SUBSETS:                                   # collect_block_qparams, :348-376
        for n in names:
            gp.collect_layer_qparams(named[n])

    def hook(m, inp, out, name):                          # cache_input_hook, gptq.py:246-251
        gp.add_batch(gp.named_layers[name], name, inp[0].data, out.data)
        if captured is not None:
            captured.setdefault(name, []).append(inp[0].data.cpu().clone())

    for names in SUBSETS:
        subset = {'layers': {n: named[n] for n in names}}
        gp.subset_init(subset)
        handles = [named[n].register_forward_hook(functools.partial(hook, name=n)) for n in names]
        with torch.no_grad():
            for x in data:                                  # block_forward, :378-401
                blk(x)
        for h in handles:
            h.remove()
        leaders.update({n: gp.layers_cache[n].get('leader', n) for n in names})
        gp.subset_transform(subset)
        errors.update({n: float(gp.last_errors[n]) for n in names})
        for n in names:
            m = named[n]
            state[n] = (m.weight.data.clone(), m.buf_scales.clone(), m.buf_zeros.clone(), m.buf_perm.clone())
            assert m.weight.data.dtype == torch.float32
            m.weight.data = gp.w_qdq(m, gp.wquantizer)      # bf16, original column order
            assert m.weight.data.dtype == gp.model_dtype and m.weight.data.shape == state[n][0].shape
    torch.cuda.synchronize()
    return state, leaders, errors


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_hooks_on_a_decoder_block(dev, dtype):
    data = _calib(dev, dtype=dtype)
    captured = {}
    blk = _block(dev, dtype=dtype)
    W0 = {n: m.weight.data.clone() for n, m in blk.named_modules() if isinstance(m, nn.Linear)}
    shared, leaders, errors = _drive(dev, blk, data, captured)
    # q/k/v and gate/up were handed one tensor per forward pass: they share; o and down stand alone
    assert leaders == {'q_proj': 'q_proj', 'k_proj': 'q_proj', 'v_proj': 'q_proj', 'o_proj': 'o_proj',
                       'gate_proj': 'gate_proj', 'up_proj': 'gate_proj', 'down_proj': 'down_proj'}
    # the same run twice: bit for bit
    again, leaders2, errors2 = _drive(dev, _block(dev, dtype=dtype), data)
    assert leaders2 == leaders and errors2 == errors
    for n in shared:
        for a, b in zip(shared[n], again[n]):
            assert torch.equal(a, b), n
    # without sharing (one Hessian, one chain, one loop per Linear, as the reference keeps them): the same results
    alone, leaders3, errors3 = _drive(dev, _block(dev, dtype=dtype), data, auto_share=False, fuse_loops=False)
    assert leaders3 == {n: n for n in leaders}
    for n in shared:
        for a, b in zip(shared[n], alone[n]):
            assert torch.equal(a, b), n
        assert abs(errors[n] - errors3[n]) <= 1e-6 * abs(errors3[n])
    # the CPU oracle on the activations the hooks saw
    for n in shared:
        xs = captured[n]
        K = xs[0].shape[-1]
        Ho, cnt = torch.zeros(K, K), 0
        for x in xs:
            cnt = G.add_batch(Ho, cnt, x)
        ref = G.gptq_layer(W0[n].cpu(), Ho, SPEC, actorder=True)
        perm = shared[n][3].cpu()
        d = torch.diag(Ho)
        assert float((d[perm] - d[ref['perm']]).abs().max()) <= 1e-6 * float(d.max())        # the same order up to ties
        if torch.equal(perm, ref['perm']):
            codes = G.codes_from(shared[n][0].cpu()[:, perm], shared[n][1].cpu(), shared[n][2].cpu(), SPEC)
            codes_o = G.codes_from(ref['tmp_perm'], ref['scales'], ref['zeros'], SPEC)
            agree = float((codes == codes_o).float().mean())
            if agree < 0.999:
                # fp32 rounding decides a few codes per thousand either way: the run has to be as close to the
                # fp64 evaluation of the same recurrence as the fp32 oracle is
                ref64 = G.gptq_layer(W0[n].cpu(), Ho.double(), SPEC, actorder=True, dtype=torch.float64)
                if torch.equal(perm, ref64['perm']):
                    codes_64 = G.codes_from(ref64['tmp_perm'].float(), ref64['scales'].float(), ref64['zeros'].float(), SPEC)
                    agree = float((codes == codes_64).float().mean())
                    assert agree >= float((codes_o == codes_64).float().mean()) - 0.001, (n, agree)
            assert agree >= 0.998, (n, agree)
        assert abs(errors[n] - ref['loss']) <= 0.01 * ref['loss'], (n, errors[n], ref['loss'])


def test_input_written_in_place_between_two_hooks_is_not_shared_silently(dev):
    """`inp[0].data` carries a fresh version counter, so an in-place write between the hooks of two Linears cannot be
    seen on the host.  The comparison on the device sees it: the follower is not given the leader's Hessian; the
    mismatch raises where the Hessian would be consumed."""
    from lightcompress_amd import _lib as L
    K = 384
    Ws = {'a': (torch.randn(32, K, generator=gen(5)) * 0.02).bfloat16(), 'b': (torch.randn(48, K, generator=gen(6)) * 0.02).bfloat16()}
    xs = [(torch.randn(1, 64, K, generator=gen(8500 + i))).bfloat16().to(dev) for i in range(3)]
    for mutate_call in (0, 2):
        gp = make_gptq(actorder=True)
        layers = {n: nn.Linear(K, w.shape[0], bias=False).to(dev).to(torch.bfloat16) for n, w in Ws.items()}
        gp.subset_init({'layers': layers})
        for i, x in enumerate(xs):
            x = x.clone()
            gp.add_batch(layers['a'], 'a', x.data, None)
            if i == mutate_call:
                x[0, 5, 7] += 1                            # one element, same memory, same version on the `.data` alias
            gp.add_batch(layers['b'], 'b', x.data, None)
        assert gp.layers_cache['b'].get('leader') == 'a'       # the host saw nothing
        with pytest.raises(L.LcqError, match='written in place'):
            gp.hessian('b')
        with pytest.raises(L.LcqError, match='written in place'):
            gp.subset_transform({'layers': layers})
        torch.cuda.synchronize()
    # share_verify: False takes the caller's word
    gp = make_gptq(actorder=True, share_verify=False)
    layers = {n: nn.Linear(K, w.shape[0], bias=False).to(dev).to(torch.bfloat16) for n, w in Ws.items()}
    gp.subset_init({'layers': layers})
    for x in xs:
        gp.add_batch(layers['a'], 'a', x.data, None)
        gp.add_batch(layers['b'], 'b', x.data, None)
    assert gp.layers_cache['b'].get('leader') == 'a' and gp.layers_cache['a'].get('share_flag') is None
    gp.subset_transform({'layers': layers})


@pytest.mark.parametrize('read_at', [0, 2, 4])
def test_hessian_read_between_the_hooks_of_one_pass(dev, read_at):
    """Reading H after the leader's hook and before the follower's folds the staged tokens; the follower, one call
    behind at that moment, is given its own Hessian first (the state before that call) and goes on alone.  Every
    result equals separate accumulation bit for bit."""
    K = 384
    Ws = {'a': (torch.randn(32, K, generator=gen(15)) * 0.02).bfloat16(), 'b': (torch.randn(48, K, generator=gen(16)) * 0.02).bfloat16()}
    xs = [(torch.randn(1, 64, K, generator=gen(8700 + i))).bfloat16().to(dev) for i in range(6)]
    out = {}
    for share in (True, False):
        gp = make_gptq(actorder=True, hessian_defer=4, auto_share=share)
        layers = {n: nn.Linear(K, w.shape[0], bias=False).to(dev).to(torch.bfloat16) for n, w in Ws.items()}
        for n, w in Ws.items():
            layers[n].weight.data = w.to(dev)
        gp.subset_init({'layers': layers})
        mid = None
        for i, x in enumerate(xs):
            gp.add_batch(layers['a'], 'a', x.data, None)
            if i == read_at:
                mid = gp.hessian('a').clone()
            gp.add_batch(layers['b'], 'b', x.data, None)
        assert gp.layers_cache['b'].get('leader', 'b') == 'b'          # released (or never joined) at the read
        Ha, Hb = gp.hessian('a').clone(), gp.hessian('b').clone()
        gp.subset_transform({'layers': layers})
        torch.cuda.synchronize()
        out[share] = (mid, Ha, Hb, layers['a'].weight.data.clone(), layers['b'].weight.data.clone())
    for a, b in zip(out[True], out[False]):
        assert torch.equal(a, b)
    ref = G.hessian_closed_form([x.cpu() for x in xs])
    assert float((out[True][2].cpu().double() - ref).abs().max() / ref.abs().max()) < 1e-5


def test_follower_that_skips_a_forward_pass(dev):
    """A Linear whose hook does not fire in one pass (a branch not taken) stops following at the leader's next call."""
    K = 256
    xs = [(torch.randn(1, 40, K, generator=gen(8800 + i))).bfloat16().to(dev) for i in range(5)]
    gp = make_gptq(actorder=False, hessian_defer=3)
    layers = {n: nn.Linear(K, 16, bias=False).to(dev).to(torch.bfloat16) for n in 'ab'}
    gp.subset_init({'layers': layers})
    for i, x in enumerate(xs):
        gp.add_batch(layers['a'], 'a', x.data, None)
        if i != 2:
            gp.add_batch(layers['b'], 'b', x.data, None)
    assert gp.layers_cache['b']['leader'] == 'b' and gp.layers_cache['b']['nsamples'] == 4
    Ha, Hb = gp.hessian('a').cpu().double(), gp.hessian('b').cpu().double()
    ra = G.hessian_closed_form([x.cpu() for x in xs])
    rb = G.hessian_closed_form([x.cpu() for i, x in enumerate(xs) if i != 2])
    assert float((Ha - ra).abs().max() / ra.abs().max()) < 1e-5
    assert float((Hb - rb).abs().max() / rb.abs().max()) < 1e-5


def test_conv1d_and_conv2d_layers(dev):
    """transformers.Conv1D keeps its weight [in, out] (gptq.py:132-133, 190-191, 302); nn.Conv2d flattens the weight
    and unfolds its inputs into patches (:130-131, 268-278).  Both against the CPU oracle on the matrices the
    reference would form."""
    try:
        from transformers.pytorch_utils import Conv1D
    except Exception as e:                                 # pragma: no cover
        pytest.skip(f'transformers.Conv1D not importable: {e}')
    K, R = 256, 48
    # --- Conv1D
    w = (torch.randn(K, R, generator=gen(41)) * 0.02)
    conv = Conv1D(R, K)
    conv.weight.data = w.clone()
    conv = conv.to(dev)
    xs = [(torch.randn(2, 40, K, generator=gen(8900 + i)) * torch.exp(0.5 * torch.randn(K, generator=gen(42)))).bfloat16() for i in range(4)]
    gp = make_gptq(actorder=True)
    gp.subset_init({'layers': {'c_fc': conv}})
    assert gp.layers_cache['c_fc']['columns'] == K and gp.layers_cache['c_fc']['kind'] == 'conv1d'
    Ho, cnt = torch.zeros(K, K), 0
    for x in xs:
        gp.add_batch(conv, 'c_fc', x.to(dev).data, None)
        cnt = G.add_batch(Ho, cnt, x)
    assert gp.layers_cache['c_fc']['nsamples'] == cnt == 8
    gp.subset_transform({'layers': {'c_fc': conv}})
    ref = G.gptq_layer(w.t().contiguous(), Ho, SPEC, actorder=True)
    assert conv.weight.data.shape == (K, R)
    got = conv.weight.data.t().cpu()
    assert torch.equal(conv.buf_perm.cpu(), ref['perm'])
    codes = G.codes_from(got[:, ref['perm']], conv.buf_scales.cpu(), conv.buf_zeros.cpu(), SPEC)
    codes_o = G.codes_from(ref['tmp_perm'], ref['scales'], ref['zeros'], SPEC)
    assert float((codes == codes_o).float().mean()) >= 0.999
    assert abs(float(gp.last_errors['c_fc']) - ref['loss']) <= 0.01 * ref['loss']
    # --- Conv2d: 8 channels, 4x4 kernel, stride 2 -> K = 128 input features per patch
    c2 = nn.Conv2d(8, 24, kernel_size=4, stride=2, padding=1, bias=False)
    w2 = torch.randn(24, 8, 4, 4, generator=gen(43)) * 0.05
    c2.weight.data = w2.clone()
    c2 = c2.to(dev)
    imgs = [torch.randn(3, 8, 12, 12, generator=gen(8950 + i)).bfloat16() for i in range(4)]
    gp = make_gptq(actorder=False)
    gp.subset_init({'layers': {'conv': c2}})
    assert gp.layers_cache['conv']['columns'] == 128 and gp.layers_cache['conv']['kind'] == 'conv2d'
    Ho, cnt = torch.zeros(128, 128), 0
    for im in imgs:
        gp.add_batch(c2, 'conv', im.to(dev).data, None)
        cnt = G.add_batch(Ho, cnt, G.conv2d_patches(im.float(), 4, 1, 1, 2).bfloat16())
    assert gp.layers_cache['conv']['nsamples'] == cnt == 12
    H = gp.hessian('conv').cpu()
    assert float((H - Ho).abs().max() / Ho.abs().max()) < 1e-5
    gp.subset_transform({'layers': {'conv': c2}})
    ref = G.gptq_layer(w2.flatten(1), Ho, SPEC, actorder=False)
    assert c2.weight.data.shape == (24, 8, 4, 4)
    codes = G.codes_from(c2.weight.data.flatten(1).cpu(), c2.buf_scales.cpu(), c2.buf_zeros.cpu(), SPEC)
    codes_o = G.codes_from(ref['tmp_perm'], ref['scales'], ref['zeros'], SPEC)
    assert float((codes == codes_o).float().mean()) >= 0.999
    assert abs(float(gp.last_errors['conv']) - ref['loss']) <= 0.01 * ref['loss']


def test_compare_bytes_and_empty_hessian_update(dev):
    """lcq_compare_bytes sets its flag on any differing bit and leaves it alone otherwise; lcq_hessian_accum with no
    tokens scales H by alpha (and does nothing for alpha == 1)."""
    from lightcompress_amd import _lib as L
    lib = L.lib()
    a = torch.randn(3 * 1024 * 1024 + 16, generator=gen(1)).bfloat16().to(dev)
    b = a.clone()
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    n = a.numel() * 2
    L.check(lib.lcq_compare_bytes(L.ptr(a), L.ptr(b), L.i64(n), L.ptr(flag), L.stream()), 'compare')
    assert int(flag.item()) == 0
    for pos in (0, 1234567, a.numel() - 1):
        b.copy_(a)
        b.view(torch.int16)[pos] ^= 1                      # one bit
        flag.zero_()
        L.check(lib.lcq_compare_bytes(L.ptr(a), L.ptr(b), L.i64(n), L.ptr(flag), L.stream()), 'compare')
        assert int(flag.item()) == 1, pos
    L.check(lib.lcq_compare_bytes(L.ptr(a), L.ptr(a), L.i64(n), L.ptr(flag), L.stream()), 'compare')
    assert int(flag.item()) == 1                           # never cleared by the call
    assert lib.lcq_compare_bytes(L.ptr(a), L.ptr(b), L.i64(n - 2), L.ptr(flag), L.stream()) == -1
    assert lib.lcq_compare_bytes(L.ptr(a), L.ptr(b), L.i64(0), L.ptr(flag), L.stream()) == 0
    K = 512
    H = torch.randn(K, K, generator=gen(2)).to(dev)
    H0 = H.clone()
    x = torch.zeros(8, K, dtype=torch.bfloat16, device=dev)
    L.check(lib.lcq_hessian_accum(L.ptr(H), L.i64(K), L.ptr(x), L.i32(L.BF16), L.i64(0), L.i64(K), L.f32(1.0), L.f32(2.0), L.stream()), 'T=0')
    assert torch.equal(H, H0)
    L.check(lib.lcq_hessian_accum(L.ptr(H), L.i64(K), L.ptr(x), L.i32(L.BF16), L.i64(0), L.i64(K), L.f32(0.5), L.f32(2.0), L.stream()), 'T=0')
    up = torch.triu(torch.ones(K, K, dtype=torch.bool, device=dev))
    assert torch.equal(H[up], (0.5 * H0)[up])
    # lcq_histc refuses an unknown element type before it touches the counters
    counts = torch.full((64,), 7, dtype=torch.int32, device=dev)
    hist = torch.zeros(64, device=dev)
    assert lib.lcq_histc(L.ptr(H), L.i32(9), L.i64(1024), L.i32(64), L.f32(-1.0), L.f32(1.0), L.ptr(counts), L.ptr(hist), L.stream()) == -3
    torch.cuda.synchronize()
    assert bool((counts == 7).all())
