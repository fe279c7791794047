"""GPTQ with the reference's method surface, running on liblcq.

Mirrors ``llmc/compression/quantization/gptq.py`` of ModelTC/LightCompress
(class ``GPTQ``): ``layer_init`` / ``add_batch`` (Hessian accumulation,
gptq.py:253-308), ``hessian_sorting`` (:58-64), ``process_hessian_and_weights``
(:128-176), ``weight_transform`` (:198-244, upstream GPTQ's "fasterquant"),
``update_layer_with_transformed_weights`` (:178-196), ``layer_transform``,
``subset_transform``, ``w_q`` / ``w_qdq`` (:411-452) and the qparam bookkeeping
(:332-409).  The model walk (blocks, hooks, deploy) of the reference's base
class is not part of this path: a "layer" here is any object with a
``weight`` tensor (an ``nn.Linear``).

Differences a caller can observe
  * one process / one GPU: the per-call all-reduce of add_batch is not issued;
  * H is kept valid on and above the diagonal only while it accumulates
    (``hessian(name)`` returns the full symmetric matrix);
  * Linears of a subset that receive the very same input tensor on every call (q/k/v, gate/up) share one Hessian
    and one Cholesky chain (``special.auto_share``, default on; detected per call by address, shape, strides and
    type, with a fallback to separate Hessians at the first call that differs; results are bit-identical either
    way).  The hooks hand over ``inp[0].data`` (gptq.py:246-251), an alias whose version counter always reads 0, so
    nothing on the host can tell whether the memory was written between two hooks of one forward pass: every
    shared call is therefore compared on the device, bit for bit, with the copy the first Linear staged
    (``special.share_verify``, default on; lcq_compare_bytes), and a difference raises ``LcqError`` where the
    Hessian is consumed (``hessian(name)``, the transform of the Linear) instead of giving the follower the
    leader's Hessian.  With ``share_verify: False`` the caller vouches that no hook input is modified in place
    between the hooks of one forward pass;
  * ``transformers.Conv1D`` (weight stored [in, out], gptq.py:132-133, 190-191, 302) and ``nn.Conv2d`` (inputs
    unfolded into patches, gptq.py:268-278) layers are taken like the reference takes them; their Hessians are
    never shared;
  * ``blocksize`` above 128 runs as passes of at most 128 columns; a group that opens in a later pass of a block
    takes its range from the weights as they were when the block started, which is what the reference's read of
    the block-stale ``W`` (gptq.py:216-222) amounts to;
  * subset_transform runs the column loops of Linears that share a chain as one loop over their stacked rows
    (``special.fuse_loops``, default on; rows are independent, so each Linear gets the result of its own loop, up to
    the rounding of the update GEMM where the larger row count selects the other GEMM kernel), and leaves every
    Linear's summed loss in ``last_errors[name]``;
  * layer_transform / subset_transform factor the damped Hessian WITHOUT the triangular inverse where every group of
    the weight quantizer lies inside one 128-column block (``special.block_factor``, default on): the loop runs on a
    block factor that has U's diagonal blocks (gptq.py:205 `Hinv1`) and carries (quantized - original) weights
    instead of errors to later columns; the same results up to fp32 rounding (closer to fp64 than the reference's
    cholesky / cholesky_inverse / cholesky chain).  process_hessian_and_weights called on its own returns the
    reference's U;
  * ``special.hessian_defer`` (default 'auto': 16 for K <= 4096, 8 for K <= 8192, else 4) add_batch calls are copied to a staging buffer and
    folded into one launch, so ``layers_cache[name]['H']`` lags behind ``nsamples`` until
    ``hessian(name)``, ``hessian_sorting`` or ``process_hessian_and_weights`` settles it
    (``hessian_defer: 1`` updates H on every call);
  * ``special.hessian_slices`` (default 'auto': 3 at K = 4096, 1 at K = 14336): a launch whose Hessian has too few
    tiles to fill the chip cuts its tokens into that many shares, each with an accumulator of its own; the same
    calls settle them into H (a sum in a fixed order; H differs from a single accumulator's by fp32 rounding);
  * per-group qparams of the loop live in two [R, G] tensors instead of a
    Python list of dicts; ``layer.buf_scales`` / ``buf_zeros`` get the same
    [R*G, 1] layout the reference writes;
  * fp32 activations are split into two bf16 halves (x = hi + lo to 2^-17) and accumulated as the four products of
    the halves on the bf16 matrix pipe; bf16 / fp16 activations go in as they are (their products are exact in fp32);
  * OWQ (`special.owq`): the Linears' outlier counts come from `special.n_outs` plus `set_block_linears(names)`
    (the reference reads the order from its model wrapper), or from a dict; Hessians and chains are not shared.
"""
from __future__ import annotations

import math

import torch

import ctypes

from . import _lib as L
from .quant import IntegerQuantizer


def C_ptr(view):
    """Device pointer of a (possibly strided) view's first element."""
    return ctypes.c_void_p(view.data_ptr())


class GPTQ:
    def __init__(self, quant_config, model_dtype=torch.bfloat16, wquantizer=None):
        self.quant_config = quant_config
        self.dev = torch.device('cuda')
        self.model_dtype = model_dtype
        wcfg = dict(quant_config['weight'])
        self.wquantizer = wquantizer or IntegerQuantizer(**wcfg)
        self.add_quant_config()
        self.layers_cache = {}
        self.qparams = {}
        self._shared = {}          # leader name -> dict(U=..., perm=..., invperm=..., status=...)

    # -- configuration (gptq.py:33-56) ---------------------------------------
    def add_quant_config(self):
        special_config = self.quant_config['special']
        self.true_sequential = special_config.get('true_sequential', True)
        self.static_groups = special_config['static_groups']
        self.actorder = special_config['actorder']
        self.percdamp = special_config['percdamp']
        self.blocksize = special_config['blocksize']
        self.owq = special_config.get('owq', False)
        self.chunk_num = special_config.get('chunk_num', 1)
        self.check_positive_definite = special_config.get('check_positive_definite', True)
        # add_batch calls folded into one Hessian launch (1 = one launch per call)
        hd = special_config.get('hessian_defer', 'auto')
        self.hessian_defer = hd if hd == 'auto' else int(hd)
        # token shares of one Hessian launch, each with an accumulator of its own ('auto': by the number of tiles)
        hs = special_config.get('hessian_slices', 'auto')
        self.hessian_slices = hs if hs == 'auto' else int(hs)
        # subset_transform starts the Cholesky chains of all Linears of a subset side by side (False: one by one)
        self.chain_overlap = bool(special_config.get('chain_overlap', True))
        self.fuse_loops = bool(special_config.get('fuse_loops', True))
        # layer_transform / subset_transform factor H without the triangular inverse where the loop allows it
        self.block_factor = bool(special_config.get('block_factor', True))
        # Linears of a subset that keep receiving the very same input tensor share one Hessian and one chain
        self.auto_share = bool(special_config.get('auto_share', True))
        # every shared add_batch call is compared on the device with the tokens the leading Linear staged
        self.share_verify = bool(special_config.get('share_verify', True))
        if self.owq:                                     # gptq.py:47-50
            self.n_outs = special_config['n_outs']
            self.static_groups = False
            self.actorder = False
        if int(self.blocksize) != self.blocksize or self.blocksize < 1:
            raise ValueError(f'blocksize: {self.blocksize}')
        self.need_perm = (
            self.wquantizer.granularity == 'per_group'
            and not self.static_groups
            and self.actorder
        ) or self.owq

    def set_block_linears(self, names):
        """OWQ: `special.n_outs` lists the number of outlier columns per Linear in the order the model names the
        Linears of a block (gptq.py:88-92, `n_out_dict`); `names` is that order.  A dict name -> count in `n_outs`
        needs no call."""
        self.n_out_dict = {name: self.n_outs[i] for i, name in enumerate(names)}

    @staticmethod
    def _layer_kind(layer):
        """'conv2d' (weight [out, in, kh, kw], inputs unfolded), 'conv1d' (transformers.Conv1D: weight [in, out]) or
        'linear' (anything else with a [out, in] weight), as gptq.py:130-133, 262-278 tell them apart."""
        if isinstance(layer, torch.nn.Conv2d):
            return 'conv2d'
        cls = type(layer)
        if cls.__name__ == 'Conv1D' and cls.__module__.split('.')[0] == 'transformers':
            return 'conv1d'
        return 'linear'

    def _weight_2d(self, layer):
        """The layer's weight as the [out_features, in_features] matrix the loop works on (gptq.py:129-133)."""
        w = layer.weight.data
        kind = self._layer_kind(layer)
        if kind == 'conv2d' or w.dim() > 2:
            w = w.flatten(1)
        elif kind == 'conv1d':
            w = w.t()
        return w

    # -- Hessian (gptq.py:253-308) ---------------------------------------------
    @torch.no_grad()
    def layer_init(self, layer, name):
        K = self._weight_2d(layer).shape[1]
        self.layers_cache.setdefault(name, {})
        slices = self.hessian_shares(K)
        acc = torch.zeros((slices, K, K), device=self.dev)
        self.layers_cache[name]['H'] = acc[0]
        self.layers_cache[name]['H_shares'] = acc if slices > 1 else None
        self.layers_cache[name]['shares_apart'] = False
        self.layers_cache[name]['nsamples'] = 0
        self.layers_cache[name]['n_in_H'] = 0
        self.layers_cache[name]['calls'] = 0
        for k in ('stage', 'stage_lo', 'stage_fill', 'stage_batches', 'last_stage', 'last_key', 'last_ref', 'manual_share',
                  'share_flag', 'hws', 'hws_key'):
            self.layers_cache[name].pop(k, None)
        self.layers_cache[name]['columns'] = K
        self.layers_cache[name]['kind'] = self._layer_kind(layer)
        self.layers_cache[name].pop('leader', None)
        self.layers_cache[name].pop('followers', None)

    @torch.no_grad()
    def subset_init(self, subset):
        self.named_layers = subset['layers']
        for name in self.named_layers:
            self.layers_cache[name] = {}
            self.layer_init(self.named_layers[name], name)

    def share_input(self, names):
        """Layers that see the same input (q/k/v, gate/up) may share one Hessian and one
        Cholesky chain: the first name accumulates, the others alias it."""
        leader = names[0]
        for n in names[1:]:
            self.layers_cache[n]['H'] = self.layers_cache[leader]['H']
            self.layers_cache[n]['H_shares'] = None
            self.layers_cache[n]['leader'] = leader
            self.layers_cache[n]['manual_share'] = True
        self.layers_cache[leader]['leader'] = leader
        self.layers_cache[leader]['manual_share'] = True

    @staticmethod
    def _input_key(t):
        """Identity of an input tensor as the hooks hand it over: same memory, same layout, same type.  (The version
        counter is left out on purpose: `inp[0].data` is a fresh alias whose counter always reads 0.)"""
        return (t.data_ptr(), tuple(t.shape), tuple(t.stride()), t.dtype)

    def _same_tokens(self, lead, inp, tokens, K):
        """Queues the comparison of a follower's tokens with the copy its leader staged from the same memory when its
        own hook ran (lcq_compare_bytes; a difference sets the leader's `share_flag`, read where the Hessian is
        consumed).  False if that copy is not there to compare with."""
        if not self.share_verify:
            return True
        t_last = lead.get('last_stage', (0, 0))[0]
        stage = lead.get('stage')
        if stage is None or t_last != tokens or lead.get('stage_fill', 0) < tokens:
            return False
        flag = lead.get('share_flag')
        if flag is None:
            flag = lead['share_flag'] = torch.zeros(1, dtype=torch.int32, device=stage.device)
        es = stage.element_size()
        off = (lead['stage_fill'] - tokens) * K * es
        nbytes = tokens * K * es
        lo = lead.get('stage_lo')
        lib, st = L.lib(), L.stream()
        if lo is not None:                               # fp32 activations: both bf16 halves
            hi_, lo_ = self._halves(inp.reshape((-1, K)).contiguous())
            L.check(lib.lcq_compare_bytes(L.ptr(hi_), ctypes.c_void_p(stage.data_ptr() + off), L.i64(nbytes), L.ptr(flag), st),
                    'lcq_compare_bytes')
            L.check(lib.lcq_compare_bytes(L.ptr(lo_), ctypes.c_void_p(lo.data_ptr() + off), L.i64(nbytes), L.ptr(flag), st),
                    'lcq_compare_bytes')
            return True
        src = inp
        if not (inp.is_contiguous() and inp.data_ptr() % 16 == 0):
            src = inp.reshape((-1, K)).contiguous()
        if nbytes % 16 != 0 or (stage.data_ptr() + off) % 16 != 0 or src.data_ptr() % 16 != 0:
            return False
        L.check(lib.lcq_compare_bytes(ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(stage.data_ptr() + off), L.i64(nbytes),
                                      L.ptr(flag), st), 'lcq_compare_bytes')
        return True

    def _follow(self, name, cache, key, separable, inp, tokens, K):
        """Identical inputs need one Hessian.  The hooks of q/k/v (or gate/up) receive the very same tensor on
        every forward pass (gptq.py:246-251), so a Linear whose every call so far got the tensor that an earlier
        Linear of the subset got for the same call follows that Linear: it owns no Hessian and no Cholesky chain
        (the results are bit-identical to separate accumulation, the arithmetic being the same).  "The same tensor"
        is decided by address, layout and type, and every such call is then compared on the device with the tokens
        the leader staged (_same_tokens), because an in-place write between two hooks leaves no trace on the host.
        Returns True if this call is covered by the Linear it follows.  The first call that differs in its key ends
        the arrangement: the follower takes a copy of the Hessian and of the staged tokens as they were before that
        call and goes on alone."""
        calls = cache['calls']
        lead_name = cache.get('leader', name)
        if cache.get('manual_share'):
            return lead_name != name
        if lead_name != name:                             # following: does this call match the leader's?
            lead = self.layers_cache.get(lead_name)
            if lead is not None and lead.get('calls', 0) == calls + 1 and lead.get('last_key') == key \
                    and self._same_tokens(lead, inp, tokens, K):
                return True
            self._unfollow(name, cache, lead)
            return False
        if not (self.auto_share and separable) or calls != 0 or self.owq or cache.get('followers'):
            return False
        for other, oc in self.layers_cache.items():       # first call: is there a Linear that just got this tensor?
            if other == name or oc.get('leader', other) != other or 'H' not in oc or oc.get('manual_share'):
                continue
            if oc.get('calls', 0) == 1 and oc.get('last_key') == key and oc.get('last_stage', (0, 0))[0] > 0 \
                    and oc['H'].shape == cache['H'].shape and self._same_tokens(oc, inp, tokens, K):
                cache['leader'] = other
                cache['H'] = oc['H']
                cache['H_shares'] = None
                oc['leader'] = other
                oc.setdefault('followers', []).append(name)
                return True
        return False

    def _unfollow(self, name, cache, lead):
        """Give a follower its own Hessian: the state of the Linear it followed, without that Linear's latest call
        when the follower has not seen it.  (That call is still in the staging buffer then: a full buffer is folded at
        the start of the next call, not at the end of the one that filled it, and whatever folds the buffer at another
        time first releases the followers that are a call behind, _release_laggards.)"""
        cache['leader'] = name
        if lead is None or 'H' not in lead:
            raise L.LcqError(f'{name} followed a Linear whose Hessian is gone')
        if name in lead.get('followers', ()):
            lead['followers'].remove(name)
        ahead = lead['calls'] - cache['calls']            # 0 or 1
        fill, batches = lead.get('stage_fill', 0), lead.get('stage_batches', 0)
        if ahead:
            t_last, b_last = lead.get('last_stage', (0, 0))
            if ahead > 1 or t_last == 0 or fill < t_last:
                raise L.LcqError(f'{name}: the input differs from the one of {lead.get("leader")} after a call that was '
                                 'folded into the shared Hessian directly; set special.auto_share: False')
            fill, batches = fill - t_last, batches - b_last
        if lead.get('H_shares') is not None:              # every share as it is: the same state, nothing summed early
            cache['H_shares'] = lead['H_shares'].clone()
            cache['H'] = cache['H_shares'][0]
        else:
            cache['H_shares'] = None
            cache['H'] = lead['H'].clone()
        cache['shares_apart'] = lead.get('shares_apart', False)
        cache['n_in_H'] = lead.get('n_in_H', 0)
        cache['upper_only'] = lead.get('upper_only', False)
        if lead.get('share_flag') is not None:            # what was compared so far concerns this Hessian too
            cache['share_flag'] = lead['share_flag'].clone()
        for k in ('stage', 'stage_lo', 'stage_fill', 'stage_batches', 'last_stage'):
            cache.pop(k, None)
        if fill > 0:
            cache['stage'] = torch.empty_like(lead['stage'])
            cache['stage'][:fill].copy_(lead['stage'][:fill])
            cache['stage_lo'] = None
            if lead.get('stage_lo') is not None:
                cache['stage_lo'] = torch.empty_like(lead['stage_lo'])
                cache['stage_lo'][:fill].copy_(lead['stage_lo'][:fill])
            cache['stage_fill'], cache['stage_batches'] = fill, batches

    def _release_laggards(self, lead_name, lead):
        """Followers that have not seen their leader's latest call yet (it skipped a forward pass, or H is being read
        between the two hooks of one pass) get their own Hessian now, while that call can still be told apart from
        the rest: it is the last one in the staging buffer."""
        for n in list(lead.get('followers', ())):
            c = self.layers_cache.get(n)
            if c is None or c.get('leader') != lead_name:
                lead['followers'].remove(n)
            elif c['calls'] < lead['calls']:
                self._unfollow(n, c, lead)

    @torch.no_grad()
    def add_batch(self, layer, name, inp, out=None):
        # Called once per Linear per calibration batch (896 times for one decoder layer): the work up to the return for
        # a Linear that follows another one, and up to the staging copy otherwise, creates no tensor views.
        cache = self.layers_cache[name]
        if not inp.is_cuda:
            raise L.LcqError('liblcq operates on GPU tensors only (no CPU fallback)')
        kind = cache.get('kind', 'linear')
        if kind == 'conv2d':                            # gptq.py:268-278: patches as tokens, [N, L, C*kh*kw]
            inp = torch.nn.functional.unfold(inp, layer.kernel_size, dilation=layer.dilation, padding=layer.padding,
                                             stride=layer.stride).transpose(1, 2)
        shape = inp.shape
        key = (inp.data_ptr(), shape, inp.stride(), inp.dtype)
        nd = len(shape)
        tmp = 1 if nd == 2 else shape[0]
        K = shape[-1]
        tokens = shape[0] if nd == 2 else (shape[0] * shape[1] if nd == 3 else shape[0])
        if nd > 3 or K != cache['columns']:
            raise L.LcqError(f'add_batch: input of shape {tuple(shape)} for a layer with {cache["columns"]} input features')
        if inp.dtype not in (torch.bfloat16, torch.float16, torch.float32):
            raise NotImplementedError(f'add_batch takes bf16 / fp16 / fp32 activations; got {inp.dtype}')
        assert tokens % self.chunk_num == 0, \
            f'Error: inp.shape[1] ({tokens}) cannot be evenly divided by chunk_num.'
        defer = self.hessian_fold(K)
        if self._follow(name, cache, key, defer > 1 and kind == 'linear', inp, tokens, K):
            cache['calls'] += 1
            cache['nsamples'] += tmp
            return                                      # the Linear it follows accumulates
        if cache.get('followers'):
            self._release_laggards(name, cache)         # a follower that skipped the previous call goes its own way
        cache['last_key'] = key
        cache['last_ref'] = inp                         # keeps the memory from being handed to another tensor meanwhile
        cache['upper_only'] = True
        # fp32 activations (gptq.py:289 `chunk.float()` keeps them fp32): staged as two bf16 halves, x = hi + lo
        split = inp.dtype == torch.float32
        sdtype = torch.bfloat16 if split else inp.dtype
        # Stage a copy of the tokens and fold several calls into one launch: the window
        # H <- H*n/(n+b1) + 2/(n+b1)*S1, then H <- H*(n+b1)/(n+b1+b2) + 2/(n+b1+b2)*S2, ...
        # telescopes to H*n/N + (2/N)*(S1+S2+...), N = n + b1 + b2 + ..., so one launch over the
        # concatenated tokens gives the same H while reading and writing it once.  A full buffer is folded at the
        # start of the next call that needs room (or when H is asked for), so the latest call can still be told
        # apart from H when a follower needs the state before it.  (`calls` counts the calls whose tokens are in
        # the buffer or in H: it moves only once this call's tokens are.)
        stage = cache.get('stage')
        if defer > 1:
            if stage is not None and (stage.dtype != sdtype or split != (cache.get('stage_lo') is not None)
                                      or cache['stage_fill'] + tokens > stage.shape[0]):
                self._flush(cache)
                if stage.dtype != sdtype or split != (cache.get('stage_lo') is not None) or tokens > stage.shape[0]:
                    stage = None                        # another type, or a call larger than the whole buffer
            if stage is None:
                stage = torch.empty((defer * tokens, K), dtype=sdtype, device=inp.device)
                cache['stage'] = stage
                cache['stage_lo'] = torch.empty_like(stage) if split else None
                cache['stage_fill'] = 0
                cache['stage_batches'] = 0
            f = cache['stage_fill']
            nbytes = tokens * K * stage.element_size()
            dst = stage.data_ptr() + f * K * stage.element_size()
            if not split and key[0] % 16 == 0 and nbytes % 16 == 0 and dst % 16 == 0 and inp.is_contiguous():
                L.check(L.lib().lcq_stage_copy(ctypes.c_void_p(key[0]), ctypes.c_void_p(dst), ctypes.c_int64(nbytes),
                                               L.stream()),
                        'lcq_stage_copy')
            else:
                x = inp.reshape((-1, K)).contiguous()
                if split:
                    self._halves(x, stage[f:f + tokens], cache['stage_lo'][f:f + tokens])
                else:
                    stage[f:f + tokens].copy_(x)
            cache['stage_fill'] = f + tokens
            cache['stage_batches'] += tmp
            cache['last_stage'] = (tokens, tmp)
            cache['calls'] += 1
            cache['nsamples'] += tmp
            return
        # one launch per call (hessian_defer: 1): nothing is staged, and nothing is shared (see _follow)
        cache['last_stage'] = (0, 0)
        cache['calls'] += 1
        cache['nsamples'] += tmp
        self._accumulate(cache, *self._halves(inp.reshape((-1, K)).contiguous()), tmp)

    def hessian_fold(self, K):
        """add_batch calls folded into one Hessian launch for a Linear with K input features.  'auto': 4 calls of 2048
        tokens at K = 14336 (1.5 ms per launch; longer launches run at a lower sustained clock and are slower per
        token), 8 up to K = 8192, 16 up to K = 4096 (the longer the launch, the smaller the share of its ramp and tail,
        and the more tokens each of its shares gets, see hessian_shares)."""
        if self.hessian_defer == 'auto':
            return 16 if K <= 4096 else (8 if K <= 8192 else 4)
        return self.hessian_defer

    def hessian_shares(self, K):
        """Token shares of one Hessian launch for K input features (lcq_hessian_accum_sliced).  A launch has one
        workgroup per 256 x 128 tile that reaches the upper triangle and the chip has 512 workgroup slots: K = 4096
        gives 272 tiles, one workgroup on most CUs, whose four waves cannot hide their own latencies.  Cutting the
        tokens of the launch into three shares with an accumulator each puts 816 workgroups on the chip; the
        accumulators are summed when H is asked for.  'auto' follows what was measured on 128 calls of 2048 tokens
        (ms, one share -> best count): K=1024 4.4 -> 1.6 (8), 2048 4.6 -> 2.0 (5), 3072 5.0 -> 3.3 (3), 4096 5.8 -> 5.1
        (3), 6144 11.9 -> 10.6 (2), 8192 18.6 -> 17.6 (2); one share is best at K = 5120, 7168, 11008, 14336 (every
        share reads and writes its accumulator once per launch)."""
        if self.hessian_slices != 'auto':
            return max(1, self.hessian_slices)
        ntr, ntc = (K + 255) // 256, (K + 127) // 128
        tiles = sum(max(ntc - 2 * r, 0) for r in range(ntr))
        if tiles <= 40:
            return 8
        if tiles <= 100:
            return 5
        if tiles <= 300:
            return 3
        if 512 < tiles < 1536 and tiles % 512 < 128:      # a round or two of workgroups and a small rest
            return 2
        return 1

    def _halves(self, x, hi=None, lo=None):
        """(x, None) for 16-bit activations; for fp32 the two bf16 halves hi = bf16(x), lo = bf16(x - hi)."""
        if x.dtype != torch.float32:
            return x, None
        hi = torch.empty(x.shape, dtype=torch.bfloat16, device=x.device) if hi is None else hi
        lo = torch.empty(x.shape, dtype=torch.bfloat16, device=x.device) if lo is None else lo
        L.check(L.lib().lcq_split_f32_bf16(L.ptr(x), L.i64(x.numel()), L.ptr(hi), L.ptr(lo), L.stream()), 'lcq_split_f32_bf16')
        return hi, lo

    def _accumulate(self, cache, x, x_lo, batches):
        """H <- H*n/(n+b) + 2/(n+b) * x^T x for the n batches already inside H (gptq.py:279-294).
        x: [tokens, K] view with unit column stride (rows may be padded); x_lo: the low halves of fp32 activations
        (then x holds the high halves and x^T x is the sum of the four products of the halves)."""
        n = cache.get('n_in_H', 0)
        alpha = n / (n + batches)
        beta = 2.0 / (n + batches)
        cache['n_in_H'] = n + batches
        H = cache['H']
        shares = cache.get('H_shares')
        cache['shares_apart'] = shares is not None
        lib, code = L.lib(), L.i32(L.dtype_code(x.dtype))
        K, T = H.shape[0], x.shape[0]
        dims = (L.i64(T), L.i64(x.stride(0)))
        if shares is None:
            # one accumulator: the launch that fills its last round of workgroups (lcq_hessian_accum_balanced), with a
            # scratch buffer kept per Linear; where no split pays the call is the plain update
            key = (K, T)
            if cache.get('hws_key') != key:
                nbytes = lib.lcq_hessian_balanced_workspace_bytes(L.i64(K), L.i64(T))
                cache['hws'] = torch.empty(nbytes, dtype=torch.uint8, device=H.device) if nbytes > 0 else None
                cache['hws_key'] = key
            ws = cache['hws']
            tail = (L.ptr(ws), L.i64(0 if ws is None else ws.numel()), L.stream())

            def launch(a, b, al):
                L.check(lib.lcq_hessian_accum_balanced(L.ptr(H), L.i64(K), L.ptr(a), L.ptr(b), code, *dims, L.f32(al), L.f32(beta),
                                                       *tail), 'lcq_hessian_accum_balanced')
        else:
            sl = (L.i32(shares.shape[0]), L.i64(shares.stride(0)), L.stream())

            def launch(a, b, al):
                L.check(lib.lcq_hessian_accum_sliced(L.ptr(H), L.i64(K), L.ptr(a), L.ptr(b), code, *dims, L.f32(al), L.f32(beta),
                                                     *sl), 'lcq_hessian_accum_sliced')
        if x_lo is None:
            launch(x, x, alpha)
            return
        for a, b, al in ((x_lo, x_lo, alpha), (x, x_lo, 1.0), (x_lo, x, 1.0), (x, x, 1.0)):      # small terms first
            launch(a, b, al)

    def _flush(self, cache):
        """Fold the staged tokens into H."""
        if cache.get('stage_fill', 0) > 0:
            lo = cache.get('stage_lo')
            self._accumulate(cache, cache['stage'][:cache['stage_fill']], None if lo is None else lo[:cache['stage_fill']],
                             cache['stage_batches'])
            cache['stage_fill'] = 0
            cache['stage_batches'] = 0
        cache['last_stage'] = (0, 0)                     # the latest call is inside H now

    def _settle(self, name):
        """H of `name` (or of the layer it aliases) with no tokens left in staging."""
        cache = self.layers_cache[name]
        lead_name = cache.get('leader', name)
        lead = self.layers_cache.get(lead_name, cache)
        if lead.get('followers'):
            self._release_laggards(lead_name, lead)
            if cache.get('leader', name) != lead_name:   # `name` itself was a call behind: it owns its Hessian now
                lead = cache
        self._flush(lead)
        lead.pop('stage', None)
        lead.pop('stage_lo', None)
        if lead.get('shares_apart'):                      # the token shares of the launches back into the one H
            sh = lead['H_shares']
            L.check(L.lib().lcq_hessian_gather_slices(L.ptr(sh), L.i64(sh.shape[1]), L.i32(sh.shape[0]), L.i64(sh.stride(0)),
                                                      L.stream()), 'lcq_hessian_gather_slices')
            lead['shares_apart'] = False
        return cache

    _SHARE_MSG = ('a Linear shared the Hessian of another Linear that was handed the same tensor, but the tensor did not '
                  'hold the same values at the two hooks (it was written in place in between); set special.auto_share: False')

    def hessian(self, name):
        """The full symmetric H of a layer (fills the lower triangle on demand)."""
        cache = self._settle(name)
        H = cache['H']
        flag = self.layers_cache.get(cache.get('leader', name), cache).get('share_flag')
        if flag is not None and int(flag.item()) != 0:
            raise L.LcqError(self._SHARE_MSG)
        if cache.get('upper_only', False) or self.layers_cache.get(cache.get('leader', name), {}).get('upper_only'):
            L.check(L.lib().lcq_symmetrize(L.ptr(H), L.i64(H.shape[0]), L.stream()), 'lcq_symmetrize')
            cache['upper_only'] = False
        return H

    def hessian_sorting(self, name):
        """gptq.py:58-64: act-order permutation from the raw diagonal."""
        H = self._settle(name)['H']
        if not self.owq:
            if self.actorder:
                self.perm = torch.argsort(torch.diag(H), descending=True)
            return
        # OWQ (gptq.py:66-83; its act-order branch is unreachable, add_quant_config switches act-order off):
        # the n_out columns with the largest Hessian diagonal go last, the others keep their order
        temp_mask = torch.full([self.columns], True, device=self.dev)
        descending_ids = torch.argsort(torch.diag(H), descending=True)
        temp_mask[descending_ids[: self.n_out]] = False
        self.perm = torch.cat([torch.arange(self.columns, device=self.dev)[temp_mask], descending_ids[: self.n_out]])

    # -- per-layer driver (gptq.py:96-196) -----------------------------------------
    @torch.no_grad()
    def subset_transform(self, subset, input_feat=None, subset_kwargs=None):
        layers_dict = subset['layers']
        self._chains_ahead(layers_dict)
        self.last_errors = {}                            # summed loss of every Linear of the subset (device scalars)
        try:
            done = set()
            for name in layers_dict:
                if name in done:
                    continue
                mates = self._loop_mates(name, layers_dict)
                if len(mates) > 1:
                    self._fused_transform(mates, layers_dict)
                    done.update(mates)
                    continue
                self.layer_transform(layers_dict[name], name)
                self.last_errors[name] = self.last_error
                self.free(name)
        finally:
            # a chain started ahead may still be running on its side stream if a Linear raised or was skipped:
            # let the current stream wait for it before its tensors can go back to the allocator
            for leader in [k for k, v in self._shared.items() if v.get('ahead')]:
                done = self._shared[leader].pop('done', None)
                if done is not None:
                    torch.cuda.current_stream().wait_event(done)
                if not any(c.get('leader', n) == leader for n, c in self.layers_cache.items()):
                    del self._shared[leader]

    def _loop_mates(self, name, layers_dict):
        """The Linears of the subset whose column loops can run as one: they share `name`'s Hessian (so its column
        order and its factor U) and have weights of the same width.  [name] alone if there are none."""
        if not self.fuse_loops or self.owq:
            return [name]
        cache = self.layers_cache.get(name)
        if cache is None:
            return [name]
        leader = cache.get('leader', name)
        mates = [n for n in layers_dict
                 if n in self.layers_cache and self.layers_cache[n].get('leader', n) == leader
                 and self.layers_cache[n].get('columns') == cache.get('columns')]
        return mates if len(mates) > 1 and name in mates else [name]

    def _chains_ahead(self, layers_dict):
        """Start the Cholesky chain of every Linear of the subset now, each on its own stream.  A chain at K = 4096 is
        a few hundred short dependent launches (diagonal blocks, panel solves) that leave most of the chip idle, so
        the chains of q/k/v (or gate/up) run in about the time of one.  layer_transform then finds the finished factor
        exactly as it finds a shared one; results are the same as one by one."""
        if not self.chain_overlap or self.owq:           # OWQ: every Linear has its own column order
            return
        todo = []
        for name in layers_dict:
            cache = self.layers_cache.get(name)
            if cache is None or 'H' not in cache:
                continue
            leader = cache.get('leader', name)
            if leader in self._shared or leader in todo:
                continue
            todo.append(leader)
        if len(todo) < 2:
            return
        if not hasattr(self, '_side_streams'):
            self._side_streams = [torch.cuda.Stream(device=self.dev) for _ in range(3)]
        main = torch.cuda.current_stream()
        for i, leader in enumerate(todo):
            H = self._settle(leader)['H']
            K = H.shape[0]
            perm = torch.argsort(torch.diag(H), descending=True) if self.actorder else None
            dead = torch.diag(H) == 0
            ws_bytes = L.lib().lcq_chol_inv_upper_workspace_bytes(L.i64(K))
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=self.dev)
            status = self._status_words(leader)
            side = self._side_streams[i % len(self._side_streams)]
            side.wait_stream(main)
            with torch.cuda.stream(side):
                direct = self._block_factor_ok(K)
                chain = L.lib().lcq_chol_block_factor if direct else L.lib().lcq_chol_inv_upper
                L.check(chain(L.ptr(H), L.i64(K), L.ptr(perm), L.f32(self.percdamp), L.ptr(None), L.i64(0), L.ptr(H), L.ptr(ws),
                              L.i64(ws_bytes), L.ptr(status), L.stream()), 'Cholesky chain')
                status_host = self._post_status(status)
                done = side.record_event()
            for t in (ws, H, status, perm):              # allocated on the main stream, used on `side`: not to be
                if t is not None:                        # handed out again before the chain has run
                    t.record_stream(side)
            del ws
            self._shared[leader] = dict(U=H, perm=perm, status=status, dead=dead, done=done, ahead=True,
                                        status_host=status_host, direct=direct)

    def _status_words(self, leader):
        """[chain status, inputs of a shared Hessian differed] as two device words; the chain writes the first, the
        second is what the comparisons of add_batch left (queued earlier on the current stream)."""
        status = torch.zeros(2, dtype=torch.int32, device=self.dev)
        flag = self.layers_cache.get(leader, {}).get('share_flag')
        if flag is not None:
            status[1:].copy_(flag)
        return status

    @staticmethod
    def _post_status(status):
        """Queues, right behind the chain on the current stream, a copy of the chain's status words to pinned host
        memory and an event after it.  The check before the weights are written back waits for that event only, so the
        host does not wait for the column loop queued after the chain and the GPU does not run dry behind it."""
        host = torch.empty(2, dtype=torch.int32, pin_memory=True)
        host.copy_(status, non_blocking=True)
        copied = torch.cuda.Event()
        copied.record()
        return host, copied

    @torch.no_grad()
    def layer_transform(self, layer, name):
        self.initialize_qparams_and_prepare_weights(layer, name)
        W, H = self.process_hessian_and_weights(layer, name, for_loop=True)
        self.update_layer_with_transformed_weights(layer, W, H, name)

    def initialize_qparams_and_prepare_weights(self, layer, name):
        self.qparams = {}
        self.columns = self.layers_cache[name]['columns']
        if self.owq:
            nd = self.n_outs if isinstance(self.n_outs, dict) else getattr(self, 'n_out_dict', None)
            if nd is None:
                raise L.LcqError('OWQ: call set_block_linears(names) first (or give special.n_outs as a dict)')
            self.n_out = nd[name]
        else:
            self.n_out = 0
        self.n_nonout = self.columns - self.n_out
        cache = self.layers_cache[name]
        leader = cache.get('leader', name)
        if leader in self._shared and not self.owq:
            self.perm = self._shared[leader].get('perm')
        elif self.actorder or self.owq:
            self.hessian_sorting(name)

    def _block_factor_ok(self, K):
        """May the loop run on the block factor P of lcq_chol_block_factor instead of U?  Every group of the
        quantizer has to lie inside one 128-column block (or the parameters are given), K in whole blocks."""
        if not self.block_factor or self.owq or self.blocksize != 128 or K % 128 != 0:
            return False
        wq = self.wquantizer
        if wq.granularity == 'per_group' and not self.static_groups:
            return wq.group_size > 0 and 128 % wq.group_size == 0
        return True

    def process_hessian_and_weights(self, layer, name, out=None, for_loop=False):
        """-> (W [R,K] fp32 in processing order, Hinv: upper factor of the damped inverse).  `out`: where W goes
        (an [R, K] fp32 tensor, e.g. the rows of a larger one), else a new tensor.
        `for_loop` (what layer_transform passes): the second result is only going to feed weight_transform, so
        where the quantizer allows it (_block_factor_ok) it is the block factor P of lcq_chol_block_factor, which has
        U's diagonal blocks but needs no triangular inverse; weight_transform recognises it."""
        w = self._weight_2d(layer).contiguous()          # Conv2d: flatten(1); transformers.Conv1D: t() (gptq.py:129-133)
        R, K = w.shape
        cache = self._settle(name) if 'H' in self.layers_cache[name] else self.layers_cache[name]
        leader = cache.get('leader', name)
        H = cache['H']
        del cache['H']
        cache.pop('H_shares', None)

        self._setup_groups(layer, R, K)

        shared = self._shared.get(leader)
        if shared is None:
            is_shared = any(c.get('leader') == leader for n, c in self.layers_cache.items() if n != name) \
                or leader != name
            perm = self.perm if (self.actorder or self.owq) else None
            dead = torch.diag(H) == 0                       # before the chain rewrites H
            ws_bytes = L.lib().lcq_chol_inv_upper_workspace_bytes(L.i64(K))
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=self.dev)
            status = self._status_words(leader)
            direct = for_loop and self._block_factor_ok(K)
            chain = L.lib().lcq_chol_block_factor if direct else L.lib().lcq_chol_inv_upper
            L.check(chain(L.ptr(H), L.i64(K), L.ptr(perm), L.f32(self.percdamp), L.ptr(None), L.i64(0), L.ptr(H), L.ptr(ws),
                          L.i64(ws_bytes), L.ptr(status), L.stream()), 'Cholesky chain')
            del ws
            shared = dict(U=H, perm=perm, status=status, dead=dead, status_host=self._post_status(status), direct=direct)
            if is_shared:
                self._shared[leader] = shared
        elif 'done' in shared:                               # started by _chains_ahead on another stream
            torch.cuda.current_stream().wait_event(shared.pop('done'))
        U = shared['U']
        if shared.get('direct') and not for_loop:
            raise L.LcqError('the chain of this Hessian was started for the column loop (block factor, no inverse): '
                             'call process_hessian_and_weights(..., for_loop=True) or set special.block_factor: False')
        self._status = shared['status'][:1]
        self._status_host = shared['status_host']
        self._loop_factor = (U.data_ptr(), bool(shared.get('direct')))      # what weight_transform is going to be handed
        self._loop_W0 = None

        # weight.clone().float(), W[:, dead] = 0 and W[:, perm] in one pass
        W = torch.empty((R, K), dtype=torch.float32, device=w.device) if out is None else out
        if W.shape != (R, K) or W.dtype != torch.float32:
            raise L.LcqError(f'process_hessian_and_weights: `out` must be fp32 [{R}, {K}]')
        dead_u8 = shared['dead'].view(torch.uint8)
        L.check(L.lib().lcq_gptq_prepare_weights(L.ptr(w), L.i32(L.dtype_code(w.dtype)), L.i64(R), L.i64(K),
                                                 L.ptr(self.perm if (self.actorder or self.owq) else None), L.ptr(dead_u8),
                                                 L.ptr(W), L.stream()), 'lcq_gptq_prepare_weights')
        if self.actorder or self.owq:
            self.invperm = torch.argsort(self.perm)
            layer.buf_perm = self.perm
            layer.buf_invperm = self.invperm
            if self.owq:                                    # gptq.py:158-167
                layer.buf_n_nonout = torch.tensor(self.n_nonout)
                if self.wquantizer.granularity == 'per_channel':
                    _, layer.buf_scales, layer.buf_zeros, _, _ = self.wquantizer.get_tensor_qparams(
                        W[:, : self.n_nonout].contiguous())
                    self._setup_groups(layer, R, K)
        if self._loop_factor[1] and out is None:
            self._loop_W0 = W.clone()                    # the block factor needs the weights as they were before the loop
        return W, U

    def _setup_groups(self, layer, R, K):
        """Storage of the loop's qparams: [R, G] scales / zeros (+ column -> group map when static)."""
        wq = self.wquantizer
        self._gidx = None
        if wq.granularity == 'per_group':
            g = wq.group_size
            G = math.ceil(self.n_nonout / g)             # groups of the quantized columns (all K without OWQ)
            self._g, self._G = g, G
            if self.static_groups:
                self._scales = layer.buf_scales.reshape(R, G).float().contiguous()
                self._zeros = None if wq.sym else layer.buf_zeros.reshape(R, G).float().contiguous()
                cols = torch.arange(K, device=self.dev)
                if self.actorder:
                    cols = self.perm
                self._gidx = (cols // g).to(torch.int32).contiguous()
                self._static = True
            else:
                self._scales = torch.empty((R, G), device=self.dev)
                self._zeros = None if wq.sym else torch.empty((R, G), device=self.dev)
                self._static = False
        else:
            self._g, self._G = 0, 1
            self._scales = layer.buf_scales.reshape(R, 1).float().contiguous()
            self._zeros = None if wq.sym else layer.buf_zeros.reshape(R, 1).float().contiguous()
            self._static = True

    def update_layer_with_transformed_weights(self, layer, W, H, name):
        Losses = torch.empty_like(W)                     # the loop writes every entry of both
        tmp = torch.empty_like(W)
        self.weight_transform(W, H, Losses, tmp)
        self._check_status()
        self._write_back(layer, W, Losses, tmp)

    def _check_status(self):
        host, copied = self._status_host
        copied.synchronize()                             # the chain and the copy behind it; the loop may still be running
        if int(host[1]) != 0:
            raise L.LcqError(self._SHARE_MSG)
        if self.check_positive_definite and int(host[0]) != 0:
            raise torch.linalg.LinAlgError('GPTQ: the damped Hessian is not positive-definite')

    def _write_back(self, layer, W, Losses, tmp):
        """gptq.py:178-196 after the loop: summed loss, outlier columns, tmp[:, invperm], the weight and the qparams."""
        self.last_error = torch.sum(Losses)              # device scalar; .item() it to log like the reference
        if self.owq and self.n_out > 0:                  # the outlier columns stay in floating point, with the
            tmp[:, self.n_nonout:] = W[:, self.n_nonout:]      # updates of the loop (gptq.py:187-188)
            Losses[:, self.n_nonout:] = 0
            self.last_error = torch.sum(Losses)
        if self.actorder or self.owq:                    # tmp[:, invperm]
            out = torch.empty_like(tmp)
            L.check(L.lib().lcq_gptq_prepare_weights(L.ptr(tmp), L.i32(L.F32), L.i64(tmp.shape[0]), L.i64(tmp.shape[1]),
                                                     L.ptr(self.invperm), L.ptr(None), L.ptr(out), L.stream()),
                    'lcq_gptq_prepare_weights')
            tmp = out
        if self._layer_kind(layer) == 'conv1d':          # gptq.py:190-191
            tmp = tmp.t().contiguous()
        elif tmp._base is not None:                      # rows of a stacked matrix: the Linear gets storage of its own
            tmp = tmp.clone()
        layer.weight.data = tmp.reshape(layer.weight.shape)
        if self.wquantizer.granularity == 'per_group' and not self.static_groups:
            self.update_model_qparams(layer)

    @torch.no_grad()
    def _fused_transform(self, names, layers_dict):
        """Linears that share one chain (the same input, hence the same H, column order and U) go through the column
        loop as ONE weight matrix, their rows stacked: the loop has no term across rows (gptq.py:229-244), so every
        row gets what it would get alone, while the block kernel, which is bound by the length of its 128 sequential
        columns and not by the number of rows, and the update GEMMs run once instead of once per Linear."""
        parts, r0 = [], 0
        rows = [self._weight_2d(layers_dict[n]).shape[0] for n in names]
        K = self.layers_cache[names[0]]['columns']
        Wall = torch.empty((sum(rows), K), dtype=torch.float32, device=self.dev)
        U = None
        for n, R in zip(names, rows):
            layer = layers_dict[n]
            self.initialize_qparams_and_prepare_weights(layer, n)
            _, U = self.process_hessian_and_weights(layer, n, out=Wall[r0:r0 + R], for_loop=True)
            parts.append((n, layer, r0, R, self._scales, self._zeros))
            r0 += R
        if self._static:                                 # given parameters: one row block per Linear
            self._scales = torch.cat([p[4] for p in parts])
            self._zeros = None if parts[0][5] is None else torch.cat([p[5] for p in parts])
        else:
            self._scales = torch.empty((r0, self._G), device=self.dev)
            self._zeros = None if self.wquantizer.sym else torch.empty((r0, self._G), device=self.dev)
        if self._loop_factor[1]:
            self._loop_W0 = Wall.clone()
        Losses, tmp = torch.empty_like(Wall), torch.empty_like(Wall)
        self.weight_transform(Wall, U, Losses, tmp)
        self._check_status()
        scales, zeros = self._scales, self._zeros
        if not hasattr(self, 'last_errors'):
            self.last_errors = {}
        for n, layer, a, R, _, _ in parts:
            self._scales = scales[a:a + R]
            self._zeros = None if zeros is None else zeros[a:a + R]
            self._write_back(layer, Wall[a:a + R], Losses[a:a + R], tmp[a:a + R])
            self.last_errors[n] = self.last_error
            self.free(n)

    @torch.no_grad()
    def weight_transform(self, W, Hinv, Losses, tmp):
        """gptq.py:198-244, in place on W, Losses, tmp."""
        R, K = W.shape
        wq = self.wquantizer
        if not hasattr(self, '_scales') or self._scales.shape[0] != R:
            raise L.LcqError('weight_transform needs process_hessian_and_weights (or _setup_groups) first')
        flags = (L.FLAG_SYM if wq.sym else 0) | (0 if wq.round_zp else L.FLAG_NO_ROUND_ZP)
        # search_column_qparams (gptq.py:358-366) is wquantizer.get_tensor_qparams: min/max ranges are found inside
        # the block kernel; any other calibrator (mse, hqq) runs on the host side before the block that opens the
        # group, on the same columns of W the kernel would read, and the kernel takes the result as given.
        host_groups = (not self._static) and wq.calib_algo in ('mse', 'hqq', 'learnable')
        # Hinv is U, or the block factor P that process_hessian_and_weights(for_loop=True) made instead: the block
        # kernel then hands (quantized - original) to the deferred updates and needs the original weights
        W0 = None
        ptr_, direct_ = getattr(self, '_loop_factor', (None, False))
        if direct_ and ptr_ == Hinv.data_ptr():
            W0 = self._loop_W0
            if W0 is None or W0.shape != W.shape:
                raise L.LcqError('weight_transform on a block factor needs the weights before the loop (_loop_W0)')
        if self._static or host_groups:
            flags |= L.FLAG_STATIC
        g = self._g
        # Two-level deferral: after every pass only the rest of the current 1024-column window is
        # updated; the columns behind the window get one update per window (8x fewer passes over W).
        B = int(self.blocksize)
        window = 8 * B if B <= 128 else B * max(1, 1024 // B)
        Err = torch.empty((R, window), device=W.device)
        lib = L.lib()
        st = L.stream()
        qmin, qmax = L.f32(wq.qmin), L.f32(wq.qmax)
        n = self.n_nonout
        searched = not self._static and g > 0            # group ranges are searched while the loop runs

        def open_groups(c0, c1):
            """search_column_qparams (gptq.py:358-366) for the groups that open in [c0, c1), on W as it is now."""
            for idx in range((c0 + g - 1) // g * g, c1, g):
                _, s_, z_, _, _ = wq.get_tensor_qparams(W[:, idx:min(idx + g, n)].contiguous())
                self._scales[:, idx // g] = s_.reshape(-1).float()
                if not wq.sym:
                    self._zeros[:, idx // g] = z_.reshape(-1).float()

        for o0 in range(0, n, window):
            o1 = min(o0 + window, n)
            # A group that opens inside the window reads its whole column range of W (gptq.py:216-222), so the
            # per-pass updates reach to the end of the last such group; the window's deep update starts there.
            hi = o1
            if searched:
                last_open = (o1 - 1) // g * g
                if last_open >= o0:
                    hi = max(o1, min(last_open + g, n))
            for b1 in range(o0, o1, B):                  # the reference's blocks
                b2 = min(b1 + B, o1)
                # A block wider than 128 columns runs as several passes.  The reference reads a group's range from
                # the global W when the group opens (gptq.py:216-222), and the global W does not see a block's own
                # updates before the block ends (they go to the block-local copy W1, gptq.py:203, 240): the groups
                # that open in the later passes are therefore searched now, before the first pass touches their columns.
                if searched and b2 - b1 > 128:
                    open_groups(b1 + 128, b2)
                for i1 in range(b1, b2, 128):
                    i2 = min(i1 + 128, b2)
                    pass_flags = flags
                    if searched and i1 > b1:
                        pass_flags |= L.FLAG_STATIC       # every group of this pass has its parameters already
                    elif host_groups:
                        open_groups(i1, i2)
                    err_blk = Err[:, i1 - o0:]
                    L.check(lib.lcq_gptq_block(L.ptr(W), L.ptr(tmp), L.ptr(Losses), C_ptr(err_blk), L.i64(window), L.ptr(Hinv),
                                               L.ptr(W0), L.i64(R), L.i64(K), L.i64(n), L.i64(i1), L.i32(i2 - i1), L.i32(self._g), qmin,
                                               qmax, L.i32(pass_flags), L.ptr(self._scales), L.ptr(self._zeros), L.ptr(self._gidx),
                                               L.i64(self._G), st), 'lcq_gptq_block')
                    if i2 < hi:
                        L.check(lib.lcq_gptq_trailing(L.ptr(W), C_ptr(err_blk), L.i64(window), L.ptr(Hinv), L.i64(R), L.i64(K),
                                                      L.i64(i1), L.i64(i2), L.i64(i2), L.i64(hi), st), 'lcq_gptq_trailing')
            if hi < K:
                L.check(lib.lcq_gptq_trailing(L.ptr(W), L.ptr(Err), L.i64(window), L.ptr(Hinv), L.i64(R), L.i64(K),
                                              L.i64(o0), L.i64(o1), L.i64(hi), L.i64(K), st), 'lcq_gptq_trailing')

    # -- qparam bookkeeping (gptq.py:332-409) ---------------------------------------
    @torch.no_grad()
    def collect_layer_qparams(self, layer):
        """What collect_block_qparams (base_blockwise_quantization.py:348-376) registers per Linear."""
        _, scales, zeros, max_int, min_int = self.wquantizer.get_tensor_qparams(layer.weight.data)
        layer.buf_scales = scales.detach()
        layer.buf_zeros = zeros.detach()
        layer.buf_qmax = max_int.clone().to(self.dev)
        layer.buf_qmin = min_int.clone().to(self.dev)

    @torch.no_grad()
    def update_model_qparams(self, layer):
        layer.buf_scales = self._scales.reshape(-1, 1).clone()
        if not self.wquantizer.sym:
            layer.buf_zeros = self._zeros.reshape(-1, 1).clone()

    @torch.no_grad()
    def split_qparams(self, qparams):
        """gptq.py:332-341: a buffer as collect_block_qparams registers it, [R * G, 1] with the G groups of a row next
        to each other, -> a list of G tensors [R, 1]."""
        group_num = math.ceil(self.columns / self.wquantizer.group_size)
        per_row = qparams.reshape(-1, group_num)
        return [per_row[:, gi].reshape(-1, 1) for gi in range(group_num)]

    @torch.no_grad()
    def merge_qparams(self, qparams):
        """gptq.py:343-356: the inverse for per_group (a list of [R, 1] -> [R * G, 1]); per_head values repeated over
        the rows of their head; anything else as it is."""
        if isinstance(qparams, int):
            return qparams
        gran = self.wquantizer.granularity
        if gran == 'per_head':
            head_size = self.rows // self.head_num
            return qparams.reshape(-1).repeat_interleave(head_size).reshape(-1, 1)
        if gran == 'per_group':
            return torch.stack(list(qparams), dim=1).reshape(-1, 1)
        return qparams

    @torch.no_grad()
    def search_column_qparams(self, c_tensor, idx):
        """gptq.py:358-366: qparams of the column slab that starts at column `idx` (one group), kept as the current
        qparams and as group idx // group_size.  (weight_transform does this inside its kernel; the method serves
        callers that drive the loop themselves.)"""
        _, scale, zero, qmax, qmin = self.wquantizer.get_tensor_qparams(c_tensor)
        self.qparams = {'scale': scale, 'zero': zero, 'qmax': qmax, 'qmin': qmin}
        gi = idx // self.wquantizer.group_size
        if getattr(self, '_scales', None) is not None and gi < self._scales.shape[1]:
            self._scales[:, gi] = scale.reshape(-1).float()
            if self._zeros is not None:
                self._zeros[:, gi] = zero.reshape(-1).float()

    @torch.no_grad()
    def search_layer_qparams(self, layer):
        """gptq.py:368-377: the registered buffers of a per_channel / per_tensor / per_head layer as the current
        qparams."""
        scales = self.merge_qparams(layer.buf_scales)
        zeros = layer.buf_zeros if self.wquantizer.sym else self.merge_qparams(layer.buf_zeros)
        self.qparams = {'scale': scales, 'zero': zeros, 'qmax': layer.buf_qmax, 'qmin': layer.buf_qmin}

    @torch.no_grad()
    def search_group_qparams(self, layer):
        """gptq.py:379-395: the registered per-group buffers as the loop's group table (`groups`)."""
        G = math.ceil(self.columns / self.wquantizer.group_size)
        self._g, self._G = self.wquantizer.group_size, G
        self._scales = layer.buf_scales.reshape(-1, G).float().contiguous()
        self._zeros = None if self.wquantizer.sym else layer.buf_zeros.reshape(-1, G).float().contiguous()

    @property
    def groups(self):
        """The reference's list of per-group dicts, materialised from the [R, G] tensors."""
        out = []
        for gi in range(self._G):
            out.append({'scale': self._scales[:, gi:gi + 1],
                        'zero': torch.tensor(0.0) if self.wquantizer.sym else self._zeros[:, gi:gi + 1],
                        'qmax': self.wquantizer.qmax, 'qmin': self.wquantizer.qmin})
        return out

    # -- deploy-time partials (gptq.py:411-452) -----------------------------------------
    @torch.no_grad()
    def w_q(self, module, wquantizer):
        weight = module.weight.data
        args = {}
        args['scales'] = module.buf_scales
        args['zeros'] = module.buf_zeros if hasattr(module, 'buf_zeros') else None
        args['qmax'] = module.buf_qmax
        args['qmin'] = module.buf_qmin
        args['scales'] = args['scales'].to(self.model_dtype)
        return wquantizer.real_quant_weight_static(weight, args)

    @torch.no_grad()
    def w_qdq(self, module, wquantizer):
        weight = module.weight
        if self.need_perm:
            weight = module.weight[:, module.buf_perm]
        args = {}
        args['scales'] = module.buf_scales
        args['zeros'] = module.buf_zeros if hasattr(module, 'buf_zeros') else None
        args['qmax'] = module.buf_qmax
        args['qmin'] = module.buf_qmin
        if self.owq:
            fp_weight = weight[:, module.buf_n_nonout:]
        weight = wquantizer.fake_quant_weight_static(weight, args).to(self.model_dtype)
        if self.owq:
            weight[:, module.buf_n_nonout:] = fp_weight.to(self.model_dtype)
        if self.need_perm:
            weight = weight[:, module.buf_invperm]
        return weight

    @torch.no_grad()
    def free(self, name):
        self.H = None
        self.Losses = None
        self.Trace = None
        leader = self.layers_cache.get(name, {}).get('leader', name)
        self.layers_cache.pop(name, None)
        if leader in self._shared and not any(c.get('leader') == leader for c in self.layers_cache.values()):
            del self._shared[leader]

    @torch.no_grad()
    def ready(self):
        if 'scale' not in self.qparams:
            return False
        return torch.all(self.qparams['scale'] != 0)
