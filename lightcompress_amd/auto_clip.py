"""AWQ weight clipping with the reference's class API, running on liblcq.

Mirrors ``llmc/compression/quantization/auto_clip.py`` of ModelTC/LightCompress (class
``AutoClipper``): ``run`` (:45-81), ``auto_clip_layer`` (:83-191), ``apply_clip`` (:193-229),
``fake_quantize_weight`` (:258-274) and ``fake_quantize_input`` (:276-281).

On this path: ``clip_version='v1'``, weight-only (``w_only=True``), a per_group weight quantizer with
``group_size`` 128 and bf16 weights / activations - the configuration of the AWQ recipes.  Everything
else raises ``NotImplementedError``.  One process, one GPU: the all-reduce of ``run`` is not issued.

The search itself is one kernel (``lcq_awq_clip_search``): the reference's [256, T, G, 128] broadcast
products, two per shrink step, are a bf16 MFMA contraction there.
"""
from __future__ import annotations

import torch

from . import _lib as L


class AutoClipper:
    def __init__(self, w_only, wquantizer, aquantizer, clip_version, clip_sym, save_clip, padding_mask):
        self.wquantizer = wquantizer
        self.aquantizer = aquantizer
        self.clip_version = clip_version
        self.clip_sym = clip_sym
        self.save_clip = save_clip
        self.padding_mask = padding_mask
        self.weight_clips = {}
        self.w_only = w_only
        self.logit = lambda x: torch.log(x / (1 - x))
        self.last_errs = None            # [R, G, n_steps] fp32 of the last auto_clip_layer call

    # -- auto_clip.py:45-81 ----------------------------------------------------------------------
    @torch.no_grad()
    def run(self, block, block_idx, input_feat, n_sample_token):
        for n, m in block.named_modules():
            if not isinstance(m, torch.nn.Linear):
                continue
            if any(_ in n for _ in ['q_', 'k_', 'query', 'key', 'Wqkv']):
                if self.clip_version == 'v2':
                    m.register_buffer('buf_upbound_factor', None)
                    m.register_buffer('buf_lowbound_factor', None)
                continue
            inputs = [torch.cat(input_feat[n])] if len(input_feat[n]) != 1 else input_feat[n]
            max_val, min_val = self.auto_clip_layer(block_idx, n, m.weight, inputs, n_sample_token=n_sample_token)
            self.apply_clip(block_idx, m, min_val, max_val, n)

    def _check(self):
        if self.clip_version != 'v1':
            raise NotImplementedError("clip_version 'v2' (learnable ranges) is not on this path")
        if not self.w_only:
            raise NotImplementedError('activation fake-quant inside the clip search (w_only=False) is not on this path')
        wq = self.wquantizer
        if wq.granularity != 'per_group' or wq.group_size != 128:
            raise NotImplementedError('the clip search kernel covers per_group quantizers with group_size 128')
        if getattr(wq, 'quant_type', 'int-quant') != 'int-quant' or not wq.round_zp:
            raise NotImplementedError('the clip search kernel covers IntegerQuantizer with round_zp')

    # -- auto_clip.py:83-191 -----------------------------------------------------------------------
    @torch.no_grad()
    def auto_clip_layer(self, block_idx, layer_name, w, inputs, n_grid=20, max_shrink=0.5, n_sample_token=512,
                        eps=0.0):
        assert w.dim() == 2
        self._check()
        wq = self.wquantizer
        group_size = wq.group_size
        w = w.data if isinstance(w, torch.nn.Parameter) else w
        R, K = w.shape
        if w.dtype != torch.bfloat16:
            raise NotImplementedError(f'the clip search kernel multiplies on bf16 MFMA; got {w.dtype}')
        if K % group_size != 0:
            raise NotImplementedError('in_features must be a multiple of the group size')
        oc_batch_size = 256 if R % 256 == 0 else 64      # the reference's batching; only its assertion matters here
        assert R % oc_batch_size == 0
        xs = []
        for i in range(len(inputs)):
            inputs[i] = inputs[i].to(w.device)
            x = inputs[i].view(-1, inputs[i].shape[-1])
            if self.padding_mask and self.padding_mask[i].numel() == x.shape[0]:
                x = x[self.padding_mask[i].flatten().bool()]
            if n_sample_token is None:
                n_sample_token = min(x.shape[0], 512)
            step_size = max(1, x.shape[0] // n_sample_token)
            xs.append(x[0::step_size])
        if len({x.shape[0] for x in xs}) != 1:
            raise NotImplementedError('inputs of different token counts: the per-input means are not one mean')
        x = torch.cat(xs).to(torch.bfloat16).contiguous()  # equal sizes: mean of the means == mean over all tokens
        wc = w.contiguous()
        G = K // group_size
        n_steps = int(max_shrink * n_grid)
        best_max = torch.empty((R, G), dtype=torch.bfloat16, device=w.device)
        best_min = torch.empty((R, G), dtype=torch.bfloat16, device=w.device)
        errs = torch.empty((R, G, n_steps), dtype=torch.float32, device=w.device)
        flags = L.FLAG_SYM if wq.sym else 0
        L.check(L.lib().lcq_awq_clip_search(L.ptr(wc), L.ptr(x), L.i64(R), L.i64(K), L.i64(x.shape[0]), L.i32(n_grid),
                                            L.i32(n_steps), L.i32(1 if self.clip_sym else 0), L.f32(float(wq.qmin)),
                                            L.f32(float(wq.qmax)), L.i32(flags), L.ptr(best_max), L.ptr(best_min),
                                            L.ptr(errs), L.stream()), 'lcq_awq_clip_search')
        self.last_errs = errs
        return best_max.unsqueeze(-1), best_min.unsqueeze(-1)       # [R, G, 1] like .squeeze(1) of [R, 1, G, 1]

    # -- auto_clip.py:193-229 ----------------------------------------------------------------------
    @torch.no_grad()
    def apply_clip(self, block_idx, layer, min_val, max_val, layer_name):
        if self.clip_version != 'v1':
            raise NotImplementedError("clip_version 'v2' (learnable ranges) is not on this path")
        w = layer.weight.data
        max_val = max_val.to(w.device)
        if self.clip_sym:
            min_val = -max_val
        layer.weight.data = self._clamp(w, min_val.to(w.device), max_val)

    def _clamp(self, w, min_val, max_val):
        R, K = w.shape
        G = max_val.shape[1]
        wc = w.contiguous()
        lo = min_val.reshape(R, G).to(w.dtype).contiguous()
        hi = max_val.reshape(R, G).to(w.dtype).contiguous()
        out = torch.empty_like(wc)
        L.check(L.lib().lcq_clamp_groups(L.ptr(wc), L.dtype_code(wc.dtype), L.i64(R), L.i64(K), L.i32(K // G), L.ptr(lo),
                                         L.ptr(hi), L.ptr(out), L.stream()), 'lcq_clamp_groups')
        return out

    # -- auto_clip.py:258-281 ----------------------------------------------------------------------
    def fake_quantize_weight(self, w, min_val, max_val, org_min_val, org_max_val):
        """v1: fake_quant_weight_dynamic(clamp(w, min_val, max_val)); w [R, K], ranges [R, G, 1]."""
        if self.clip_version != 'v1':
            raise NotImplementedError("clip_version 'v2' (learnable ranges) is not on this path")
        return self.wquantizer.fake_quant_weight_dynamic(self._clamp(w, min_val, max_val))

    def fake_quantize_input(self, block_idx, x, layer_name):
        if not self.w_only:
            return self.aquantizer.fake_quant_act_dynamic(x)
        return x
