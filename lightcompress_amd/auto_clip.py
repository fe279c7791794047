"""AWQ weight clipping with the reference's class API, running on liblcq.

Mirrors ``llmc/compression/quantization/auto_clip.py`` of ModelTC/LightCompress (class
``AutoClipper``): ``run`` (:45-81), ``auto_clip_layer`` (:83-191), ``apply_clip`` (:193-229),
``get_clip_factor`` (:231-256), ``fake_quantize_weight`` (:258-274) and ``fake_quantize_input`` (:276-281).
One process, one GPU: the all-reduce of ``run`` is not issued.

Two search paths:

* the default follows the reference's rounding sequence: every product of ``(x * w)`` rounded to the tensors' type,
  fp32 sums per group, the two sums rounded before they are subtracted, the squared difference rounded, the mean over
  tokens rounded (``lcq_group_dots``); weights go through the quantizer classes exactly as the reference's
  ``fake_quantize_weight`` / ``fake_quantize_input`` do.  It covers ``clip_version`` v1 and v2, ``w_only`` True and
  False, any group size or per_channel weights, bf16 and fp32, several inputs;
* ``AutoClipper.fast = True`` selects, where it applies (v1, weight-only, per_group 128, bf16, min/max integer
  quantizer), one bf16 MFMA kernel (``lcq_awq_clip_search``) that contracts the weight *difference* with the tokens
  and does not reproduce the rounding of the two sums: about 50x faster, same range on > 90 % of the groups.

``clip_version='v2'`` with a per_group quantizer fails in the reference (its static fake quant broadcasts
[ocb * G, gs] rows against [ocb, 1, G, 1] qparams); here it runs, with the qparams matched to the groups.
per_tensor weight quantizers are rejected: their range in the reference spans the 256 output rows of one search batch.
"""
from __future__ import annotations

import torch

from . import _lib as L
from .kernel import weight_cast_to_bf16, weight_cast_to_fp8
from .quant import _scaled


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
        self.fast = False                # True: the bf16 MFMA search kernel where it applies (see the module docstring)
        self.fp8_block_size = 128

    # -- auto_clip.py:45-81 ----------------------------------------------------------------------
    @torch.no_grad()
    def run(self, block, block_idx, input_feat, n_sample_token):
        for n, m in block.named_modules():
            if not isinstance(m, torch.nn.Linear):
                continue
            is_fp8_weight = m.weight.data.dtype == torch.float8_e4m3fn
            if is_fp8_weight:                              # block-wise float8 checkpoint: search on the bf16 weights
                m.weight.data = weight_cast_to_bf16(m.weight.data.contiguous(), m.weight_scale_inv.data.contiguous(),
                                                    self.fp8_block_size).to(torch.bfloat16)
            if any(_ in n for _ in ['q_', 'k_', 'query', 'key', 'Wqkv']):
                if self.clip_version == 'v2':
                    m.register_buffer('buf_upbound_factor', None)
                    m.register_buffer('buf_lowbound_factor', None)
                continue
            inputs = [torch.cat(input_feat[n])] if len(input_feat[n]) != 1 else input_feat[n]
            max_val, min_val = self.auto_clip_layer(block_idx, n, m.weight, inputs, n_sample_token=n_sample_token)
            self.apply_clip(block_idx, m, min_val, max_val, n)
            if is_fp8_weight:
                m.weight.data, m.weight_scale_inv.data = weight_cast_to_fp8(m.weight.data.contiguous(), self.fp8_block_size)

    def _fast_applies(self, w, inputs):
        wq = self.wquantizer
        return (self.fast and self.clip_version == 'v1' and self.w_only and wq.granularity == 'per_group'
                and wq.group_size == 128 and getattr(wq, 'quant_type', 'int-quant') == 'int-quant' and wq.round_zp
                and wq.calib_algo == 'minmax' and w.dtype == torch.bfloat16
                and all(x.dtype == torch.bfloat16 for x in inputs))

    @staticmethod
    def _rows_minmax(t2d):
        """amin / amax over the last dimension of a contiguous [rows, cols] tensor -> two [rows] tensors."""
        rows, cols = t2d.shape
        mn = torch.empty(rows, dtype=t2d.dtype, device=t2d.device)
        mx = torch.empty(rows, dtype=t2d.dtype, device=t2d.device)
        L.check(L.lib().lcq_minmax_rows(L.ptr(t2d), L.dtype_code(t2d.dtype), L.i64(rows), L.i64(cols), L.ptr(mn),
                                        L.ptr(mx), L.stream()), 'lcq_minmax_rows')
        return mn, mx

    @staticmethod
    def _group_dots(x, w, group_size, org=None):
        """(x * w).sum(dim=-1) of auto_clip.py:141,160 as [R, G, T]; with `org` the rounded error of :163 as [R, G]."""
        R, K = w.shape
        T, G = x.shape[0], K // group_size
        out = torch.empty((R, G) if org is not None else (R, G, T), dtype=w.dtype, device=w.device)
        L.check(L.lib().lcq_group_dots(L.ptr(x), L.ptr(w), L.dtype_code(w.dtype), L.i64(R), L.i64(K), L.i64(T),
                                       L.i32(group_size), L.ptr(None if org is not None else out), L.ptr(org),
                                       L.ptr(out if org is not None else None), L.stream()), 'lcq_group_dots')
        return out

    # -- auto_clip.py:83-191 -----------------------------------------------------------------------
    @torch.no_grad()
    def auto_clip_layer(self, block_idx, layer_name, w, inputs, n_grid=20, max_shrink=0.5, n_sample_token=512,
                        eps=0.0):
        assert w.dim() == 2
        wq = self.wquantizer
        if self.clip_version not in ('v1', 'v2'):
            raise Exception('Not support other clip version')
        if wq.granularity == 'per_tensor':
            raise NotImplementedError('per_tensor weight ranges span one 256-row search batch in the reference; '
                                      'not on this path')
        w = w.data if isinstance(w, torch.nn.Parameter) else w
        R, K = w.shape
        group_size = wq.group_size if wq.granularity == 'per_group' else K
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
            xs.append(x[0::step_size].contiguous())
        n_steps = int(max_shrink * n_grid)
        wc = w.contiguous()
        if self._fast_applies(wc, xs):
            if len({x.shape[0] for x in xs}) != 1:
                raise NotImplementedError('inputs of different token counts: the per-input means are not one mean '
                                          '(use fast = False)')
            return self._search_mfma(wc, torch.cat(xs) if len(xs) > 1 else xs[0], n_grid, n_steps)
        return self._search_exact(block_idx, layer_name, wc, xs, group_size, n_grid, n_steps, eps)

    def _search_mfma(self, wc, x, n_grid, n_steps):
        """Equal token counts: the mean of the per-input means is the mean over all tokens."""
        wq = self.wquantizer
        R, K = wc.shape
        G = K // 128
        best_max = torch.empty((R, G), dtype=torch.bfloat16, device=wc.device)
        best_min = torch.empty((R, G), dtype=torch.bfloat16, device=wc.device)
        errs = torch.empty((R, G, n_steps), dtype=torch.float32, device=wc.device)
        flags = L.FLAG_SYM if wq.sym else 0
        L.check(L.lib().lcq_awq_clip_search(L.ptr(wc), L.ptr(x), L.i64(R), L.i64(K), L.i64(x.shape[0]), L.i32(n_grid),
                                            L.i32(n_steps), L.i32(1 if self.clip_sym else 0), L.f32(float(wq.qmin)),
                                            L.f32(float(wq.qmax)), L.i32(flags), L.ptr(best_max), L.ptr(best_min),
                                            L.ptr(errs), L.stream()), 'lcq_awq_clip_search')
        self.last_errs = errs
        return best_max.unsqueeze(-1), best_min.unsqueeze(-1)       # [R, G, 1] like .squeeze(1) of [R, 1, G, 1]

    def _search_exact(self, block_idx, layer_name, wc, xs, group_size, n_grid, n_steps, eps):
        """The reference's loop with all output rows at once (rows are independent: its batches of 256 only bound
        memory).  Ranges and errors are [R, G, 1] tensors handled with the reference's own torch expressions; the
        [R, T, G, gs]-sized work is in kernels."""
        R, K = wc.shape
        G = K // group_size
        if wc.dtype not in (torch.bfloat16, torch.float32, torch.float16):
            raise NotImplementedError(f'the clip search covers bf16, fp16 and fp32 weights; got {wc.dtype}')
        if any(x.dtype != wc.dtype for x in xs):
            raise NotImplementedError('activations and weights of different types')
        mn, mx = self._rows_minmax(wc.view(R * G, group_size))
        org_min_val = mn.view(R, G, 1)
        org_max_val = torch.maximum(mx.abs(), mn.abs()).view(R, G, 1) if self.clip_sym else mx.view(R, G, 1)
        best_max_val = org_max_val.clone()
        best_min_val = org_min_val.clone()
        min_errs = torch.ones_like(org_max_val) * 1e9
        org_out = [self._group_dots(x, wc, group_size) for x in xs]
        # the quantized activations do not change from step to step (the reference recomputes them every time)
        q_xs = [self.fake_quantize_input(block_idx, x.view(1, x.shape[0], G, group_size), layer_name)
                .reshape(x.shape[0], K).contiguous() if not self.w_only else x for x in xs]
        errs = []
        for i_s in range(n_steps):
            if i_s == 0:
                if self.clip_version == 'v2' and not self.w_only:
                    i_s += eps
            max_val = _scaled(org_max_val, 1 - i_s / n_grid)       # (fp16: the fp32 product rounded, then the cast)
            min_val = -max_val if self.clip_sym else _scaled(org_min_val, 1 - i_s / n_grid)
            q_w = self.fake_quantize_weight(wc, min_val, max_val, org_min_val, org_max_val).contiguous()
            err_mean = 0
            for i in range(len(xs)):
                err = self._group_dots(q_xs[i], q_w, group_size, org=org_out[i]).view(min_errs.shape)
                err_mean = err_mean + err
            err_mean /= len(xs)
            errs.append(err_mean.float())
            cur_best_idx = err_mean < min_errs
            min_errs[cur_best_idx] = err_mean[cur_best_idx]
            best_max_val[cur_best_idx] = max_val[cur_best_idx]
            best_min_val[cur_best_idx] = min_val[cur_best_idx]
        self.last_errs = torch.cat(errs, dim=-1)
        return best_max_val, best_min_val

    # -- auto_clip.py:193-229 ----------------------------------------------------------------------
    @torch.no_grad()
    def apply_clip(self, block_idx, layer, min_val, max_val, layer_name):
        if self.clip_version == 'v1':
            w = layer.weight.data
            max_val = max_val.to(w.device)
            if self.clip_sym:
                min_val = -max_val
            layer.weight.data = self._clamp(w, min_val.to(w.device), max_val)
        elif self.clip_version == 'v2':
            up_factor, low_factor = self.get_clip_factor(block_idx, layer, min_val, max_val, layer_name)
            layer.register_buffer('buf_upbound_factor', up_factor)
            layer.register_buffer('buf_lowbound_factor', low_factor)
            if self.save_clip:
                if block_idx not in self.weight_clips:
                    self.weight_clips[block_idx] = dict()
                n = f'{layer_name}.weight_quantizer.'
                self.weight_clips[block_idx][n + 'upbound_factor'] = up_factor.cpu()
                self.weight_clips[block_idx][n + 'lowbound_factor'] = low_factor.cpu() if low_factor is not None else None
        else:
            raise Exception('Not support other clip version')

    # -- auto_clip.py:231-256 ----------------------------------------------------------------------
    def get_clip_factor(self, block_idx, layer, min_val, max_val, layer_name):
        org_min_val, org_max_val = self.wquantizer.get_minmax_range(self.wquantizer.reshape_tensor(layer.weight.data))
        org_val_shape = org_max_val.shape
        if self.clip_sym:
            abs_max_val = torch.max(org_max_val.abs(), org_min_val.abs())
            abs_max_val = abs_max_val.clamp(min=1e-5)
            abs_max_val = abs_max_val.reshape(*max_val.shape[:2], -1)
            up_factor = self.logit((max_val / abs_max_val))
            up_factor = up_factor.reshape(org_val_shape)
            low_factor = None
        else:
            org_max_val = org_max_val.reshape(*max_val.shape[:2], -1)
            up_factor = self.logit((max_val / org_max_val))
            up_factor = up_factor.reshape(org_val_shape)
            org_min_val = org_min_val.reshape(*min_val.shape[:2], -1)
            low_factor = self.logit((min_val / org_min_val))
            low_factor = low_factor.reshape(org_val_shape)
        return up_factor, low_factor

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
        """w [R, K]; ranges [R, G, 1] (the reference's [ocb, 1, G, 1] without the broadcast axis)."""
        if self.clip_version == 'v1':
            cur_w = self._clamp(w, min_val, max_val)
            q_w = self.wquantizer.fake_quant_weight_dynamic(cur_w)
        elif self.clip_version == 'v2':
            low_factor = self.logit((min_val / org_min_val))
            up_factor = self.logit((max_val / org_max_val))
            R, G = max_val.shape[:2]
            w3 = w.view(R, G, -1)
            tensor_range = self.wquantizer.get_learnable_range(w3, low_factor, up_factor)
            scales, zeros, qmax, qmin = self.wquantizer.get_qparams(tensor_range, w.device)
            args = {'scales': scales, 'zeros': zeros, 'qmax': qmax, 'qmin': qmin}
            q_w = self.wquantizer.fake_quant_weight_static(w3, args).view(w.shape)
        else:
            raise Exception('Not support other clip version')
        return q_w

    def fake_quantize_input(self, block_idx, x, layer_name):
        if not self.w_only:
            return self.aquantizer.fake_quant_act_dynamic(x)
        return x
