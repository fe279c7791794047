"""AWQ scale search with the reference's method surface, running on liblcq.

Mirrors ``llmc/compression/quantization/awq.py`` of ModelTC/LightCompress
(class ``Awq``): ``get_weight_scale`` (:48-72), ``get_act_scale`` (:74-85),
``get_scales`` (:87-108), ``fake_quantize_weight`` (:147-164),
``calculate_loss`` (:134-145), ``search_scale_subset`` (:178-278) and
``scaling_input`` (base_blockwise_quantization.py:899-912).

What changes under the API
  * W*s and the fake quantization are one kernel writing a scratch tensor, so
    the layer weights are never modified and never restored from a host copy
    (the reference multiplies in place and reloads the state dict from CPU at
    every grid point);
  * mean|x| is computed once per input instead of once per grid point;
  * the 20 losses stay on the device and are compared once (first minimum
    wins, as ``loss < best`` does), instead of one ``.item()`` per point;
  * the inspect-module forward itself (library GEMMs) is whatever the caller
    passes; the O(K) scale arithmetic (pow / clamp / normalise) uses torch ops
    on the [K] vector like the reference;
  * one process / one GPU: no all_reduce / broadcast of the winner;
  * float8 block-wise checkpoints (``weight`` float8_e4m3fn with ``weight_scale_inv``, awq.py:53-56, 148-160): the
    weight is brought to bf16 once per search (``weight_cast_to_bf16``, the block-wise casts of kernel.py), every
    grid point's scaled + fake-quantized weight is cast back with fresh block scales (``weight_cast_to_fp8``), and
    both buffers are put back afterwards;
  * GQA (``is_gqa``: v_proj feeding o_proj, base_blockwise_quantization.py:281-295, 614-618): the scales have
    one entry per key/value channel and are repeated per query group before they meet o_proj's columns;
    ``set_model_config`` takes the three sizes from a config object instead of ``self.model``.
"""
from __future__ import annotations

import torch

from . import _lib as L
from .blockwise import ScaleFolding, is_linear_like
from .quant import IntegerQuantizer


class Awq(ScaleFolding):
    def __init__(self, quant_config, wquantizer=None, aquantizer=None):
        self.quant_config = quant_config
        special_config = quant_config.get('special', {})
        self.save_scale = special_config.get('save_scale', False)
        self.act_scales = {}
        self.do_gqa_trans = special_config.get('do_gqa_trans', False)
        self.trans = special_config.get('trans', True)
        self.trans_version = special_config.get('trans_version', 'v2')
        self.awq_bs = special_config.get('awq_bs', None)
        self.save_mem = special_config.get('save_mem', True)
        # Several input tensors: the reference tests `loss_mean < best_error` inside the loop over inputs
        # (awq.py:245-248), so the grid point is picked by the FIRST input's weighted loss (later partial sums only
        # grow), while `best_scales` aliases `scales_mean`, which the in-place `+=` of the later inputs completes to
        # the mean over all inputs.  'first_input' reproduces that; 'mean' compares the mean loss over all inputs.
        self.multi_input_select = special_config.get('multi_input_select', 'first_input')
        if self.multi_input_select not in ('first_input', 'mean'):
            raise ValueError(f'multi_input_select: {self.multi_input_select}')
        self.wquantizer = wquantizer or IntegerQuantizer(**quant_config['weight'])
        self.aquantizer = aquantizer
        self.w_only = aquantizer is None
        self.padding_mask = None
        self.fp8_block_size = special_config.get('fp8_block_size', 128)
        self._ws = {}

    def _workspace(self, K, device):
        key = (int(K), str(device))
        if key not in self._ws:
            n = L.lib().lcq_awq_workspace_bytes(L.i64(K))
            self._ws[key] = torch.empty(n, dtype=torch.uint8, device=device)
        return self._ws[key]

    # -- awq.py:39-46 -----------------------------------------------------------
    @torch.no_grad()
    def set_model_config(self, model_config=None):
        """base_blockwise_quantization.py:281-295; ``model_config`` defaults to ``self.model.model_config``."""
        cfg = model_config if model_config is not None else self.model.model_config
        self.hidden_size = cfg.hidden_size
        self.num_heads = cfg.num_attention_heads
        self.head_dim = self.hidden_size // self.num_heads
        if hasattr(cfg, 'intermediate_size'):
            self.intermediate_size = cfg.intermediate_size
        if hasattr(cfg, 'num_key_value_heads'):
            self.num_key_value_heads = cfg.num_key_value_heads
            self.num_key_value_groups = self.num_heads // self.num_key_value_heads
            self.has_gqa = self.num_key_value_groups > 1
        else:
            self.has_gqa = False

    @torch.no_grad()
    def repeat_gqa_scales(self, scales):
        """base_blockwise_quantization.py:614-618: [kv_heads * head_dim] -> [1, heads, head_dim] (index plumbing on a
        vector of K values)."""
        scales = scales.view(1, self.num_key_value_heads, self.head_dim)
        return torch.repeat_interleave(scales, dim=1, repeats=self.num_key_value_groups)

    def scaling_weight(self, w, scales, is_gqa):
        scales_tmp = self.repeat_gqa_scales(scales) if is_gqa else scales
        w.mul_(scales_tmp.view(1, -1))
        return w

    def _bf16_weight(self, fc):
        """The layer weight; a float8 block-wise weight as bf16 (awq.py:53-56, 148-151)."""
        w = fc.weight.data
        if w.dtype == torch.float8_e4m3fn:
            from .kernel import weight_cast_to_bf16
            w = weight_cast_to_bf16(w.contiguous(), fc.weight_scale_inv.data.contiguous(), self.fp8_block_size).to(torch.bfloat16)
        return w

    def _store_weight(self, fc, w):
        """fc.weight.data = w; for a float8 block-wise layer the block-wise cast of w (awq.py:158-162)."""
        if fc.weight.data.dtype == torch.float8_e4m3fn:
            from .kernel import weight_cast_to_fp8
            fc.weight.data, fc.weight_scale_inv.data = weight_cast_to_fp8(w.contiguous(), self.fp8_block_size)
        else:
            fc.weight.data = w

    # -- awq.py:48-72 -------------------------------------------------------------
    def get_weight_scale(self, layers_dict):
        layers = list(layers_dict.values())
        total_scale = None
        wq = self.wquantizer
        for _m in layers:
            w = self._bf16_weight(_m).contiguous()
            R, K = w.shape
            g = wq.group_size if wq.granularity == 'per_group' else K
            out = torch.empty(K, dtype=w.dtype, device=w.device)
            L.check(L.lib().lcq_awq_weight_scale(L.ptr(w), L.i32(L.dtype_code(w.dtype)), L.i64(R), L.i64(K), L.i32(g),
                                                 L.ptr(out), L.ptr(self._workspace(K, w.device)), L.stream()),
                    'lcq_awq_weight_scale')
            if total_scale is None:
                total_scale = out
            else:
                total_scale.add_(out)
        return total_scale.div_(len(layers))

    # -- awq.py:74-85 ---------------------------------------------------------------
    def _absmean(self, x):
        K = x.shape[-1]
        x2 = x.reshape(-1, K).contiguous()
        out = torch.empty(K, dtype=x.dtype, device=x.device)
        L.check(L.lib().lcq_absmean_cols(L.ptr(x2), L.i32(L.dtype_code(x.dtype)), L.i64(x2.shape[0]), L.i64(K),
                                         L.ptr(out), L.ptr(self._workspace(K, x.device)), L.stream()),
                'lcq_absmean_cols')
        return out

    def get_act_scale(self, x):
        if x.shape[0] == self._bs:
            return self._absmean(x)
        batch_means = []
        b_num = x.shape[0] // self._bs
        for num in range(b_num):
            batch_means.append(self._absmean(x[num * self._bs:(num + 1) * self._bs]))
        return sum(batch_means) / len(batch_means)

    # -- awq.py:87-108 -----------------------------------------------------------------
    @torch.no_grad()
    def get_scales(self, prev_op, x, w_max, is_gqa, ratio, x_mean=None):
        """``x_mean``: mean|x| computed earlier (of ``prev_op(x)`` when is_gqa), so that the grid does not redo it."""
        if x_mean is not None:
            x_tmp = x_mean
        elif is_gqa:
            # statistics of v_proj's OUTPUT (its forward is the caller's library GEMM); the reference also calls
            # get_weight_scale on v_proj here and never uses the result (awq.py:90-91, 104-105)
            x_tmp = self.get_act_scale(prev_op(x))
        else:
            x_tmp = self.get_act_scale(x)
        if self.trans_version == 'v1' and not is_gqa:
            scales = (x_tmp.pow(ratio) / w_max.pow(1 - ratio)).clamp(min=1e-4).view(-1)
        else:
            scales = x_tmp.pow(ratio).clamp(min=1e-4).view(-1)
        scales = scales / (scales.max() * scales.min()).sqrt()
        return scales

    # -- awq.py:110-145 ------------------------------------------------------------------
    def inspect_module_forward(self, x, inspect_module, kwargs):
        if self._bs == x.shape[0]:
            with torch.no_grad():
                out = inspect_module(x, **kwargs)
                if isinstance(out, tuple):
                    out = out[0]
            return out
        outs = []
        b_num = x.shape[0] // self._bs
        for num in range(b_num):
            _x = x[num * self._bs:(num + 1) * self._bs]
            out = inspect_module(_x, **kwargs)
            if isinstance(out, tuple):
                out = out[0]
            outs.append(out)
        return torch.cat(outs, dim=0)

    @torch.no_grad()
    def get_original_out(self, x, inspect_module, subset_kwargs):
        return self.inspect_module_forward(x, inspect_module, subset_kwargs)

    def _loss_device(self, org_out, out):
        """mean squared difference as a 1-element device tensor (no host sync)."""
        def one(a, b):
            a, b = a.contiguous(), b.contiguous()
            res = torch.empty(1, dtype=torch.float32, device=a.device)
            L.check(L.lib().lcq_sq_err_mean(L.ptr(a), L.ptr(b), L.i32(L.dtype_code(a.dtype)), L.i64(a.numel()),
                                            L.ptr(res), L.ptr(self._workspace(a.shape[-1], a.device)), L.stream()),
                    'lcq_sq_err_mean')
            return res
        if out.shape[0] == self._bs:
            return one(org_out, out)
        b_num = org_out.shape[0] // self._bs
        total = None
        for num in range(b_num):
            l = one(org_out[num * self._bs:(num + 1) * self._bs], out[num * self._bs:(num + 1) * self._bs])
            total = l if total is None else total + l
        return total / b_num

    def calculate_loss(self, org_out, out):
        return self._loss_device(org_out, out).item()

    # -- awq.py:147-176 ----------------------------------------------------------------------
    def _scale_quant(self, weight, scales):
        """fake_quant_weight_dynamic(W * s) (awq.py:147-164) into a new tensor.  Min/max calibration with rounded zero
        points is one fused kernel; any other weight quantizer setting (calib_algo mse / hqq, round_zp False, other
        granularities) multiplies first and then goes through the quantizer's own fake_quant_weight_dynamic."""
        wq = self.wquantizer
        w = weight.contiguous()
        R, K = w.shape
        s = scales.to(w.dtype).contiguous()
        fused = (wq.calib_algo not in ('mse', 'hqq', 'learnable') and wq.round_zp
                 and wq.granularity in ('per_group', 'per_channel') and getattr(wq, 'quant_type', '') == 'int-quant')
        if not fused:
            ws = torch.empty_like(w)
            L.check(L.lib().lcq_scale_matrix(L.ptr(w), L.i32(L.dtype_code(w.dtype)), L.i64(R), L.i64(K), L.ptr(s), L.i32(0),
                                             L.ptr(ws), L.stream()), 'lcq_scale_matrix')
            return wq.fake_quant_weight_dynamic(ws)
        g = wq.group_size if wq.granularity == 'per_group' else 0
        out = torch.empty_like(w)
        L.check(L.lib().lcq_awq_scale_quant(L.ptr(w), L.i32(L.dtype_code(w.dtype)), L.i64(R), L.i64(K), L.ptr(s), L.i32(g),
                                            L.f32(wq.qmin), L.f32(wq.qmax), L.i32(L.FLAG_SYM if wq.sym else 0),
                                            L.ptr(out), L.stream()), 'lcq_awq_scale_quant')
        return out

    def fake_quantize_weight(self, fc, scales, is_gqa, layer_name):
        if is_gqa:
            scales = self.repeat_gqa_scales(scales).reshape(-1)
        self._store_weight(fc, self._scale_quant(self._bf16_weight(fc), scales))
        return fc.weight

    def fake_quantize_input(self, x_tmp, layers_dict):
        if self._bs == x_tmp.shape[0]:
            return self.aquantizer.fake_quant_act_dynamic(x_tmp)
        return torch.stack([self.aquantizer.fake_quant_act_dynamic(x_tmp[i]) for i in range(x_tmp.shape[0])])

    # -- base_blockwise_quantization.py:899-912 --------------------------------------------------
    @torch.no_grad()
    def scaling_input(self, x, scales, is_gqa):
        if is_gqa:
            scales = self.repeat_gqa_scales(scales).reshape(-1)
        K = x.shape[-1]
        x2 = x.contiguous()
        s = scales.to(x.dtype).contiguous()
        out = torch.empty_like(x2)
        L.check(L.lib().lcq_div_cols(L.ptr(x2), L.i32(L.dtype_code(x.dtype)), L.i64(x2.numel() // K), L.i64(K), L.ptr(s),
                                     L.ptr(out), L.stream()), 'lcq_div_cols')
        return out

    # -- awq.py:178-278 ------------------------------------------------------------------------------
    @torch.no_grad()
    def search_scale_subset(self, prev_op, layers_dict, input, inspect_module, is_gqa, subset_kwargs):
        if self.awq_bs is None:
            self._bs = input[0].shape[0]
        else:
            self._bs = self.awq_bs
        # the reference computes w_max for every version (awq.py:190) and reads it only in v1
        w_max = self.get_weight_scale(layers_dict) if self.trans_version == 'v1' else None
        n_grid = 20
        # what the reference saves and reloads as a host state dict: the tensors themselves, never modified here
        saved = {name: (fc.weight.data, fc.weight_scale_inv.data if fc.weight.data.dtype == torch.float8_e4m3fn else None)
                 for name, fc in layers_dict.items()}
        originals = {name: self._bf16_weight(fc) for name, fc in layers_dict.items()}
        device = next(iter(originals.values())).device
        n_samples = input[0].shape[0] if len(input) == 1 else sum(x.shape[0] for x in input)

        org_out_dict, x_mean_dict = {}, {}
        loss_rows, scale_rows = [], []
        for n in range(n_grid):
            loss_mean = 0
            scales_mean = 0
            loss_select = None
            for i in range(len(input)):
                input[i] = input[i].to(device)
                x = input[i]
                kwargs = subset_kwargs[i] if isinstance(subset_kwargs, list) else (subset_kwargs or {})
                if i not in org_out_dict:
                    org_out_dict[i] = self.get_original_out(x, inspect_module, kwargs)
                    x_mean_dict[i] = self.get_act_scale(prev_op(x) if is_gqa else x)
                org_out = org_out_dict[i]
                ratio = n * 1 / n_grid
                scales = self.get_scales(prev_op, x, w_max, is_gqa, ratio, x_mean=x_mean_dict[i])
                col_scales = self.repeat_gqa_scales(scales).reshape(-1) if is_gqa else scales
                for layer_name, fc in layers_dict.items():
                    self._store_weight(fc, self._scale_quant(originals[layer_name], col_scales))
                x_tmp = self.scaling_input(x, scales, is_gqa)
                if not self.w_only:
                    x_tmp = self.fake_quantize_input(x_tmp, layers_dict)
                out = self.inspect_module_forward(x_tmp, inspect_module, kwargs)
                if self.padding_mask and org_out.shape[1] == self.padding_mask[i].shape[-1]:
                    m = self.padding_mask[i].unsqueeze(dim=-1).to(org_out.device)
                    org_out, out = org_out * m, out * m
                loss = self._loss_device(org_out, out)
                loss_mean = loss_mean + x.shape[0] * 1.0 / n_samples * loss
                if i == 0:
                    loss_select = loss_mean
                scales_mean = scales_mean + x.shape[0] * 1.0 / n_samples * scales
                for layer_name, fc in layers_dict.items():      # the originals were never touched
                    fc.weight.data = saved[layer_name][0]
                    if saved[layer_name][1] is not None:
                        fc.weight_scale_inv.data = saved[layer_name][1]
            if len(input) > 1 and self.multi_input_select == 'mean':
                loss_select = loss_mean
            loss_rows.append(loss_select.reshape(1))
            scale_rows.append(scales_mean)
        losses = torch.cat(loss_rows)
        best = torch.argmin(losses)                              # first minimum, like `loss < best_error`
        self.search_losses = losses
        best_scales = torch.stack(scale_rows)[best]
        return best_scales

    # -- awq.py:299-373 ---------------------------------------------------------------------------------
    @torch.no_grad()
    def subset_transform(self, subset, input_feat, subset_kwargs):
        """Search the scales of one subset, fold them into the operator in front of it and rescale the cached inputs.
        ``subset``: {'layers': {name: Linear}, 'prev_op': [module], 'input': [name], 'inspect': module, 'do_trans':
        bool}.  Subsets without a single LayerNorm-like or Linear operator in front are left alone, as are Linear
        predecessors whose width fits none of the fc-fc cases unless grouped-query scaling is on (then the statistics
        come from the input recorded one entry earlier, the predecessor's own input)."""
        layers_dict = subset['layers']
        prev_op = subset['prev_op']
        input_name = subset['input'][0]
        inspect_module = subset['inspect']
        if not subset.get('do_trans', True):
            return
        config = getattr(self, 'config', None)
        if config is not None and config['model']['type'] == 'Starcoder' and is_linear_like(prev_op[0]):
            return
        assert len(prev_op) in (0, 1), 'Only support single prev_op. If multi prev_ops, code need to be updated.'
        if len(prev_op) == 0 or prev_op[0] is None:
            return
        op = prev_op[0]
        is_linear = is_linear_like(op)
        is_norm = not is_linear and hasattr(op, 'weight') and op.weight.dim() == 1
        if not (is_linear or is_norm):
            return
        layers = list(layers_dict.values())
        is_gqa = False
        if is_linear:
            width = layers[0].in_features
            if op.out_features not in (width * 3, width * 2, width):
                if not (self.has_gqa and self.do_gqa_trans):
                    return
                is_gqa = True
                keys = list(input_feat.keys())
                input_name = keys[keys.index(input_name) - 1]
        scale = self.search_scale_subset(op, layers_dict, input_feat[input_name], inspect_module, is_gqa, subset_kwargs)
        self.apply_scale(scale, prev_op, layers)
        self.update_input_feat(scale, input_feat, layers_dict, is_gqa)
        if self.save_scale:
            for n in layers_dict:
                self.act_scales[f'{self.model.block_name_prefix}.{self.block_idx}.{n}'] = scale
