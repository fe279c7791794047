"""Oracle: AWQ scale search (test infrastructure only).

Restates awq.py of the reference on CPU tensors: get_weight_scale (:48-72),
get_act_scale (:74-85), get_scales (:87-108), fake_quantize_weight (:147-164),
calculate_loss (:134-145), search_scale_subset (:178-278, one process; ``search_scale``
for one input tensor, ``search_scale_inputs`` for several tensors / ``awq_bs``
micro-batches) and scaling_input (base_blockwise_quantization.py:899-912).
The inspect module is any callable taking (x, weights_dict) so the tests can
use a SwiGLU MLP without nn.Module plumbing.
"""
from __future__ import annotations

import torch

from . import quant_ref as Q


def weight_scale(weights, spec):
    total = None
    for w in weights:
        w = w.clone()
        shape = w.shape
        rows = Q.reshape_rows(spec, w)
        a = rows.abs()
        mx = a.amax(dim=1, keepdim=True)
        ls = a.div_(mx).view(shape)
        total = Q.mean_rows(ls) if total is None else total.add_(Q.mean_rows(ls))
    return total.div_(len(weights))


def act_scale(x):
    return Q.mean_rows(x.abs().view(-1, x.shape[-1]))


def get_scales(x, w_max, ratio, version='v2'):
    xm = act_scale(x)
    if version == 'v1':
        s = (xm.pow(ratio) / w_max.pow(1 - ratio)).clamp(min=1e-4).view(-1)
    else:
        s = xm.pow(ratio).clamp(min=1e-4).view(-1)
    return s / (s.max() * s.min()).sqrt()


def scale_and_fake_quant(w, scales, spec):
    w = w.clone()
    w.mul_(scales.view(1, -1))
    return Q.int_fake_quant_dynamic(spec, w)


def scaling_input(x, scales):
    return x / scales.view(1, -1)


def loss(org_out, out):
    return (org_out - out).float().pow(2).mean().item()


def repeat_gqa(scales, kv_heads, head_dim, groups):
    """repeat_gqa_scales, base_blockwise_quantization.py:614-618 -> flat [kv_heads * groups * head_dim]."""
    return torch.repeat_interleave(scales.view(1, kv_heads, head_dim), dim=1, repeats=groups).reshape(-1)


def search_scale(weights: dict, x, forward, spec, n_grid=20, version='v2', gqa=None):
    """-> (best_scales, losses per grid point).  `forward(x, weights_dict)` is the inspect module.
    ``gqa=(prev_op, kv_heads, head_dim, groups)``: awq.py:88-93, 104-105 with is_gqa - the scales come from the
    statistics of prev_op(x) in the v2 form and are repeated per query group before they meet the columns."""
    w_max = weight_scale(list(weights.values()), spec) if spec.granularity == 'per_group' else None
    org_out = forward(x, weights)
    best_err, best_scales, losses = float('inf'), None, []
    for n in range(n_grid):
        ratio = n * 1 / n_grid
        if gqa is not None:
            prev_op, kvh, hd, groups = gqa
            s_kv = get_scales(prev_op(x), None, ratio, 'v2')
            s = repeat_gqa(s_kv, kvh, hd, groups)
        else:
            s = s_kv = get_scales(x, w_max, ratio, version)
        wq = {k: scale_and_fake_quant(w, s, spec) for k, w in weights.items()}
        out = forward(scaling_input(x, s), wq)
        l = loss(org_out, out)
        losses.append(l)
        if l < best_err:
            best_err, best_scales = l, s_kv
    return best_scales, losses


def search_scale_inputs(weights: dict, inputs: list, forward, spec, n_grid=20, version='v2', bs=None):
    """search_scale_subset (awq.py:178-278) for a LIST of input tensors and micro-batches of ``bs`` samples
    (``awq_bs``), statement for statement: ``loss_mean`` and ``scales_mean`` accumulate over the inputs, and
    ``is_best`` is evaluated inside that loop (awq.py:245-248) - with Python floats for the losses and an in-place
    ``+=`` on ``scales_mean`` from the second input on, so ``best_scales`` (an alias of ``scales_mean``) keeps
    growing after it was chosen.  -> (best_scales, per grid point the list of ``loss_mean`` after each input)."""
    bs = inputs[0].shape[0] if bs is None else bs

    def act_scale_bs(x):                                     # get_act_scale, awq.py:74-85
        if x.shape[0] == bs:
            return act_scale(x)
        means = [act_scale(x[k * bs:(k + 1) * bs]) for k in range(x.shape[0] // bs)]
        return sum(means) / len(means)

    def fwd_bs(x, w):                                        # inspect_module_forward, awq.py:110-126
        if x.shape[0] == bs:
            return forward(x, w)
        return torch.cat([forward(x[k * bs:(k + 1) * bs], w) for k in range(x.shape[0] // bs)], dim=0)

    def loss_bs(a, b):                                       # calculate_loss, awq.py:134-145
        if b.shape[0] == bs:
            return (a - b).float().pow(2).mean().item()
        total = 0.0
        for k in range(a.shape[0] // bs):
            total += (a[k * bs:(k + 1) * bs] - b[k * bs:(k + 1) * bs]).float().pow(2).mean().item()
        return total / (a.shape[0] // bs)

    w_max = weight_scale(list(weights.values()), spec)
    n_samples = inputs[0].shape[0] if len(inputs) == 1 else sum(x.shape[0] for x in inputs)
    best_error, best_scales, trace = float('inf'), None, []
    org_out = {}
    for n in range(n_grid):
        loss_mean = 0
        scales_mean = 0
        row = []
        for i, x in enumerate(inputs):
            if i not in org_out:
                org_out[i] = fwd_bs(x, weights)
            ratio = n * 1 / n_grid
            xm = act_scale_bs(x)
            if version == 'v1':
                scales = (xm.pow(ratio) / w_max.pow(1 - ratio)).clamp(min=1e-4).view(-1)
            else:
                scales = xm.pow(ratio).clamp(min=1e-4).view(-1)
            scales = scales / (scales.max() * scales.min()).sqrt()
            wq = {k: scale_and_fake_quant(w, scales, spec) for k, w in weights.items()}
            out = fwd_bs(scaling_input(x, scales), wq)
            l = loss_bs(org_out[i], out)
            loss_mean += x.shape[0] * 1.0 / n_samples * l
            scales_mean += x.shape[0] * 1.0 / n_samples * scales      # in place from the second input on
            row.append(loss_mean)
            if loss_mean < best_error:
                best_error = loss_mean
                best_scales = scales_mean
        trace.append(row)
    return best_scales, trace


# ----------------------------------------------------------------------------
# AutoClipper
# ----------------------------------------------------------------------------
def _logit(x):
    return torch.log(x / (1 - x))                       # auto_clip.py:42


def learnable_range(spec, tensor, lowbound_factor=None, upbound_factor=None):
    """get_learnable_range, quant.py:207-221: the min/max range scaled by sigmoid(factor)."""
    min_val, max_val = Q.minmax_range(spec, tensor)
    if spec.symmetric:
        if upbound_factor is not None:
            abs_max = torch.max(max_val.abs(), min_val.abs())
            abs_max = abs_max.clamp(min=1e-5)
            abs_max = torch.sigmoid(upbound_factor) * abs_max
            min_val = -abs_max
            max_val = abs_max
    else:
        if upbound_factor is not None and lowbound_factor is not None:
            min_val = torch.sigmoid(lowbound_factor) * min_val
            max_val = torch.sigmoid(upbound_factor) * max_val
    return min_val, max_val


def clip_fake_quantize_weight(spec, w, min_val, max_val, org_min_val, org_max_val, clip_version='v1'):
    """AutoClipper.fake_quantize_weight, auto_clip.py:258-274, on w [ocb, 1, G, gs].  v2 quantizes with the qparams of
    the learnable range; the reference's static fake quant flattens w to [ocb * G, gs] rows first, which only
    broadcasts against the [ocb, 1, G, 1] qparams when they hold one entry per row in the same order - written here
    with the qparams flattened the same way (identical for per_channel, G = 1; the reference fails for G > 1)."""
    if clip_version == 'v1':
        cur_w = torch.clamp(w, min_val, max_val)
        return Q.int_fake_quant_dynamic(spec, cur_w)
    low_factor = _logit(min_val / org_min_val)
    up_factor = _logit(max_val / org_max_val)
    lo, hi = learnable_range(spec, w, low_factor, up_factor)
    scales, zeros, qmax, qmin = Q.int_qparams(spec, lo, hi)
    rows = Q.reshape_rows(spec, w)
    zr = zeros if zeros.dim() == 0 else zeros.reshape(-1, 1)
    out = Q.int_quant_dequant(spec, rows.reshape(-1, rows.shape[-1]), scales.reshape(-1, 1), zr, qmax, qmin)
    return out.reshape(w.shape).to(w.dtype)


def auto_clip_layer(spec, w, inputs, clip_sym=False, n_grid=20, max_shrink=0.5, n_sample_token=512,
                    clip_version='v1', aspec=None, eps=0.0):
    """auto_clip.py:83-191 on CPU tensors, op for op: for each batch of output rows the [ocb, T, G, g] products of the
    sampled inputs with the original and with the clamped (v1) / range-scaled (v2) fake-quantized weights, their sums
    over g, the mean squared difference over tokens, and the running `err < min_errs` selection over the shrink
    steps.  `aspec` (an IntSpec, per_token) switches the activation fake quant of w_only=False on: it sees
    [1, T, G, g], i.e. one range per token AND group.  Returns (best_max [R, G, 1], best_min [R, G, 1],
    errs [R, G, n_steps] as computed)."""
    assert w.dim() == 2
    group_size = spec.group_size if spec.granularity == 'per_group' else w.shape[1]
    w = w.reshape(w.shape[0], 1, -1, group_size)
    oc_batch_size = 256 if w.shape[0] % 256 == 0 else 64
    assert w.shape[0] % oc_batch_size == 0
    w_all = w
    best_max_val_all, best_min_val_all, errs_all = [], [], []
    for i_b in range(w.shape[0] // oc_batch_size):
        w = w_all[i_b * oc_batch_size:(i_b + 1) * oc_batch_size]
        org_max_val = w.abs().amax(dim=-1, keepdim=True) if clip_sym else w.amax(dim=-1, keepdim=True)
        org_min_val = w.amin(dim=-1, keepdim=True)
        best_max_val = org_max_val.clone()
        best_min_val = org_min_val.clone()
        min_errs = torch.ones_like(org_max_val) * 1e9
        org_out_dict = {}
        errs_b = []
        for i_s in range(int(max_shrink * n_grid)):
            if i_s == 0:
                if clip_version == 'v2' and aspec is not None:
                    i_s += eps
            err_mean = 0
            for i in range(len(inputs)):
                x = inputs[i]
                x = x.view(-1, x.shape[-1])
                x = x.reshape(1, x.shape[0], -1, group_size)
                nst = n_sample_token if n_sample_token is not None else min(x.shape[1], 512)
                step_size = max(1, x.shape[1] // nst)
                x = x[:, 0::step_size]
                if i in org_out_dict:
                    org_out = org_out_dict[i]
                else:
                    org_out = (x * w).sum(dim=-1)
                    org_out_dict[i] = org_out
                max_val = org_max_val * (1 - i_s / n_grid)
                min_val = -max_val if clip_sym else org_min_val * (1 - i_s / n_grid)
                q_w = clip_fake_quantize_weight(spec, w, min_val, max_val, org_min_val, org_max_val, clip_version)
                q_x = Q.int_fake_quant_dynamic(aspec, x) if aspec is not None else x
                cur_out = (q_x * q_w).sum(dim=-1)
                err = (cur_out - org_out).pow(2).mean(dim=1).view(min_errs.shape)
                err_mean += err
            err_mean /= len(inputs)
            errs_b.append(err_mean.clone())
            cur_best_idx = err_mean < min_errs
            min_errs[cur_best_idx] = err_mean[cur_best_idx]
            best_max_val[cur_best_idx] = max_val[cur_best_idx]
            best_min_val[cur_best_idx] = min_val[cur_best_idx]
        best_max_val_all.append(best_max_val)
        best_min_val_all.append(best_min_val)
        errs_all.append(torch.cat(errs_b, dim=-1))          # [ocb, 1, G, n_steps]
    best_max_val = torch.cat(best_max_val_all, dim=0)
    best_min_val = torch.cat(best_min_val_all, dim=0)
    return best_max_val.squeeze(1), best_min_val.squeeze(1), torch.cat(errs_all, dim=0).squeeze(1)


def clip_factor(spec, w, min_val, max_val, clip_sym=False):
    """AutoClipper.get_clip_factor, auto_clip.py:231-256 -> (up_factor, low_factor) shaped like the quantizer's ranges."""
    org_min_val, org_max_val = Q.minmax_range(spec, Q.reshape_rows(spec, w))
    org_val_shape = org_max_val.shape
    if clip_sym:
        abs_max_val = torch.max(org_max_val.abs(), org_min_val.abs()).clamp(min=1e-5)
        abs_max_val = abs_max_val.reshape(*max_val.shape[:2], -1)
        return _logit(max_val / abs_max_val).reshape(org_val_shape), None
    org_max_val = org_max_val.reshape(*max_val.shape[:2], -1)
    up = _logit(max_val / org_max_val).reshape(org_val_shape)
    org_min_val = org_min_val.reshape(*min_val.shape[:2], -1)
    low = _logit(min_val / org_min_val).reshape(org_val_shape)
    return up, low


def apply_clip_v1(w, min_val, max_val, clip_sym=False):
    """auto_clip.py:194-211: clamp the weight group-wise to the found range."""
    org_shape = w.shape
    x = w.reshape(*max_val.shape[:2], -1)
    if clip_sym:
        min_val = -max_val
    return torch.clamp(x, min_val, max_val).reshape(org_shape)
