"""Oracle: AWQ scale search (test infrastructure only).

Restates awq.py of the reference on CPU tensors: get_weight_scale (:48-72),
get_act_scale (:74-85), get_scales (:87-108), fake_quantize_weight (:147-164),
calculate_loss (:134-145), search_scale_subset (:178-278, single input batch,
one process) and scaling_input (base_blockwise_quantization.py:899-912).
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
        total = ls.mean(0) if total is None else total.add_(ls.mean(0))
    return total.div_(len(weights))


def act_scale(x):
    return x.abs().view(-1, x.shape[-1]).mean(0)


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


def search_scale(weights: dict, x, forward, spec, n_grid=20, version='v2'):
    """-> (best_scales, losses per grid point).  `forward(x, weights_dict)` is the inspect module."""
    w_max = weight_scale(list(weights.values()), spec) if spec.granularity == 'per_group' else None
    org_out = forward(x, weights)
    best_err, best_scales, losses = float('inf'), None, []
    for n in range(n_grid):
        ratio = n * 1 / n_grid
        s = get_scales(x, w_max, ratio, version)
        wq = {k: scale_and_fake_quant(w, s, spec) for k, w in weights.items()}
        out = forward(scaling_input(x, s), wq)
        l = loss(org_out, out)
        losses.append(l)
        if l < best_err:
            best_err, best_scales = l, s
    return best_scales, losses
