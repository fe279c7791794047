"""Oracle: GPTQ Hessian, Cholesky chain and lazy-batch column loop
(test infrastructure only).

Restates gptq.py of the reference on CPU tensors: ``add_batch`` (:253-295,
without the all-reduce — one process), ``hessian_sorting`` (:58-64),
``process_hessian_and_weights`` (:128-176) and ``weight_transform``
(:198-244) with the per-group parameter refresh of ``search_column_qparams``
(:358-366).  ``dtype=torch.float64`` runs the same recurrences in double
precision for the closed-form / invariant checks that pin this file.
"""
from __future__ import annotations

import math

import torch

from . import quant_ref as Q


# ---------------------------------------------------------------------------
# Hessian   (gptq.py:253-295)
# ---------------------------------------------------------------------------
def add_batch(H: torch.Tensor, nsamples: int, inp: torch.Tensor, chunk_num: int = 1) -> int:
    """In-place running-mean update of H with one calibration batch; returns the new count."""
    if inp.dim() == 2:
        inp = inp.unsqueeze(0)
    b = inp.shape[0]
    x = inp.reshape(-1, inp.shape[-1]).t()
    assert x.shape[1] % chunk_num == 0
    H *= nsamples / (nsamples + b)
    nsamples += b
    for chunk in torch.chunk(x, chunk_num, dim=1):
        chunk = math.sqrt(2 / nsamples) * chunk.to(H.dtype)
        H += chunk.matmul(chunk.t())
    return nsamples


def conv2d_patches(inp: torch.Tensor, kernel_size, dilation=1, padding=0, stride=1) -> torch.Tensor:
    """What add_batch makes of a Conv2d input (gptq.py:268-278): nn.Unfold -> [N, C*kh*kw, L], permuted and flattened
    to [C*kh*kw, N*L]; returned here as [N, L, C*kh*kw] so that add_batch above (which transposes) sees the same
    matrix, with N as the batch count."""
    cols = torch.nn.functional.unfold(inp, kernel_size, dilation=dilation, padding=padding, stride=stride)
    return cols.transpose(1, 2).contiguous()


def hessian_closed_form(batches, dtype=torch.float64) -> torch.Tensor:
    """(2/N) * sum_b X_b^T X_b — what the running rescale telescopes to (N = number of batches)."""
    n = sum(1 if b.dim() == 2 else b.shape[0] for b in batches)
    K = batches[0].shape[-1]
    H = torch.zeros(K, K, dtype=dtype)
    for b in batches:
        x = b.reshape(-1, K).to(dtype)
        H += x.t() @ x
    return H * (2.0 / n)


# ---------------------------------------------------------------------------
# permutation, dead columns, damping, Cholesky chain   (gptq.py:58-64, 128-176)
# ---------------------------------------------------------------------------
def act_order(H: torch.Tensor) -> torch.Tensor:
    return torch.argsort(torch.diag(H), descending=True)


def owq_order(H: torch.Tensor, n_out: int) -> torch.Tensor:
    """hessian_sorting with owq, gptq.py:66-83 (act-order is off whenever owq is on, :47-50): the n_out columns with
    the largest diagonal move to the end, the rest keep their order."""
    K = H.shape[0]
    mask = torch.full([K], True)
    descending_ids = torch.argsort(torch.diag(H), descending=True)
    mask[descending_ids[:n_out]] = False
    return torch.cat([torch.arange(K)[mask], descending_ids[:n_out]])


def process_hessian_and_weights(weight: torch.Tensor, H: torch.Tensor, percdamp: float, perm=None,
                                dtype=torch.float32):
    """-> (W [R,K] in `dtype`, Hinv upper Cholesky factor of the damped inverse, invperm|None)."""
    W = weight.clone().to(dtype)
    H = H.clone().to(dtype)
    dead = torch.diag(H) == 0
    H[dead, dead] = 1
    W[:, dead] = 0
    invperm = None
    if perm is not None:
        W = W[:, perm]
        H = H[perm][:, perm]
        invperm = torch.argsort(perm)
    damp = percdamp * torch.mean(torch.diag(H))
    idx = torch.arange(H.shape[0])
    H[idx, idx] += damp
    H = torch.linalg.cholesky(H)
    H = torch.cholesky_inverse(H)
    H = torch.linalg.cholesky(H, upper=True)
    return W, H, invperm


# ---------------------------------------------------------------------------
# lazy-batch column loop   (gptq.py:198-244)
# ---------------------------------------------------------------------------
def block_factor(U, blocksize=128):
    """The block upper triangular P that stands in for U in the column loop (no counterpart in the reference, which
    always forms U; the product's chain builds P without a triangular inverse).  With M = U^-1:
    P[b, b] = U[b, b] (gptq.py:205 takes exactly this block as Hinv1), P[p, b] = M[p, b] U[b, b] for p < b."""
    K = U.shape[0]
    assert K % blocksize == 0
    M = torch.linalg.solve_triangular(U, torch.eye(K, dtype=U.dtype), upper=True)
    P = torch.zeros_like(U)
    for b in range(K // blocksize):
        sl = slice(b * blocksize, (b + 1) * blocksize)
        P[sl, sl] = U[sl, sl]
        P[:b * blocksize, sl] = M[:b * blocksize, sl] @ U[sl, sl]
    return P


def weight_transform(W, Hinv, spec, blocksize=128, static_qparams=None, static_groups=None, qparams_fn=None, n_out=0,
                     block_factor_W0=None):
    """Runs the loop in place on W (as the reference does) and returns
    (tmp, Losses, groups) where groups is the list of per-group
    (scale [R,1], zero [R,1]|0-dim) refreshed at every group boundary.

    ``spec`` is an oracle IntSpec (per_group or per_channel).  For
    per_channel, ``static_qparams=(scale, zero)`` are the fixed row
    parameters the reference takes from the layer's RTN buffers.
    ``static_groups=(scales [R,G], zeros [R,G] | None, perm | None)``: per_group with
    ``static_groups: True`` - the RTN parameters of the ORIGINAL column order, looked up as
    ``groups[perm[idx] // g]`` (gptq.py:143-148, 224-227); nothing is refreshed.
    ``qparams_fn(spec, cols) -> (rows, scale, zero, qmax, qmin)`` stands for ``wquantizer.get_tensor_qparams``
    (gptq.py:358-366 calls it, so ``calib_algo`` reaches the loop); default: min/max calibration.
    ``n_out``: OWQ - the last n_out columns are not quantized (the loop and the group ranges stop before them) but
    still receive every block's update.
    ``block_factor_W0``: Hinv is block_factor(U) and this is a copy of W as it was before the loop; a block then hands
    (quantized - original) instead of Err1 to the update of the later columns, everything else is the reference's loop.
    """
    qparams_fn = qparams_fn or Q.int_tensor_qparams
    R, K = W.shape
    Losses = torch.zeros_like(W)
    tmp = torch.zeros_like(W)
    groups = []
    per_group = spec.granularity == 'per_group'
    if not per_group:
        scale, zero = static_qparams
    qmax, qmin = spec.qmax, spec.qmin
    n_nonout = K - n_out
    for i1 in range(0, n_nonout, blocksize):
        i2 = min(i1 + blocksize, n_nonout)
        count = i2 - i1
        W1, Hinv1 = W[:, i1:i2].clone(), Hinv[i1:i2, i1:i2]
        tmp1, Err1, Losses1 = torch.zeros_like(W1), torch.zeros_like(W1), torch.zeros_like(W1)
        Q1 = torch.zeros_like(W1)
        for i in range(count):
            w, d = W1[:, i], Hinv1[i, i]
            if per_group and static_groups is not None:
                sg, zg, perm = static_groups
                idx = i1 + i
                if perm is not None:
                    idx = int(perm[idx])
                scale = sg[:, idx // spec.group_size].unsqueeze(1)
                zero = torch.tensor(0.0) if zg is None else zg[:, idx // spec.group_size].unsqueeze(1)
            elif per_group and (i1 + i) % spec.group_size == 0:
                cols = W[:, (i1 + i): min(i1 + i + spec.group_size, K - n_out)]      # W, not W1 (gptq.py:216-222)
                _, scale, zero, qmax, qmin = qparams_fn(spec, cols)
                groups.append((scale.clone(), zero.clone()))
            q = Q.int_quant_dequant(spec, w.unsqueeze(1), scale, zero, qmax, qmin).squeeze(1)
            tmp1[:, i] = w
            Q1[:, i] = q
            Losses1[:, i] = ((w - q) ** 2) / (2 * d ** 2)
            err1 = (w - q) / d
            W1[:, i:] -= err1.unsqueeze(1).matmul(Hinv1[i, i:].unsqueeze(0))
            Err1[:, i] = err1
        tmp[:, i1:i2], Losses[:, i1:i2] = tmp1, Losses1
        if block_factor_W0 is not None:
            Err1 = Q1 - block_factor_W0[:, i1:i2]
        W[:, i2:] -= Err1.matmul(Hinv[i1:i2, i2:])
    return tmp, Losses, groups


def merge_groups(groups):
    """update_model_qparams / merge_qparams (gptq.py:343-356, 397-409): [R*G, 1], row-major [R, G]."""
    scales = torch.stack([g[0] for g in groups], dim=1).reshape(-1, 1)
    zeros = None
    if groups[0][1].dim() > 0:
        zeros = torch.stack([g[1] for g in groups], dim=1).reshape(-1, 1)
    return scales, zeros


def mse_tensor_qparams(spec, t, **mse):
    """get_tensor_qparams with calib_algo 'mse' (quant.py:689-696 with :147-205)."""
    rows = Q.reshape_rows(spec, t)
    lo, hi = Q.int_mse_range(spec, rows.clone(), **mse)
    s, z, qmax, qmin = Q.int_qparams(spec, lo, hi)
    return rows, s, z, qmax, qmin


def gptq_layer(weight, H, spec, percdamp=0.01, blocksize=128, actorder=False, dtype=torch.float32,
               static_qparams=None, qparams_fn=None, owq_n_out=None):
    """layer_transform (gptq.py:113-196): -> dict(weight=tmp un-permuted, scales, zeros, perm, loss, Hinv).
    ``owq_n_out`` (an int) switches OWQ on: outlier-last column order, per_channel qparams from the non-outlier
    columns of the permuted weight (:158-167), outlier columns written back un-quantized (:187-188)."""
    owq = owq_n_out is not None
    n_out = owq_n_out if owq else 0
    perm = owq_order(H, n_out) if owq else (act_order(H) if actorder else None)
    W, Hinv, invperm = process_hessian_and_weights(weight, H, percdamp, perm, dtype)
    if owq and spec.granularity == 'per_channel':
        _, s_, z_, _, _ = Q.int_tensor_qparams(spec, W[:, :W.shape[1] - n_out])
        static_qparams = (s_, z_)
    tmp, Losses, groups = weight_transform(W, Hinv, spec, blocksize, static_qparams, qparams_fn=qparams_fn, n_out=n_out)
    out = dict(loss=float(Losses.sum()), perm=perm, Hinv=Hinv, tmp_perm=tmp)
    if owq:
        tmp[:, W.shape[1] - n_out:] = W[:, W.shape[1] - n_out:]
        out['static_qparams'] = static_qparams
    if actorder or owq:
        tmp = tmp[:, invperm]
    out['weight'] = tmp
    if groups:
        out['scales'], out['zeros'] = merge_groups(groups)
    return out


def codes_from(tmp_perm, scales, zeros, spec):
    """Integer codes the deploy step derives from the compensated weights and the
    loop's qparams (gptq.py:411-452, in processing order), fp32 arithmetic.
    Handles a ragged last group (K % group_size != 0) group by group."""
    R, K = tmp_perm.shape
    g = spec.group_size if spec.granularity == 'per_group' else K
    Gn = -(-K // g)
    s = scales.reshape(R, Gn)
    z = zeros.reshape(R, Gn) if zeros is not None else None
    out = torch.empty_like(tmp_perm)
    for gi in range(Gn):
        sl = slice(gi * g, min((gi + 1) * g, K))
        zg = z[:, gi:gi + 1] if z is not None else torch.tensor(0.0)
        out[:, sl] = Q.int_quant(spec, tmp_perm[:, sl], s[:, gi:gi + 1], zg, spec.qmax, spec.qmin)
    return out


def recon_loss(W0, What, X):
    """|| (W0 - What) X^T ||_F^2 for X [T, K]."""
    d = (W0.double() - What.double()) @ X.double().t()
    return float((d * d).sum())
