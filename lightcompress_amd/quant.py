"""Quantizer primitives with the reference's class API, running on liblcq.

Mirrors ``llmc/compression/quantization/quant.py`` of ModelTC/LightCompress:
``IntegerQuantizer`` (quant.py:660-959) and ``FloatQuantizer`` (quant.py:962-1228)
with the same constructor kwargs, method names, argument order and return
tuples, so algorithm code written against the reference runs unchanged.

Every arithmetic method launches hand-written gfx950 kernels through the C
ABI in ``include/lcq.h``.  There is no CPU path: CPU tensors raise
``LcqError``.  Reshapes/views, index mixing and dtype casts stay in torch.

``calib_algo``: ``minmax``, ``mse``, ``hqq``, ``learnable`` (the sigmoid-scaled range with GIVEN factors; training
them needs autograd and is not here), ``static_minmax`` / ``static_moving_minmax`` / ``static_hist`` for activations.
Not carried over (they raise ``NotImplementedError``): STE rounding (training only) and the ``rounding`` override of
``fake_quant_weight_static``.  ``per_block`` granularity runs for
``FloatQuantizer('e4m3')`` weights only (``real_quant_weight_dynamic`` / ``fake_quant_weight_dynamic``).
"""
from __future__ import annotations

import math

import torch

from . import _lib as L


def ceil_div(x, y):
    return (x + y - 1) // y


def _scaled(scales, factor):
    """scales * output_scale_factor as torch computes it for a number: the fp32 product, rounded, then the cast to the
    tensor's type.  (For fp16 the GPU's fused multiply-and-convert would round the exact product once; the two differ
    when the fp32 rounding lands on an fp16 tie, which x * 1.7 often does.)"""
    if factor == 1 or not torch.is_tensor(scales) or scales.dtype != torch.float16:
        return scales * factor
    return (scales.float() * factor).to(torch.float16)


class BaseQuantizer(object):
    """Constructor surface of quant.py:48-103."""

    def __init__(self, bit, symmetric, granularity, **kwargs):
        self.bit = bit
        self.sym = symmetric
        self.granularity = granularity
        self.kwargs = kwargs

        self.calib_algo = self.kwargs.get('calib_algo', 'minmax')
        # mse config (quant.py:78-81)
        self.mse_b_num = self.kwargs.get('mse_b_num', 1)
        self.maxshrink = self.kwargs.get('maxshrink', 0.8)
        self.mse_grid = self.kwargs.get('mse_grid', 100)
        # hist config (quant.py:83-87)
        self.bins = self.kwargs.get('bins', 2048)
        self.upsample_rate = 16
        # hqq config (quant.py:89-93)
        self.lp_norm = self.kwargs.get('lp_norm', 0.7)
        self.beta = self.kwargs.get('beta', 10)
        self.kappa = self.kwargs.get('kappa', 1.01)
        self.iters = self.kwargs.get('iters', 20)
        if self.granularity == 'per_group':
            self.group_size = self.kwargs['group_size']
        elif self.granularity == 'per_head':
            self.head_num = self.kwargs['head_num']
        elif self.granularity == 'per_block':
            assert self.calib_algo == 'minmax' and self.sym
            self.block_size = self.kwargs['block_size']

        if self.kwargs.get('ste', False) or self.kwargs.get('ste_all', False):
            raise NotImplementedError('straight-through rounding is a training feature; not on this path')
        self.round_func = torch.round
        self.sigmoid = torch.nn.Sigmoid()
        self.ste_all = False
        self.round_zp = self.kwargs.get('round_zp', True)

    # -- calibration -------------------------------------------------------
    def get_tensor_range(self, tensor, args={}):
        if self.calib_algo == 'minmax':
            return self.get_minmax_range(tensor)
        if self.calib_algo == 'mse':
            return self.get_mse_range(tensor)
        if self.calib_algo == 'learnable':
            return self.get_learnable_range(tensor, **args)
        return self.get_minmax_range(tensor)                 # quant.py:131-132: anything else falls back to minmax

    def get_learnable_range(self, tensor, lowbound_factor=None, upbound_factor=None):
        """quant.py:207-221: the min/max range scaled by sigmoid(factor).  The factors are inputs here (found by
        AutoClipper v2 or loaded); training them needs autograd and is not on this path.  Range kernels on the
        tensor, the handful of per-row scalars in torch like the reference."""
        min_val, max_val = self.get_minmax_range(tensor)
        if self.sym:
            if upbound_factor is not None:
                abs_max = torch.max(max_val.abs(), min_val.abs())
                abs_max = abs_max.clamp(min=1e-5)
                abs_max = self.sigmoid(upbound_factor) * abs_max
                min_val = -abs_max
                max_val = abs_max
        else:
            if upbound_factor is not None and lowbound_factor is not None:
                min_val = self.sigmoid(lowbound_factor) * min_val
                max_val = self.sigmoid(upbound_factor) * max_val
        return (min_val, max_val)

    def get_mse_range(self, tensor, norm=2.4, bs=256):
        """quant.py:147-205 -> fp32 (min_val, max_val) [rows, 1]: the shrunken range with the smallest
        sum |quant_dequant(x) - x| ** norm per row, one kernel instead of 80 rounds of ~10 torch ops."""
        if self.granularity == 'per_tensor' or tensor.dim() != 2:
            raise NotImplementedError('get_mse_range runs on a 2-D reshaped tensor')
        assert self.mse_b_num >= 1 and tensor.shape[0] % self.mse_b_num == 0, \
            'Batch number must be divisible by tensor.shape[0],'
        if getattr(self, 'quant_type', 'int-quant') != 'int-quant':
            return self._mse_range_float(tensor, norm)
        t = tensor.contiguous()
        rows, cols = t.shape
        mn = torch.empty((rows, 1), dtype=torch.float32, device=t.device)
        mx = torch.empty((rows, 1), dtype=torch.float32, device=t.device)
        L.check(L.lib().lcq_mse_range(L.ptr(t), L.dtype_code(t.dtype), L.i64(rows), L.i64(cols), L.f32(float(self.qmin)),
                                      L.f32(float(self.qmax)), L.i32(self._int_flags()),
                                      L.i32(int(self.maxshrink * self.mse_grid)), L.i32(int(self.mse_grid)),
                                      L.f32(norm), L.ptr(mn), L.ptr(mx), L.stream()), 'lcq_mse_range')
        return (mn, mx)

    def get_minmax_range(self, tensor):
        """quant.py:134-145 -> (min_val, max_val)."""
        dt = L.dtype_code(tensor.dtype)
        t = tensor.contiguous()
        if self.granularity == 'per_tensor':
            mn = torch.empty((), dtype=t.dtype, device=t.device)
            mx = torch.empty((), dtype=t.dtype, device=t.device)
            ws = torch.empty(L.lib().lcq_minmax_all_workspace_bytes(), dtype=torch.uint8, device=t.device)
            L.check(L.lib().lcq_minmax_all(L.ptr(t), dt, L.i64(t.numel()), L.ptr(mn), L.ptr(mx), L.ptr(ws),
                                           L.stream()), 'lcq_minmax_all')
            return (mn, mx)
        cols = t.shape[-1]
        rows = t.numel() // cols
        shape = (*t.shape[:-1], 1)
        mn = torch.empty(shape, dtype=t.dtype, device=t.device)
        mx = torch.empty(shape, dtype=t.dtype, device=t.device)
        L.check(L.lib().lcq_minmax_rows(L.ptr(t), dt, L.i64(rows), L.i64(cols), L.ptr(mn), L.ptr(mx), L.stream()),
                'lcq_minmax_rows')
        return (mn, mx)

    def _int_flags(self):
        return (L.FLAG_SYM if self.sym else 0) | (0 if self.round_zp else L.FLAG_NO_ROUND_ZP)

    def get_qparams(self, tensor_range, device):
        """quant.py:544-558 -> (scales, zeros, qmax, qmin)."""
        min_val, max_val = tensor_range[0].contiguous(), tensor_range[1].contiguous()
        qmin = self.qmin.to(device)
        qmax = self.qmax.to(device)
        flags = self._int_flags()
        # 0-dim ranges (per_tensor) meet the 0-dim fp32 (qmax - qmin): torch promotes the result to fp32
        if max_val.dim() == 0 and not self.sym and max_val.dtype != torch.float32:
            flags |= L.FLAG_RANGE_BF16 if max_val.dtype == torch.bfloat16 else L.FLAG_RANGE_F16
            min_val, max_val = min_val.float(), max_val.float()
        scales = torch.empty_like(max_val)
        zeros = torch.tensor(0.0) if self.sym else torch.empty_like(max_val)
        L.check(L.lib().lcq_qparams_int(L.ptr(min_val), L.ptr(max_val), L.dtype_code(max_val.dtype),
                                        L.i64(max_val.numel()), L.f32(self.qmin), L.f32(self.qmax),
                                        L.i32(flags), L.ptr(scales),
                                        L.ptr(None if self.sym else zeros), L.stream()), 'lcq_qparams_int')
        return scales, zeros, qmax, qmin

    # -- static activation calibration (quant.py:105-124, 223-262, 523-585) -------------------
    def reshape_batch_tensors(self, act_tensors):
        """quant.py:105-124: calibration inputs -> list (one entry per module input) of lists of tensors."""
        assert len(act_tensors) > 0, (
            'Calibration data is insufficient. Please provide more data to ensure '
            'all experts in the MOE receive an adequate number of tokens.'
        )
        if isinstance(act_tensors[0], tuple):
            act_tensors = [torch.stack(tensor_list) for tensor_list in zip(*act_tensors)]
        elif len(act_tensors) == 1:
            act_tensors[0] = [act_tensors[0][i] for i in range(act_tensors[0].size(0))]
        else:
            act_tensors = [act_tensors]
        return act_tensors

    def get_minmax_stats(self, act_tensors):
        """quant.py:223-250: per input, the stacked fp32 CPU ranges of every calibration tensor (range kernels on
        the GPU; like the reference the handful of scalars is collected on the host)."""
        stats_min_max = {}
        for input_idx, tensors in enumerate(act_tensors):
            mins, maxs = [], []
            for tensor in tensors:
                lo, hi = self.get_minmax_range(self.reshape_tensor(tensor))
                mins.append(lo.detach().cpu().to(torch.float32).unsqueeze(0))
                maxs.append(hi.detach().cpu().to(torch.float32).unsqueeze(0))
            stats_min_max[input_idx] = {'min': torch.cat(mins), 'max': torch.cat(maxs)}
        return stats_min_max

    def get_static_minmax_range(self, act_tensors):
        """quant.py:252-262: mean of the per-tensor ranges."""
        stats = self.get_minmax_stats(self.reshape_batch_tensors(act_tensors))
        min_vals = [r['min'].mean(dim=0) for r in stats.values()]
        max_vals = [r['max'].mean(dim=0) for r in stats.values()]
        return min_vals, max_vals

    # -- histogram observer (calib_algo 'static_hist', quant.py:264-521) ---------------------------------------
    # The passes over the activations (range, histogram) are kernels.  What follows them works on `bins` numbers per
    # module input and stays host-side fp32 torch arithmetic on CPU tensors, as in the reference, whose histograms
    # live on the CPU as well (quant.py:468): the search below compares sums that differ in their last bits, so it
    # keeps the reference's operation order.
    def _histc(self, tensor, lo, hi):
        t = tensor.contiguous()
        counts = torch.empty(self.bins, dtype=torch.int32, device=t.device)
        hist = torch.empty(self.bins, dtype=torch.float32, device=t.device)
        L.check(L.lib().lcq_histc(L.ptr(t), L.dtype_code(t.dtype), L.i64(t.numel()), L.i32(self.bins), L.f32(lo),
                                  L.f32(hi), L.ptr(counts), L.ptr(hist), L.stream()), 'lcq_histc')
        return hist.cpu()

    def get_norm(self, delta_begin, delta_end, density):
        """quant.py:264-277: density times the integral of x^2 over [delta_begin, delta_end]."""
        return density * ((delta_end * delta_end * delta_end - delta_begin * delta_begin * delta_begin) / 3)

    def get_quantization_error(self, histogram, min_val, max_val, next_start_bin, next_end_bin):
        """quant.py:279-328: L2 error of quantizing the histogram's mass with 2**bit levels spread over the source
        bins next_start_bin..next_end_bin; every source bin is a uniform density."""
        bin_width = (max_val.item() - min_val.item()) / self.bins
        dst_bin_width = bin_width * (next_end_bin - next_start_bin + 1) / self.dst_nbins
        if dst_bin_width == 0.0:
            return 0.0
        half = dst_bin_width / 2
        begin = (torch.arange(self.bins) - next_start_bin) * bin_width      # source bin edges from the first level's start
        end = begin + bin_width
        first = torch.clamp(torch.div(begin, dst_bin_width, rounding_mode='floor'), 0, self.dst_nbins - 1)
        last = torch.clamp(torch.div(end, dst_bin_width, rounding_mode='floor'), 0, self.dst_nbins - 1)
        density = histogram / bin_width
        norm = torch.zeros(self.bins)
        norm += self.get_norm(begin - (first + 0.5) * dst_bin_width, torch.ones(self.bins) * half, density)
        norm += (last - first - 1) * self.get_norm(torch.tensor(-half), torch.tensor(half), density)
        norm += self.get_norm(torch.tensor(-half), end - (last * dst_bin_width + half), density)
        return norm.sum().item()

    def _upscale_histogram(self, histogram, orig_min, orig_max, update_min, update_max):
        """quant.py:330-366: the old histogram, `upsample_rate` sub-bins per bin, dropped into the bins of the
        wider range."""
        fine = histogram.repeat_interleave(self.upsample_rate) / self.upsample_rate
        n_fine = self.bins * self.upsample_rate
        mids = torch.linspace(orig_min, orig_max, n_fine + 1)[:-1] + 0.5 * ((orig_max - orig_min) / n_fine)
        edges = torch.linspace(update_min, update_max, self.bins + 1)
        where = torch.bucketize(mids, edges, right=True) - 1
        where[where >= self.bins] = self.bins - 1
        where[where < 0] = 0
        return torch.bincount(where, weights=fine, minlength=self.bins)

    def _combine_histograms(self, orig_hist, orig_min, orig_max, update_hist, update_min, update_max):
        """quant.py:368-400."""
        if update_min == orig_min and update_max == orig_max:
            return orig_hist + update_hist
        if orig_min == orig_max:                               # a single value so far: its bin, weighted (quant.py:380-388)
            one = torch.histc(orig_min, bins=self.bins, min=update_min, max=update_max) * torch.sum(update_hist)
            return one + update_hist
        assert update_min <= orig_min
        assert update_max >= orig_max
        return update_hist + self._upscale_histogram(orig_hist, orig_min, orig_max, update_min, update_max)

    def get_hist_threshold(self, histogram, min_val, max_val):
        """quant.py:402-459: shrink the range one quantile step (1e-8 of the mass) at a time from whichever side
        gives up fewer bins, until the quantization error stops falling."""
        assert histogram.size()[0] == self.bins, 'bins mismatch'
        bin_width = (max_val - min_val) / self.bins
        total = torch.sum(histogram).item()
        csum = torch.cumsum(histogram, dim=0).tolist()         # fp32 values; a 0-dim fp32 tensor compares with a
        f32 = lambda v: torch.tensor(v, dtype=torch.float32).item()       # python number in fp32
        stepsize = 1e-8
        alpha, beta = 0.0, 1.0
        start_bin, end_bin = 0, self.bins - 1
        norm_min = float('inf')
        while alpha < beta:
            next_alpha, next_beta = alpha + stepsize, beta - stepsize
            lo_mass, hi_mass = f32(next_alpha * total), f32(next_beta * total)
            left, right = start_bin, end_bin
            while left < end_bin and csum[left] < lo_mass:
                left += 1
            while right > start_bin and csum[right] > hi_mass:
                right -= 1
            next_start_bin, next_end_bin = start_bin, end_bin
            if (left - start_bin) > (end_bin - right):
                next_start_bin, alpha = left, next_alpha
            else:
                next_end_bin, beta = right, next_beta
            if next_start_bin == start_bin and next_end_bin == end_bin:
                # Neither end moved: the reference goes on lowering beta by one step per iteration until the right
                # end does move - 1e8 steps per unit of mass, minutes for a histogram whose last bin is heavy
                # (clamped or rectified activations).  The same iterations, taken at once.
                beta = self._skip_idle_steps(alpha, beta, stepsize, csum[end_bin], total)
                continue
            norm = self.get_quantization_error(histogram, min_val, max_val, next_start_bin, next_end_bin)
            if norm > norm_min:
                break
            norm_min = norm
            start_bin, end_bin = next_start_bin, next_end_bin
        return min_val + bin_width * start_bin, min_val + bin_width * (end_bin + 1)

    @staticmethod
    def _beta_after(beta, n, step):
        """beta after n iterations of `beta = beta - step` in double precision, exactly: inside one binade every
        subtraction removes the same whole number of ulps, so runs of steps collapse into one product."""
        while n > 0:
            nxt = beta - step                              # one literal step (it may cross into the next binade)
            n -= 1
            beta = nxt
            if n == 0 or beta <= 0.0:
                break
            d = beta - (beta - step)                       # exact (Sterbenz): the effective step in this binade
            lo = 2.0 ** math.floor(math.log2(beta))        # beta in [lo, 2 lo)
            m = min(n, int((beta - lo) / d))               # steps whose results stay >= lo
            if m > 0 and beta - (beta - step) == d and (beta - m * d) >= lo:
                beta, n = beta - m * d, n - m              # m * d is exact: d is a few thousand ulps, m < 2**40
        return beta

    def _skip_idle_steps(self, alpha, beta, step, cs_end, total):
        """`beta` at the start of the first iteration in which the right end of get_hist_threshold moves, given that
        it does not move now (iteration i tests csum[end] > fp32((beta_i - step) * total), beta_i = i steps below
        beta); stops early where the loop would (alpha >= beta)."""
        f32 = lambda v: torch.tensor(v, dtype=torch.float32).item()
        idle = lambda b: b > alpha and not (cs_end > f32((b - step) * total))     # monotone: once False, False below
        if not idle(beta):
            return beta
        lo, hi = 0, max(1, int((beta - alpha) / step) + 2)      # idle(beta_lo) holds; beta_hi <= alpha, so it does not
        while hi - lo > 1:
            mid = (lo + hi) // 2
            if idle(self._beta_after(beta, mid, step)):
                lo = mid
            else:
                hi = mid
        return self._beta_after(beta, hi, step)

    def get_static_hist_range(self, act_tensors):
        """quant.py:461-521 -> (min_vals, max_vals), 0-dim fp32 CPU tensors, one per module input."""
        act_tensors = self.reshape_batch_tensors(act_tensors)
        stats = self.get_minmax_stats(act_tensors)
        new_min_vals, new_max_vals = [], []
        for input_idx, tensors in enumerate(act_tensors):
            histogram, min_val, max_val = None, None, None
            for idx, tensor in enumerate(tensors):
                x_min, x_max = stats[input_idx]['min'][idx], stats[input_idx]['max'][idx]
                if histogram is None:
                    histogram = self._histc(tensor, x_min.item(), x_max.item())
                    min_val, max_val = x_min, x_max
                    continue
                new_min, new_max = torch.min(min_val, x_min), torch.max(max_val, x_max)
                update = self._histc(tensor, new_min.item(), new_max.item())
                if new_min == min_val and new_max == max_val:
                    histogram = histogram + update
                else:
                    histogram = self._combine_histograms(histogram, min_val, max_val, update, new_min, new_max)
                min_val, max_val = new_min, new_max
            new_min, new_max = self.get_hist_threshold(histogram, min_val, max_val)
            new_min_vals.append(new_min)
            new_max_vals.append(new_max)
        return new_min_vals, new_max_vals

    def get_static_moving_minmax_range(self, act_tensors, alpha):
        """quant.py:523-542: exponential moving average of the per-tensor ranges, in the tensors' dtype."""
        act_tensors = self.reshape_batch_tensors(act_tensors)
        moving_min_vals, moving_max_vals = [], []
        for tensors in act_tensors:
            moving_min_val, moving_max_val = None, None
            for tensor in tensors:
                min_val, max_val = self.get_minmax_range(self.reshape_tensor(tensor))
                if moving_min_val is None or moving_max_val is None:
                    moving_min_val, moving_max_val = min_val, max_val
                else:
                    moving_min_val = moving_min_val + alpha * (min_val - moving_min_val)
                    moving_max_val = moving_max_val + alpha * (max_val - moving_max_val)
            moving_min_vals.append(moving_min_val)
            moving_max_vals.append(moving_max_val)
        return moving_min_vals, moving_max_vals

    def get_batch_tensors_qparams(self, act_tensors, alpha=0.01, args={}):
        """quant.py:559-585 -> (scales_list, zeros_list, qmin_list, qmax_list), one entry per module input."""
        if self.calib_algo == 'static_hist':
            assert (
                self.sym is True and self.granularity == 'per_tensor'
            ), 'Only support per tensor static symmetric int quantize.'
            min_vals, max_vals = self.get_static_hist_range(act_tensors)
        elif self.calib_algo == 'static_minmax':
            min_vals, max_vals = self.get_static_minmax_range(act_tensors)
        elif self.calib_algo == 'static_moving_minmax':
            min_vals, max_vals = self.get_static_moving_minmax_range(act_tensors, alpha)
        else:
            raise ValueError(f'Unsupported calibration algorithm: {self.calib_algo}')
        scales_list, zeros_list, qmin_list, qmax_list = [], [], [], []
        for min_val, max_val in zip(min_vals, max_vals):
            dev = min_val.device if min_val.is_cuda else torch.device('cuda', torch.cuda.current_device())
            scales, zeros, qmax, qmin = self.get_qparams((min_val.to(dev), max_val.to(dev)), dev)
            if not min_val.is_cuda:                          # host statistics give host qparams, as in the reference
                scales, qmax, qmin = scales.cpu(), qmax.cpu(), qmin.cpu()
                zeros = zeros.cpu()
            scales_list.append(scales)
            zeros_list.append(zeros)
            qmin_list.append(qmin)
            qmax_list.append(qmax)
        return scales_list, zeros_list, qmin_list, qmax_list

    # -- several experts in one launch --------------------------------------------------------------
    def real_quant_weight_dynamic_experts(self, weights, args={}):
        """real_quant_weight_dynamic of every matrix in `weights` (equal shapes) with ONE launch over their stacked
        rows -> list of (codes, scales, zeros) per expert, bit-identical to separate calls.  per_channel / per_group."""
        if self.granularity not in ('per_channel', 'per_group'):
            raise NotImplementedError('experts are stacked along the rows: per_channel / per_group only')
        E, (R, K) = len(weights), weights[0].shape
        codes, scales, zeros = self.real_quant_weight_dynamic(experts_as_rows(weights), dict(args))
        cs, ss = codes.view(E, R, -1), scales.view(E, R, -1)
        zs = None if zeros is None else zeros.view(E, R, -1)
        return [(cs[e], ss[e], None if zs is None else zs[e]) for e in range(E)]

    # -- HQQ (quant.py:587-609) -----------------------------------------------------------------
    def optimize_weights_proximal(self, tensor, scales, zeros, qmax, qmin):
        """Half-quadratic zero-point refinement: every iteration is one fused pass (lcq_hqq_step) where the
        reference runs about a dozen elementwise kernels; the loop and its early stop stay on the host, with the
        same one scalar read-back per iteration."""
        t = tensor.contiguous()
        if t.dtype != torch.float32 or t.dim() != 2:
            raise NotImplementedError('optimize_weights_proximal runs on the 2-D fp32 tensor get_hqq_qparams builds')
        rows, cols = t.shape
        s = scales.to(device=t.device, dtype=torch.float32).reshape(-1).contiguous()
        if s.numel() != rows:
            raise NotImplementedError('hqq needs one scale per row (per_channel / per_group)')
        z_in = None if _is_cpu_zero(zeros) else zeros.to(device=t.device, dtype=torch.float32).reshape(-1).contiguous()
        bufs = [torch.empty(rows, dtype=torch.float32, device=t.device) for _ in range(2)]
        err_rows = torch.empty(rows, dtype=torch.float32, device=t.device)
        scales_rt = torch.empty(rows, dtype=torch.float32, device=t.device)
        best_error = 1e4
        z_cur = z_in
        for i in range(self.iters):
            z_out = bufs[i & 1]
            L.check(L.lib().lcq_hqq_step(L.ptr(t), L.i64(rows), L.i64(cols), L.ptr(s), L.ptr(z_cur), L.ptr(z_out),
                                         L.ptr(err_rows), L.ptr(scales_rt), L.f32(1.0 / self.beta), L.f32(self.lp_norm),
                                         L.f32(float(qmin)), L.f32(float(qmax)), L.stream()), 'lcq_hqq_step')
            z_cur = z_out
            current_error = float(err_rows.sum()) / t.numel()
            if current_error < best_error:
                best_error = current_error
            else:
                break
        if z_cur is None:                                    # iters == 0
            z_cur = torch.zeros(rows, dtype=torch.float32, device=t.device) if z_in is None else z_in
            scales_rt = 1 / (1 / s)
        return scales_rt.view(rows, 1), z_cur.view(rows, 1)

    def get_hqq_qparams(self, tensor, args):
        """quant.py:679-687."""
        tensor = self.reshape_tensor(tensor.float())
        tensor_range = self.get_minmax_range(tensor)
        scales, zeros, qmax, qmin = self.get_qparams(tensor_range, tensor.device)
        best_scales, best_zeros = self.optimize_weights_proximal(tensor, scales, zeros, qmax, qmin)
        return tensor, best_scales, best_zeros, qmax, qmin

    # -- views (quant.py:611-657); torch view ops only ----------------------
    def reshape_tensor(self, tensor, allow_padding=False):
        if self.granularity == 'per_group':
            if tensor.shape[-1] >= self.group_size:
                if tensor.shape[-1] % self.group_size == 0:
                    t = tensor.reshape(-1, self.group_size)
                elif allow_padding:
                    deficiency = self.group_size - tensor.shape[1] % self.group_size
                    pad = torch.zeros((*tensor.shape[:-1], deficiency), device=tensor.device, dtype=tensor.dtype)
                    t = torch.cat((tensor, pad), dim=-1).reshape(-1, self.group_size)
                else:
                    raise ValueError(
                        f'Dimension {tensor.shape[-1]} '
                        f'not divisible by group size {self.group_size}'
                    )
            else:
                t = tensor
        elif self.granularity == 'per_head':
            t = tensor.reshape(self.head_num, -1)
        elif self.granularity == 'per_block':             # quant.py:634-638: zero-padded [M/b, b, N/b, b] view
            m, n = tensor.shape
            b = self.block_size
            t_padded = torch.zeros((ceil_div(m, b) * b, ceil_div(n, b) * b), dtype=tensor.dtype, device=tensor.device)
            t_padded[:m, :n] = tensor
            t = t_padded.view(-1, b, t_padded.size(1) // b, b)
        else:
            t = tensor
        return t

    def restore_tensor(self, tensor, shape):
        if tensor.shape == shape:
            return tensor
        if self.granularity == 'per_block':                # quant.py:646-650
            try:
                return tensor.reshape(-1, shape[-1])[:shape[0], :]
            except RuntimeError:
                return tensor.reshape(shape[0], -1)[:, :shape[1]]
        try:
            return tensor.reshape(shape)
        except RuntimeError:
            deficiency = self.group_size - shape[1] % self.group_size
            return tensor.reshape(*shape[:-1], -1)[..., :-deficiency]


def experts_as_rows(weights):
    """The [R, K] matrices of several experts as one [E * R, K] matrix: a view when they lie one behind the other in
    one tensor (slices of a stacked expert weight), a copy otherwise.  Row-wise granularities (per_channel, per_group)
    do not care which expert a row belongs to, and one launch over 16 experts runs at 0.72 - 0.75 of the HBM peak where
    a launch over one expert (29 MB) reaches 0.46 - 0.50: its ramp and tail are half of a 10 us kernel."""
    w0 = weights[0]
    if any(w.shape != w0.shape or w.dtype != w0.dtype or w.dim() != 2 for w in weights):
        raise ValueError('experts_as_rows: 2-D matrices of one shape and type')
    step = w0.numel() * w0.element_size()
    if all(w.is_contiguous() and w.untyped_storage().data_ptr() == w0.untyped_storage().data_ptr()
           and w.data_ptr() == w0.data_ptr() + i * step for i, w in enumerate(weights)):
        return w0.as_strided((len(weights) * w0.shape[0], w0.shape[1]), (w0.shape[1], 1))
    return torch.cat(list(weights), dim=0)


def _rows_cols(t):
    """A reshaped tensor as (rows, cols) for the row kernels."""
    if t.dim() == 0:
        return 1, 1
    cols = t.shape[-1]
    return (t.numel() // cols if cols else 0), cols


def _static_layout(t, scales):
    """How static qparams map onto rows of `t`: one per row, or one scalar."""
    rows, cols = _rows_cols(t)
    n = scales.numel()
    if n == 1:
        return rows, cols, True
    if n == rows:
        return rows, cols, False
    raise L.LcqError(f'qparams of shape {tuple(scales.shape)} do not match rows of tensor {tuple(t.shape)}')


def _is_cpu_zero(z):
    return z.device.type == 'cpu' and z.numel() == 1 and float(z) == 0.0


class IntegerQuantizer(BaseQuantizer):
    """quant.py:660-959."""

    def __init__(self, bit, symmetric, granularity, **kwargs):
        super().__init__(bit, symmetric, granularity, **kwargs)
        self.quant_type = 'int-quant'
        if 'int_range' in self.kwargs:
            self.qmin = self.kwargs['int_range'][0]
            self.qmax = self.kwargs['int_range'][1]
        else:
            if self.sym:
                self.qmin = -(2 ** (self.bit - 1))
                self.qmax = 2 ** (self.bit - 1) - 1
            else:
                self.qmin = 0.0
                self.qmax = 2 ** self.bit - 1
        self.qmin = torch.tensor(self.qmin)
        self.qmax = torch.tensor(self.qmax)
        self.dst_nbins = 2 ** bit
        self._bounds_dev = {}

    def _dev_bounds(self, device):
        """qmax / qmin as 0-dim tensors on `device` (what the reference hands out), cached."""
        key = str(device)
        if key not in self._bounds_dev:
            self._bounds_dev[key] = (self.qmax.to(device), self.qmin.to(device))
        return self._bounds_dev[key]

    def _bound(self, v):
        """Python float of a qmin/qmax argument without a device sync for our own tensors."""
        if not torch.is_tensor(v):
            return float(v)
        for qmax_d, qmin_d in self._bounds_dev.values():
            if v is qmax_d:
                return float(self.qmax)
            if v is qmin_d:
                return float(self.qmin)
        return float(v)

    # -- one fused launch -----------------------------------------------------
    def _launch(self, rows_t, *, static, scales=None, zeros=None, want_dq=False, want_codes=None,
                osf=1.0, qmin=None, qmax=None):
        """Run lcq_quant_int over a reshaped tensor.

        Returns (dq | None, codes | None, scales, zeros).  Dynamic mode creates
        scales / zeros of shape [rows, 1] (0-dim for per_tensor).
        """
        t = rows_t.contiguous()
        flags = self._int_flags()
        qmin = self._bound(self.qmin if qmin is None else qmin)
        qmax = self._bound(self.qmax if qmax is None else qmax)
        if static:
            # dimensioned qparams of another float type promote the computation like torch would
            if scales.dim() > 0 and scales.dtype != t.dtype:
                common = torch.promote_types(t.dtype, scales.dtype)
                t = t.to(common)
            # a 0-dim fp32 qparam next to a bf16 tensor (per_tensor, quant.py:544-558) goes in as fp32: torch on a GPU
            # reads a 0-dim tensor operand through a cast to the result type, which the kernel does where the
            # parameter meets the rows, while scales * output_scale_factor is still formed in fp32
            qp_dtype = t.dtype
            if scales.dim() == 0 and scales.dtype == torch.float32 and t.dtype != torch.float32:
                flags |= L.FLAG_SCALE_F32
                qp_dtype = torch.float32
            scales = scales.to(device=t.device, dtype=qp_dtype).contiguous()
            rows, cols, scalar = _static_layout(t, scales)
            flags |= L.FLAG_STATIC | (L.FLAG_SCALAR_QP if scalar else 0)
            z = None
            if zeros is not None and not _is_cpu_zero(zeros):
                z = zeros.to(device=t.device, dtype=qp_dtype).contiguous()
                if z.numel() != scales.numel():
                    z = z.expand_as(scales).contiguous()
        else:
            if self.granularity == 'per_tensor':
                lo, hi = self.get_minmax_range(t)
                scales, zeros, _, _ = self.get_qparams((lo, hi), t.device)
                return self._launch(t, static=True, scales=scales, zeros=zeros, want_dq=want_dq,
                                    want_codes=want_codes, osf=osf)
            rows, cols = _rows_cols(t)
            scales = torch.empty((rows, 1), dtype=t.dtype, device=t.device)
            z = None if self.sym else torch.empty((rows, 1), dtype=t.dtype, device=t.device)
        dq = torch.empty_like(t) if want_dq else None
        codes, cd = None, L.CODE_NONE
        if want_codes is not None:
            if want_codes == 'same':
                codes, cd = torch.empty_like(t), L.CODE_SAME
            elif want_codes == 'ct4':                    # eight 4-bit codes (+8) per int32, in row order
                codes, cd = torch.empty(t.numel() // 8, dtype=torch.int32, device=t.device), L.CODE_CT4
            else:
                codes = torch.empty(t.shape, dtype=want_codes, device=t.device)
                cd = {torch.int32: L.CODE_I32, torch.int8: L.CODE_I8, torch.uint8: L.CODE_U8}[want_codes]
        L.check(L.lib().lcq_quant_int(L.ptr(t), L.dtype_code(t.dtype), L.i64(rows), L.i64(cols), L.f32(qmin),
                                      L.f32(qmax), L.i32(flags), L.f32(osf), L.ptr(dq), L.ptr(codes), L.i32(cd),
                                      L.ptr(scales), L.ptr(z), L.stream()), 'lcq_quant_int')
        if not static:
            zeros = torch.tensor(0.0) if self.sym else z
        return dq, codes, scales, zeros

    # -- reference API ----------------------------------------------------------
    def get_tensor_qparams(self, tensor, args={}):
        """quant.py:689-696 -> (tensor_reshaped, scales, zeros, qmax, qmin)."""
        if self.calib_algo == 'hqq':
            return self.get_hqq_qparams(tensor, args)
        tensor = self.reshape_tensor(tensor)
        if self.calib_algo != 'minmax':
            scales, zeros, qmax, qmin = self.get_qparams(self.get_tensor_range(tensor, args), tensor.device)
            return tensor, scales, zeros, qmax, qmin
        if self.granularity == 'per_tensor':
            scales, zeros, qmax, qmin = self.get_qparams(self.get_minmax_range(tensor), tensor.device)
            return tensor, scales, zeros, qmax, qmin
        _, _, scales, zeros = self._launch(tensor, static=False)
        if tensor.dim() != 2:
            scales = scales.view(*tensor.shape[:-1], 1)
            if not self.sym:
                zeros = zeros.view(*tensor.shape[:-1], 1)
        qmax, qmin = self._dev_bounds(tensor.device)
        return tensor, scales, zeros, qmax, qmin

    def quant(self, tensor, scales, zeros, qmax, qmin):
        """quant.py:698-707: integer codes stored as floats."""
        _, codes, _, _ = self._launch(tensor, static=True, scales=scales, zeros=zeros, want_codes='same',
                                      qmin=qmin, qmax=qmax)
        return codes.view(tensor.shape)

    def dequant(self, tensor, scales, zeros):
        """quant.py:709-711."""
        t = tensor.contiguous()
        if scales.dim() > 0 and scales.dtype != t.dtype:
            t = t.to(torch.promote_types(t.dtype, scales.dtype))
        qp_dtype, flags = t.dtype, 0
        if scales.dim() == 0 and scales.dtype == torch.float32 and t.dtype != torch.float32:
            qp_dtype, flags = torch.float32, L.FLAG_SCALE_F32
        s = scales.to(device=t.device, dtype=qp_dtype).contiguous()
        rows, cols, scalar = _static_layout(t, s)
        z = None
        if zeros is not None and not _is_cpu_zero(zeros):
            z = zeros.to(device=t.device, dtype=qp_dtype).contiguous()
        out = torch.empty_like(t)
        L.check(L.lib().lcq_dequant_int(L.ptr(t), L.dtype_code(t.dtype), L.i64(rows), L.i64(cols), L.ptr(s), L.ptr(z),
                                        L.i32(flags | (L.FLAG_SCALAR_QP if scalar else 0)), L.f32(1.0), L.ptr(out),
                                        L.stream()), 'lcq_dequant_int')
        return out

    def quant_dequant(self, tensor, scales, zeros, qmax, qmin, output_scale_factor=1):
        """quant.py:713-716."""
        dq, _, _, _ = self._launch(tensor, static=True, scales=scales, zeros=zeros, want_dq=True,
                                   osf=output_scale_factor, qmin=qmin, qmax=qmax)
        return dq.view(tensor.shape)

    def _fake_dynamic(self, t, args={}):
        shape, dtype = t.shape, t.dtype
        rows_t = self.reshape_tensor(t)
        if self.calib_algo != 'minmax':                  # calibrated ranges, then the static path (quant.py:853-860)
            rargs = {k: args[k] for k in ('lowbound_factor', 'upbound_factor') if k in args} \
                if self.calib_algo == 'learnable' else {}
            rows_t, scales, zeros, qmax, qmin = self.get_tensor_qparams(t, rargs)
            dq, _, _, _ = self._launch(rows_t, static=True, scales=scales, zeros=zeros, want_dq=True, qmin=qmin, qmax=qmax)
            return self.restore_tensor(dq.view(rows_t.shape), shape).to(dtype)
        dq, _, _, _ = self._launch(rows_t, static=False, want_dq=True)
        return self.restore_tensor(dq.view(rows_t.shape), shape).to(dtype)

    def _fake_static(self, t, args):
        shape, dtype = t.shape, t.dtype
        rows_t = self.reshape_tensor(t)
        dq, _, _, _ = self._launch(rows_t, static=True, scales=args['scales'], zeros=args['zeros'], want_dq=True,
                                   osf=args.get('output_scale_factor', 1), qmin=args['qmin'], qmax=args['qmax'])
        return self.restore_tensor(dq.view(rows_t.shape), shape).to(dtype)

    def fake_quant_act_static(self, act, args={}):
        """quant.py:718-751.  `args['current_bit']` is accepted and changes nothing, as in the reference: it swaps
        `self.bit` for the duration of the call (:725-727, :742-743), which no arithmetic reads (qmin / qmax are
        fixed at construction and the given ones are used here)."""
        if 'int_indices' in args:
            q_act = act[:, :, args['int_indices']]
            fp_act = act[:, :, args['fp_indices']]
        else:
            q_act = act
        q_act = self._fake_static(q_act, args)
        if 'int_indices' in args:
            mix_act = torch.zeros_like(act)
            mix_act[:, :, args['int_indices']] = q_act
            mix_act[:, :, args['fp_indices']] = fp_act
            return mix_act
        return q_act

    def fake_quant_act_dynamic(self, act, args={}):
        """quant.py:753-782."""
        if 'int_indices' in args:
            q_act = act[:, :, args['int_indices']]
            fp_act = act[:, :, args['fp_indices']]
        else:
            q_act = act
        q_act = self._fake_dynamic(q_act)
        if 'int_indices' in args:
            mix_act = torch.zeros_like(act)
            mix_act[:, :, args['int_indices']] = q_act
            mix_act[:, :, args['fp_indices']] = fp_act
            return mix_act
        return q_act

    def _weight_view(self, weight, args):
        if 'int_indices' in args:
            if self.granularity == 'per_group':
                assert len(args['int_indices']) % self.group_size == 0
            return weight[:, args['int_indices']], weight[:, args['fp_indices']]
        if 'dim' in args and 'ic' in args['dim']:
            return weight.T, None
        return weight, None

    def _weight_merge(self, weight, q_weight, fp_weight, args):
        if 'int_indices' in args:
            mix_weight = torch.zeros_like(weight)
            mix_weight[:, args['int_indices']] = q_weight
            mix_weight[:, args['fp_indices']] = fp_weight
            return mix_weight
        if 'dim' in args and 'ic' in args['dim']:
            return q_weight.T
        return q_weight

    def fake_quant_weight_static(self, weight, args):
        """quant.py:784-830."""
        if 'rounding' in args:
            raise NotImplementedError("the 'rounding' override is not on this path")
        q_weight, fp_weight = self._weight_view(weight, args)
        q_weight = self._fake_static(q_weight, args)
        return self._weight_merge(weight, q_weight, fp_weight, args)

    def fake_quant_weight_dynamic(self, weight, args={}):
        """quant.py:832-868."""
        q_weight, fp_weight = self._weight_view(weight, args)
        q_weight = self._fake_dynamic(q_weight, args)
        return self._weight_merge(weight, q_weight, fp_weight, args)

    def _code_dtype(self):
        if self.bit == 8:
            return torch.int8 if self.qmin != 0 else torch.uint8
        return torch.int32

    def _finish_real(self, codes, scales, zeros, output_scale_factor):
        scales = _scaled(scales, output_scale_factor)
        dtype = self._code_dtype()
        if not self.sym and self.round_zp:
            zeros = zeros.to(dtype)
        elif self.sym:
            zeros = None
        qparams_shape = 1 if self.granularity == 'per_tensor' else (codes.shape[0], -1)
        if zeros is not None:
            zeros = zeros.view(qparams_shape)
        scales = scales.view(qparams_shape)
        return codes, scales, zeros

    def real_quant_weight_static(self, weight, args):
        """quant.py:870-913 -> (codes, scales, zeros|None)."""
        org_w_shape = weight.shape
        output_scale_factor = args.pop('output_scale_factor', 1)
        rows_t = self.reshape_tensor(weight)
        _, codes, _, _ = self._launch(rows_t, static=True, scales=args['scales'], zeros=args['zeros'],
                                      want_codes=self._code_dtype(), qmin=args['qmin'], qmax=args['qmax'])
        codes = self.restore_tensor(codes.view(rows_t.shape), org_w_shape)
        return self._finish_real(codes, args['scales'], args['zeros'], output_scale_factor)

    def real_quant_weight_dynamic(self, weight, args={}):
        """quant.py:915-952 -> (codes, scales, zeros|None)."""
        org_w_shape = weight.shape
        output_scale_factor = args.pop('output_scale_factor', 1) if 'output_scale_factor' in args else 1
        rows_t = self.reshape_tensor(weight)
        if self.calib_algo != 'minmax':
            rows_t, scales, zeros, qmax, qmin = self.get_tensor_qparams(weight)
            _, codes, _, _ = self._launch(rows_t, static=True, scales=scales, zeros=zeros, want_codes=self._code_dtype(),
                                          qmin=qmin, qmax=qmax)
        else:
            _, codes, scales, zeros = self._launch(rows_t, static=False, want_codes=self._code_dtype())
        codes = self.restore_tensor(codes.view(rows_t.shape), org_w_shape)
        return self._finish_real(codes, scales, zeros, output_scale_factor)

    def real_quant_pack_dynamic(self, weight):
        """Quantize and pack in one pass: what VllmRealQuantLinear.pack(*real_quant_weight_dynamic(w)[:2])
        returns for a symmetric 4-bit quantizer (module_utils.py:929-955 after quant.py:915-952), without
        the int32 codes ever reaching HBM -> (int32 [R, K/8], scales [R, -1], None)."""
        if self.bit != 4 or not self.sym or weight.dim() != 2 or weight.shape[1] % 8 != 0:
            raise NotImplementedError('fused quantize+pack: symmetric 4-bit, 2-D weight, in_features % 8 == 0')
        if weight.dtype == torch.float16:                   # fp16 rows have no fused kernel: quantize, then pack
            codes, scales, _ = self.real_quant_weight_dynamic(weight)
            packed = torch.empty((weight.shape[0], weight.shape[1] // 8), dtype=torch.int32, device=weight.device)
            cd = {torch.int32: L.CODE_I32, torch.int8: L.CODE_I8, torch.uint8: L.CODE_U8}[codes.dtype]
            L.check(L.lib().lcq_pack_ct(L.ptr(codes.contiguous()), L.i32(cd), L.i64(weight.shape[0]), L.i64(weight.shape[1]),
                                        L.i32(4), L.ptr(packed), L.stream()), 'lcq_pack_ct')
            return packed, scales, None
        rows_t = self.reshape_tensor(weight)
        _, packed, scales, _ = self._launch(rows_t, static=False, want_codes='ct4')
        qparams_shape = 1 if self.granularity == 'per_tensor' else (weight.shape[0], -1)
        return packed.view(weight.shape[0], weight.shape[1] // 8), scales.view(qparams_shape), None

    def real_quant_pack_dynamic_experts(self, weights):
        """real_quant_pack_dynamic of every matrix in `weights` with one launch -> list of (packed, scales, None)."""
        if self.granularity not in ('per_channel', 'per_group'):
            raise NotImplementedError('experts are stacked along the rows: per_channel / per_group only')
        E, (R, K) = len(weights), weights[0].shape
        packed, scales, _ = self.real_quant_pack_dynamic(experts_as_rows(weights))
        ps, ss = packed.view(E, R, -1), scales.view(E, R, -1)
        return [(ps[e], ss[e], None) for e in range(E)]

    def __repr__(self):
        return (
            f'IntegerQuantizer(bit={self.bit}, sym={self.sym},'
            f'granularity={self.granularity},'
            f'kwargs={self.kwargs}, qmin={self.qmin}, qmax={self.qmax})'
        )


class FloatQuantizer(BaseQuantizer):
    """quant.py:962-1228, qtorch branch.

    The minifloat rounding the reference delegates to QPyTorch's
    ``float_quantize(x, e, m, rounding='nearest')`` runs inside the kernel.  Two
    extra kwargs select its unpinned details: ``fp_tie`` ('away' default |
    'even') and ``fp_subnormals`` (True default).
    """

    _RANGES = {('e4m3', 8): torch.float8_e4m3fn, ('e5m2', 8): torch.float8_e5m2,
               ('e3m2', 6): (-28, 28), ('e4m7', 12): (-510, 510), ('e2m1', 4): (-6, 6)}

    def __init__(self, bit, symmetric, granularity, **kwargs):
        super().__init__(bit, symmetric, granularity, **kwargs)
        self.sym = True
        self.quant_type = 'float-quant'
        self.e_bits = int(self.bit[1])
        self.m_bits = int(self.bit[-1])
        self.sign_bits = 1
        self.num_bits = self.e_bits + self.m_bits + self.sign_bits
        self.default_bias = 2 ** (self.e_bits - 1)
        self.dst_nbins = 2 ** self.num_bits
        self.use_qtorch = self.kwargs.get('use_qtorch')
        self.fp_tie = self.kwargs.get('fp_tie', 'away')
        self.fp_subnormals = self.kwargs.get('fp_subnormals', True)
        if not self.use_qtorch:
            self.qmin = self.qmax = None                 # quant.py:972-1002 sets them only with qtorch
            return
        if 'float_range' in self.kwargs:
            self.qmin, self.qmax = self.kwargs['float_range']
        else:
            key = (self.bit, self.num_bits)
            if key not in self._RANGES:
                raise NotImplementedError('Only 4, 6, 8, and 12-bit quantization is supported.')
            if isinstance(self._RANGES[key], tuple):
                self.qmin, self.qmax = self._RANGES[key]
            else:
                finfo = torch.finfo(self._RANGES[key])
                self.qmin, self.qmax = finfo.min, finfo.max
        self.qmax = torch.tensor(self.qmax)
        self.qmin = torch.tensor(self.qmin)

    # -- use_qtorch=False: per-element steps (quant.py:1004-1026) ----------------------------------
    def _emu(self, rows_t, scales=None, want=(), rng=None):
        """One launch of lcq_quant_fp_emu -> dict with the requested outputs out of
        'xc', 'scales', 'q', 'q_fp8', 'dq'.  scales=None: dynamic (per-row ranges of rows_t, or `rng` = (min, max))."""
        t = rows_t.contiguous()
        flags = 0
        mn = mx = s_in = None
        if scales is None:
            if self.granularity == 'per_tensor':
                # the reference indexes maxval.shape[0] of a 0-dim range here (quant.py:1011)
                raise IndexError('tuple index out of range')
            mn, mx = self.get_minmax_range(t) if rng is None else (rng[0].to(t.dtype), rng[1].to(t.dtype))
            if self.e_bits >= 5 and t.dtype != torch.float32:
                t, mn, mx = t.float(), mn.float(), mx.float()        # maxval.to(float32), quant.py:1014-1015
            mn, mx = mn.contiguous(), mx.contiguous()
            rows, cols = _rows_cols(t)
        else:
            scales[scales == 0] = 1                                  # quant.py:1061 mutates the caller's tensor
            if scales.dim() > 0 and scales.dtype != t.dtype:
                t = t.to(torch.promote_types(t.dtype, scales.dtype))
            s_in = scales.to(t.dtype).contiguous()
            flags |= L.FLAG_STATIC
            if s_in.numel() == t.numel():
                rows, cols = _rows_cols(t)
            else:
                rows, cols, scalar = _static_layout(t, s_in)
                flags |= L.FLAG_SCALAR_QP if scalar else L.FLAG_ROW_QP
        out = {}
        for k in want:
            if k == 'q_fp8':
                out[k] = torch.empty(t.shape, dtype=torch.float8_e4m3fn if self.e_bits == 4 else torch.float8_e5m2,
                                     device=t.device)
            else:
                out[k] = torch.empty_like(t)
        q = out.get('q_fp8', out.get('q'))
        L.check(L.lib().lcq_quant_fp_emu(L.ptr(t), L.dtype_code(t.dtype), L.i64(rows), L.i64(cols), L.i32(self.e_bits),
                                         L.i32(self.m_bits), L.i32(flags), L.ptr(mn), L.ptr(mx), L.ptr(s_in),
                                         L.ptr(out.get('xc')), L.ptr(out.get('scales')), L.ptr(q),
                                         L.i32(L.CODE_FP8 if 'q_fp8' in out else L.CODE_SAME), L.ptr(out.get('dq')),
                                         L.stream()), 'lcq_quant_fp_emu')
        return out

    def get_float_qparams(self, tensor, tensor_range, device):
        """quant.py:1004-1026 -> (clamped tensor, elementwise scales).  `tensor_range` None: the per-row min / max of
        `tensor` (what get_tensor_range returns for it with calib_algo minmax); otherwise the given (min, max)."""
        o = self._emu(tensor, want=('xc', 'scales'), rng=tensor_range)
        return o['xc'].view(tensor.shape), o['scales'].view(tensor.shape)

    def _mse_range_float(self, tensor, norm):
        """get_mse_range (quant.py:147-205) for the minifloat quantizer: the shrink grid stays a host loop, every step
        is one range -> scale launch, one quantize-dequantize launch and the reference's elementwise error
        (|q - x| ** norm summed per row, fp32 torch ops).  `lo` / `hi` are views of the returned ranges and a row
        that improves overwrites them, so the next steps shrink the improved range - the reference's aliasing of
        best_min_val with min_val (quant.py:170, 196-198)."""
        t = tensor.float().contiguous()
        mn, mx = self.get_minmax_range(t)
        bs = t.shape[0] // self.mse_b_num
        for b in range(self.mse_b_num):
            x = t[b * bs:(b + 1) * bs]
            lo, hi = mn[b * bs:(b + 1) * bs], mx[b * bs:(b + 1) * bs]
            best = torch.full((x.shape[0], 1), float('inf'), device=t.device)
            for i in range(int(self.maxshrink * self.mse_grid)):
                p = 1 - i / self.mse_grid
                xmin, xmax = p * lo, p * hi
                if self.use_qtorch:
                    scales, zeros, qmax, qmin = self.get_qparams((xmin, xmax), t.device)
                    q = self.quant_dequant(x, scales, zeros, qmax, qmin)
                else:
                    q = self._emu(x, want=('dq',), rng=(xmin, xmax))['dq'].view(x.shape)
                err = q.sub_(x).abs_().pow_(norm).sum(1, keepdim=True)
                better = err < best
                best = torch.where(better, err, best)
                lo.copy_(torch.where(better, xmin, lo))
                hi.copy_(torch.where(better, xmax, hi))
        return (mn, mx)

    def get_hqq_qparams(self, tensor, args):
        """quant.py:1028-1040: the HQQ solver returns non-zero zero points, which the minifloat quantize kernels
        (zero point 0, as every other calibration of this class gives) do not take."""
        raise NotImplementedError("calib_algo='hqq' with FloatQuantizer: zero points other than 0 are not on this path")

    def _fp_flags(self):
        return ((L.FLAG_TIE_EVEN if self.fp_tie == 'even' else 0)
                | (0 if self.fp_subnormals else L.FLAG_NO_SUBNORMALS))

    def get_qparams(self, tensor_range, device):
        """Symmetric branch of quant.py:544-552 with the float qmax."""
        min_val, max_val = tensor_range[0].contiguous(), tensor_range[1].contiguous()
        flags = L.FLAG_SYM
        # 0-dim ranges (per_tensor) divided by the 0-dim fp32 qmax promote to fp32
        if max_val.dim() == 0 and max_val.dtype != torch.float32:
            flags |= L.FLAG_RANGE_BF16 if max_val.dtype == torch.bfloat16 else L.FLAG_RANGE_F16
            min_val, max_val = min_val.float(), max_val.float()
        scales = torch.empty_like(max_val)
        L.check(L.lib().lcq_qparams_int(L.ptr(min_val), L.ptr(max_val), L.dtype_code(max_val.dtype),
                                        L.i64(max_val.numel()), L.f32(-float(self.qmax)), L.f32(self.qmax),
                                        L.i32(flags), L.ptr(scales), L.ptr(None), L.stream()),
                'lcq_qparams_int')
        return scales, torch.tensor(0.0), self.qmax.to(device), self.qmin.to(device)

    def _launch(self, rows_t, *, static, scales=None, want_dq=None, want_codes=None):
        t = rows_t.contiguous()
        flags = self._fp_flags()
        if static:
            scales[scales == 0] = 1                      # quant.py:1061 mutates the caller's tensor
            if scales.dim() > 0 and scales.dtype != t.dtype:
                t = t.to(torch.promote_types(t.dtype, scales.dtype))
            if scales.dim() == 0 and scales.dtype == torch.float32 and t.dtype != torch.float32:
                s = scales.contiguous()                  # x / s rounds s to the row type, dq keeps fp32
                flags |= L.FLAG_SCALE_F32
            else:
                s = scales.to(t.dtype).contiguous()
            rows, cols, scalar = _static_layout(t, s)
            flags |= L.FLAG_STATIC | (L.FLAG_SCALAR_QP if scalar else 0)
        else:
            if self.granularity == 'per_tensor':
                s, _, _, _ = self.get_qparams(self.get_minmax_range(t), t.device)
                return self._launch(t, static=True, scales=s, want_dq=want_dq, want_codes=want_codes)
            rows, cols = _rows_cols(t)
            s = torch.empty((rows, 1), dtype=t.dtype, device=t.device)
        dq = None
        if want_dq == 'f32':
            dq = torch.empty(t.shape, dtype=torch.float32, device=t.device)
            flags |= L.FLAG_DQ_F32
        elif want_dq:
            dq = torch.empty_like(t)
        codes, cd = None, L.CODE_NONE
        if want_codes == 'f32':
            codes, cd = torch.empty(t.shape, dtype=torch.float32, device=t.device), L.CODE_F32
        elif want_codes is not None:
            codes, cd = torch.empty(t.shape, dtype=want_codes, device=t.device), L.CODE_FP8
        L.check(L.lib().lcq_quant_fp(L.ptr(t), L.dtype_code(t.dtype), L.i64(rows), L.i64(cols), L.i32(self.e_bits),
                                     L.i32(self.m_bits), L.f32(self.qmax), L.i32(flags), L.ptr(dq), L.ptr(codes),
                                     L.i32(cd), L.ptr(s), L.stream()), 'lcq_quant_fp')
        return dq, codes, s

    def get_tensor_qparams(self, tensor, args={}):
        """quant.py:1042-1058 -> (tensor_reshaped, scales, zeros, qmax, qmin)."""
        if self.calib_algo == 'hqq':
            return self.get_hqq_qparams(tensor, args)
        if self.granularity == 'per_block':
            raise NotImplementedError('per_block ranges are taken inside the block-wise cast (fake / real quant methods)')
        tensor = self.reshape_tensor(tensor)
        if self.calib_algo in ('mse', 'learnable'):          # the shared dispatch of quant.py:124-132
            tensor_range = self.get_tensor_range(tensor, args)
            if not self.use_qtorch:
                xc, s = self.get_float_qparams(tensor, tensor_range, tensor.device)
                return xc, s, torch.tensor(0), None, None
            s, z, qmax, qmin = self.get_qparams(tensor_range, tensor.device)
            return tensor, s, z, qmax, qmin
        if not self.use_qtorch:
            xc, s = self.get_float_qparams(tensor, None, tensor.device)
            return xc, s, torch.tensor(0), None, None
        if self.granularity == 'per_tensor':
            s, z, qmax, qmin = self.get_qparams(self.get_minmax_range(tensor), tensor.device)
            return tensor, s, z, qmax, qmin
        _, _, s = self._launch(tensor, static=False)
        if tensor.dim() != 2:
            s = s.view(*tensor.shape[:-1], 1)
        return tensor, s, torch.tensor(0.0), self.qmax.to(tensor.device), self.qmin.to(tensor.device)

    def quant(self, tensor, scales, zeros, qmax, qmin):
        """quant.py:1060-1071: fp32 values on the minifloat grid (qtorch) / round(t / s) in the
        tensor's type (no qtorch)."""
        if not self.use_qtorch:
            return self._emu(tensor, scales, want=('q',))['q'].view(tensor.shape)
        _, codes, _ = self._launch(tensor, static=True, scales=scales, want_codes='f32')
        return codes.view(tensor.shape)

    def dequant(self, tensor, scales, zeros):
        """quant.py:1073-1075 on fp32 codes."""
        if not self.use_qtorch:
            t = tensor.contiguous()
            s = scales.to(t.dtype).contiguous()
            if s.numel() == t.numel():
                rows, cols, flags = t.numel(), 1, 0
            else:
                rows, cols, scalar = _static_layout(t, s)
                flags = L.FLAG_SCALAR_QP if scalar else 0
            out = torch.empty_like(t)
            L.check(L.lib().lcq_dequant_int(L.ptr(t), L.dtype_code(t.dtype), L.i64(rows), L.i64(cols), L.ptr(s),
                                            L.ptr(None), L.i32(flags | L.FLAG_SYM), L.f32(1.0), L.ptr(out), L.stream()),
                    'lcq_dequant_int')
            return out
        t = tensor.float().contiguous()
        s = scales.contiguous()
        rows, cols, scalar = _static_layout(t, s)
        out = torch.empty_like(t)
        L.check(L.lib().lcq_dequant_fp(L.ptr(t), L.i64(rows), L.i64(cols), L.ptr(s), L.dtype_code(s.dtype),
                                       L.i32(L.FLAG_SCALAR_QP if scalar else 0), L.ptr(out), L.stream()),
                'lcq_dequant_fp')
        return out

    def quant_dequant(self, tensor, scales, zeros, qmax, qmin):
        """quant.py:1077-1080: fp32 result (the float codes promote it); the tensor's type without qtorch."""
        if not self.use_qtorch:
            return self._emu(tensor, scales, want=('dq',))['dq'].view(tensor.shape)
        dq, _, _ = self._launch(tensor, static=True, scales=scales, want_dq='f32')
        return dq.view(tensor.shape)

    def _calibrated(self, t, args):
        """Dynamic quantization with calib_algo mse / learnable: (rows, scales, zeros, qmax, qmin) through
        get_tensor_qparams, as quant.py:1099-1108, 1137-1155, 1194-1206 do."""
        rargs = {k: args[k] for k in ('lowbound_factor', 'upbound_factor') if k in args} \
            if self.calib_algo == 'learnable' else {}
        return self.get_tensor_qparams(t, rargs)

    def _fake(self, t, static_scales=None, args={}):
        if self.granularity == 'per_block':
            if static_scales is not None:
                return self._per_block_static(t, static_scales, True)
            return self._per_block(t, True)
        shape, dtype = t.shape, t.dtype
        if static_scales is None and self.calib_algo != 'minmax':
            rows_t, scales, zeros, qmax, qmin = self._calibrated(t, args)
            dq = self.quant_dequant(rows_t, scales, zeros, qmax, qmin)
            return self.restore_tensor(dq.view(rows_t.shape), shape).to(dtype)
        rows_t = self.reshape_tensor(t)
        if not self.use_qtorch:
            dq = self._emu(rows_t, static_scales, want=('dq',))['dq']
            return self.restore_tensor(dq.view(rows_t.shape), shape).to(dtype)
        if static_scales is None:
            dq, _, _ = self._launch(rows_t, static=False, want_dq=True)
        else:
            dq, _, _ = self._launch(rows_t, static=True, scales=static_scales, want_dq=True)
        return self.restore_tensor(dq.view(rows_t.shape), shape).to(dtype)

    def fake_quant_act_static(self, act, args={}):
        return self._fake(act, args['scales'])

    def fake_quant_act_dynamic(self, act, args={}):
        return self._fake(act, None, args)

    def fake_quant_weight_static(self, weight, args):
        if 'rounding' in args:
            raise NotImplementedError("the 'rounding' override is not on this path")
        ic = 'dim' in args and 'ic' in args['dim']
        q = self._fake(weight.T if ic else weight, args['scales'])
        return q.T if ic else q

    def fake_quant_weight_dynamic(self, weight, args={}):
        ic = 'dim' in args and 'ic' in args['dim']
        q = self._fake(weight.T if ic else weight, None, args)
        return q.T if ic else q

    def _per_block(self, weight, want_dq):
        """per_block granularity (quant.py:138-140, 634-638): 128 x 128 blocks, fp32 ranges and scales."""
        from .kernel import FLAG_CLAMP_RANGE, FLAG_TIE_AWAY, _block_quant, _block_dequant
        if self.bit != 'e4m3' or self.block_size != 128 or not self.use_qtorch or not self.fp_subnormals:
            raise NotImplementedError('per_block runs for e4m3, block_size 128, use_qtorch=True')
        if weight.dim() != 2:
            raise NotImplementedError('per_block expects a 2-D weight')
        flags = FLAG_CLAMP_RANGE | (0 if self.fp_tie == 'even' else FLAG_TIE_AWAY)
        y, s = _block_quant(weight.contiguous(), 128, flags)
        if want_dq:
            return _block_dequant(y, s, torch.float32).to(weight.dtype)
        return y, s

    def _per_block_static(self, weight, scales, want_dq):
        """per_block with GIVEN block scales (fake / real_quant_weight_static, quant.py:1113-1139, 1160-1192 on the
        zero-padded [mb, bs, nb, bs] view of reshape_tensor :634-638 with scales [mb, 1, nb, 1]): every block becomes
        one row of bs * bs elements with its scale, the row kernel does the rest, and the rows go back into place.
        -> the dequantized weight in the weight's type, or float8 codes."""
        if not self.use_qtorch or weight.dim() != 2:
            raise NotImplementedError('static per_block scales: 2-D weights, use_qtorch=True')
        bs = self.block_size
        m, n = weight.shape
        mb, nb = -(-m // bs), -(-n // bs)
        if scales.numel() != mb * nb:
            raise L.LcqError(f'per_block: {scales.numel()} scales for {mb} x {nb} blocks')
        scales[scales == 0] = 1                          # quant.py:1061 mutates the caller's tensor
        w = weight
        if (m, n) != (mb * bs, nb * bs):
            w = torch.zeros((mb * bs, nb * bs), dtype=weight.dtype, device=weight.device)
            w[:m, :n] = weight
        rows = w.view(mb, bs, nb, bs).permute(0, 2, 1, 3).reshape(mb * nb, bs * bs)
        s_rows = scales.reshape(mb * nb, 1).clone()
        if want_dq:
            out, _, _ = self._launch(rows, static=True, scales=s_rows, want_dq=True)
        else:
            _, out, _ = self._launch(rows, static=True, scales=s_rows,
                                     want_codes=torch.float8_e4m3fn if self.e_bits == 4 else torch.float8_e5m2)
        out = out.view(mb, nb, bs, bs).permute(0, 2, 1, 3).reshape(mb * bs, nb * bs)[:m, :n]
        return out.to(weight.dtype) if want_dq else out.contiguous()

    def _real(self, weight, static_scales, output_scale_factor, args={}):
        assert self.bit in ['e4m3', 'e5m2'], 'Only FP8 E4M3 and E5M2 support real quant'
        if self.granularity == 'per_block':
            if static_scales is not None:
                y = self._per_block_static(weight, static_scales, False)
                s = _scaled(static_scales, output_scale_factor)
                return y, (s.view(s.shape[0], s.shape[2]) if s.dim() == 4 else s), None
            y, s = self._per_block(weight, False)
            return y, _scaled(s, output_scale_factor), None
        dtype = torch.float8_e4m3fn if self.e_bits == 4 else torch.float8_e5m2
        org_w_shape = weight.shape
        if static_scales is None and self.calib_algo != 'minmax':
            rows_t, static_scales, _, _, _ = self._calibrated(weight, args)      # then as with given scales
            weight = rows_t
        rows_t = self.reshape_tensor(weight)
        if not self.use_qtorch:
            if static_scales is None:
                o = self._emu(rows_t, want=('q_fp8', 'scales'))
                scales = o['scales']
            else:
                o = self._emu(rows_t, static_scales, want=('q_fp8',))
                scales = static_scales
            codes = self.restore_tensor(o['q_fp8'].view(rows_t.shape), org_w_shape)
            scales = _scaled(scales, output_scale_factor)
            return codes, scales.view(1 if self.granularity == 'per_tensor' else (codes.shape[0], -1)), None
        if static_scales is None:
            _, codes, scales = self._launch(rows_t, static=False, want_codes=dtype)
        else:
            _, codes, _ = self._launch(rows_t, static=True, scales=static_scales, want_codes=dtype)
            scales = static_scales
        codes = self.restore_tensor(codes.view(rows_t.shape), org_w_shape)
        scales = _scaled(scales, output_scale_factor)
        qparams_shape = 1 if self.granularity == 'per_tensor' else (codes.shape[0], -1)
        return codes, scales.view(qparams_shape), None

    def real_quant_weight_static(self, weight, args):
        """quant.py:1160-1192."""
        return self._real(weight, args['scales'], args.pop('output_scale_factor', 1))

    def real_quant_weight_dynamic(self, weight, args={}):
        """quant.py:1194-1220."""
        osf = args.pop('output_scale_factor', 1) if 'output_scale_factor' in args else 1
        return self._real(weight, None, osf, args)

    def __repr__(self):
        return (
            f'FloatQuantizer(bit={self.bit},'
            f'e_bits={self.e_bits}, m_bits={self.m_bits},'
            f'granularity={self.granularity},'
            f'kwargs={self.kwargs}, qmin={self.qmin}, qmax={self.qmax})'
        )


# -- quant.py:20-45 of the reference: the block-wise float8 casts it uses where its Triton kernels do not run ----
class Weight48IntegerQuantizer(BaseQuantizer):
    """quant.py:1230-1367: weights to 8-bit integers, those integers to 4-bit integers (second-level
    scales / zero points optionally confined to an integer range), and back.  Both levels run on the
    integer quantizer's kernels: range -> lcq_minmax_rows, qparams -> lcq_qparams_int, codes kept in the
    tensor's dtype -> lcq_quant_int, back -> lcq_dequant_int."""

    def __init__(self, bit, bit4, bit8, **kwargs):
        super().__init__(bit, None, None, **kwargs)
        self.quant_type = 'int-quant-w48'
        assert self.bit == 48, 'Only support 48-bit quantization'
        self.bit_settings = {4: bit4, 8: bit8}
        self._stage = {}
        for b, cfg in self.bit_settings.items():
            if 'zeros_bit' in cfg:
                raise NotImplementedError('zeros_bit: zero points outside [qmin, qmax] are not on this path')
            extra = {k: cfg[k] for k in ('int_range', 'group_size') if k in cfg}
            q = IntegerQuantizer(b, cfg['symmetric'], cfg.get('granularity'), **extra)
            self._stage[b] = q
            cfg['qmin'], cfg['qmax'] = q.qmin, q.qmax
            if 'scales_bit' in cfg:
                n = cfg['scales_bit']
                cfg['scales_qmin'] = -(2 ** (n - 1)) if cfg['scales_symmetric'] else 0
                cfg['scales_qmax'] = 2 ** (n - 1) - 1 if cfg['scales_symmetric'] else 2 ** n - 1
            else:
                cfg['scales_qmin'], cfg['scales_qmax'] = -torch.inf, torch.inf
            cfg['zeros_qmin'], cfg['zeros_qmax'] = cfg['qmin'], cfg['qmax']

    def reshape_tensor(self, tensor, bit=4):
        cfg = self.bit_settings[bit]
        if cfg.get('granularity') == 'per_group':
            group_size = cfg.get('group_size')
            if tensor.shape[-1] % group_size != 0:
                raise ValueError(f'Dimension {tensor.shape[-1]} not divisible by group size {group_size}')
            return tensor.reshape(-1, group_size)
        return tensor

    def get_minmax_range(self, tensor):
        cols = tensor.shape[-1]
        t = tensor.contiguous()
        mn = torch.empty((*t.shape[:-1], 1), dtype=t.dtype, device=t.device)
        mx = torch.empty_like(mn)
        L.check(L.lib().lcq_minmax_rows(L.ptr(t), L.dtype_code(t.dtype), L.i64(t.numel() // cols), L.i64(cols),
                                        L.ptr(mn), L.ptr(mx), L.stream()), 'lcq_minmax_rows')
        return (mn, mx)

    def get_qparams(self, tensor_range, device, bit):
        cfg = self.bit_settings[bit]
        scales, zeros, qmax, qmin = self._stage[bit].get_qparams(tensor_range, device)
        if 'scales_bit' in cfg:                                   # a clamp of [rows, 1] parameters
            scales = scales.clamp(cfg['scales_qmin'], cfg['scales_qmax'])
        return scales, zeros, qmax, qmin

    def quant(self, tensor, scales, zeros, qmax, qmin):
        return self._stage[4].quant(tensor, scales, zeros, qmax, qmin)

    def dequant(self, tensor, scales, zeros):
        return self._stage[4].dequant(tensor, scales, zeros)

    def quant_dequant(self, tensor, scales, zeros, qmax, qmin):
        return self.dequant(self.quant(tensor, scales, zeros, qmax, qmin), scales, zeros)

    def fake_quant_weight_dynamic(self, weight, args={}):
        org_shape16, org_dtype16 = weight.shape, weight.dtype
        # 16 -> 8 bit
        weight = self.reshape_tensor(weight, bit=8)
        scales816, zeros816, qmax816, qmin816 = self.get_qparams(self.get_tensor_range(weight), weight.device, bit=8)
        weight = self.quant(weight, scales816, zeros816, qmax816, qmin816)
        # 8 -> 4 bit
        org_shape8, org_dtype8 = weight.shape, weight.dtype
        weight = self.reshape_tensor(weight, bit=4)
        scales48, zeros48, qmax48, qmin48 = self.get_qparams(self.get_tensor_range(weight), weight.device, bit=4)
        weight = self.quant(weight, scales48, zeros48, qmax48, qmin48)
        # 4 -> 8 -> 16 bit
        weight = self.restore_tensor(self.dequant(weight, scales48, zeros48), org_shape8).to(org_dtype8)
        weight = self.restore_tensor(self.dequant(weight, scales816, zeros816), org_shape16).to(org_dtype16)
        return weight

    def restore_tensor(self, tensor, shape):
        return tensor.reshape(shape) if tensor.shape != shape else tensor


def weight_cast_to_bf16(weight, scale, block_size):
    """float8 block-wise weight -> bf16: FloatQuantizer('e4m3', per_block).dequant(weight.float(), scale, 0)."""
    from .kernel import _block_dequant
    if block_size != 128:
        raise NotImplementedError('block_size 128 only')
    return _block_dequant(weight.contiguous(), scale, torch.bfloat16)


def weight_cast_to_fp8(weight, block_size):
    """bf16 / fp32 weight -> (float8_e4m3fn, fp32 scales [nbm, nbn]): real_quant_weight_dynamic of
    FloatQuantizer('e4m3', per_block, use_qtorch=True): s = clamp(max|x|, 1e-5) / 448, float_quantize's
    ties-away rounding (parameter ``fp_tie`` of FloatQuantizer; this function keeps the default)."""
    q = FloatQuantizer('e4m3', True, 'per_block', block_size=block_size, use_qtorch=True)
    fp8_weight, fp8_scale, _ = q.real_quant_weight_dynamic(weight)
    return fp8_weight, fp8_scale
