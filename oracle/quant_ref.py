"""Oracle: integer / minifloat quantizer arithmetic (test infrastructure only).

Restates quant.py of the reference as free functions over CPU torch tensors.
The op ORDER and the dtype each op runs in are what make results bit-exact,
so every line keeps the reference's op sequence (one torch op per arithmetic
step, no fusing) while the structure (functions + a small spec object instead
of a class hierarchy) is this repo's own.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import numpy as np
import torch


# ----------------------------------------------------------------------------
# spec
# ----------------------------------------------------------------------------
@dataclass
class IntSpec:
    """Mirror of the ctor surface, quant.py:49-103 and 660-677."""
    bit: int
    symmetric: bool
    granularity: str                      # per_tensor|per_channel|per_group|per_head|per_token
    group_size: int = 0
    head_num: int = 0
    round_zp: bool = True
    int_range: tuple | None = None
    qmin: torch.Tensor = field(init=False)
    qmax: torch.Tensor = field(init=False)

    def __post_init__(self):
        if self.int_range is not None:
            lo, hi = self.int_range
        elif self.symmetric:
            lo, hi = -(2 ** (self.bit - 1)), 2 ** (self.bit - 1) - 1
        else:
            lo, hi = 0.0, 2 ** self.bit - 1          # qmin is a python float there (quant.py:672)
        self.qmin = torch.tensor(lo)
        self.qmax = torch.tensor(hi)


# ----------------------------------------------------------------------------
# reshape / restore   (quant.py:611-657)
# ----------------------------------------------------------------------------
def reshape_rows(spec, t: torch.Tensor, allow_padding=False) -> torch.Tensor:
    if spec.granularity == 'per_group':
        g = spec.group_size
        if t.shape[-1] < g:
            return t
        if t.shape[-1] % g == 0:
            return t.reshape(-1, g)
        if not allow_padding:
            raise ValueError(f'Dimension {t.shape[-1]} not divisible by group size {g}')
        lack = g - t.shape[1] % g
        pad = torch.zeros((*t.shape[:-1], lack), dtype=t.dtype)
        return torch.cat((t, pad), dim=-1).reshape(-1, g)
    if spec.granularity == 'per_head':
        return t.reshape(spec.head_num, -1)
    return t


def restore_rows(spec, t: torch.Tensor, shape) -> torch.Tensor:
    if t.shape == shape:
        return t
    try:
        return t.reshape(shape)
    except RuntimeError:
        lack = spec.group_size - shape[1] % spec.group_size
        return t.reshape(*shape[:-1], -1)[..., :-lack]


# ----------------------------------------------------------------------------
# range -> qparams   (quant.py:134-145, 544-558)
# ----------------------------------------------------------------------------
def minmax_range(spec, t: torch.Tensor):
    if spec.granularity == 'per_tensor':
        return torch.min(t), torch.max(t)
    return t.amin(dim=-1, keepdim=True), t.amax(dim=-1, keepdim=True)


def int_qparams(spec, lo: torch.Tensor, hi: torch.Tensor):
    qmin, qmax = spec.qmin, spec.qmax
    if spec.symmetric:
        span = torch.max(hi.abs(), lo.abs())
        span = span.clamp(min=1e-5)
        scales = span / qmax
        zeros = torch.tensor(0.0)
    else:
        scales = (hi - lo).clamp(min=1e-5) / (qmax - qmin)
        zeros = (qmin - torch.round(lo / scales)).clamp(qmin, qmax)
        if not spec.round_zp:
            zeros = qmin - (lo / scales)
    return scales, zeros, qmax, qmin


def int_tensor_qparams(spec, t: torch.Tensor):
    """quant.py:689-696 (minmax calibration)."""
    rows = reshape_rows(spec, t)
    lo, hi = minmax_range(spec, rows)
    s, z, qmax, qmin = int_qparams(spec, lo, hi)
    return rows, s, z, qmax, qmin


# ----------------------------------------------------------------------------
# quant / dequant   (quant.py:698-716)
# ----------------------------------------------------------------------------
def as_operand(t, q):
    """A 0-dim floating tensor `q` as an operand of an element-wise operation with the 16-bit tensor `t`, the way the
    reference's platform treats it.  torch on a GPU reads a 0-dim *tensor* operand through a cast to the type of the
    result, so a 0-dim fp32 scale or zero point (per_tensor: quant.py:544-558 builds them from 0-dim ranges and the
    0-dim fp32 qmax / qmin) is rounded to bf16 / fp16 before the division, sum or product; torch on the CPU does that
    for sums and differences only and keeps the fp32 value in products and quotients.  The reference runs on the GPU:
    the conversion is written out here so that the CPU evaluation gives the GPU's result
    (tests/test_torch_gpu_semantics_gpu.py evaluates the reference's expressions with torch on the GPU)."""
    if torch.is_tensor(q) and q.dim() == 0 and q.is_floating_point() and torch.is_tensor(t) and t.dim() > 0 \
            and t.dtype in (torch.bfloat16, torch.float16) and q.dtype != t.dtype:
        return q.to(t.dtype)
    return q


def mean_rows(t):
    """``t.mean(0)`` of a [N, ...] tensor (K elements per slice) the way the reference's platform computes it.  torch's
    GPU reduction multiplies the fp32 sum by the fp32 factor float(K) / (N * K) and casts the fp32 product to the
    tensor's type; torch's CPU kernel divides the sum by N.  The two differ in the last place for about a third of the
    fp32 results when N is not a power of two.  On a GPU tensor of fp32 or bf16 this is torch itself.  For fp16 the
    rule is written out on either device: torch's ROCm build fuses the multiply with the cast (one rounding of the
    exact product, different where sum * factor is an fp16 tie) while its CUDA build rounds twice, which is what the
    restatement and the library do (tests/test_torch_gpu_semantics_gpu.py compares all of them on sums that are exact
    in fp32)."""
    if t.dtype not in (torch.float32, torch.float16, torch.bfloat16) or (t.is_cuda and t.dtype != torch.float16):
        return t.mean(0)
    n, k = t.shape[0], t[0].numel()
    factor = float(np.float32(k) / np.float32(n * k))
    return (t.float().sum(0) * factor).to(t.dtype)


def int_quant(spec, t, scales, zeros, qmax, qmin):
    if spec.round_zp:
        return torch.clamp(torch.round(t / as_operand(t, scales)) + as_operand(t, zeros), qmin, qmax)
    return torch.clamp(torch.round(t / as_operand(t, scales.clamp_min(1e-9)) + as_operand(t, zeros)), qmin, qmax)


def int_dequant(t, scales, zeros):
    return (t - as_operand(t, zeros)) * as_operand(t, scales)


def int_quant_dequant(spec, t, scales, zeros, qmax, qmin, output_scale_factor=1):
    q = int_quant(spec, t, scales, zeros, qmax, qmin)
    return int_dequant(q, scales * output_scale_factor, zeros)


def int_fake_quant_dynamic(spec, w: torch.Tensor) -> torch.Tensor:
    """fake_quant_weight_dynamic / fake_quant_act_dynamic, quant.py:753-782, 832-868."""
    shape, dtype = w.shape, w.dtype
    rows, s, z, qmax, qmin = int_tensor_qparams(spec, w)
    out = int_quant_dequant(spec, rows, s, z, qmax, qmin)
    return restore_rows(spec, out, shape).to(dtype)


def int_fake_quant_static(spec, w, scales, zeros, qmax, qmin, output_scale_factor=1):
    """fake_quant_weight_static, quant.py:784-830 (no index mixing)."""
    shape, dtype = w.shape, w.dtype
    rows = reshape_rows(spec, w)
    out = int_quant_dequant(spec, rows, scales, zeros, qmax, qmin, output_scale_factor)
    return restore_rows(spec, out, shape).to(dtype)


def _code_dtype(spec):
    if spec.bit == 8:
        return torch.int8 if spec.qmin != 0 else torch.uint8
    return torch.int32


def _qparam_shape(spec, codes):
    return 1 if spec.granularity == 'per_tensor' else (codes.shape[0], -1)


def int_real_quant_dynamic(spec, w, output_scale_factor=1):
    """real_quant_weight_dynamic, quant.py:915-952."""
    shape = w.shape
    rows, s, z, qmax, qmin = int_tensor_qparams(spec, w)
    codes = restore_rows(spec, int_quant(spec, rows, s, z, qmax, qmin), shape)
    s = s * output_scale_factor
    dt = _code_dtype(spec)
    codes = codes.to(dt)
    if not spec.symmetric and spec.round_zp:
        z = z.to(dt)
    elif spec.symmetric:
        z = None
    shp = _qparam_shape(spec, codes)
    if z is not None:
        z = z.view(shp)
    return codes, s.view(shp), z


def int_real_quant_static(spec, w, scales, zeros, qmax, qmin, output_scale_factor=1):
    """real_quant_weight_static, quant.py:870-913."""
    shape = w.shape
    rows = reshape_rows(spec, w)
    codes = restore_rows(spec, int_quant(spec, rows, scales, zeros, qmax, qmin), shape)
    s = scales * output_scale_factor
    dt = _code_dtype(spec)
    codes = codes.to(dt)
    z = zeros
    if not spec.symmetric and spec.round_zp:
        z = z.to(dt)
    elif spec.symmetric:
        z = None
    shp = _qparam_shape(spec, codes)
    if z is not None:
        z = z.view(shp)
    return codes, s.view(shp), z


# ----------------------------------------------------------------------------
# minifloat ("FPx") quantizer, qtorch mode   (quant.py:962-1002, 1042-1080)
# ----------------------------------------------------------------------------
_FLOAT_RANGE = {'e4m3': 448.0, 'e5m2': 57344.0, 'e3m2': 28.0, 'e4m7': 510.0, 'e2m1': 6.0}


@dataclass
class FloatSpec:
    bit: str                       # 'e4m3' ...
    granularity: str
    group_size: int = 0
    head_num: int = 0
    float_range: tuple | None = None
    # rounding model of the third-party float_quantize (parity unpinned)
    tie: str = 'away'              # 'away' (add-half-then-truncate) | 'even'
    subnormals: bool = True
    symmetric: bool = True         # forced, quant.py:965
    round_zp: bool = True

    def __post_init__(self):
        self.e_bits = int(self.bit[1])
        self.m_bits = int(self.bit[-1])
        if self.float_range is not None:
            lo, hi = self.float_range
        else:
            hi = _FLOAT_RANGE[self.bit]
            lo = -hi
        self.qmin = torch.tensor(float(lo))
        self.qmax = torch.tensor(float(hi))


def float_quantize_nearest(x: torch.Tensor, e_bits: int, m_bits: int,
                           tie: str = 'away', subnormals: bool = True) -> torch.Tensor:
    """Round fp32 ``x`` to a (1, e_bits, m_bits) minifloat grid, result in fp32.

    Restates the *published* algorithm of QPyTorch's ``float_quantize(...,
    rounding='nearest')`` (third-party, absent from the reference tree;
    call site quant.py:1065-1067), working on the fp32 bit pattern:

    * normal range: add half of the dropped-mantissa ulp to the raw bits and
      truncate (``tie='away'``: ties go away from zero) — or RNE for
      ``tie='even'`` (what a native float8 cast does);
    * below the minimum normal 2**(2 - 2**(e_bits-1)): with ``subnormals`` the
      value is rounded on the fixed step  min_normal * 2**-m_bits  (by adding
      +-min_normal, rounding the mantissa, subtracting again); without, it is
      flushed to 0 or +-min_normal whichever is nearer;
    * the exponent is clipped at 2**(e_bits-1): the largest magnitude is
      2**(2**(e_bits-1)) * (2 - 2**-m_bits)  (480 for e4m3, above the 448 the
      reference scales to, so saturation never fires on in-range inputs).
    """
    assert x.dtype == torch.float32
    a = np.ascontiguousarray(x.detach().numpy())
    bits = a.view(np.uint32).astype(np.uint64)
    sign = bits & 0x80000000
    mag = bits & 0x7FFFFFFF
    drop = 23 - m_bits
    half = np.uint64(1 << (drop - 1))
    keep = np.uint64(~((1 << drop) - 1) & 0xFFFFFFFF)

    def round_mag(m):
        if tie == 'away':
            return (m + half) & keep
        lsb = (m >> np.uint64(drop)) & np.uint64(1)
        return (m + half - np.uint64(1) + lsb) & keep

    min_exp = -((1 << (e_bits - 1)) - 2)              # exponent of the minimum normal
    max_exp = 1 << (e_bits - 1)
    exp_field = (mag >> np.uint64(23)).astype(np.int64) - 127
    is_sub = exp_field < min_exp
    finite = (mag >> np.uint64(23)) != 0xFF

    out_norm = round_mag(mag)
    # exponent clipping (saturate to the largest representable magnitude)
    max_mag = np.uint64(((max_exp + 127) << 23) | (((1 << m_bits) - 1) << drop))
    out_norm = np.where((out_norm >> np.uint64(23)).astype(np.int64) - 127 > max_exp, max_mag, out_norm)

    mn = np.float32(2.0 ** min_exp)
    absx = np.abs(a)
    if subnormals:
        shifted = (absx.astype(np.float32) + mn).astype(np.float32)
        sb = round_mag(shifted.view(np.uint32).astype(np.uint64))
        sub_val = (sb.astype(np.uint32).view(np.float32) - mn).astype(np.float32)
    else:
        sub_val = np.where(absx > mn / 2, mn, np.float32(0)).astype(np.float32)
    sub_bits = sub_val.view(np.uint32).astype(np.uint64)

    out = np.where(is_sub, sub_bits, out_norm)
    out = np.where(finite, out, mag)                   # inf / nan pass through
    res = (out | sign).astype(np.uint32).view(np.float32)
    return torch.from_numpy(res.copy()).reshape(x.shape)


def float_qparams(spec, lo, hi):
    """get_qparams (symmetric branch) as used by FloatQuantizer, quant.py:544-552, 1048-1051."""
    span = torch.max(hi.abs(), lo.abs())
    span = span.clamp(min=1e-5)
    scales = span / spec.qmax
    zeros = torch.tensor(0.0)
    return scales, zeros, spec.qmax, spec.qmin


def float_tensor_qparams(spec, t):
    rows = reshape_rows(spec, t)
    lo, hi = minmax_range(spec, rows)
    s, z, qmax, qmin = float_qparams(spec, lo, hi)
    return rows, s, z, qmax, qmin


def float_quant(spec, t, scales, zeros):
    """quant.py:1060-1071 (qtorch branch): result is fp32 whatever the input dtype."""
    scales[scales == 0] = 1
    scaled = t / as_operand(t, scales) + zeros
    return float_quantize_nearest(scaled.float(), spec.e_bits, spec.m_bits, spec.tie, spec.subnormals)


def float_dequant(t, scales, zeros):
    return (t - zeros) * scales


def float_fake_quant_dynamic(spec, w):
    """quant.py:1099-1108, 1141-1158."""
    shape, dtype = w.shape, w.dtype
    rows, s, z, _, _ = float_tensor_qparams(spec, w)
    q = float_quant(spec, rows, s, z)
    out = float_dequant(q, s, z)
    return restore_rows(spec, out, shape).to(dtype)


def float_real_quant_dynamic(spec, w, output_scale_factor=1):
    """quant.py:1194-1220."""
    assert spec.bit in ('e4m3', 'e5m2')
    dt = torch.float8_e4m3fn if spec.e_bits == 4 else torch.float8_e5m2
    shape = w.shape
    rows, s, z, _, _ = float_tensor_qparams(spec, w)
    q = restore_rows(spec, float_quant(spec, rows, s, z), shape)
    s = s * output_scale_factor
    q = q.to(dt)
    shp = 1 if spec.granularity == 'per_tensor' else (q.shape[0], -1)
    return q, s.view(shp), None


# ----------------------------------------------------------------------------
# FloatQuantizer(use_qtorch=False): per-element power-of-two-like steps
# ----------------------------------------------------------------------------
def float_emu_qparams(spec, rows: torch.Tensor, lo: torch.Tensor, hi: torch.Tensor):
    """get_float_qparams, quant.py:1004-1026, one torch op per step (the two 0-dim fp32 tensors
    the reference creates with .cuda() live where the rows live).  Returns (clamped rows, elementwise
    scales).  On GPU tensors this is the reference's own evaluation (torch's GPU log2 / pow), on CPU tensors
    the same formula through the CPU math library: bf16 rows give the same bits either way, fp32 rows differ
    in the last place of log2 for about a quarter of the rows.  Pinned by test_oracle_quant.py: the row maximum is a fixed point, results are
    idempotent, relative step 2**-m_bits in the normal range, fixed step below it, and an fp64
    evaluation of the same formula on exactly representable inputs."""
    maxval = torch.max(hi, -lo)
    e_bits = torch.tensor(spec.e_bits, dtype=torch.float32).to(rows.device)      # `.cuda()` in the reference
    m_bits = torch.tensor(spec.m_bits, dtype=torch.float32).to(rows.device)
    if maxval.shape[0] != 1 and len(maxval.shape) != len(rows.shape):
        maxval = maxval.view([-1] + [1] * (len(rows.shape) - 1))
    if e_bits >= 5:
        maxval = maxval.to(dtype=torch.float32)
    bias = 2 ** e_bits - torch.log2(maxval) + torch.log2(2 - 2 ** (-m_bits)) - 1
    xc = torch.min(torch.max(rows, -maxval), maxval)
    log_scales = torch.clamp(torch.floor(torch.log2(torch.abs(xc)) + bias), 1.0)
    scales = 2.0 ** (log_scales - m_bits - bias)
    return xc, scales


def float_emu_quant(t, scales, zeros):
    """quant.py:1060-1071 with round_func = torch.round."""
    scales[scales == 0] = 1
    return torch.round(t / scales + zeros)


def float_emu_tensor_qparams(spec, t):
    """get_tensor_qparams, quant.py:1042-1058 (non-qtorch branch): zeros is an int64 0-dim 0."""
    rows = reshape_rows(spec, t)
    lo, hi = minmax_range(spec, rows)
    xc, scales = float_emu_qparams(spec, rows, lo, hi)
    return xc, scales, torch.tensor(0), None, None


def float_emu_fake_quant_dynamic(spec, w):
    """quant.py:1099-1108 / 1141-1158 without qtorch."""
    shape, dtype = w.shape, w.dtype
    xc, s, z, _, _ = float_emu_tensor_qparams(spec, w)
    q = float_emu_quant(xc, s, z)
    out = float_dequant(q, s, z)
    return restore_rows(spec, out, shape).to(dtype)


def float_emu_real_quant_dynamic(spec, w, output_scale_factor=1):
    """quant.py:1194-1220 without qtorch: integer-valued codes stored as float8, elementwise scales."""
    assert spec.bit in ('e4m3', 'e5m2')
    dt = torch.float8_e4m3fn if spec.e_bits == 4 else torch.float8_e5m2
    shape = w.shape
    xc, s, z, _, _ = float_emu_tensor_qparams(spec, w)
    q = restore_rows(spec, float_emu_quant(xc, s, z), shape)
    s = s * output_scale_factor
    q = q.to(dt)
    return q, s.view(q.shape[0], -1), None


# ----------------------------------------------------------------------------
# block-wise float8 (e4m3) casts
# ----------------------------------------------------------------------------
def triton_weight_cast_to_fp8(x: torch.Tensor, block_size: int = 128):
    """kernel.py:57-85 (weight_cast_to_fp8_kernel) as torch ops: per block s = max|x| / 448 in fp32,
    y = (x.float() / s).to(float8_e4m3fn) - the cast rounds to nearest even like Triton's."""
    M, N = x.shape
    mb, nb = -(-M // block_size), -(-N // block_size)
    y = torch.empty(M, N, dtype=torch.float8_e4m3fn)
    s = torch.empty(mb, nb, dtype=torch.float32)
    for i in range(mb):
        for j in range(nb):
            blk = x[i * block_size:(i + 1) * block_size, j * block_size:(j + 1) * block_size].float()
            sc = blk.abs().max() / 448.0
            s[i, j] = sc
            y[i * block_size:(i + 1) * block_size, j * block_size:(j + 1) * block_size] = (blk / sc).to(torch.float8_e4m3fn)
    return y, s


def triton_act_quant(x: torch.Tensor, block_size: int = 128):
    """kernel.py:7-54: one scale per block_size elements of the last dimension."""
    xb = x.float().reshape(-1, block_size)
    s = xb.abs().amax(dim=-1) / 448.0
    y = (xb / s.unsqueeze(-1)).to(torch.float8_e4m3fn).reshape(x.shape)
    return y, s.reshape(*x.shape[:-1], x.shape[-1] // block_size)


def triton_weight_cast_to_bf16(y: torch.Tensor, s: torch.Tensor, block_size: int = 128, dtype=torch.bfloat16):
    """kernel.py:88-138: float(y) * s per block, stored in `dtype`."""
    M, N = y.shape
    se = s.repeat_interleave(block_size, 0)[:M].repeat_interleave(block_size, 1)[:, :N]
    return (y.float() * se).to(dtype)


def float_per_block_real_quant(spec, w: torch.Tensor, block_size: int = 128):
    """weight_cast_to_fp8 of quant.py:33-45: FloatQuantizer('e4m3', per_block).real_quant_weight_dynamic, i.e.
    reshape_tensor (zero-padded [mb, bs, nb, bs], :634-638), abs().float() block ranges (:138-140), symmetric
    qparams (:548-552), float_quantize on x / s in fp32 (:1060-1068), cast to float8, restore (:647-651)."""
    m, n = w.shape
    mb, nb = -(-m // block_size), -(-n // block_size)
    t_padded = torch.zeros((mb * block_size, nb * block_size), dtype=w.dtype)
    t_padded[:m, :n] = w
    t = t_padded.view(-1, block_size, t_padded.size(1) // block_size, block_size)
    min_val = t.abs().float().amin(dim=(1, 3), keepdim=True)
    max_val = t.abs().float().amax(dim=(1, 3), keepdim=True)
    scales, zeros, _, _ = float_qparams(spec, min_val, max_val)
    q = float_quant(spec, t, scales, zeros)
    q = q.reshape(-1, n if nb * block_size == n else nb * block_size)[:m, :n]
    return q.to(torch.float8_e4m3fn), scales.view(scales.shape[0], scales.shape[2]), None


def float_per_block_static(spec, w: torch.Tensor, scales: torch.Tensor, block_size: int = 128, real=False):
    """fake_quant_weight_static / real_quant_weight_static of FloatQuantizer with per_block granularity and GIVEN
    scales [mb, 1, nb, 1] (quant.py:1113-1139, 1160-1192): reshape_tensor's zero-padded 4-D view (:634-638), x / s
    broadcast per block, float_quantize, (dequantize,) restore_tensor (:647-651), cast."""
    m, n = w.shape
    mb, nb = -(-m // block_size), -(-n // block_size)
    t_padded = torch.zeros((mb * block_size, nb * block_size), dtype=w.dtype)
    t_padded[:m, :n] = w
    t = t_padded.view(-1, block_size, t_padded.size(1) // block_size, block_size)
    zeros = torch.tensor(0.0)
    q = float_quant(spec, t, scales, zeros)
    if not real:
        q = float_dequant(q, scales, zeros)
    q = q.reshape(-1, nb * block_size)[:m, :n]
    return q.to(torch.float8_e4m3fn if spec.e_bits == 4 else torch.float8_e5m2) if real else q.to(w.dtype)


# ----------------------------------------------------------------------------
# calib_algo 'mse'
# ----------------------------------------------------------------------------
def int_mse_range(spec, tensor: torch.Tensor, norm=2.4, maxshrink=0.8, mse_grid=100, mse_b_num=1):
    """get_mse_range, quant.py:147-205, op for op - including its aliasing: `best_min_val, best_max_val = _min_val,
    _max_val` are views of the range tensors, so an improving step overwrites the range that the following
    steps shrink."""
    assert mse_b_num >= 1 and tensor.shape[0] % mse_b_num == 0
    bs = tensor.shape[0] // mse_b_num
    tensor = tensor.float()
    min_val, max_val = minmax_range(spec, tensor)
    for b_num in range(mse_b_num):
        _tensor = tensor[b_num * bs:(b_num + 1) * bs, :]
        _min_val, _max_val = min_val[b_num * bs:(b_num + 1) * bs, :], max_val[b_num * bs:(b_num + 1) * bs, :]
        best = torch.full([_tensor.shape[0]], float('inf'), device=_tensor.device)
        best_min_val, best_max_val = _min_val, _max_val
        for i in range(int(maxshrink * mse_grid)):
            p = 1 - i / mse_grid
            xmin = p * _min_val
            xmax = p * _max_val
            scales, zeros, qmax, qmin = int_qparams(spec, xmin, xmax)
            q_tensor = int_quant_dequant(spec, _tensor, scales, zeros, qmax, qmin)
            q_tensor -= _tensor
            q_tensor.abs_()
            q_tensor.pow_(norm)
            err = torch.sum(q_tensor, 1)
            tmp = err < best
            if torch.any(tmp):
                best[tmp] = err[tmp]
                best_min_val[tmp] = xmin[tmp]
                best_max_val[tmp] = xmax[tmp]
        min_val[b_num * bs:(b_num + 1) * bs, :], max_val[b_num * bs:(b_num + 1) * bs, :] = best_min_val, best_max_val
    return min_val, max_val


def float_mse_range(spec, tensor: torch.Tensor, norm=2.4, maxshrink=0.8, mse_grid=100, mse_b_num=1):
    """get_mse_range, quant.py:147-205, for FloatQuantizer(use_qtorch=True): the same recurrence (aliasing included)
    with the symmetric float qparams (:544-552) and float_quantize in quant_dequant (:1060-1080)."""
    assert mse_b_num >= 1 and tensor.shape[0] % mse_b_num == 0
    bs = tensor.shape[0] // mse_b_num
    tensor = tensor.float()
    min_val, max_val = minmax_range(spec, tensor)
    for b_num in range(mse_b_num):
        _tensor = tensor[b_num * bs:(b_num + 1) * bs, :]
        _min_val, _max_val = min_val[b_num * bs:(b_num + 1) * bs, :], max_val[b_num * bs:(b_num + 1) * bs, :]
        best = torch.full([_tensor.shape[0]], float('inf'), device=_tensor.device)
        best_min_val, best_max_val = _min_val, _max_val
        for i in range(int(maxshrink * mse_grid)):
            p = 1 - i / mse_grid
            xmin = p * _min_val
            xmax = p * _max_val
            scales, zeros, _, _ = float_qparams(spec, xmin, xmax)
            q_tensor = float_dequant(float_quant(spec, _tensor, scales, zeros), scales, zeros)
            q_tensor -= _tensor
            q_tensor.abs_()
            q_tensor.pow_(norm)
            err = torch.sum(q_tensor, 1)
            tmp = err < best
            if torch.any(tmp):
                best[tmp] = err[tmp]
                best_min_val[tmp] = xmin[tmp]
                best_max_val[tmp] = xmax[tmp]
        min_val[b_num * bs:(b_num + 1) * bs, :], max_val[b_num * bs:(b_num + 1) * bs, :] = best_min_val, best_max_val
    return min_val, max_val


def float_fake_quant_with_range(spec, w, lo, hi):
    """fake_quant_weight_dynamic of FloatQuantizer once get_tensor_range has given (lo, hi) - calib_algo mse or
    learnable, quant.py:1042-1058, 1141-1158."""
    shape, dtype = w.shape, w.dtype
    rows = reshape_rows(spec, w)
    s, z, _, _ = float_qparams(spec, lo, hi)
    out = float_dequant(float_quant(spec, rows, s, z), s, z)
    return restore_rows(spec, out, shape).to(dtype)


def learnable_range(spec, rows, lowbound_factor=None, upbound_factor=None):
    """get_learnable_range, quant.py:207-221."""
    lo, hi = minmax_range(spec, rows)
    if spec.symmetric:
        if upbound_factor is not None:
            abs_max = torch.max(hi.abs(), lo.abs()).clamp(min=1e-5)
            abs_max = torch.sigmoid(upbound_factor) * abs_max
            lo, hi = -abs_max, abs_max
    elif upbound_factor is not None and lowbound_factor is not None:
        lo, hi = torch.sigmoid(lowbound_factor) * lo, torch.sigmoid(upbound_factor) * hi
    return lo, hi


# ----------------------------------------------------------------------------
# HQQ zero-point refinement   (quant.py:94-103, 587-609, 679-687)
# ----------------------------------------------------------------------------
def hqq_shrink(x: torch.Tensor, beta_ctor: float, lp_norm: float) -> torch.Tensor:
    """shrink_op, quant.py:94-103.  Both lambdas read self.beta (the constructor value): the annealed beta the
    solver hands them is ignored."""
    if lp_norm == 1:
        return torch.sign(x) * torch.nn.functional.relu(torch.abs(x) - 1.0 / beta_ctor)
    return torch.sign(x) * torch.nn.functional.relu(
        torch.abs(x) - (1.0 / beta_ctor) * torch.pow(torch.abs(x), lp_norm - 1))


def hqq_optimize(tensor, scales, zeros, qmax, qmin, lp_norm=0.7, beta=10, kappa=1.01, iters=20):
    """optimize_weights_proximal, quant.py:587-609 -> (scales, zeros, iterations run)."""
    best_error = 1e4
    current_beta = beta
    scales = 1 / scales
    n_run = 0
    for i in range(iters):
        n_run += 1
        W_q = torch.round(tensor * scales + zeros).clamp(qmin, qmax)
        W_r = (W_q - zeros) / scales
        W_e = hqq_shrink(tensor - W_r, beta, lp_norm)
        zeros = torch.mean(W_q - (tensor - W_e) * scales, axis=-1, keepdim=True)
        current_beta *= kappa
        current_error = float(torch.abs(tensor - W_r).mean())
        if current_error < best_error:
            best_error = current_error
        else:
            break
    scales = 1 / scales
    return scales, zeros, n_run


def int_hqq_qparams(spec, t: torch.Tensor, **hqq):
    """get_hqq_qparams, quant.py:679-687 -> (rows fp32, scales, zeros, qmax, qmin)."""
    rows = reshape_rows(spec, t.float())
    lo, hi = minmax_range(spec, rows)
    s, z, qmax, qmin = int_qparams(spec, lo, hi)
    s, z, _ = hqq_optimize(rows, s, z, qmax, qmin, **hqq)
    return rows, s, z, qmax, qmin


# ----------------------------------------------------------------------------
# static activation calibration   (quant.py:105-124, 223-262, 523-585)
# ----------------------------------------------------------------------------
def _batch_lists(act_tensors):
    if isinstance(act_tensors[0], tuple):
        return [torch.stack(ts) for ts in zip(*act_tensors)]
    if len(act_tensors) == 1:
        return [[act_tensors[0][i] for i in range(act_tensors[0].size(0))]]
    return [act_tensors]


def static_minmax_ranges(spec, act_tensors):
    """get_static_minmax_range, quant.py:252-262: fp32 mean of the per-tensor ranges, per module input."""
    mins, maxs = [], []
    for tensors in _batch_lists(act_tensors):
        lo = torch.stack([minmax_range(spec, reshape_rows(spec, t))[0].float() for t in tensors])
        hi = torch.stack([minmax_range(spec, reshape_rows(spec, t))[1].float() for t in tensors])
        mins.append(lo.mean(dim=0))                       # (the reference has moved the ranges to the host by now:
        maxs.append(hi.mean(dim=0))                       # this is torch's CPU mean on either platform)
    return mins, maxs


def static_moving_minmax_ranges(spec, act_tensors, alpha):
    """get_static_moving_minmax_range, quant.py:523-542."""
    mins, maxs = [], []
    for tensors in _batch_lists(act_tensors):
        m_lo = m_hi = None
        for t in tensors:
            lo, hi = minmax_range(spec, reshape_rows(spec, t))
            if m_lo is None:
                m_lo, m_hi = lo, hi
            else:
                m_lo = m_lo + alpha * (lo - m_lo)
                m_hi = m_hi + alpha * (hi - m_hi)
        mins.append(m_lo)
        maxs.append(m_hi)
    return mins, maxs


# ----------------------------------------------------------------------------
# histogram observer, calib_algo 'static_hist'   (quant.py:264-521)
# ----------------------------------------------------------------------------
def histc_device(x: torch.Tensor, bins: int, lo: float, hi: float) -> torch.Tensor:
    """torch.histc as torch's DEVICE kernel bins (the reference's activations are on the GPU, quant.py:473-487):
    bin = (int)((v - lo) * bins / (hi - lo)) in fp32, multiply first, the top edge counted into the last bin,
    values outside [lo, hi] dropped, lo == hi widened by one to each side.  Restated from ATen's published
    SummaryOps kernel; the CPU torch.histc divides first and so differs on values next to a bin edge - the
    CPU test pins this function against it up to exactly those values, and the GPU test
    (tests/test_quant_gpu.py::test_histogram_kernel) against torch.histc on GPU tensors, count for count."""
    lo32, hi32 = np.float32(lo), np.float32(hi)
    if lo32 == hi32:
        lo32, hi32 = lo32 - np.float32(1), hi32 + np.float32(1)
    v = x.detach().float().flatten().numpy()
    v = v[(v >= lo32) & (v <= hi32)]
    b = ((v - lo32) * np.float32(bins) / (hi32 - lo32)).astype(np.int64)
    b[b == bins] = bins - 1
    return torch.from_numpy(np.bincount(b, minlength=bins).astype(np.float32))


def hist_quantization_error(hist, min_val, max_val, start_bin, end_bin, bins, dst_nbins):
    """get_quantization_error + get_norm, quant.py:264-328, op for op on CPU fp32 tensors."""
    def get_norm(delta_begin, delta_end, density):
        norm = (delta_end * delta_end * delta_end - delta_begin * delta_begin * delta_begin) / 3
        return density * norm
    bin_width = (max_val.item() - min_val.item()) / bins
    dst_bin_width = bin_width * (end_bin - start_bin + 1) / dst_nbins
    if dst_bin_width == 0.0:
        return 0.0
    src_bin = torch.arange(bins)
    src_bin_begin = (src_bin - start_bin) * bin_width
    src_bin_end = src_bin_begin + bin_width
    dst_bin_of_begin = torch.clamp(torch.div(src_bin_begin, dst_bin_width, rounding_mode='floor'), 0, dst_nbins - 1)
    dst_bin_of_begin_center = (dst_bin_of_begin + 0.5) * dst_bin_width
    dst_bin_of_end = torch.clamp(torch.div(src_bin_end, dst_bin_width, rounding_mode='floor'), 0, dst_nbins - 1)
    density = hist / bin_width
    norm = torch.zeros(bins)
    delta_begin = src_bin_begin - dst_bin_of_begin_center
    delta_end = dst_bin_width / 2
    norm += get_norm(delta_begin, torch.ones(bins) * delta_end, density)
    norm += (dst_bin_of_end - dst_bin_of_begin - 1) * get_norm(torch.tensor(-dst_bin_width / 2),
                                                              torch.tensor(dst_bin_width / 2), density)
    dst_bin_of_end_center = dst_bin_of_end * dst_bin_width + dst_bin_width / 2
    delta_begin = -dst_bin_width / 2
    delta_end = src_bin_end - dst_bin_of_end_center
    norm += get_norm(torch.tensor(delta_begin), delta_end, density)
    return norm.sum().item()


def hist_combine(orig_hist, orig_min, orig_max, update_hist, update_min, update_max, bins, upsample_rate=16):
    """_combine_histograms + _upscale_histogram, quant.py:330-400."""
    if update_min == orig_min and update_max == orig_max:
        return orig_hist + update_hist
    if orig_min == orig_max:
        bin_value = torch.sum(update_hist)
        return torch.histc(orig_min, bins=bins, min=update_min, max=update_max) * bin_value + update_hist
    assert update_min <= orig_min and update_max >= orig_max
    histogram = orig_hist.repeat_interleave(upsample_rate) / upsample_rate
    bin_size = (orig_max - orig_min) / (bins * upsample_rate)
    mid_points = torch.linspace(orig_min, orig_max, bins * upsample_rate + 1)[:-1] + 0.5 * bin_size
    boundaries = torch.linspace(update_min, update_max, bins + 1)
    bucket = torch.bucketize(mid_points, boundaries, right=True) - 1
    bucket[bucket >= bins] = bins - 1
    bucket[bucket < 0] = 0
    return update_hist + torch.bincount(bucket, weights=histogram, minlength=bins)


def hist_threshold(hist, min_val, max_val, bins, dst_nbins):
    """get_hist_threshold, quant.py:402-459, the loop as written.  Its `cSum[i] < next_alpha * total` compares a 0-dim
    fp32 tensor with a python number, which torch evaluates in fp32: written here as a comparison of python floats
    with the right-hand side rounded to fp32 (the loop takes one step per 1e-8 of the mass, millions for a
    histogram with heavy edge bins; as tensor operations that is minutes)."""
    bin_width = (max_val - min_val) / bins
    total = torch.sum(hist).item()
    cSum = torch.cumsum(hist, dim=0).tolist()
    f32 = lambda v: float(np.float32(v))
    stepsize = 1e-8
    alpha, beta = 0.0, 1.0
    start_bin, end_bin = 0, bins - 1
    norm_min = float('inf')
    while alpha < beta:
        next_alpha = alpha + stepsize
        next_beta = beta - stepsize
        left, right = start_bin, end_bin
        while left < end_bin and cSum[left] < f32(next_alpha * total):
            left = left + 1
        while right > start_bin and cSum[right] > f32(next_beta * total):
            right = right - 1
        next_start_bin, next_end_bin = start_bin, end_bin
        if (left - start_bin) > (end_bin - right):
            next_start_bin = left
            alpha = next_alpha
        else:
            next_end_bin = right
            beta = next_beta
        if next_start_bin == start_bin and next_end_bin == end_bin:
            continue
        norm = hist_quantization_error(hist, min_val, max_val, next_start_bin, next_end_bin, bins, dst_nbins)
        if norm > norm_min:
            break
        norm_min = norm
        start_bin, end_bin = next_start_bin, next_end_bin
    return min_val + bin_width * start_bin, min_val + bin_width * (end_bin + 1)


def static_hist_ranges(act_tensors, bit, bins=2048):
    """get_static_hist_range, quant.py:461-521 (per_tensor, symmetric - what get_batch_tensors_qparams asserts)."""
    mins, maxs = [], []
    for tensors in _batch_lists(act_tensors):
        hist = min_val = max_val = None
        for t in tensors:
            x_min, x_max = torch.min(t).float(), torch.max(t).float()
            if hist is None:
                hist = histc_device(t, bins, x_min.item(), x_max.item())
                min_val, max_val = x_min, x_max
                continue
            new_min, new_max = torch.min(min_val, x_min), torch.max(max_val, x_max)
            upd = histc_device(t, bins, new_min.item(), new_max.item())
            if new_min == min_val and new_max == max_val:
                hist = hist + upd
            else:
                hist = hist_combine(hist, min_val, max_val, upd, new_min, new_max, bins)
            min_val, max_val = new_min, new_max
        lo, hi = hist_threshold(hist, min_val, max_val, bins, 2 ** bit)
        mins.append(lo)
        maxs.append(hi)
    return mins, maxs


# ----------------------------------------------------------------------------
# Weight48IntegerQuantizer   (quant.py:1230-1367)
# ----------------------------------------------------------------------------
def w48_fake_quant(w: torch.Tensor, bit4: dict, bit8: dict) -> torch.Tensor:
    """fake_quant_weight_dynamic, quant.py:1338-1367: 16 -> 8 -> 4 -> 8 -> 16 bit.  Settings: symmetric,
    granularity ('per_group' + group_size, else rows as they are), int_range, scales_bit + scales_symmetric."""
    def bounds(cfg, bit):
        if 'int_range' in cfg:
            return torch.tensor(cfg['int_range'][0]), torch.tensor(cfg['int_range'][1])
        if cfg['symmetric']:
            return torch.tensor(-(2 ** (bit - 1))), torch.tensor(2 ** (bit - 1) - 1)
        return torch.tensor(0), torch.tensor(2 ** bit - 1)

    def rows_of(t, cfg):
        return t.reshape(-1, cfg['group_size']) if cfg.get('granularity') == 'per_group' else t

    def qparams(t, cfg, bit):
        qmin, qmax = bounds(cfg, bit)
        lo, hi = t.amin(dim=-1, keepdim=True), t.amax(dim=-1, keepdim=True)
        if cfg['symmetric']:
            scales = torch.max(hi.abs(), lo.abs()).clamp(min=1e-5) / qmax
            zeros = torch.tensor(0.0)
        else:
            scales = (hi - lo).clamp(min=1e-5) / (qmax - qmin)
            zeros = qmin - torch.round(lo / scales)
        if 'scales_bit' in cfg:
            n = cfg['scales_bit']
            s_lo, s_hi = (-(2 ** (n - 1)), 2 ** (n - 1) - 1) if cfg['scales_symmetric'] else (0, 2 ** n - 1)
            scales = scales.clamp(s_lo, s_hi)
        zeros = zeros.clamp(qmin, qmax)
        return scales, zeros, qmax, qmin

    shape16, dtype16 = w.shape, w.dtype
    t = rows_of(w, bit8)
    s8, z8, qmax8, qmin8 = qparams(t, bit8, 8)
    t = torch.clamp(torch.round(t / s8) + z8, qmin8, qmax8)
    shape8, dtype8 = t.shape, t.dtype
    t = rows_of(t, bit4)
    s4, z4, qmax4, qmin4 = qparams(t, bit4, 4)
    t = torch.clamp(torch.round(t / s4) + z4, qmin4, qmax4)
    t = ((t - z4) * s4).reshape(shape8).to(dtype8)
    t = ((t - z8) * s8).reshape(shape16).to(dtype16)
    return t
