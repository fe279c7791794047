"""Block-wise float8 casts with the reference's function names, running on liblcq.

Mirrors ``llmc/compression/quantization/kernel.py`` of ModelTC/LightCompress (Triton kernels used when the
checkpoint itself is block-wise FP8, e.g. DeepSeek-V3): ``act_quant`` (:29-54), ``weight_cast_to_fp8`` (:57-85) and
``weight_cast_to_bf16`` (:88-138).  One fp32 scale per 128-element activation block / 128x128 weight block,
``s = max|x| / 448``, ``y = (x / s).to(float8_e4m3fn)`` in fp32 arithmetic.
"""
from __future__ import annotations

import torch

from . import _lib as L

FLAG_CLAMP_RANGE, FLAG_TIE_AWAY = 1024, 2048


def _pad_cols(x, mult=8):
    """x with its last dimension zero-padded to a multiple of `mult` (the kernels take whole 16-byte pieces of a row;
    zeros change no block maximum and a pad of fewer than 8 columns never opens another 128-column block)."""
    N = x.shape[-1]
    if N % mult == 0:
        return x
    out = torch.zeros((*x.shape[:-1], (N + mult - 1) // mult * mult), dtype=x.dtype, device=x.device)
    out[..., :N] = x
    return out


def _block_quant(x, block_rows, flags):
    if x.dtype == torch.float16:                            # the casts compute in fp32 (kernel.py:43, 74): an exact widening
        return _block_quant(x.float(), block_rows, flags)
    if x.shape[-1] % 8 and block_rows != 1:
        y, s = _block_quant(_pad_cols(x), block_rows, flags)
        return y[..., :x.shape[-1]].contiguous(), s
    M, N = x.numel() // x.shape[-1], x.shape[-1]
    y = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device)
    if block_rows == 1:
        s = torch.empty((*x.shape[:-1], N // 128), dtype=torch.float32, device=x.device)
    else:
        s = torch.empty(((M + 127) // 128, (N + 127) // 128), dtype=torch.float32, device=x.device)
    L.check(L.lib().lcq_fp8_block_quant(L.ptr(x), L.i32(L.dtype_code(x.dtype)), L.i64(M), L.i64(N), L.i32(block_rows),
                                        L.i32(flags), L.ptr(y), L.ptr(s), L.stream()), 'lcq_fp8_block_quant')
    return y, s


def act_quant(x, block_size=128):
    """-> (float8_e4m3fn tensor like x, fp32 scales [..., last_dim / block_size])."""
    assert x.is_contiguous(), 'Input tensor must be contiguous'
    assert x.size(-1) % block_size == 0, \
        f'Last dimension size must be divisible by block_size (block_size={block_size})'
    if block_size != 128:
        raise NotImplementedError('block_size 128 only')
    return _block_quant(x, 1, 0)


def weight_cast_to_fp8(x, block_size=128):
    """-> (float8_e4m3fn [M, N], fp32 scales [ceil(M/128), ceil(N/128)])."""
    assert x.is_contiguous()
    assert x.dim() == 2
    if block_size != 128:
        raise NotImplementedError('block_size 128 only')
    return _block_quant(x, 128, 0)


def weight_cast_to_bf16(x, s, block_size=128):
    """-> x * s per block, in torch's default dtype (as the reference's `torch.empty_like(x, dtype=torch.get_default_dtype())`)."""
    assert x.is_contiguous() and s.is_contiguous(), 'Input tensors must be contiguous'
    assert x.dim() == 2 and s.dim() == 2, 'Input tensors must have 2 dimensions'
    if block_size != 128:
        raise NotImplementedError('block_size 128 only')
    return _block_dequant(x, s, torch.get_default_dtype())


def _block_dequant(x, s, out_dtype):
    M, N = x.shape
    if out_dtype == torch.float16:                          # float(y) * s in fp32, then the cast of the store (kernel.py:106)
        return _block_dequant(x, s, torch.float32).to(torch.float16)
    if out_dtype not in (torch.float32, torch.bfloat16):
        raise NotImplementedError(f'output dtype {out_dtype}')
    if N % 8:
        xp = _pad_cols(x.view(torch.uint8)).view(torch.float8_e4m3fn)
        return _block_dequant(xp, s, out_dtype)[:, :N].contiguous()
    out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    sf = s.to(torch.float32).contiguous()
    L.check(L.lib().lcq_fp8_block_dequant(L.ptr(x), L.ptr(sf), L.i64(M), L.i64(N), L.ptr(out), L.i32(L.dtype_code(out_dtype)),
                                          L.stream()), 'lcq_fp8_block_dequant')
    return out
