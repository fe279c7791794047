"""Oracle: int4/int8 packing (test infrastructure only).

Restates VllmRealQuantLinear.pack (module_utils.py:929-955) and
AutoawqRealQuantLinear.gemm_pack (module_utils.py:1097-1158) with numpy /
CPU torch, vectorised instead of the reference's per-column Python loops.
"""
from __future__ import annotations

import math

import numpy as np
import torch

AWQ_ORDER = (0, 2, 4, 6, 1, 3, 5, 7)


def pack_ct(codes: torch.Tensor, scales: torch.Tensor, num_bits: int):
    """compressed-tensors layout: nibble i of word j = uint8(code + 2^(b-1)) at column pf*j+i."""
    offset = pow(2, num_bits) // 2
    u = (codes + offset).to(torch.uint8).numpy().astype(np.uint32)
    pf = 32 // num_bits
    words = math.ceil(u.shape[1] / pf)
    u = np.pad(u, [(0, 0), (0, words * pf - u.shape[1])], constant_values=0)
    packed = np.zeros((u.shape[0], words), dtype=np.uint32)
    for i in range(pf):
        packed |= u[:, i::pf] << np.uint32(num_bits * i)
    return torch.from_numpy(np.ascontiguousarray(packed).view(np.int32)), scales.to(torch.float16)


def unpack_ct(packed: torch.Tensor, num_bits: int, cols: int) -> torch.Tensor:
    """Inverse of pack_ct for in-range codes (independent check)."""
    pf = 32 // num_bits
    w = packed.numpy().view(np.uint32)
    out = np.zeros((w.shape[0], w.shape[1] * pf), dtype=np.int32)
    for i in range(pf):
        out[:, i::pf] = (w >> np.uint32(num_bits * i)) & np.uint32((1 << num_bits) - 1)
    return torch.from_numpy(out[:, :cols] - (1 << (num_bits - 1)))


def gemm_pack(weight: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor, group_size: int, bit: int = 4):
    """AutoAWQ layout.  weight [R,K]; scales/zeros [R, K/g] as real_quant returns them."""
    assert bit == 4
    s = scales.t().contiguous().to(torch.float16)           # [K/g, R]
    z = zeros.t().contiguous()
    sz = z * s                                              # fp16
    gi = torch.arange(weight.shape[1]) // group_size
    # (w[:, k] + sz[g(k)]) / s[g(k)] column by column == broadcast over the [R, K] matrix
    iw = torch.round((weight + sz[gi].t()) / s[gi].t()).to(torch.int)
    iw = iw.t().contiguous().to(torch.int32)                # [K, R]
    pack_num = 32 // bit
    qweight = torch.zeros((iw.shape[0], iw.shape[1] // 32 * bit), dtype=torch.int32)
    for i in range(pack_num):
        qweight |= iw[:, AWQ_ORDER[i]::pack_num] << (i * bit)
    z32 = z.to(torch.int32)
    qzeros = torch.zeros((z32.shape[0], z32.shape[1] // 32 * bit), dtype=torch.int32)
    for i in range(pack_num):
        qzeros |= z32[:, AWQ_ORDER[i]::pack_num] << (i * bit)
    return qweight, s, qzeros


def gemm_unpack(qweight: torch.Tensor, bit: int = 4) -> torch.Tensor:
    """qweight [K, R/8] -> iw [K, R] for in-range nibbles (independent check)."""
    w = qweight.numpy().view(np.uint32)
    out = np.zeros((w.shape[0], w.shape[1] * 8), dtype=np.int32)
    for i in range(8):
        out[:, AWQ_ORDER[i]::8] = (w >> np.uint32(4 * i)) & np.uint32(15)
    return torch.from_numpy(out)
