"""CPU oracle for the GPTQ int3/int4 QuantLinear path.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU, what the reference computes on its torch
fallback path.  It is the checker that the HIP kernels are compared with; it is
never part of the product path.  Only tests, the smoke check and the
``cpu_baseline`` leg of the benchmark may import it.

Each function names the reference lines it follows (paths relative to the
reference checkout):

* ``pack_qweight_loop`` / ``pack_qzeros_loop``  auto_gptq/nn_modules/qlinear.py:105-139, :141-175
* ``unpack_qweight_ref`` / ``unpack_qzeros_ref`` auto_gptq/nn_modules/qlinear.py:62-70, :201-240
* ``dequant_ref``                               auto_gptq/nn_modules/qlinear.py:242
* ``forward_ref``                               auto_gptq/nn_modules/qlinear.py:177-247
* ``unpack_bitstream``                          closed form: code j of a 32-code block sits at
                                                bit ``bits*j`` of a little-endian stream of int32
                                                words (cross-check: auto_gptq/nn_modules/tvm_untils/
                                                workloads.py:298 states the same stream over bytes)

Pinning status.  The reference holds no golden vectors for this path (its
tests only print).  The functions here are pinned by tests/test_oracle.py:
unpack against the closed-form bit stream, against the loop packer (round
trip) and against the C restatement in oracle/gptq_oracle.c; the zero-point
``+1`` against hand-worked words; dequant against exact integer cases and an
fp32-product/RNE-to-fp16 restatement; forward against an fp64 matmul and
integer-exact column sums.  ``pack`` applied to real float weights
(rounding of ``(W + s*z)/s``) is covered by the fixture in tests/golden/ when
present, otherwise it is "parity unpinned".
"""
from __future__ import annotations

import math

import numpy as np
import torch

SUPPORTED_BITS = (3, 4)


# --------------------------------------------------------------------------
# Packing (defines the on-disk format).  Loop versions follow the reference
# statement by statement; they are slow and meant for small cases.
# --------------------------------------------------------------------------
def pack_qweight_loop(intweight: np.ndarray, bits: int) -> np.ndarray:
    """codes [K, N] (values < 2**bits) -> int32 [K//32*bits, N].  qlinear.py:105-139."""
    intweight = np.ascontiguousarray(intweight).astype(np.uint32)
    qweight = np.zeros((intweight.shape[0] // 32 * bits, intweight.shape[1]), dtype=np.uint32)
    i = 0
    row = 0
    while row < qweight.shape[0]:
        if bits in (2, 4, 8):
            for j in range(i, i + (32 // bits)):
                qweight[row] |= intweight[j] << np.uint32(bits * (j - i))
            i += 32 // bits
            row += 1
        elif bits == 3:
            for j in range(i, i + 10):
                qweight[row] |= intweight[j] << np.uint32(3 * (j - i))
            i += 10
            qweight[row] |= intweight[i] << np.uint32(30)
            row += 1
            qweight[row] |= (intweight[i] >> np.uint32(2)) & np.uint32(1)
            i += 1
            for j in range(i, i + 10):
                qweight[row] |= intweight[j] << np.uint32(3 * (j - i) + 1)
            i += 10
            qweight[row] |= intweight[i] << np.uint32(31)
            row += 1
            qweight[row] |= (intweight[i] >> np.uint32(1)) & np.uint32(3)
            i += 1
            for j in range(i, i + 10):
                qweight[row] |= intweight[j] << np.uint32(3 * (j - i) + 2)
            i += 10
            row += 1
        else:
            raise NotImplementedError("Only 2,3,4,8 bits are supported.")
    return qweight.view(np.int32)


def pack_qzeros_loop(zeros: np.ndarray, bits: int) -> np.ndarray:
    """zero points [G, N] (1..2**bits) -> int32 [G, N//32*bits]; stores ``z - 1``.

    qlinear.py:141-175 (the same bit layout as the weights, along N).
    """
    z = (np.ascontiguousarray(zeros).astype(np.int64) - 1).astype(np.uint32)
    return np.ascontiguousarray(pack_qweight_loop(np.ascontiguousarray(z.T), bits).T)


# --------------------------------------------------------------------------
# Closed-form statement of the layout, independent of the reference's tables.
# --------------------------------------------------------------------------
def unpack_bitstream(packed: np.ndarray, bits: int, axis: int = 0) -> np.ndarray:
    """Read ``bits``-wide codes from little-endian streams of int32 words along ``axis``."""
    p = np.moveaxis(np.ascontiguousarray(packed).view(np.uint32), axis, 0)
    nwords = p.shape[0]
    ncodes = nwords * 32 // bits
    out = np.empty((ncodes,) + p.shape[1:], dtype=np.int32)
    p64 = p.astype(np.uint64)
    mask = np.uint64((1 << bits) - 1)
    for j in range(ncodes):
        bit = bits * j
        w, sh = divmod(bit, 32)
        v = p64[w] >> np.uint64(sh)
        if sh + bits > 32:
            v = v | (p64[w + 1] << np.uint64(32 - sh))
        out[j] = (v & mask).astype(np.int32)
    return np.moveaxis(out, 0, axis)


# --------------------------------------------------------------------------
# The reference's torch fallback, same ops in the same order (prints removed).
# --------------------------------------------------------------------------
def _wf(bits: int) -> torch.Tensor:
    # qlinear.py:62-70
    if bits in (2, 4, 8):
        return torch.tensor(list(range(0, 32, bits)), dtype=torch.int32).unsqueeze(0)
    if bits == 3:
        return torch.tensor(
            [
                [0, 3, 6, 9, 12, 15, 18, 21, 24, 27, 30, 0],
                [0, 1, 4, 7, 10, 13, 16, 19, 22, 25, 28, 31],
                [0, 2, 5, 8, 11, 14, 17, 20, 23, 26, 29, 0],
            ],
            dtype=torch.int32,
        ).reshape(1, 3, 12)
    raise NotImplementedError("Only 2,3,4,8 bits are supported.")


def unpack_qzeros_ref(qzeros: torch.Tensor, bits: int, n: int) -> torch.Tensor:
    """int32 [G, N//32*bits] -> zero points [G, N] (already ``+1``).  qlinear.py:202-209, :217-227."""
    wf = _wf(bits)
    if bits in (2, 4, 8):
        zeros = torch.bitwise_right_shift(
            torch.unsqueeze(qzeros, 2).expand(-1, -1, 32 // bits), wf.unsqueeze(0)
        ).to(torch.int16 if bits == 8 else torch.int8)
        torch.bitwise_and(zeros, (2 ** bits) - 1, out=zeros)
        zeros = zeros + 1
        return zeros.reshape(qzeros.shape[0], n)
    zeros = qzeros.reshape(qzeros.shape[0], qzeros.shape[1] // 3, 3, 1).expand(-1, -1, -1, 12)
    zeros = zeros >> wf.unsqueeze(0)
    zeros[:, :, 0, 10] = (zeros[:, :, 0, 10] & 0x3) | ((zeros[:, :, 1, 0] << 2) & 0x4)
    zeros[:, :, 1, 11] = (zeros[:, :, 1, 11] & 0x1) | ((zeros[:, :, 2, 0] << 1) & 0x6)
    zeros = zeros & 0x7
    zeros = torch.cat([zeros[:, :, 0, :11], zeros[:, :, 1, 1:12], zeros[:, :, 2, 1:11]], dim=2)
    zeros = zeros + 1
    return zeros.reshape(qzeros.shape[0], n)


def unpack_qweight_ref(qweight: torch.Tensor, bits: int) -> torch.Tensor:
    """int32 [K//32*bits, N] -> codes [K, N].  qlinear.py:211-215, :229-240."""
    wf = _wf(bits)
    if bits in (2, 4, 8):
        weight = torch.bitwise_right_shift(
            torch.unsqueeze(qweight, 1).expand(-1, 32 // bits, -1), wf.unsqueeze(-1)
        ).to(torch.int16 if bits == 8 else torch.int8)
        torch.bitwise_and(weight, (2 ** bits) - 1, out=weight)
    else:
        weight = qweight.reshape(qweight.shape[0] // 3, 3, 1, qweight.shape[1]).expand(-1, -1, 12, -1)
        weight = (weight >> wf.unsqueeze(-1)) & 0x7
        weight[:, 0, 10] = (weight[:, 0, 10] & 0x3) | ((weight[:, 1, 0] << 2) & 0x4)
        weight[:, 1, 11] = (weight[:, 1, 11] & 0x1) | ((weight[:, 2, 0] << 1) & 0x6)
        weight = weight & 0x7
        weight = torch.cat([weight[:, 0, :11], weight[:, 1, 1:12], weight[:, 2, 1:11]], dim=1)
    return weight.reshape(weight.shape[0] * weight.shape[1], weight.shape[2])


def dequant_ref(qweight, qzeros, scales, g_idx, bits: int) -> torch.Tensor:
    """fp16 [K, N] = scales[g] * (q - zero[g]), one fp16 rounding per element.  qlinear.py:242."""
    n = qweight.shape[1]
    zeros = unpack_qzeros_ref(qzeros, bits, n)
    weight = unpack_qweight_ref(qweight, bits)
    g = g_idx.long()
    return scales[g] * (weight - zeros[g])


def forward_ref(x, qweight, qzeros, scales, g_idx, bias, bits: int) -> torch.Tensor:
    """QuantLinear.forward on the torch branch.  qlinear.py:177-247."""
    outfeatures = qweight.shape[1]
    out_shape = x.shape[:-1] + (outfeatures,)
    x = x.reshape(-1, x.shape[-1])
    weights = dequant_ref(qweight, qzeros, scales, g_idx, bits)
    out = torch.matmul(x.half(), weights)
    out = out.reshape(out_shape)
    out = out + bias if bias is not None else out
    return out


def matmul_only_ref(x, weights) -> torch.Tensor:
    """The S6 step alone on a pre-dequantised fp16 ``weights``.  qlinear.py:243."""
    return torch.matmul(x.reshape(-1, x.shape[-1]).half(), weights)


# --------------------------------------------------------------------------
# Independent restatements used to pin the functions above.
# --------------------------------------------------------------------------
def dequant_exact(qweight: np.ndarray, qzeros: np.ndarray, scales: np.ndarray, g_idx: np.ndarray,
                  bits: int) -> np.ndarray:
    """Closed-form dequant: bit-stream unpack, fp32 product (exact), one RNE to fp16."""
    q = unpack_bitstream(qweight, bits, axis=0)
    z = unpack_bitstream(qzeros, bits, axis=1) + 1
    g = np.asarray(g_idx).astype(np.int64)
    prod = scales.astype(np.float32)[g] * (q - z[g]).astype(np.float32)
    return prod.astype(np.float16)


def forward_f64(x: np.ndarray, w16: np.ndarray, bias=None) -> np.ndarray:
    """fp64 matmul of fp16 operands: the tight reference that outputs are compared with."""
    y = x.reshape(-1, x.shape[-1]).astype(np.float64) @ w16.astype(np.float64)
    if bias is not None:
        y = y + bias.astype(np.float64)
    return y


def n_groups(k: int, group_size: int) -> int:
    gs = group_size if group_size != -1 else k
    return math.ceil(k / gs)
