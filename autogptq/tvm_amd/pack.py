"""Vectorised packers for the AutoGPTQ int3/int4 tensor format, and seeded synthetic layers.

Format (reference: auto_gptq/nn_modules/qlinear.py:105-175): along the packed axis, every
``bits`` consecutive int32 words are one little-endian bit stream of 32 codes, code ``j`` at
bit ``bits*j``.  ``qweight`` packs the codes along K, ``qzeros`` packs ``zero - 1`` along N.
"""
from __future__ import annotations

import math

import numpy as np
import torch


def pack_along_axis0(codes: np.ndarray, bits: int) -> np.ndarray:
    """codes [R, C] with values in [0, 2**bits) -> int32 [R//32*bits, C]; R must divide by 32."""
    codes = np.ascontiguousarray(codes)
    rows, cols = codes.shape
    if rows % 32 != 0:
        raise ValueError(f"packed axis length {rows} is not a multiple of 32")
    if bits not in (2, 3, 4, 8):
        raise NotImplementedError("Only 2, 3, 4 and 8 bits are supported.")
    blocks = codes.reshape(rows // 32, 32, cols).astype(np.uint64)
    if bits != 3:
        # widths that divide a word: 32 codes -> `bits` words of 32 / bits codes each
        per = 32 // bits
        b = blocks.reshape(rows // 32, bits, per, cols)
        shifts = (bits * np.arange(per, dtype=np.uint64)).reshape(1, 1, per, 1)
        words = np.bitwise_or.reduce(b << shifts, axis=2)
        return words.reshape(rows // per, cols).astype(np.uint32).view(np.int32)
    # 3 bits: a 96-bit stream; build it in two 64-bit halves that overlap nowhere
    out = np.zeros((rows // 32, 3, cols), dtype=np.uint64)
    for j in range(32):
        bit = 3 * j
        w, sh = divmod(bit, 32)
        v = blocks[:, j, :] << np.uint64(sh)
        out[:, w, :] |= v & np.uint64(0xFFFFFFFF)
        if sh + 3 > 32:
            out[:, w + 1, :] |= v >> np.uint64(32)
    return out.reshape(rows // 32 * 3, cols).astype(np.uint32).view(np.int32)


def pack_qweight(codes: np.ndarray, bits: int) -> np.ndarray:
    """codes [K, N] -> qweight int32 [K//32*bits, N]."""
    return pack_along_axis0(codes, bits)


def pack_qzeros(zeros: np.ndarray, bits: int) -> np.ndarray:
    """zero points [G, N] in [1, 2**bits] -> qzeros int32 [G, N//32*bits] (stores zero - 1)."""
    z = np.asarray(zeros).astype(np.int64) - 1
    if z.min() < 0 or z.max() >= (1 << bits):
        raise ValueError("zero points must lie in [1, 2**bits]")
    return np.ascontiguousarray(pack_along_axis0(np.ascontiguousarray(z.T), bits).T)


def unpack_along_axis0(words: np.ndarray, bits: int) -> np.ndarray:
    """Inverse of pack_along_axis0: int32 [R//32*bits, C] -> codes uint8 [R, C]."""
    if bits not in (2, 3, 4, 8):
        raise NotImplementedError("Only 2, 3, 4 and 8 bits are supported.")
    w = np.ascontiguousarray(words).view(np.uint32)
    rows, cols = w.shape
    if rows % bits != 0:
        raise ValueError(f"{rows} packed rows are not a multiple of bits={bits}")
    if bits != 3:
        per = 32 // bits
        shifts = (bits * np.arange(per, dtype=np.uint32)).reshape(1, per, 1)
        mask = np.uint32((1 << bits) - 1)
        return ((w[:, None, :] >> shifts) & mask).astype(np.uint8).reshape(rows * per, cols)
    b = w.reshape(rows // 3, 3, cols).astype(np.uint64)
    lo = b[:, 0, :] | (b[:, 1, :] << np.uint64(32))       # stream bits 0..63
    hi = (b[:, 1, :] >> np.uint64(31)) | (b[:, 2, :] << np.uint64(1))  # stream bits 63..95 at bit 0
    out = np.empty((rows // 3, 32, cols), dtype=np.uint8)
    for j in range(32):
        bit = 3 * j
        if bit + 3 <= 64:
            out[:, j, :] = ((lo >> np.uint64(bit)) & np.uint64(7)).astype(np.uint8)
        else:
            out[:, j, :] = ((hi >> np.uint64(bit - 63)) & np.uint64(7)).astype(np.uint8)
    return out.reshape(rows // 3 * 32, cols)


def unpack_rows_torch(words: torch.Tensor, bits: int) -> torch.Tensor:
    """``unpack_along_axis0`` with torch ops, on whatever device ``words`` is: int32
    [R//32*bits, C] -> codes int64 [R, C]."""
    rows, cols = words.shape
    w = words.to(torch.int64) & 0xFFFFFFFF
    if bits != 3:
        per = 32 // bits
        shifts = (bits * torch.arange(per, device=words.device)).view(1, per, 1)
        return ((w.unsqueeze(1) >> shifts) & ((1 << bits) - 1)).reshape(rows * per, cols)
    b = w.view(rows // 3, 3, cols)
    out = torch.empty((rows // 3, 32, cols), dtype=torch.int64, device=words.device)
    for j in range(32):
        wi, sh = divmod(3 * j, 32)
        v = b[:, wi, :] >> sh
        if sh > 29:  # the code continues in the next word
            v = v | (b[:, wi + 1, :] << (32 - sh))
        out[:, j, :] = v & 7
    return out.reshape(rows // 3 * 32, cols)


def pack_rows_torch(codes: torch.Tensor, bits: int) -> torch.Tensor:
    """``pack_along_axis0`` with torch ops: codes [R, C] (any integer dtype, values < 2**bits) ->
    int32 [R//32*bits, C]."""
    R, cols = codes.shape
    c = codes.to(torch.int64).view(R // 32, 32, cols)
    words = torch.zeros((R // 32, bits, cols), dtype=torch.int64, device=codes.device)
    for j in range(32):
        wi, sh = divmod(bits * j, 32)
        words[:, wi, :] |= (c[:, j, :] << sh) & 0xFFFFFFFF
        if sh + bits > 32:
            words[:, wi + 1, :] |= c[:, j, :] >> (32 - sh)
    words = torch.where(words >= (1 << 31), words - (1 << 32), words)
    return words.to(torch.int32).view(R // 32 * bits, cols)


def sort_channels_by_group(qweight: torch.Tensor, g_idx: torch.Tensor, bits: int, group_size: int):
    """Load-time preparation for activation-order checkpoints: reorders the input channels so that
    every group is contiguous, which lets the decode kernel treat the layer like one without
    ``g_idx``.  Returns ``(qweight_sorted int32 [K//32*bits, N], kmap int32 [2K])`` on the device of
    ``qweight``, or ``None`` when the layer does not qualify.

    Sorted position j holds original channel perm[j] (stable sort by group).  ``kmap[k]`` tells the
    kernel where original channel k goes: low 16 bits = its position inside the sorted K range with
    the codes of each lane block (8 channels for int4, 32 for int3) already in the order the
    kernels' register unpack produces them, high 16 bits = its group.  ``kmap[K + j]`` is
    perm[j], the original channel whose codes are j-th along K in ``qweight_sorted``.  Requires K < 65536, every
    group to hold exactly ``group_size`` channels, and ``group_size`` to be a multiple of the lane
    block."""
    from . import _slots

    K = int(g_idx.numel())
    gs = K if group_size == -1 else group_size
    klane = 8 if bits == 4 else 32
    if K >= 65536 or gs % klane != 0 or K % 32 != 0 or K % gs != 0:
        return None
    dev = qweight.device
    g = g_idx.detach().to(device=dev, dtype=torch.int64)
    perm = torch.argsort(g, stable=True)
    ar = torch.arange(K, dtype=torch.int64, device=dev)
    if not torch.equal(g[perm], ar // gs):
        return None
    qweight_sorted = pack_rows_torch(unpack_rows_torch(qweight.detach(), bits)[perm], bits)
    inv = torch.empty(K, dtype=torch.int64, device=dev)
    inv[perm] = ar                                          # original k -> sorted position
    slot_of_code = torch.tensor(_slots.slot_of_code(bits), dtype=torch.int64, device=dev)
    pos = (inv // klane) * klane + slot_of_code[inv % klane]
    kmap = torch.cat([pos | ((inv // gs) << 16), perm]).to(torch.int32)
    return qweight_sorted.contiguous(), kmap.contiguous()


TILE_COLS = 32     # columns of one tile of the tiled format: the N extent of one 32x32x16 matrix instruction
TILE_CHANNELS = 64  # input channels of one block of the tiled format: two lane halves x 32 codes


def tiled_qualifies(K: int, N: int, bits: int, group_size: int) -> bool:
    """Layers the tiled format covers: 3 or 4 bits, whole groups made of whole 32-channel lane blocks."""
    gs = K if group_size == -1 else group_size
    return bits in (2, 3, 4, 8) and K % 32 == 0 and N % 32 == 0 and gs % 32 == 0 and K % gs == 0 and K <= 65536


def tile_layout(qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor, g_idx, bits: int, group_size: int):
    """The load-time re-layout for the tiled kernels, in torch ops (the statement the library's own
    preparation, ``gptq_hip_tile_prepare``, is tested against; the reference's TVM module re-lays its
    weights once in the same spirit, auto_gptq/nn_modules/qlinear_tvm.py:25-40,105-107).

    Returns ``(qtile int32 [N/32 * Kp/64 * 64 * bits], sz int32 [G, N], xsrc int32 [Kp], kinv int16 [K])``
    with Kp = K rounded up to 64, or None when the layer does not qualify (K must not exceed 65536: ``kinv``
    holds the position of every channel, the inverse of ``xsrc``, as an unsigned 16-bit value).

    * The input channels are sorted by group (stable; the identity for contiguous groups); position p of
      the sorted order holds channel ``xsrc[p]`` (-1 for the padding positions p >= K, whose codes are 0).
    * ``qtile`` is a sequence of blocks, column tile T (32 columns) outermost, then block S (64 positions):
      block (T, S) is 64 lanes x ``bits`` words; lane (n = lane % 32, h = lane // 32) holds the 32 codes of
      column 32 T + n at positions 64 S + 32 h .. + 31 as the usual little-endian stream of ``bits``-bit
      fields, with the codes permuted inside the lane (each 4 / 8 / 16 positions for 8 / 4 / 2 bits, all 32
      for 3 bits) so that the kernels' register unpack yields them in position order: stream field
      ``_slots.lane_field_of_position(bits)[s]`` holds position s.  Word i of lane l sits at l * bits + i of the block,
      except for 8 bits, whose block is two halves of 64 lanes x 4 words: (i // 4) * 256 + l * 4 + i % 4.
    * ``sz[g, n]`` = fp16 bits of ``scales[g, n]`` | fp16 bits of the zero point (stored value + 1) << 16.
    """
    rows, N = qweight.shape
    K = rows * 32 // bits
    if not tiled_qualifies(K, N, bits, group_size):
        return None
    gs = K if group_size == -1 else group_size
    dev = qweight.device
    ar = torch.arange(K, dtype=torch.int64, device=dev)
    if g_idx is None:
        perm = ar
    else:
        g = g_idx.detach().to(device=dev, dtype=torch.int64)
        perm = torch.argsort(g, stable=True)
        if not torch.equal(g[perm], ar // gs):
            return None
    Kp = (K + TILE_CHANNELS - 1) // TILE_CHANNELS * TILE_CHANNELS
    codes = unpack_rows_torch(qweight.detach(), bits)[perm]                      # [K, N], sorted order
    qtile = _tile_words(codes, bits)
    zeros = unpack_rows_torch(qzeros.detach().t().contiguous(), bits).t() + 1     # [G, N]
    zbits = zeros.to(torch.float16).view(torch.int16).to(torch.int64) & 0xFFFF
    sbits = scales.detach().contiguous().view(torch.int16).to(torch.int64) & 0xFFFF
    both = sbits | (zbits << 16)
    sz = torch.where(both >= (1 << 31), both - (1 << 32), both).to(torch.int32).contiguous()
    xsrc = torch.full((Kp,), -1, dtype=torch.int32, device=dev)
    xsrc[:K] = perm.to(torch.int32)
    inv = torch.empty(K, dtype=torch.int64, device=dev)
    inv[perm] = ar
    kinv = torch.where(inv >= (1 << 15), inv - (1 << 16), inv).to(torch.int16)   # unsigned 16-bit positions
    return qtile, sz, xsrc, kinv


def _tile_words(codes: torch.Tensor, bits: int) -> torch.Tensor:
    """The blocks of the tiled format for a code matrix [positions, columns] (columns a multiple of 32; the
    positions are padded with zero codes to a multiple of 64): int32, 1-D."""
    from . import _slots

    P, C = codes.shape
    dev = codes.device
    Pp = (P + TILE_CHANNELS - 1) // TILE_CHANNELS * TILE_CHANNELS
    S, T = Pp // TILE_CHANNELS, C // TILE_COLS
    if Pp > P:
        codes = torch.cat([codes, torch.zeros((Pp - P, C), dtype=codes.dtype, device=dev)])
    # stream field f of a lane holds the position order[f]
    field_of = _slots.lane_field_of_position(bits)
    order = torch.empty(32, dtype=torch.int64, device=dev)
    order[torch.tensor(field_of, dtype=torch.int64, device=dev)] = torch.arange(32, device=dev)
    blocks = codes.reshape(S * 2, 32, C)[:, order, :]                             # [(S, h), field, C]
    words = pack_rows_torch(blocks.reshape(S * 2 * 32, C), bits)                  # [(S, h, word), C]
    words = words.view(S, 2, bits, T, TILE_COLS)
    if bits == 8:   # [T, S, word // 4, (h, n), word % 4]
        return words.view(S, 2, 2, 4, T, TILE_COLS).permute(4, 0, 2, 1, 5, 3).contiguous().view(-1)
    return words.permute(3, 0, 1, 4, 2).contiguous().view(-1)                     # [T, S, (h, n), word]


def tile_layout_transposed(qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor, g_idx, bits: int,
                           group_size: int):
    """The second prepared copy, for the transposed product gx = gy @ W^T (the gradient with respect to x; the
    reference's Triton back end, auto_gptq/nn_modules/qlinear_triton.py:195-273,298-317), in torch ops: the
    statement ``gptq_hip_tile_prepare_transposed`` is tested against.

    Returns ``(qtile_t int32 [K/32 * Np/64 * 64 * bits], szt int32 [G, Np/8, 8])`` with Np = N rounded up to 64,
    or None when the tiled format does not cover the layer.

    * ``qtile_t`` is the tiled format of the TRANSPOSED code matrix: its positions are the layer's columns n (padded
      with zero codes to Np), its columns are the layer's sorted positions p; block (T, S) holds, in lane
      (lane % 32, h), the codes of position 32 T + lane % 32 at columns 64 S + 32 h .. + 31.
    * ``szt[g, o]``, for the octet of columns 8 o .. 8 o + 7: words r = 0..3 are the fp16 pairs
      (scale[g, 8 o + 2 r], scale[g, 8 o + 2 r + 1]), words 4 + r the pairs (base + zero) of the same columns, with
      the bases of the register unpack (``_slots.BASE_OF_POSITION``); zeros for columns past N.
    """
    from . import _slots

    rows, N = qweight.shape
    K = rows * 32 // bits
    if not tiled_qualifies(K, N, bits, group_size):
        return None
    gs = K if group_size == -1 else group_size
    dev = qweight.device
    ar = torch.arange(K, dtype=torch.int64, device=dev)
    if g_idx is None:
        perm = ar
    else:
        g = g_idx.detach().to(device=dev, dtype=torch.int64)
        perm = torch.argsort(g, stable=True)
        if not torch.equal(g[perm], ar // gs):
            return None
    codes = unpack_rows_torch(qweight.detach(), bits)[perm]                      # [K, N], sorted order
    qtile_t = _tile_words(codes.t().contiguous(), bits)
    G = K // gs
    Np = (N + 63) // 64 * 64
    zeros = (unpack_rows_torch(qzeros.detach().t().contiguous(), bits).t() + 1).to(torch.float32)   # [G, N]
    base = torch.tensor(_slots.BASE_OF_POSITION[bits], dtype=torch.float32, device=dev).repeat(N // 8)
    zb = (zeros + base[None, :]).to(torch.float16)                               # exact: small integers
    s = scales.detach().contiguous()

    def pairs(v):   # fp16 [G, N] -> int64 [G, Np/8, 4]: (v[2 i], v[2 i + 1]) as one word
        bits16 = v.view(torch.int16).to(torch.int64) & 0xFFFF
        if Np > N:
            bits16 = torch.cat([bits16, torch.zeros((G, Np - N), dtype=torch.int64, device=dev)], dim=1)
        b = bits16.view(G, Np // 8, 4, 2)
        return b[..., 0] | (b[..., 1] << 16)

    both = torch.cat([pairs(s), pairs(zb)], dim=2)                               # [G, Np/8, 8]
    szt = torch.where(both >= (1 << 31), both - (1 << 32), both).to(torch.int32).contiguous()
    return qtile_t, szt


def num_groups(k: int, group_size: int) -> int:
    gs = k if group_size == -1 else group_size
    return math.ceil(k / gs)


def make_g_idx(k: int, group_size: int, desc_act: bool, gen: torch.Generator) -> torch.Tensor:
    gs = k if group_size == -1 else group_size
    if desc_act:
        return (torch.randperm(k, generator=gen) // gs).to(torch.int32)
    return (torch.arange(k) // gs).to(torch.int32)


def synth_layer(seed: int, K: int, N: int, bits: int, group_size: int, desc_act: bool, M: int = 1,
                bias: bool = False) -> dict:
    """Seeded synthetic QuantLinear tensors (CPU): uniform codes and zero codes, scales in
    [1e-3, 1e-2], x ~ N(0, 1).  The dict also keeps the unpacked ``codes`` and ``zeros``."""
    gen = torch.Generator().manual_seed(seed)
    G = num_groups(K, group_size)
    codes = torch.randint(0, 1 << bits, (K, N), generator=gen, dtype=torch.int32)
    zeros = torch.randint(0, 1 << bits, (G, N), generator=gen, dtype=torch.int32) + 1
    scales = (torch.rand((G, N), generator=gen) * (1e-2 - 1e-3) + 1e-3).to(torch.float16)
    g_idx = make_g_idx(K, group_size, desc_act, gen)
    x = torch.randn((M, K), generator=gen).to(torch.float16)
    b = torch.randn((N,), generator=gen).to(torch.float16) if bias else None
    return {
        "bits": bits, "group_size": group_size, "K": K, "N": N, "G": G, "desc_act": desc_act,
        "codes": codes, "zeros": zeros,
        "qweight": torch.from_numpy(pack_qweight(codes.numpy(), bits)),
        "qzeros": torch.from_numpy(pack_qzeros(zeros.numpy(), bits)),
        "scales": scales, "g_idx": g_idx, "x": x, "bias": b,
    }
