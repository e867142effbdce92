"""The tiled format's definition (pack.tile_layout), pinned on the CPU: decoding every lane of every block by
plain bit extraction, with the register unpack's slot table, must give back the codes of the layer in the
order xsrc states; xsrc must be the stable sort of the channels by group; sz must hold the scales and the
zero points (+1) the oracle unpacks."""
import numpy as np
import pytest
import torch

from autogptq.tvm_amd import _slots, pack
from oracle import gptq_oracle as orc


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("K,N,gs,act", [(64, 32, 32, False), (192, 64, 64, True), (1056, 96, 32, True),
                                        (2048, 64, 128, True), (96, 32, -1, True), (160, 32, 32, False)])
def test_tile_layout_decodes_to_the_layer(bits, K, N, gs, act):
    L = pack.synth_layer(5 + K, K, N, bits, gs, act)
    qtile, sz, xsrc, kinv = pack.tile_layout(L["qweight"], L["qzeros"], L["scales"], L["g_idx"] if act else None, bits, gs)
    Kp = (K + 63) // 64 * 64
    S, T = Kp // 64, N // 32
    assert qtile.numel() == T * S * 64 * bits and tuple(xsrc.shape) == (Kp,)
    if bits == 8:   # the block is two halves of 64 lanes x 4 words
        qt = qtile.numpy().view(np.uint32).reshape(T, S, 2, 64, 4).transpose(0, 1, 3, 2, 4).reshape(T, S, 64, 8)
    else:
        qt = qtile.numpy().view(np.uint32).reshape(T, S, 64, bits)
    qt = np.concatenate([qt, np.zeros_like(qt[..., :1])], axis=-1).astype(np.uint64)   # (a zero word past the end)
    codes = orc.unpack_qweight_ref(L["qweight"], bits).numpy()      # the oracle's unpack, [K, N]
    assert np.array_equal(codes, L["codes"].numpy())
    field_of = _slots.lane_field_of_position(bits)
    assert sorted(field_of) == list(range(32))
    x = xsrc.numpy()
    for s in range(32):
        bit = bits * field_of[s]
        wd, sh = bit // 32, bit % 32
        two = qt[..., wd] | (qt[..., wd + 1] << np.uint64(32))       # the field may straddle two words (3 bits)
        q = (two >> np.uint64(sh)) & np.uint64((1 << bits) - 1)
        for h in range(2):
            pos = 64 * np.arange(S) + 32 * h + s                     # [S]
            src = x[pos]
            want = np.where(src[None, :, None] >= 0, codes[np.maximum(src, 0)].reshape(S, T, 32).transpose(1, 0, 2), 0)
            got = q[:, :, 32 * h: 32 * h + 32]                        # [T, S, n]
            assert np.array_equal(got, want), (s, h)
    g = L["g_idx"].numpy().astype(np.int64)
    perm = np.argsort(g, kind="stable") if act else np.arange(K)
    assert np.array_equal(x[:K], perm) and (x[K:] == -1).all()
    assert np.array_equal(kinv.numpy().view(np.uint16).astype(np.int64)[perm], np.arange(K))   # the inverse map
    szn = sz.numpy().view(np.uint32)
    assert np.array_equal((szn & 0xFFFF).astype(np.uint16).view(np.float16), L["scales"].numpy())
    zeros = orc.unpack_qzeros_ref(L["qzeros"], bits, N).numpy()       # already +1
    assert np.array_equal((szn >> 16).astype(np.uint16).view(np.float16).astype(np.int64), zeros)


def test_tile_layout_refuses_what_the_format_does_not_cover():
    L = pack.synth_layer(9, 96, 32, 4, 16, False)      # groups narrower than a 32-channel lane block
    assert pack.tile_layout(L["qweight"], L["qzeros"], L["scales"], None, 4, 16) is None
    L = pack.synth_layer(9, 128, 32, 4, 64, True)
    bad = L["g_idx"].clone()
    bad[:] = 0                                          # not an activation order of equal groups
    assert pack.tile_layout(L["qweight"], L["qzeros"], L["scales"], bad, 4, 64) is None


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("K,N,gs,act", [(64, 32, 32, False), (192, 96, 64, True), (1056, 96, 32, True),
                                        (256, 416, 128, True), (96, 160, -1, False)])
def test_transposed_layout_decodes_to_the_layer(bits, K, N, gs, act):
    """The copy of the transposed product (pack.tile_layout_transposed): lane (p, h) of block (T, S) holds the codes
    of sorted position 32 T + p at columns 64 S + 32 h .. + 31 (zeros past N); the table holds, per group and octet
    of columns, the scales and (base + zero) of the register unpack as fp16 pairs."""
    L = pack.synth_layer(7 + K, K, N, bits, gs, act)
    g_idx = L["g_idx"] if act else None
    qtile_t, szt = pack.tile_layout_transposed(L["qweight"], L["qzeros"], L["scales"], g_idx, bits, gs)
    Np = (N + 63) // 64 * 64
    S, T = Np // 64, K // 32
    assert qtile_t.numel() == T * S * 64 * bits
    if bits == 8:
        qt = qtile_t.numpy().view(np.uint32).reshape(T, S, 2, 64, 4).transpose(0, 1, 3, 2, 4).reshape(T, S, 64, 8)
    else:
        qt = qtile_t.numpy().view(np.uint32).reshape(T, S, 64, bits)
    qt = np.concatenate([qt, np.zeros_like(qt[..., :1])], axis=-1).astype(np.uint64)
    codes = orc.unpack_qweight_ref(L["qweight"], bits).numpy()      # [K, N]
    g = L["g_idx"].numpy().astype(np.int64)
    perm = np.argsort(g, kind="stable") if act else np.arange(K)
    sorted_codes = np.zeros((K, Np), dtype=np.int64)
    sorted_codes[:, :N] = codes[perm]
    field_of = _slots.lane_field_of_position(bits)
    for s in range(32):
        bit = bits * field_of[s]
        wd, sh = bit // 32, bit % 32
        two = qt[..., wd] | (qt[..., wd + 1] << np.uint64(32))
        q = (two >> np.uint64(sh)) & np.uint64((1 << bits) - 1)      # [T, S, lane]
        for h in range(2):
            cols = 64 * np.arange(S) + 32 * h + s                    # [S]
            want = sorted_codes[:, cols].reshape(T, 32, S).transpose(0, 2, 1)   # [T, S, p]
            assert np.array_equal(q[:, :, 32 * h: 32 * h + 32], want), (s, h)
    # the table
    G = L["scales"].shape[0]
    assert tuple(szt.shape) == (G, Np // 8, 8)
    t = szt.numpy().view(np.uint32)
    lo = (t & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float32)
    hi = (t >> 16).astype(np.uint16).view(np.float16).astype(np.float32)
    pairs = np.stack([lo, hi], axis=-1)                               # [G, Np/8, 8, 2]
    s_got = pairs[:, :, :4, :].reshape(G, Np)
    z_got = pairs[:, :, 4:, :].reshape(G, Np)
    zeros = orc.unpack_qzeros_ref(L["qzeros"], bits, N).numpy().astype(np.float32)   # already +1
    base = np.tile(np.array(_slots.BASE_OF_POSITION[bits], dtype=np.float32), N // 8)
    assert np.array_equal(s_got[:, :N], L["scales"].numpy().astype(np.float32))
    assert np.array_equal(z_got[:, :N], zeros + base[None, :])
    assert (s_got[:, N:] == 0).all() and (z_got[:, N:] == 0).all()
