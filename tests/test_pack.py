"""The product's vectorised packers against the oracle's loop packers (which follow the
reference's pack statement by statement) and against the closed-form unpack."""
import numpy as np
import pytest
import torch

from autogptq.tvm_amd import pack
from oracle import gptq_oracle as orc


@pytest.mark.parametrize("bits", [3, 4])
def test_pack_qweight_equals_reference_loops(bits):
    rng = np.random.default_rng(bits)
    codes = rng.integers(0, 1 << bits, size=(160, 9))
    assert np.array_equal(pack.pack_qweight(codes, bits), orc.pack_qweight_loop(codes, bits))


@pytest.mark.parametrize("bits", [3, 4])
def test_pack_qzeros_equals_reference_loops(bits):
    rng = np.random.default_rng(bits + 10)
    zeros = rng.integers(1, (1 << bits) + 1, size=(4, 96))
    got = pack.pack_qzeros(zeros, bits)
    assert np.array_equal(got, orc.pack_qzeros_loop(zeros, bits))
    assert np.array_equal(orc.unpack_bitstream(got, bits, axis=1) + 1, zeros)


def test_pack_rejects_bad_input():
    with pytest.raises(ValueError):
        pack.pack_qweight(np.zeros((33, 4), dtype=np.int64), 4)
    with pytest.raises(NotImplementedError):
        pack.pack_qweight(np.zeros((32, 4), dtype=np.int64), 5)
    with pytest.raises(ValueError):
        pack.pack_qzeros(np.zeros((1, 32), dtype=np.int64), 4)  # zero point 0 is not storable


def test_synth_layer_shapes_and_determinism():
    a = pack.synth_layer(1234, 4096, 64, 3, 128, True, M=2)
    b = pack.synth_layer(1234, 4096, 64, 3, 128, True, M=2)
    assert a["qweight"].shape == (384, 64) and a["qweight"].dtype == torch.int32
    assert a["qzeros"].shape == (32, 6) and a["scales"].shape == (32, 64)
    assert a["g_idx"].shape == (4096,) and a["x"].shape == (2, 4096)
    assert torch.equal(a["qweight"], b["qweight"]) and torch.equal(a["g_idx"], b["g_idx"])
    assert sorted(a["g_idx"].tolist()) == sorted((torch.arange(4096) // 128).tolist())
    assert float(a["scales"].min()) >= 1e-3 * 0.999 and float(a["scales"].max()) <= 1e-2 * 1.001
    c = pack.synth_layer(5, 64, 32, 4, -1, False)
    assert c["G"] == 1 and c["qzeros"].shape == (1, 4) and int(c["g_idx"].max()) == 0


@pytest.mark.parametrize("bits", [3, 4])
def test_quantlinear_pack_round_trips_through_the_oracle(bits):
    """QuantLinear.pack (reference: qlinear.py:77-175) on weights that sit exactly on the
    quantisation grid: dequantising the packed tensors must give those weights back."""
    from autogptq.tvm_amd import QuantLinear

    K, N, gs = 64, 32, 32
    G = K // gs
    gen = torch.Generator().manual_seed(bits)
    scales = (torch.rand((N, G), generator=gen) * 0.009 + 0.001).half().float()
    zeros = torch.randint(1, (1 << bits) + 1, (N, G), generator=gen).float()
    codes = torch.randint(0, 1 << bits, (N, K), generator=gen)
    g = torch.arange(K) // gs
    W = scales[:, g] * (codes.float() - zeros[:, g])  # exact in fp32
    lin = torch.nn.Linear(K, N, bias=True)
    lin.weight.data = W
    q = QuantLinear(bits, gs, K, N, True)
    q.pack(lin, scales.clone(), zeros.clone())
    assert q.qweight.shape == (K // 32 * bits, N) and q.qzeros.shape == (G, N // 32 * bits)
    assert np.array_equal(orc.unpack_bitstream(q.qweight.numpy(), bits, 0), codes.t().numpy())
    assert np.array_equal(orc.unpack_bitstream(q.qzeros.numpy(), bits, 1) + 1, zeros.t().numpy().astype(np.int32))
    w16 = orc.dequant_ref(q.qweight, q.qzeros, q.scales, q.g_idx, bits)
    assert torch.equal(w16, W.t().half())
    assert torch.equal(q.bias, lin.bias.half())


# ---------------------------------------------------------------------------------------------
# Golden vectors written by the reference's own QuantLinear.pack (tests/golden/make_pack_vectors.py):
# real-valued weights, so the rounding of (W + scale * zero) / scale is what is being pinned.
def _golden_cases():
    import os

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "pack_vectors.npz")
    data = np.load(path, allow_pickle=False)
    names = sorted({k.rsplit(".", 1)[0] for k in data.files})
    return data, names


_GOLD, _GOLD_NAMES = _golden_cases()


@pytest.mark.parametrize("name", _GOLD_NAMES)
def test_quantlinear_pack_matches_reference_vectors(name):
    from autogptq.tvm_amd import QuantLinear

    bits, K, N, gs, act, has_bias = (int(v) for v in _GOLD[name + ".meta"])
    linear = torch.nn.Linear(K, N, bias=bool(has_bias))
    with torch.no_grad():
        linear.weight.copy_(torch.from_numpy(_GOLD[name + ".weight"]))
        if has_bias:
            linear.bias.copy_(torch.from_numpy(_GOLD[name + ".bias_in"]))
    q = QuantLinear(bits, gs, K, N, bool(has_bias))
    q.pack(linear, torch.from_numpy(_GOLD[name + ".scales_in"]).clone(),
           torch.from_numpy(_GOLD[name + ".zeros_in"]).clone(), torch.from_numpy(_GOLD[name + ".g_idx"]).clone())
    assert np.array_equal(q.qweight.numpy(), _GOLD[name + ".qweight"])
    assert np.array_equal(q.qzeros.numpy(), _GOLD[name + ".qzeros"])
    assert np.array_equal(q.scales.numpy().view(np.uint16), _GOLD[name + ".scales"])
    assert np.array_equal(q.g_idx.numpy(), _GOLD[name + ".g_idx"])
    if has_bias:
        assert np.array_equal(q.bias.detach().numpy().view(np.uint16), _GOLD[name + ".bias"])


@pytest.mark.parametrize("name", _GOLD_NAMES)
def test_oracle_unpacks_reference_packed_tensors(name):
    """The oracle's unpack and dequant applied to tensors the reference packed: the codes must be
    round((W + s z) / s) and the dequantised weight within half a quantisation step of W wherever
    the code did not saturate."""
    bits, K, N, gs, act, has_bias = (int(v) for v in _GOLD[name + ".meta"])
    qweight, qzeros = _GOLD[name + ".qweight"], _GOLD[name + ".qzeros"]
    scales16 = _GOLD[name + ".scales"].view(np.float16)
    g_idx = _GOLD[name + ".g_idx"]
    codes = orc.unpack_bitstream(qweight, bits, axis=0)            # [K, N]
    zeros = orc.unpack_bitstream(qzeros, bits, axis=1) + 1         # [G, N]
    assert np.array_equal(zeros, _GOLD[name + ".zeros_in"].T.astype(np.int64))
    W = _GOLD[name + ".weight"].T.astype(np.float32)               # [K, N]
    s = scales16.astype(np.float32)[g_idx]                          # [K, N]
    z = zeros[g_idx].astype(np.float32)
    s_in = _GOLD[name + ".scales_in"].T.astype(np.float32)[g_idx]
    want = np.rint((W + z * s_in) / s).astype(np.int64)             # the reference's expression
    assert want.min() >= 0 and want.max() < (1 << bits)             # the fixture keeps codes in range
    assert np.array_equal(codes, want)
    deq = orc.dequant_ref(torch.from_numpy(qweight), torch.from_numpy(qzeros),
                          torch.from_numpy(scales16.copy()), torch.from_numpy(g_idx), bits).float().numpy()
    assert np.all(np.abs(deq - W) <= 0.5 * s * 1.01 + 1e-3)         # within half a quantisation step


# ---------------------------------------------------------------------------------------------
# Load-time preparation of activation-order layers: channels sorted by group.
@pytest.mark.parametrize("bits", [3, 4])
def test_unpack_is_the_inverse_of_pack(bits):
    rng = np.random.default_rng(bits + 40)
    codes = rng.integers(0, 1 << bits, size=(224, 7)).astype(np.uint8)
    assert np.array_equal(pack.unpack_along_axis0(pack.pack_along_axis0(codes, bits), bits), codes)
    words = rng.integers(-(1 << 31), 1 << 31, size=(12, 5)).astype(np.int32)
    assert np.array_equal(pack.unpack_along_axis0(words, bits), orc.unpack_bitstream(words, bits, axis=0))
    # the torch versions (they run on the GPU when a layer is prepared) agree with the numpy ones
    assert np.array_equal(pack.unpack_rows_torch(torch.from_numpy(words), bits).numpy(),
                          pack.unpack_along_axis0(words, bits))
    assert np.array_equal(pack.pack_rows_torch(torch.from_numpy(codes.astype(np.int64)), bits).numpy(),
                          pack.pack_along_axis0(codes, bits))


@pytest.mark.parametrize("bits,K,gs", [(4, 256, 32), (3, 256, 64), (3, 128, -1), (4, 96, 8)])
def test_sort_channels_by_group_preserves_the_layer(bits, K, gs):
    from autogptq.tvm_amd import _slots

    N = 32
    L = pack.synth_layer(90 + bits, K, N, bits, gs, True)
    res = pack.sort_channels_by_group(L["qweight"], L["g_idx"], bits, gs)
    assert res is not None
    qs, kmap = res
    assert qs.shape == L["qweight"].shape and qs.dtype == torch.int32 and kmap.shape == (2 * K,)
    kmap, src = kmap[:K], kmap[K:].long()
    g = K if gs == -1 else gs
    klane = 8 if bits == 4 else 32
    pos, grp = (kmap & 0xFFFF).long(), (kmap >> 16).long()
    assert torch.equal(grp, L["g_idx"].long())
    # undo the slot order to get the sorted position of every original channel
    code_of_slot = torch.tensor(_slots.code_of_slot(bits))
    sorted_pos = (pos // klane) * klane + code_of_slot[pos % klane]
    assert sorted(sorted_pos.tolist()) == list(range(K))            # a permutation
    assert torch.equal(sorted_pos[src], torch.arange(K))            # second half: channel at each sorted index
    assert torch.equal(sorted_pos // g, L["g_idx"].long())           # groups became contiguous
    # the sorted layer with contiguous groups dequantises to the original weight rows, permuted
    w_orig = orc.dequant_ref(L["qweight"], L["qzeros"], L["scales"], L["g_idx"], bits)
    contiguous = (torch.arange(K) // g).to(torch.int32)
    w_sorted = orc.dequant_ref(qs, L["qzeros"], L["scales"], contiguous, bits)
    assert torch.equal(w_sorted[sorted_pos], w_orig)


def test_sort_channels_declines_what_it_cannot_sort():
    L = pack.synth_layer(7, 128, 32, 4, 32, True)
    g = L["g_idx"].clone()
    g[g == 3] = 2                                   # uneven groups
    assert pack.sort_channels_by_group(L["qweight"], g, 4, 32) is None
    assert pack.sort_channels_by_group(L["qweight"], L["g_idx"], 3, 16) is None   # group narrower than a lane block
