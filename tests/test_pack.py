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
        pack.pack_qweight(np.zeros((32, 4), dtype=np.int64), 2)
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
