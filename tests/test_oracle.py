"""Pins the CPU oracle (oracle/) without a GPU.

The reference holds no golden vectors for this path, so each oracle function is pinned by
checks a plausible mistake would fail: hand-worked words, an independent closed form, three
independent statements agreeing (torch table unpack, closed-form bit stream, C restatement),
exact-integer cases and an fp64 matmul.
"""
import numpy as np
import pytest
import torch

from oracle import gptq_oracle as orc


def rand_words(rng, shape):
    return rng.integers(0, 1 << 32, size=shape, dtype=np.uint64).astype(np.uint32).view(np.int32)


# ---------------------------------------------------------------- hand-worked known answers
def test_int4_known_word():
    # nibbles 0..7 of 0x76543210 are 0,1,..,7 (code j at bit 4j)
    q = np.array([[0x76543210]], dtype=np.uint32).view(np.int32)
    assert orc.unpack_bitstream(q, 4, axis=0)[:, 0].tolist() == list(range(8))
    assert orc.unpack_qweight_ref(torch.from_numpy(q), 4)[:, 0].tolist() == list(range(8))
    # a word with the sign bit set: arithmetic shift must not leak into the top nibble
    q = np.array([[0xF0000000]], dtype=np.uint32).view(np.int32)
    assert orc.unpack_qweight_ref(torch.from_numpy(q), 4)[:, 0].tolist() == [0] * 7 + [15]


def test_int3_straddling_codes_known_words():
    # code 10 = 7 alone: bits 30,31 of word 0 and bit 0 of word 1 (reference pack :120-122)
    codes = np.zeros((32, 1), dtype=np.int64)
    codes[10] = 7
    packed = orc.pack_qweight_loop(codes, 3).view(np.uint32)
    assert packed[:, 0].tolist() == [0xC0000000, 0x00000001, 0x00000000]
    # code 21 = 7 alone: bit 31 of word 1 and bits 0,1 of word 2 (reference pack :127-129)
    codes[:] = 0
    codes[21] = 7
    packed = orc.pack_qweight_loop(codes, 3).view(np.uint32)
    assert packed[:, 0].tolist() == [0x00000000, 0x80000000, 0x00000003]
    # code 10 = 5 (0b101): low two bits 01 at 30..31, high bit 1 in word 1
    codes[:] = 0
    codes[10] = 5
    packed = orc.pack_qweight_loop(codes, 3).view(np.uint32)
    assert packed[:, 0].tolist() == [0x40000000, 0x00000001, 0x00000000]
    # code 0 = 1, code 11 = 1, code 22 = 1: bit 0 of w0, bit 1 of w1, bit 2 of w2
    codes[:] = 0
    codes[[0, 11, 22]] = 1
    packed = orc.pack_qweight_loop(codes, 3).view(np.uint32)
    assert packed[:, 0].tolist() == [1, 2, 4]


def test_known_words_two_and_eight_bits():
    # 8 bits: word 0x04030201 holds codes 1, 2, 3, 4; 2 bits: 0xE4 = 0b11100100 holds 0, 1, 2, 3
    w8 = np.array([[0x04030201], [0x7FFFFF80 - (1 << 32) + (1 << 31)]], dtype=np.int64).astype(np.int32)
    got = orc.unpack_bitstream(w8, 8, axis=0)[:, 0].tolist()
    assert got[:4] == [1, 2, 3, 4] and got[4:] == [0x80, 0xFF, 0xFF, 0xFF]
    w2 = np.array([[0xE4], [-1]], dtype=np.int32)
    got = orc.unpack_bitstream(w2, 2, axis=0)[:, 0].tolist()
    assert got[:4] == [0, 1, 2, 3] and got[4:16] == [0] * 12 and got[16:] == [3] * 16
    assert np.array_equal(orc.unpack_qweight_ref(torch.from_numpy(w8), 8).numpy()[:, 0], orc.unpack_bitstream(w8, 8)[:, 0])
    assert np.array_equal(orc.unpack_qweight_ref(torch.from_numpy(w2), 2).numpy()[:, 0], orc.unpack_bitstream(w2, 2)[:, 0])


def test_zero_point_plus_one_known():
    for bits in (2, 3, 4, 8):
        n = 64
        qz = np.zeros((2, n // 32 * bits), dtype=np.int32)
        assert (orc.unpack_qzeros_ref(torch.from_numpy(qz), bits, n).numpy() == 1).all()
        qz = np.full((2, n // 32 * bits), -1, dtype=np.int32)  # all bits set
        assert (orc.unpack_qzeros_ref(torch.from_numpy(qz), bits, n).numpy() == (1 << bits)).all()


# ---------------------------------------------------------------- three statements agree
@pytest.mark.parametrize("bits", [2, 3, 4, 8])
def test_unpack_statements_agree_on_random_words(bits, c_oracle):
    rng = np.random.default_rng(10 + bits)
    qw = rand_words(rng, (bits * 6, 40))  # 6 blocks of 32 channels, arbitrary bit patterns
    a = orc.unpack_bitstream(qw, bits, axis=0)
    b = orc.unpack_qweight_ref(torch.from_numpy(qw), bits).numpy().astype(np.int32)
    c = c_oracle.unpack_rows(qw, bits)
    assert a.shape == (192, 40)
    assert np.array_equal(a, b)
    assert np.array_equal(a, c)
    assert a.min() >= 0 and a.max() < (1 << bits)


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
def test_unpack_zeros_statements_agree(bits, c_oracle):
    rng = np.random.default_rng(20 + bits)
    n = 96
    qz = rand_words(rng, (5, n // 32 * bits))
    a = orc.unpack_bitstream(qz, bits, axis=1) + 1
    b = orc.unpack_qzeros_ref(torch.from_numpy(qz), bits, n).numpy().astype(np.int32)
    c = c_oracle.unpack_zeros(qz, bits)
    assert np.array_equal(a, b)
    assert np.array_equal(a, c)


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
def test_pack_unpack_round_trip(bits):
    rng = np.random.default_rng(30 + bits)
    codes = rng.integers(0, 1 << bits, size=(96, 7))
    qw = orc.pack_qweight_loop(codes, bits)
    assert qw.shape == (96 // 32 * bits, 7)
    assert np.array_equal(orc.unpack_bitstream(qw, bits, axis=0), codes)
    assert np.array_equal(orc.unpack_qweight_ref(torch.from_numpy(qw), bits).numpy(), codes)
    zeros = rng.integers(1, (1 << bits) + 1, size=(3, 64))
    qz = orc.pack_qzeros_loop(zeros, bits)
    assert qz.shape == (3, 64 // 32 * bits)
    assert np.array_equal(orc.unpack_qzeros_ref(torch.from_numpy(qz), bits, 64).numpy(), zeros)


def test_int3_single_code_positions():
    # every code position in turn holds 7: the packed block must have exactly bits 3j..3j+2 set
    for j in range(32):
        codes = np.zeros((32, 1), dtype=np.int64)
        codes[j] = 7
        w = orc.pack_qweight_loop(codes, 3).view(np.uint32)[:, 0].astype(object)
        stream = int(w[0]) | (int(w[1]) << 32) | (int(w[2]) << 64)
        assert stream == 7 << (3 * j), j


# ---------------------------------------------------------------- dequant
def _layer(bits, K, N, gs, desc_act, seed):
    from autogptq.tvm_amd.pack import synth_layer

    return synth_layer(seed, K, N, bits, gs, desc_act, M=3)


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("desc_act", [False, True])
def test_dequant_statements_agree(bits, desc_act, c_oracle):
    L = _layer(bits, 128, 64, 32, desc_act, 40 + bits)
    a = orc.dequant_ref(L["qweight"], L["qzeros"], L["scales"], L["g_idx"], bits).numpy()
    b = orc.dequant_exact(L["qweight"].numpy(), L["qzeros"].numpy(), L["scales"].numpy(), L["g_idx"].numpy(), bits)
    c = c_oracle.dequant(L["qweight"].numpy(), L["qzeros"].numpy(), L["scales"].numpy(), L["g_idx"].numpy(), bits)
    assert a.dtype == np.float16
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
    assert np.array_equal(a.view(np.uint16), c.view(np.uint16))
    # and from first principles, element by element on a few entries
    codes, zeros = L["codes"].numpy(), L["zeros"].numpy()
    g = L["g_idx"].numpy()
    for (k, n) in [(0, 0), (10, 5), (21, 63), (127, 31), (64, 17)]:
        want = np.float16(np.float32(L["scales"].numpy()[g[k], n]) * np.float32(codes[k, n] - zeros[g[k], n]))
        assert a[k, n] == want


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
def test_dequant_unit_scale_is_integer_exact(bits):
    L = _layer(bits, 64, 32, -1, False, 50 + bits)
    ones = torch.ones_like(L["scales"])
    w = orc.dequant_ref(L["qweight"], L["qzeros"], ones, L["g_idx"], bits).numpy().astype(np.int64)
    assert np.array_equal(w, L["codes"].numpy() - L["zeros"].numpy()[L["g_idx"].numpy().astype(np.int64)])


def test_fp16_multiply_equals_fp32_product_rounded_once(c_oracle):
    # the claim the kernels and the C oracle rely on, over all scale bit patterns that are finite
    s_bits = np.arange(0, 0x7C00, 7, dtype=np.uint16)
    s = torch.from_numpy(s_bits.view(np.float16).copy())
    for d in list(range(-16, 16)) + [-256, -255, -129, -100, 97, 127, 200, 254]:   # 8-bit layers reach +-256
        torch_prod = (s * torch.tensor(d, dtype=torch.int32)).numpy()  # fp16 tensor * int tensor -> fp16
        restated = (s.numpy().astype(np.float32) * np.float32(d)).astype(np.float16)
        assert np.array_equal(torch_prod.view(np.uint16), restated.view(np.uint16)), d
    lib = c_oracle.lib()
    rng = np.random.default_rng(5)
    for f in rng.standard_normal(2000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 2000):
        assert lib.oracle_float_to_half(float(f)) == int(np.float32(f).astype(np.float16).view(np.uint16)), f
    for h in range(0, 0x7C00, 13):
        assert lib.oracle_half_to_float(h) == float(np.uint16(h).view(np.float16))


def test_permuted_g_idx_regroups_rows():
    bits = 4
    L = _layer(bits, 128, 32, 32, False, 77)
    gen = torch.Generator().manual_seed(3)
    g_perm = (torch.randperm(128, generator=gen) // 32).to(torch.int32)
    w_perm = orc.dequant_ref(L["qweight"], L["qzeros"], L["scales"], g_perm, bits).numpy()
    codes, zeros, sc = L["codes"].numpy(), L["zeros"].numpy(), L["scales"].numpy()
    for k in range(128):
        g = int(g_perm[k])
        want = (sc[g].astype(np.float32) * (codes[k] - zeros[g]).astype(np.float32)).astype(np.float16)
        assert np.array_equal(w_perm[k], want)


# ---------------------------------------------------------------- forward
@pytest.mark.parametrize("bits", [3, 4])
def test_forward_matches_fp64_and_c(bits, c_oracle):
    L = _layer(bits, 256, 64, 64, True, 60 + bits)
    bias = torch.randn(64, generator=torch.Generator().manual_seed(1)).half()
    y = orc.forward_ref(L["x"], L["qweight"], L["qzeros"], L["scales"], L["g_idx"], bias, bits).float().numpy()
    w = orc.dequant_exact(L["qweight"].numpy(), L["qzeros"].numpy(), L["scales"].numpy(), L["g_idx"].numpy(), bits)
    y64 = orc.forward_f64(L["x"].numpy(), w, bias.numpy())
    assert np.allclose(y, y64, rtol=1e-2, atol=1e-2)
    yc = c_oracle.forward(L["x"].numpy(), L["qweight"].numpy(), L["qzeros"].numpy(), L["scales"].numpy(),
                          L["g_idx"].numpy(), bias.numpy(), bits)
    assert np.allclose(yc, y64, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("bits", [3, 4])
def test_forward_integer_exact_column_sums(bits):
    # x = 1, scales = 1: y[n] = sum_k (q[k, n] - zero[n]) exactly (the reference's own sanity pattern:
    # ones input, unit scales; auto_gptq/nn_modules/tvm_untils/pycuda_warpper.py:357-365)
    L = _layer(bits, 64, 32, -1, False, 70 + bits)
    x = torch.ones((1, 64), dtype=torch.float16)
    ones = torch.ones_like(L["scales"])
    y = orc.forward_ref(x, L["qweight"], L["qzeros"], ones, L["g_idx"], None, bits).float().numpy()
    want = (L["codes"].numpy() - L["zeros"].numpy()[0][None, :]).sum(axis=0)
    assert np.array_equal(y[0], want.astype(np.float32))


def test_forward_keeps_leading_dims():
    L = _layer(4, 64, 32, 32, False, 80)
    x = torch.randn((2, 3, 64), generator=torch.Generator().manual_seed(2)).half()
    y = orc.forward_ref(x, L["qweight"], L["qzeros"], L["scales"], L["g_idx"], None, 4)
    assert y.shape == (2, 3, 32) and y.dtype == torch.float16


# Vectors written by the reference's own QuantLinear.forward on the CPU (tests/golden/make_forward_vectors.py):
# forward(I) without the bias is the reference's dequantised weight, forward(x) its output.
def _forward_vectors():
    import os

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "forward_vectors.npz")
    data = np.load(path)
    return data, sorted({k.split(".")[0] for k in data.files})


_FWD, _FWD_NAMES = _forward_vectors()


def test_forward_vectors_cover_every_width_with_and_without_an_activation_order():
    seen = {(int(_FWD[n + ".meta"][0]), bool(_FWD[n + ".meta"][4])) for n in _FWD_NAMES}
    assert seen == {(b, a) for b in (2, 3, 4, 8) for a in (False, True)}
    assert any(int(_FWD[n + ".meta"][3]) == -1 for n in _FWD_NAMES)


@pytest.mark.parametrize("name", _FWD_NAMES)
def test_oracle_reproduces_the_reference_forward(name, c_oracle):
    bits, K, N, gs, act, has_bias = (int(v) for v in _FWD[name + ".meta"])
    qweight, qzeros, g_idx = _FWD[name + ".qweight"], _FWD[name + ".qzeros"], _FWD[name + ".g_idx"]
    scales = _FWD[name + ".scales"].view(np.float16)
    bias = _FWD[name + ".bias"].view(np.float16) if has_bias else None
    x = _FWD[name + ".x"].view(np.float16)
    w_ref, y_ref = _FWD[name + ".w"], _FWD[name + ".y"].view(np.float16)
    tq, tz, ts, tg = (torch.from_numpy(a.copy()) for a in (qweight, qzeros, scales, g_idx))
    # the dequantised weight: bit for bit, from all three statements of the oracle
    assert np.array_equal(orc.dequant_ref(tq, tz, ts, tg, bits).numpy().view(np.uint16), w_ref)
    assert np.array_equal(orc.dequant_exact(qweight, qzeros, scales, g_idx, bits).view(np.uint16), w_ref)
    assert np.array_equal(c_oracle.dequant(qweight, qzeros, scales, g_idx, bits).view(np.uint16), w_ref)
    # the output: the torch restatement runs the reference's own operations in its order (same bits on the same
    # torch build; one fp16 ulp of slack for another build's summation order); the C restatement sums in double
    tb = torch.from_numpy(bias.copy()) if bias is not None else None
    y = orc.forward_ref(torch.from_numpy(x.copy()), tq, tz, ts, tg, tb, bits).numpy()
    assert y.dtype == np.float16 and y.shape == y_ref.shape
    ulp = np.maximum(np.abs(y_ref.astype(np.float32)), 2.0 ** -14) * 2.0 ** -10
    assert np.all(np.abs(y.astype(np.float32) - y_ref.astype(np.float32)) <= ulp)
    yc = c_oracle.forward(x, qweight, qzeros, scales, g_idx, bias, bits)
    # (the reference adds in fp16-rounded steps the CPU backend chooses: K products of magnitude <= |x| |w|)
    bound = 2e-3 + 2e-3 * np.abs(yc)
    assert np.all(np.abs(yc - y_ref.astype(np.float32)) <= bound)
