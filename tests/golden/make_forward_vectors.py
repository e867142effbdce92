"""Writes tests/golden/forward_vectors.npz: what the reference's own QuantLinear.forward
(auto_gptq/nn_modules/qlinear.py:177-247, its torch branch on the CPU) returns for small packed layers of every
width of the format, with and without an activation order:

  * ``forward(I)`` for the K x K fp16 identity, bias removed: the dequantised weight W itself (a product with the
    identity adds nothing but exact zeros), i.e. the reference's unpack + zeros + 1 + gather + one-rounding dequant;
  * ``forward(x)`` for a seeded fp16 x of five rows, with the layer's bias.

The layers are packed by the reference's own ``pack`` from real-valued weights, as in make_pack_vectors.py.  Run
once, in a container that holds the reference checkout:

    python tests/golden/make_forward_vectors.py /root/reference

Only the reference's qlinear.py is loaded (by file path, not through the package), it runs on the CPU, and nothing
but the .npz fixture is kept.  The fixture pins the oracle's ``dequant_ref`` (bit for bit) and ``forward_ref``.
"""
import contextlib
import io
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from make_pack_vectors import load_reference_qlinear  # noqa: E402

CASES = [  # name, bits, K, N, group_size, act_order, bias
    ("int2_k128_n64_g32", 2, 128, 64, 32, False, True),
    ("int2_k128_n64_g64_act", 2, 128, 64, 64, True, False),
    ("int3_k128_n64_g32", 3, 128, 64, 32, False, False),
    ("int3_k128_n64_g32_act", 3, 128, 64, 32, True, True),
    ("int3_k96_n32_gall_act", 3, 96, 32, -1, True, False),
    ("int4_k128_n64_g32", 4, 128, 64, 32, False, True),
    ("int4_k128_n96_g64_act", 4, 128, 96, 64, True, True),
    ("int4_k64_n32_gall", 4, 64, 32, -1, False, False),
    ("int8_k128_n64_g32", 8, 128, 64, 32, False, False),
    ("int8_k64_n32_g32_act", 8, 64, 32, 32, True, True),
]


def main():
    ref = load_reference_qlinear(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    out = {}
    for case_no, (name, bits, K, N, gs, act, bias) in enumerate(CASES):
        gen = torch.Generator().manual_seed(9100 + case_no)
        maxq = 2 ** bits - 1
        g = K if gs == -1 else gs
        G = (K + g - 1) // g
        scales = (torch.rand(N, G, generator=gen) * 0.02 + 0.005)
        zeros = torch.randint(1, maxq + 1, (N, G), generator=gen).float()
        g_idx = (torch.randperm(K, generator=gen).to(torch.int32) // g) if act else (torch.arange(K, dtype=torch.int32) // g)
        codes = torch.randint(0, maxq + 1, (N, K), generator=gen).float()
        gl = g_idx.long()
        noise = (torch.rand(N, K, generator=gen) * 2 - 1) * 0.45
        linear = torch.nn.Linear(K, N, bias=bias)
        with torch.no_grad():
            linear.weight.copy_(scales[:, gl] * (codes - zeros[:, gl] + noise))
            if bias:
                linear.bias.copy_(torch.randn(N, generator=gen) * 0.1)
        q = ref.QuantLinear(bits, gs, K, N, bias)
        q.pack(linear, scales.clone(), zeros.clone(), g_idx.clone())
        x = torch.randn(5, K, generator=gen).half()
        with contextlib.redirect_stdout(io.StringIO()):      # (the reference's forward prints its input and output)
            y = q.forward(x)
            kept, q.bias = q.bias, None
            w = q.forward(torch.eye(K, dtype=torch.float16))
            q.bias = kept
        assert y.dtype == torch.float16 and w.dtype == torch.float16 and tuple(w.shape) == (K, N)
        out[name + ".meta"] = np.array([bits, K, N, gs, int(act), int(bias)], dtype=np.int64)
        out[name + ".qweight"] = q.qweight.numpy().astype(np.int32)
        out[name + ".qzeros"] = q.qzeros.numpy().astype(np.int32)
        out[name + ".scales"] = q.scales.numpy().view(np.uint16)
        out[name + ".g_idx"] = q.g_idx.numpy().astype(np.int32)
        if bias:
            out[name + ".bias"] = q.bias.detach().numpy().view(np.uint16)
        out[name + ".x"] = x.numpy().view(np.uint16)
        out[name + ".w"] = w.numpy().view(np.uint16)       # forward(I) without the bias = dequantised W
        out[name + ".y"] = y.detach().numpy().view(np.uint16)
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "forward_vectors.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes;", len(CASES), "cases")


if __name__ == "__main__":
    main()
