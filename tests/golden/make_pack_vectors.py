"""Writes tests/golden/pack_vectors.npz: inputs and outputs of the reference's QuantLinear.pack
(auto_gptq/nn_modules/qlinear.py:77-175) on small layers with real-valued weights.

This is the one function of the path whose result on arbitrary float weights no closed form or
fixture of the reference pins (the rounding of (W + scale * zero) / scale), so its vectors come
from the reference itself.  Run once, in a container that holds the reference checkout:

    python tests/golden/make_pack_vectors.py /root/reference

Only the reference's qlinear.py is loaded (by file path, not through the package), it runs on the
CPU, and nothing but the .npz fixture is kept.
"""
import importlib.util
import os
import sys

import numpy as np
import torch


def load_reference_qlinear(ref_root: str):
    path = os.path.join(ref_root, "auto_gptq", "nn_modules", "qlinear.py")
    spec = importlib.util.spec_from_file_location("_reference_qlinear", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


CASES = [  # name, bits, K, N, group_size, act_order, bias
    ("int4_k128_n64_g32", 4, 128, 64, 32, False, True),
    ("int4_k128_n64_g32_act", 4, 128, 64, 32, True, False),
    ("int3_k128_n64_g32_act", 3, 128, 64, 32, True, True),
    ("int3_k96_n32_gall", 3, 96, 32, -1, False, False),
    ("int4_k64_n96_g16", 4, 64, 96, 16, False, False),
]


def main():
    ref = load_reference_qlinear(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    out = {}
    for case_no, (name, bits, K, N, gs, act, bias) in enumerate(CASES):
        gen = torch.Generator().manual_seed(9000 + case_no)
        maxq = 2 ** bits - 1
        g = K if gs == -1 else gs
        G = (K + g - 1) // g
        # what a GPTQ quantiser hands to pack: per (column, group) fp scales and integer zero points,
        # and weights that sit near (not on) the quantisation grid, codes inside [0, maxq]
        scales = (torch.rand(N, G, generator=gen) * 0.02 + 0.005)
        zeros = torch.randint(1, maxq + 1, (N, G), generator=gen).float()
        if act:
            g_idx = torch.randperm(K, generator=gen).to(torch.int32) // g
        else:
            g_idx = (torch.arange(K, dtype=torch.int32) // g)
        codes = torch.randint(0, maxq + 1, (N, K), generator=gen).float()
        gl = g_idx.long()
        noise = (torch.rand(N, K, generator=gen) * 2 - 1) * 0.45
        weight = scales[:, gl] * (codes - zeros[:, gl] + noise)
        linear = torch.nn.Linear(K, N, bias=bias)
        with torch.no_grad():
            linear.weight.copy_(weight)
            if bias:
                linear.bias.copy_(torch.randn(N, generator=gen) * 0.1)
        q = ref.QuantLinear(bits, gs, K, N, bias)
        q.pack(linear, scales.clone(), zeros.clone(), g_idx.clone())
        out[name + ".meta"] = np.array([bits, K, N, gs, int(act), int(bias)], dtype=np.int64)
        out[name + ".weight"] = linear.weight.detach().numpy().astype(np.float32)
        if bias:
            out[name + ".bias_in"] = linear.bias.detach().numpy().astype(np.float32)
            out[name + ".bias"] = q.bias.detach().numpy().view(np.uint16)
        out[name + ".scales_in"] = scales.numpy().astype(np.float32)
        out[name + ".zeros_in"] = zeros.numpy().astype(np.float32)
        out[name + ".g_idx"] = g_idx.numpy().astype(np.int32)
        out[name + ".qweight"] = q.qweight.numpy().astype(np.int32)
        out[name + ".qzeros"] = q.qzeros.numpy().astype(np.int32)
        out[name + ".scales"] = q.scales.numpy().view(np.uint16)
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "pack_vectors.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes;", len(CASES), "cases")


if __name__ == "__main__":
    main()
