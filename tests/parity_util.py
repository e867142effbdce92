"""Helpers shared by the GPU parity tests: oracle-side expected values for a synthetic layer."""
import numpy as np
import torch

from autogptq.tvm_amd.pack import synth_layer
from oracle import c_oracle

RTOL = 1e-2  # the tolerance the path's contract states for y (fp16 in/out, fp32 accumulate)
ATOL = 1e-2


def to_dev(L, dev):
    out = dict(L)
    for k in ("qweight", "qzeros", "scales", "g_idx", "x", "bias"):
        if L.get(k) is not None:
            out[k] = L[k].to(dev)
    return out


def expected_weight(L) -> torch.Tensor:
    """fp16 [K, N] from the C oracle (bit-exact target)."""
    w = c_oracle.dequant(L["qweight"].numpy(), L["qzeros"].numpy(), L["scales"].numpy(), L["g_idx"].numpy(),
                         L["bits"])
    return torch.from_numpy(w.copy())


def expected_output(L, x=None, w16=None) -> torch.Tensor:
    """fp32 [M, N]: x @ W with W the oracle's fp16 weight, accumulated in fp32 or wider."""
    if w16 is None:
        w16 = expected_weight(L)
    x = L["x"] if x is None else x
    y = x.reshape(-1, x.shape[-1]).float() @ w16.float()
    if L.get("bias") is not None:
        y = y + L["bias"].float()
    return y


def assert_close(got: torch.Tensor, want: torch.Tensor, what: str, rtol=RTOL, atol=ATOL):
    got = got.detach().float().cpu()
    want = want.detach().float().cpu()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    err = (got - want).abs()
    bound = atol + rtol * want.abs()
    bad = err > bound
    assert not bool(bad.any()), (
        f"{what}: {int(bad.sum())} of {bad.numel()} outside rtol={rtol} atol={atol}; "
        f"max abs err {float(err.max()):.4g} at {np.unravel_index(int(err.argmax()), err.shape)}"
    )
    return float(err.max())


def layer(seed, K, N, bits, gs, desc_act, M=1, bias=False):
    return synth_layer(seed, K, N, bits, gs, desc_act, M=M, bias=bias)


def assert_tight(got: torch.Tensor, want: torch.Tensor, what: str):
    """A bound much tighter than the contract's, so that an indexing slip cannot hide inside
    the tolerance: one fp16 rounding of y (relative 2^-11) plus fp32 accumulation noise and, for
    the kernels that apply scales per group, the reference's own weight-rounding noise."""
    return assert_close(got, want, what + " (tight)", rtol=2e-3, atol=3e-3)
