"""Mint golden vectors for the E2M1 / E8M0 encoders from the reference's own format classes.

Run once in a container that has the reference checkout (it is absent on GPU machines):

    python tests/golden/make_mxfp_vectors.py [/path/to/reference]

Only ``ours/mxfp.py`` is loaded (pure torch, CPU).  The vectors cover what closed forms do not
pin: the float32 ``1e-6`` tie-break bias of ``MXFP4Tensor._from_float`` around every midpoint of
the E2M1 grid, and ``MXScaleTensor``'s float32 ``floor(log2(v))``.  Output:
``tests/golden/mxfp_vectors.npz`` (inputs and the reference's outputs, nothing else).
"""

import importlib.util
import os
import sys

import numpy as np
import torch


def load_reference_mxfp(ref_root):
    path = os.path.join(ref_root, "ours", "mxfp.py")
    spec = importlib.util.spec_from_file_location("reference_mxfp", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def e2m1_inputs():
    g = torch.Generator().manual_seed(1234)
    parts = []
    mids = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0]
    grid = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    for m in mids + grid:
        base = torch.tensor([m], dtype=torch.float32)
        # every float32 within +-64 ulp of the point
        bits = base.view(torch.int32).item()
        nb = torch.arange(-64, 65, dtype=torch.int32) + bits
        nb = nb[nb >= 0]
        parts.append(nb.view(torch.float32))
        # absolute offsets around the bias magnitude
        offs = torch.tensor([0.0, 2.5e-7, 4.9e-7, 5e-7, 5.1e-7, 9e-7, 9.9e-7, 1e-6, 1.01e-6, 1.1e-6, 1.5e-6,
                             2e-6, 3e-6, 1e-5, 1e-4], dtype=torch.float32)
        parts.append(base + offs)
        parts.append(base - offs)
    parts.append(torch.tensor([0.0, -0.0, float("inf"), float("-inf"), float("nan"), 6.5, 7.0, 8.0, 100.0, 1e-30,
                              1e-45, 0.1, 0.2499999, 5.9999995], dtype=torch.float32))
    # large magnitudes: float32 cancellation makes the distances to several candidates equal there
    big = torch.ldexp(torch.ones(20), torch.arange(20, 40, dtype=torch.int32))
    parts.append(torch.cat([big, big * 1.25, big + 6.0, big + 2.0, torch.tensor([1e9, 3e38, 16777222.0, 33554438.0])]))
    parts.append(torch.rand(4096, generator=g) * 8.0)
    parts.append(torch.randn(4096, generator=g) * 2.0)
    x = torch.cat(parts)
    x = torch.cat([x, -x])
    return x.contiguous()


def e8m0_inputs():
    g = torch.Generator().manual_seed(4321)
    pw = torch.ldexp(torch.ones(277, dtype=torch.float64), torch.arange(-149, 128, dtype=torch.int32)).to(torch.float32)
    rnd = torch.exp2(torch.rand(4096, generator=g) * 250.0 - 125.0)
    special = torch.tensor([0.0, -1.0, float("inf"), float("nan"), 1.5, 3.0, 0.75, 1e-40], dtype=torch.float32)
    # bf16-valued inputs, the only non-power-of-two scale inputs the path ever produces upstream
    bf = (torch.rand(4096, generator=g) * 100.0).to(torch.bfloat16).to(torch.float32) + 2.0 ** -20
    return torch.cat([pw, rnd, special, bf]).contiguous()


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    mx = load_reference_mxfp(ref_root)
    x4 = e2m1_inputs()
    codes = mx.MXFP4Tensor(data=x4.clone()).data
    decoded = mx.MXFP4Tensor(data=torch.arange(16, dtype=torch.uint8), dtype=torch.uint8).to(torch.float32)
    pk_in = torch.arange(16, dtype=torch.uint8).repeat(4).reshape(4, 16)
    packed = mx.MXFP4Tensor(data=pk_in, dtype=torch.uint8).to_packed_tensor(dim=1)
    x8 = e8m0_inputs()
    sc = mx.MXScaleTensor(data=x8.clone())
    sc_dec = mx.MXScaleTensor(size=(256,))
    sc_dec.data = torch.arange(256, dtype=torch.uint8)
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "mxfp_vectors.npz")
    np.savez_compressed(
        out,
        e2m1_in_bits=x4.view(torch.int32).numpy(), e2m1_codes=codes.numpy(),
        e2m1_decode_all16_bits=decoded.view(torch.int32).numpy(),
        pack_in=pk_in.numpy(), pack_out=packed.numpy(),
        e8m0_in_bits=x8.view(torch.int32).numpy(), e8m0_codes=sc.data.numpy(),
        e8m0_decode_all256_bits=sc_dec.to(torch.float32).view(torch.int32).numpy(),
    )
    print("wrote", out, "e2m1", x4.numel(), "e8m0", x8.numel())


if __name__ == "__main__":
    main()
