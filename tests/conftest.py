import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "mp-sparse-attn_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (HIP device); run with -m gpu")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no HIP device")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def make_qkv(B, Hq, Hkv, N, D, seed, dtype=torch.bfloat16, sigma=1.0, outliers=False):
    """Seeded synthetic q/k/v on the CPU (float32 draw, then cast), so the oracle and the GPU see the same
    bits.  ``outliers``: per head one channel (1% of 128 rounds to 1) of q and of k is multiplied by 20."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, N, D, generator=g) * sigma
    k = torch.randn(B, Hkv, N, D, generator=g) * sigma
    v = torch.randn(B, Hkv, N, D, generator=g) * sigma
    if outliers:
        n_out = max(1, round(0.01 * D))
        for t, H in ((q, Hq), (k, Hkv)):
            for h in range(H):
                idx = torch.randint(0, D, (n_out,), generator=g)
                t[:, h, :, idx] *= 20.0
    return q.to(dtype), k.to(dtype), v.to(dtype)


COS_MIN, MAXABS_MAX = 0.999, 2e-2


def attention_close(got, want, what=""):
    """The acceptance bar of the attention path: cosine >= 0.999 over the flattened tensors and max-abs error <= 2e-2.
    The bar is a bar on the arithmetic.  A 16-bit OUTPUT adds its own rounding: two float32 results 1e-3 apart can fall
    on different sides of a rounding boundary, and for an output of magnitude 4 or more one bf16 step is 2^-5 = 0.031.
    So each side that is a 16-bit tensor gets half a unit in its last place, at the oracle value's magnitude, on top
    of the 2e-2; float32 tensors get nothing."""
    import oracle as O
    g, w = got.detach().cpu(), want.detach().cpu()
    m = O.precision_metric(g, w)
    wd = w.double()
    allow = torch.full_like(wd, MAXABS_MAX)
    for t in (g, w):
        bits = {torch.bfloat16: 8, torch.float16: 11}.get(t.dtype)
        if bits is not None:
            allow = allow + torch.exp2(torch.floor(torch.log2(wd.abs().clamp_min(2.0 ** -24))) - bits)
    err = (g.double() - wd).abs()
    assert m["cos"] >= COS_MIN and bool((err <= allow).all()), f"{what}: {m}, worst excess {(err - allow).max().item():.4g}"
    return m
