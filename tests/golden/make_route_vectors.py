"""Write the tile router's golden vectors: scale bytes in, class map / visiting lists / run lengths out.

The routing rule is this build's own (the reference keeps or skips tiles but does not choose a precision), so
these vectors pin the rule against drift rather than against the reference: they were written from the integer
formulation in ``oracle/mx_route.py`` after that was checked against an exact rational evaluation of the score bound
it stands for (``tests/test_oracle_route.py``).  The CPU oracle and the HIP kernels are both tested against the file.

    python tests/golden/make_route_vectors.py          # writes tests/golden/route_vectors.npz
"""

import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle as O  # noqa: E402


def cases():
    rng = np.random.default_rng(20240607)
    out = {}
    specs = [  # name, B, Hq, Hkv, query tiles, key tiles, tile, D, valid keys in the last key tile, causal, hi, lo
        ("a", 1, 4, 2, 5, 5, 64, 128, 64, 0, 0.5, 0.05),
        ("b", 1, 4, 2, 5, 5, 64, 128, 37, 1, 0.5, 0.05),
        ("c", 2, 2, 2, 3, 70, 64, 64, 11, 0, 0.9, 0.6),
        ("d", 1, 2, 1, 4, 4, 128, 128, 128, 1, 0.0, 0.3),
        ("e", 1, 2, 1, 4, 4, 128, 64, 5, 0, 0.25, 0.0),
    ]
    for name, B, Hq, Hkv, ntq, ntk, tile, D, last, causal, hi, lo in specs:
        nb = D // 32

        def scales(H, nt, valid_last):
            top = rng.integers(112, 132, size=(B, H, nt, 1, nb))
            rows = np.clip(top - rng.integers(0, 6, size=(B, H, nt, tile, nb)), 1, 255)
            rows[:, :, -1, valid_last:, :] = 0            # padding rows of a ragged last tile
            return rows.reshape(B, H, nt * tile, nb).astype(np.uint8)

        qs = scales(Hq, ntq, last if ntq == ntk else tile)
        ks = scales(Hkv, ntk, last)
        n_keys = (ntk - 1) * tile + last
        cls = O.route_tiles(qs, ks, tile, bool(causal), hi, lo)
        order, counts = O.route_order(cls, n_keys, tile, bool(causal))
        out.update({f"{name}_qs": qs, f"{name}_ks": ks, f"{name}_cls": cls, f"{name}_order": order, f"{name}_counts": counts,
                    f"{name}_meta": np.array([tile, D, n_keys, causal], dtype=np.int64),
                    f"{name}_thresh": np.array([hi, lo], dtype=np.float32)})
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "route_vectors.npz")
    np.savez_compressed(path, **cases())
    print(path, os.path.getsize(path), "bytes")
