"""Writes the small golden fixtures of tests/golden/ from the pure-Python
float64 brute-force statements in oracle/brute.py.

Run from the repository root:  python tests/golden/make_golden.py
Inputs are drawn from a seeded numpy generator and rounded to float32 (WE) or
bfloat16 (attention operands) BEFORE the brute force sees them, so every
implementation under test starts from the same bits.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import brute  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def to_bf16(x):
    """Round float32 -> bfloat16 (nearest even), returned as float32."""
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def we_golden():
    rng = np.random.default_rng(20240607)
    Z, N, K = 2, 24, 6
    steps = rng.normal(size=(Z, N, 3))
    steps = 3.8 * steps / np.linalg.norm(steps, axis=-1, keepdims=True)
    coords = np.cumsum(steps, axis=1).astype(np.float32)
    coords[0, 7] = coords[0, 3]              # a coincident pair: excluded like the self pair
    wl = 3.7 + (20 - 3.7) * (20 ** (np.arange(K) / K) - 1) / 19
    wn = (2 * np.pi / wl).astype(np.float32)
    wn[2] = -wn[2]                           # the reference test feeds signed wavenumbers
    mask = np.zeros((Z, N), bool)
    mask[1, 18:] = True                      # tail padding
    mask[1, 4] = True                        # and one interior padded token
    out, cs, ss = brute.we_brute(coords.astype(np.float64).tolist(), wn.astype(np.float64).tolist(), mask.tolist())
    np.savez(os.path.join(HERE, "we_small.npz"), coords=coords, wavenumbers=wn, mask=mask,
             out=np.array(out), cos_sums=np.array(cs), sin_sums=np.array(ss))


def we_aniso_golden():
    rng = np.random.default_rng(20240609)
    Z, N, K = 2, 21, 5
    steps = rng.normal(size=(Z, N, 3))
    steps = 3.8 * steps / np.linalg.norm(steps, axis=-1, keepdims=True)
    a = np.cumsum(steps, axis=1).astype(np.float32)
    a[0, 9] = a[0, 2]                        # a coincident pair
    b = rng.normal(size=(Z, N, 3))
    b = (b / np.linalg.norm(b, axis=-1, keepdims=True)).astype(np.float32)
    b[1, 0] = 0                              # chain ends carry no C-beta vector
    wl = 3.7 + (20 - 3.7) * (20 ** (np.arange(K) / K) - 1) / 19
    wn = (2 * np.pi / wl).astype(np.float32)
    cb = rng.uniform(0.5, 2.5, K).astype(np.float32)
    cb[3] = -cb[3]
    mask = np.zeros((Z, N), bool)
    mask[1, 16:] = True
    mask[1, 5] = True
    out, d_cb, d_k = brute.we_aniso_brute(a.astype(np.float64).tolist(), b.astype(np.float64).tolist(),
                                          cb.astype(np.float64).tolist(), wn.astype(np.float64).tolist(), mask.tolist())
    np.savez(os.path.join(HERE, "we_aniso_small.npz"), coordsA=a, coordsB=b, cb_magnitudes=cb, wavenumbers=wn,
             mask=mask, out=np.array(out), d_cb=np.array(d_cb), d_k=np.array(d_k))


def attn_golden():
    rng = np.random.default_rng(20240608)
    Z, H, N, d = 2, 2, 20, 64
    Q = to_bf16(rng.normal(size=(Z, H, N, d)).astype(np.float32))
    K = to_bf16(rng.normal(size=(Z, H, N, d)).astype(np.float32))
    V = to_bf16(rng.normal(size=(Z, H, N, d)).astype(np.float32))
    steps = rng.normal(size=(Z, N, 3))
    steps = 3.8 * steps / np.linalg.norm(steps, axis=-1, keepdims=True)
    coords = np.cumsum(steps, axis=1).astype(np.float32)
    sigma = np.array([3.0, 12.5], np.float32)
    mask = np.zeros((Z, N), bool)
    mask[1, 13:] = True
    mask[1, 2] = True
    O, L = brute.geo_attn_brute(Q.astype(np.float64).tolist(), K.astype(np.float64).tolist(),
                                V.astype(np.float64).tolist(), coords.astype(np.float64).tolist(),
                                sigma.astype(np.float64).tolist(), mask.tolist())
    np.savez(os.path.join(HERE, "geo_attn_small.npz"), Q=Q, K=K, V=V, coords=coords, sigma=sigma, mask=mask,
             O=np.array(O), L=np.array(L))


if __name__ == "__main__":
    we_golden()
    we_aniso_golden()
    attn_golden()
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
