"""ctypes front end of oracle/_build/liboracle.so (TEST INFRASTRUCTURE).

The C sources cite the reference lines they follow; this file only marshals
numpy arrays.
"""
import ctypes
import os

import numpy as np

from . import build as _build

_lib = None


def lib():
    global _lib
    if _lib is None:
        path = _build.LIB
        srcs = [os.path.join(_build.HERE, f) for f in _build.SOURCES]
        if not os.path.exists(path) or any(os.path.getmtime(f) > os.path.getmtime(path) for f in srcs):
            _build.build()
        _lib = ctypes.CDLL(path)
    return _lib


def _p(a, ct):
    return None if a is None else a.ctypes.data_as(ctypes.POINTER(ct))


def _rows(rows, N):
    if rows is None:
        return None, N
    r = np.ascontiguousarray(np.asarray(rows, dtype=np.int32))
    assert r.ndim == 1 and (r >= 0).all() and (r < N).all()
    return r, int(r.shape[0])


def we(coords, wavenumbers, mask=None, rows=None, precision="f64", mag_type=1):
    """coords [Z,N,3], wavenumbers [K], mask [Z,N] bool (True = padded).

    mag_type other than 1 (the reference's other source weights) is evaluated in f64 only.

    Returns (out [Z,R,2K], cos_sums [Z,R,K], sin_sums [Z,R,K]) for the selected
    rows (all rows when rows is None), float64 for precision 'f64' and float32
    for 'f32' (terms evaluated in float the way the PyTorch statement does).
    """
    c = np.ascontiguousarray(np.asarray(coords, dtype=np.float32))
    w = np.ascontiguousarray(np.asarray(wavenumbers, dtype=np.float32))
    Z, N, three = c.shape
    assert three == 3
    K = int(w.shape[0])
    m = None if mask is None else np.ascontiguousarray(np.asarray(mask).astype(np.uint8))
    if m is not None:
        assert m.shape == (Z, N)
    r, R = _rows(rows, N)
    dt, ct, fn = (np.float64, ctypes.c_double, lib().we_oracle_f64) if precision == "f64" else \
                 (np.float32, ctypes.c_float, lib().we_oracle_f32)
    out = np.empty((Z, R, 2 * K), dt)
    cs = np.empty((Z, R, K), dt)
    ss = np.empty((Z, R, K), dt)
    if mag_type != 1:
        assert precision == "f64" and mag_type in (0, 2, 3)
        fn = lib().we_oracle_mag_f64
        fn.restype = None
        fn(_p(c, ctypes.c_float), _p(w, ctypes.c_float), _p(m, ctypes.c_uint8),
           ctypes.c_int(Z), ctypes.c_int(N), ctypes.c_int(K), ctypes.c_int(mag_type),
           _p(r, ctypes.c_int), ctypes.c_int(R), _p(out, ct), _p(cs, ct), _p(ss, ct))
        return out, cs, ss
    fn.restype = None
    fn(_p(c, ctypes.c_float), _p(w, ctypes.c_float), _p(m, ctypes.c_uint8),
       ctypes.c_int(Z), ctypes.c_int(N), ctypes.c_int(K), _p(r, ctypes.c_int), ctypes.c_int(R),
       _p(out, ct), _p(cs, ct), _p(ss, ct))
    return out, cs, ss


def we_dropout(coords, wavenumbers, mask, dropout_p, seed, rows=None, mag_type=1):
    """The embedding with the reference kernel's in-kernel dropout (isotropic/cuda/wf_embedding_kernel.cu:27-46,
    :227-238) for an explicit 32-bit seed; float64 (out [Z,R,2K], cos_sums, sin_sums [Z,R,K])."""
    c = np.ascontiguousarray(np.asarray(coords, dtype=np.float32))
    w = np.ascontiguousarray(np.asarray(wavenumbers, dtype=np.float32))
    Z, N, three = c.shape
    assert three == 3 and mag_type in (0, 1, 2, 3)
    K = int(w.shape[0])
    m = None if mask is None else np.ascontiguousarray(np.asarray(mask).astype(np.uint8))
    r, R = _rows(rows, N)
    out = np.empty((Z, R, 2 * K), np.float64)
    cs = np.empty((Z, R, K), np.float64)
    ss = np.empty((Z, R, K), np.float64)
    fn = lib().we_oracle_dropout_f64
    fn.restype = None
    fn(_p(c, ctypes.c_float), _p(w, ctypes.c_float), _p(m, ctypes.c_uint8), ctypes.c_int(Z), ctypes.c_int(N), ctypes.c_int(K),
       ctypes.c_int(mag_type), ctypes.c_float(dropout_p), ctypes.c_uint32(int(seed) & 0xffffffff),
       _p(r, ctypes.c_int), ctypes.c_int(R), _p(out, ctypes.c_double), _p(cs, ctypes.c_double), _p(ss, ctypes.c_double))
    return out, cs, ss


def we_hash5(a, b, c, d, seed):
    fn = lib().we_oracle_hash5
    fn.restype = ctypes.c_uint32
    return int(fn(ctypes.c_int(a), ctypes.c_int(b), ctypes.c_int(c), ctypes.c_int(d), ctypes.c_uint32(int(seed) & 0xffffffff)))


def we_dropout_keep(z, i, j, k, seed, dropout_p):
    fn = lib().we_oracle_dropout_keep
    fn.restype = ctypes.c_int
    return bool(fn(ctypes.c_int(z), ctypes.c_int(i), ctypes.c_int(j), ctypes.c_int(k), ctypes.c_uint32(int(seed) & 0xffffffff),
                   ctypes.c_float(dropout_p)))


def we_aniso(coordsA, coordsB, cb_magnitudes, wavenumbers, mask=None, rows=None):
    """coordsA, coordsB [Z,N,3], cb_magnitudes, wavenumbers [K], mask [Z,N] bool (True = padded).

    Returns (out, d_cb, d_k), each [Z,R,2K] float64, for the selected rows.
    """
    a = np.ascontiguousarray(np.asarray(coordsA, dtype=np.float32))
    b = np.ascontiguousarray(np.asarray(coordsB, dtype=np.float32))
    w = np.ascontiguousarray(np.asarray(wavenumbers, dtype=np.float32))
    cb = np.ascontiguousarray(np.asarray(cb_magnitudes, dtype=np.float32))
    Z, N, three = a.shape
    assert three == 3 and b.shape == a.shape and cb.shape == w.shape and w.ndim == 1
    K = int(w.shape[0])
    m = None if mask is None else np.ascontiguousarray(np.asarray(mask).astype(np.uint8))
    if m is not None:
        assert m.shape == (Z, N)
    r, R = _rows(rows, N)
    out = np.empty((Z, R, 2 * K), np.float64)
    d_cb = np.empty_like(out)
    d_k = np.empty_like(out)
    fn = lib().we_aniso_oracle_f64
    fn.restype = None
    cf, cd = ctypes.c_float, ctypes.c_double
    fn(_p(a, cf), _p(b, cf), _p(cb, cf), _p(w, cf), _p(m, ctypes.c_uint8),
       ctypes.c_int(Z), ctypes.c_int(N), ctypes.c_int(K), _p(r, ctypes.c_int), ctypes.c_int(R),
       _p(out, cd), _p(d_cb, cd), _p(d_k, cd))
    return out, d_cb, d_k


def geo_attn(Q, K, V, coords, sigma, key_padding_mask=None, rows=None):
    """Q,K,V [Z,H,N,d] (float values, already rounded to the kernel's operand
    type by the caller), coords [Z,N,3], sigma [H], key_padding_mask [Z,N] bool.

    Returns (O [Z,H,R,d], L [Z,H,R]) in float64.
    """
    q = np.ascontiguousarray(np.asarray(Q, dtype=np.float32))
    k = np.ascontiguousarray(np.asarray(K, dtype=np.float32))
    v = np.ascontiguousarray(np.asarray(V, dtype=np.float32))
    c = np.ascontiguousarray(np.asarray(coords, dtype=np.float32))
    s = np.ascontiguousarray(np.asarray(sigma, dtype=np.float32))
    Z, H, N, d = q.shape
    assert k.shape == q.shape and v.shape == q.shape and c.shape == (Z, N, 3) and s.shape == (H,)
    m = None if key_padding_mask is None else np.ascontiguousarray(np.asarray(key_padding_mask).astype(np.uint8))
    r, R = _rows(rows, N)
    O = np.empty((Z, H, R, d), np.float64)
    L = np.empty((Z, H, R), np.float64)
    fn = lib().geo_attn_oracle_f64
    fn.restype = None
    fn(_p(q, ctypes.c_float), _p(k, ctypes.c_float), _p(v, ctypes.c_float), _p(c, ctypes.c_float),
       _p(s, ctypes.c_float), _p(m, ctypes.c_uint8),
       ctypes.c_int(Z), ctypes.c_int(H), ctypes.c_int(N), ctypes.c_int(d),
       _p(r, ctypes.c_int), ctypes.c_int(R), _p(O, ctypes.c_double), _p(L, ctypes.c_double))
    return O, L


def geo_attn_legacy(Q, K, V, coords, sigma, beta, key_padding_mask=None, min_rbf=0.0, max_rbf=1.0, rows=None):
    """The reference kernel's own logits, S + beta*rbf_norm*|S| with the [min_rbf, max_rbf] pair mask.
    Same conventions as geo_attn.  Returns (O, L) in float64."""
    q = np.ascontiguousarray(np.asarray(Q, dtype=np.float32))
    k = np.ascontiguousarray(np.asarray(K, dtype=np.float32))
    v = np.ascontiguousarray(np.asarray(V, dtype=np.float32))
    c = np.ascontiguousarray(np.asarray(coords, dtype=np.float32))
    s = np.ascontiguousarray(np.asarray(sigma, dtype=np.float32))
    b = np.ascontiguousarray(np.asarray(beta, dtype=np.float32))
    Z, H, N, d = q.shape
    assert k.shape == q.shape and v.shape == q.shape and c.shape == (Z, N, 3) and s.shape == (H,) and b.shape == (H,)
    m = None if key_padding_mask is None else np.ascontiguousarray(np.asarray(key_padding_mask).astype(np.uint8))
    r, R = _rows(rows, N)
    O = np.empty((Z, H, R, d), np.float64)
    L = np.empty((Z, H, R), np.float64)
    fn = lib().geo_attn_legacy_oracle_f64
    fn.restype = None
    fn(_p(q, ctypes.c_float), _p(k, ctypes.c_float), _p(v, ctypes.c_float), _p(c, ctypes.c_float),
       _p(s, ctypes.c_float), _p(b, ctypes.c_float), _p(m, ctypes.c_uint8),
       ctypes.c_int(Z), ctypes.c_int(H), ctypes.c_int(N), ctypes.c_int(d),
       ctypes.c_double(min_rbf), ctypes.c_double(max_rbf),
       _p(r, ctypes.c_int), ctypes.c_int(R), _p(O, ctypes.c_double), _p(L, ctypes.c_double))
    return O, L
