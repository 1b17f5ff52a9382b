"""GPU tests of the WE forward with the reference kernel's in-kernel dropout (proteus_we_dropout_fwd) against the CPU
oracle on the same seed: the dropout mask is integer arithmetic and must be the same to the bit, so the bars are the
forward's own (rel-L2 <= 1e-4 for out, cos_sums and sin_sums)."""
import ctypes

import numpy as np
import pytest
import torch

import proteusai_amd as pa
from oracle import c_oracle
from proteusai_amd import _lib, synth

pytestmark = pytest.mark.gpu

REL_L2_TOL = 1e-4


def rel_l2(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    nb = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / nb) if nb > 0 else float(np.linalg.norm(a - b))


def inputs(seed, Z, N, K):
    g = torch.Generator().manual_seed(seed)
    coords = torch.stack([synth.random_walk_chain(N, g) for _ in range(Z)])
    wn = torch.exp(torch.linspace(np.log(0.02), np.log(2.0), K))
    return coords, wn


def check(gpu, coords, wn, mask, p, seed, mag=1, rows=None):
    out, cs, ss = pa.we_forward(coords.to(gpu), wn.to(gpu), None if mask is None else mask.to(gpu),
                                magnitude_type=mag, dropout_p=p, rng_seed=seed)
    torch.cuda.synchronize()
    ro, rc, rs = c_oracle.we_dropout(coords.numpy(), wn.numpy(), None if mask is None else mask.numpy(), p, seed, rows=rows, mag_type=mag)
    sel = slice(None) if rows is None else np.asarray(rows)
    for got, want, name in ((out, ro, "out"), (cs, rc, "cos_sums"), (ss, rs, "sin_sums")):
        got = got.cpu().numpy()[:, sel]
        assert np.isfinite(got).all(), name
        e = rel_l2(got, want)
        assert e <= REL_L2_TOL, f"{name}: rel-L2 {e:.3e} (p={p}, seed={seed}, mag={mag})"
        if mask is not None:
            m = mask.numpy()[:, sel] if rows is None else mask.numpy()[:, rows]
            assert (got[m] == 0).all(), f"{name}: padded observers must get zeros"
    return out, cs, ss


@pytest.mark.parametrize("p", [0.1, 0.5, 0.9])
@pytest.mark.parametrize("N,K", [(1, 4), (63, 5), (64, 64), (200, 33), (513, 70)])
def test_mask_and_sums_equal_the_oracle(gpu, N, K, p):
    coords, wn = inputs(N + K, 2, N, K)
    mask = torch.zeros(2, N, dtype=torch.bool)
    if N > 8:
        mask[1, N // 2:] = True
        mask[0, 3] = True
    check(gpu, coords, wn, mask, p, seed=1000 * N + K)


@pytest.mark.parametrize("mag", [0, 2, 3])
def test_other_source_weights(gpu, mag):
    coords, wn = inputs(5, 2, 150, 20)
    check(gpu, coords, wn, None, 0.3, seed=77, mag=mag)


def test_the_mask_is_a_function_of_the_four_indices_and_the_seed(gpu):
    # zero wavenumbers: cos = 1 and weight 1 (magnitude_type 0), so out[z, i, 2k] * (1 - p) counts the kept partners of
    # (z, i, k) -- an integer that must equal the oracle's count exactly, for every row, wavenumber and batch item
    Z, N, K = 3, 130, 9
    coords, _ = inputs(9, Z, N, K)
    wn = torch.zeros(K)
    p, seed = 0.4, 0xdeadbeef
    out, _, _ = pa.we_forward(coords.to(gpu), wn.to(gpu), None, magnitude_type=0, dropout_p=p, rng_seed=seed)
    kept = out.cpu().numpy()[:, :, 0::2].astype(np.float64) * (1.0 - float(np.float32(p)))
    want = np.zeros((Z, N, K))
    for z in range(Z):
        for i in range(N):
            for k in range(K):
                want[z, i, k] = sum(c_oracle.we_dropout_keep(z, i, j, k, seed, p) for j in range(N) if j != i)
    assert np.abs(kept - want).max() < 1e-3          # integers, up to the rounding of the factor 1 / (1 - p)
    # the same seed gives the same result to the bit, another seed another mask
    again, _, _ = pa.we_forward(coords.to(gpu), wn.to(gpu), None, magnitude_type=0, dropout_p=p, rng_seed=seed)
    other, _, _ = pa.we_forward(coords.to(gpu), wn.to(gpu), None, magnitude_type=0, dropout_p=p, rng_seed=seed + 1)
    assert torch.equal(out, again) and not torch.equal(out, other)
    # a fresh seed per call when none is given (isotropic/cuda/wf_embedding.py:48-49)
    a, _, _ = pa.we_forward(coords.to(gpu), wn.to(gpu), None, magnitude_type=0, dropout_p=p)
    b, _, _ = pa.we_forward(coords.to(gpu), wn.to(gpu), None, magnitude_type=0, dropout_p=p)
    assert not torch.equal(a, b)


def test_large_indices_sampled_rows(gpu):
    # token indices up to 5000 and 300 wavenumbers enter the hash; rows are independent
    N, K = 5000, 300
    coords, wn = inputs(3, 1, N, K)
    rows = np.unique(np.concatenate([np.random.default_rng(0).choice(N, 40, replace=False), [0, 63, 64, N - 1]])).astype(np.int32)
    check(gpu, coords, wn, None, 0.25, seed=2 ** 32 - 5, rows=rows)


def test_operator_gradient_is_that_of_the_masked_sum(gpu):
    # the saved sums carry the mask, so d/dk of sum(out * G) is the backward's contraction of the masked sums: compare
    # with central differences of the operator at a fixed seed
    coords, wn = inputs(11, 2, 90, 6)
    c = coords.to(gpu)
    w = wn.to(gpu).double().requires_grad_(True)
    G = torch.randn(2, 90, 12, generator=torch.Generator().manual_seed(1)).to(gpu)
    out = pa.wf_embedding(c, w, 1, 0.35, None, rng_seed=4242)
    (out.double() * G.double()).sum().backward()
    eps = 1e-3
    for k in (0, 3, 5):
        wp, wm = wn.clone(), wn.clone()
        wp[k] += eps
        wm[k] -= eps
        fp = (pa.wf_embedding(c, wp.to(gpu), 1, 0.35, None, rng_seed=4242).double() * G.double()).sum()
        fm = (pa.wf_embedding(c, wm.to(gpu), 1, 0.35, None, rng_seed=4242).double() * G.double()).sum()
        fd = float((fp - fm) / (2 * eps))
        assert abs(float(w.grad[k]) - fd) <= 2e-3 * max(1.0, abs(fd)), (k, float(w.grad[k]), fd)


def test_argument_errors_and_the_threshold(gpu):
    lib = _lib.load()
    coords, wn = inputs(1, 1, 10, 2)
    with pytest.raises(ValueError):
        pa.we_forward(coords.to(gpu), wn.to(gpu), None, dropout_p=1.0)
    with pytest.raises(ValueError):
        pa.we_forward(coords.to(gpu), wn.to(gpu), None, dropout_p=-0.1)
    c, w = coords.to(gpu), wn.to(gpu)
    o = torch.empty(1, 10, 4, device=gpu)
    s = torch.empty(1, 10, 2, device=gpu)
    args = (c.data_ptr(), _lib.COORDS_AOS, w.data_ptr(), None, o.data_ptr(), s.data_ptr(), s.data_ptr(), 1, 10, 2)
    assert lib.proteus_we_dropout_fwd_check(*args, 1, ctypes.c_float(0.5)) == 0
    assert lib.proteus_we_dropout_fwd_check(*args, 1, ctypes.c_float(1.0)) == -2
    assert lib.proteus_we_dropout_fwd_check(*args, 1, ctypes.c_float(float("nan"))) == -2
    assert lib.proteus_we_dropout_fwd_check(*args, 4, ctypes.c_float(0.5)) == -7
    assert lib.proteus_we_dropout_fwd_check(c.data_ptr(), _lib.COORDS_AOS, w.data_ptr(), None, o.data_ptr(), None, None, 1, 10, 2,
                                            1, ctypes.c_float(0.5)) == -1
    # the smallest kept hash value: exactly where the reference's float test turns
    for p in (1e-9, 0.1, 0.5, 0.75, 0.999):
        h = lib.proteus_we_dropout_threshold(ctypes.c_float(p))
        keep = lambda v: np.float32(v) / np.float32(2.0 ** 32) >= np.float32(p)
        assert keep(h) and (h == 0 or not keep(h - 1))
    assert lib.proteus_we_dropout_threshold(ctypes.c_float(0.0)) == 0
