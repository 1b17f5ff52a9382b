"""Pins the WE oracles (C f64/f32, tiled torch, pure-Python brute force) without
a GPU: closed forms, invariants, the derivative identity that ties the cos/sin
sums to the embedding, the k -> 0 limit, and the committed golden fixture.
None of these tests re-types the oracle's formula: each checks it against
something the mathematics fixes independently."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import brute, c_oracle, torch_oracle


def _all_oracles(coords, wn, mask=None):
    """Every oracle flavour on the same input, as float64 numpy triples."""
    c = np.asarray(coords, np.float32)
    w = np.asarray(wn, np.float32)
    res = {}
    res["c_f64"] = c_oracle.we(c, w, mask, precision="f64")
    res["c_f32"] = tuple(a.astype(np.float64) for a in c_oracle.we(c, w, mask, precision="f32"))
    m = None if mask is None else torch.as_tensor(np.asarray(mask))
    res["torch_f64"] = tuple(a.numpy() for a in torch_oracle.we_torch(torch.from_numpy(c), torch.from_numpy(w), m, dtype=torch.float64))
    res["torch_f32"] = tuple(a.double().numpy() for a in torch_oracle.we_torch(torch.from_numpy(c), torch.from_numpy(w), m, dtype=torch.float32, row_chunk=5))
    return res


TOL = {"c_f64": 1e-12, "torch_f64": 1e-12, "c_f32": 2e-5, "torch_f32": 2e-5}


def test_two_points_closed_form():
    # N = 2 at distance r: out = [cos(kr)/r, sin(kr)/r], sums = [cos kr, sin kr], for both tokens
    r = 5.0
    coords = np.array([[[1.0, 2.0, 3.0], [1.0 + 3.0, 2.0 + 4.0, 3.0]]], np.float32)   # 3-4-5 triangle
    wn = np.array([0.3, 1.7, -0.9], np.float32)
    for name, (out, cs, ss) in _all_oracles(coords, wn).items():
        for i in range(2):
            for k, kv in enumerate(wn.astype(np.float64)):
                assert out[0, i, 2 * k] == pytest.approx(math.cos(kv * r) / r, abs=TOL[name] * 10), name
                assert out[0, i, 2 * k + 1] == pytest.approx(math.sin(kv * r) / r, abs=TOL[name] * 10), name
                assert cs[0, i, k] == pytest.approx(math.cos(kv * r), abs=TOL[name] * 10), name
                assert ss[0, i, k] == pytest.approx(math.sin(kv * r), abs=TOL[name] * 10), name


def test_lattice_closed_form():
    # tokens on a 1-D lattice with spacing a: token 0 sees distances a, 2a, ..., (N-1)a, so
    # cos_sums = Re sum_{m=1}^{N-1} e^{i k a m} = Re[ e^{ika} (1 - e^{ika(N-1)}) / (1 - e^{ika}) ]
    a, N = 2.0, 33
    coords = np.zeros((1, N, 3), np.float32)
    coords[0, :, 1] = a * np.arange(N)
    wn = np.array([0.37, 1.1], np.float32)
    for name, (out, cs, ss) in _all_oracles(coords, wn).items():
        for k, kv in enumerate(wn.astype(np.float64)):
            zeta = np.exp(1j * kv * a)
            geo = zeta * (1 - zeta ** (N - 1)) / (1 - zeta)
            assert cs[0, 0, k] == pytest.approx(geo.real, abs=TOL[name] * 50), name
            assert ss[0, 0, k] == pytest.approx(geo.imag, abs=TOL[name] * 50), name
            harm = sum(np.exp(1j * kv * a * m) / (a * m) for m in range(1, N))
            assert out[0, 0, 2 * k] == pytest.approx(harm.real, abs=TOL[name] * 50), name
            assert out[0, 0, 2 * k + 1] == pytest.approx(harm.imag, abs=TOL[name] * 50), name


def test_equilateral_triangle():
    s = 4.2
    coords = np.array([[[0, 0, 0], [s, 0, 0], [s / 2, s * math.sqrt(3) / 2, 0]]], np.float32)
    wn = np.array([0.8], np.float32)
    k = float(wn[0])
    for name, (out, cs, ss) in _all_oracles(coords, wn).items():
        for i in range(3):
            assert out[0, i, 0] == pytest.approx(2 * math.cos(k * s) / s, abs=1e-5), name
            assert out[0, i, 1] == pytest.approx(2 * math.sin(k * s) / s, abs=1e-5), name
            assert cs[0, i, 0] == pytest.approx(2 * math.cos(k * s), abs=1e-5), name


def _random_case(seed, Z=2, N=40, K=7, maskfrac=0.25):
    rng = np.random.default_rng(seed)
    coords = (rng.normal(size=(Z, N, 3)) * 12).astype(np.float32)
    wn = rng.normal(size=K).astype(np.float32)            # signed, like tests/wf_embed/wf_embed.py:24
    mask = rng.random((Z, N)) < maskfrac
    return coords, wn, mask


def test_oracles_agree_with_brute_force():
    coords, wn, mask = _random_case(3, Z=2, N=18, K=4)
    coords[0, 5] = coords[0, 11]          # coincident points
    ref = tuple(np.array(a) for a in brute.we_brute(coords.astype(np.float64).tolist(), wn.astype(np.float64).tolist(), mask.tolist()))
    for name, got in _all_oracles(coords, wn, mask).items():
        for g, r in zip(got, ref):
            assert np.abs(g - r).max() <= TOL[name] * 20 * max(1.0, np.abs(r).max()), name


def test_golden_fixture(golden_dir):
    g = np.load(os.path.join(golden_dir, "we_small.npz"))
    for name, got in _all_oracles(g["coords"], g["wavenumbers"], g["mask"]).items():
        for a, key in zip(got, ("out", "cos_sums", "sin_sums")):
            assert np.abs(a - g[key]).max() <= TOL[name] * 20 * max(1.0, np.abs(g[key]).max()), (name, key)
    # the fixture holds a coincident pair and padded tokens: their conventions are part of it
    assert (g["out"][1][g["mask"][1]] == 0).all() and (g["cos_sums"][1][g["mask"][1]] == 0).all()


def test_rigid_motion_invariance_and_permutation_equivariance():
    coords, wn, mask = _random_case(5)
    base = c_oracle.we(coords, wn, mask)
    rng = np.random.default_rng(0)
    q, _ = np.linalg.qr(rng.normal(size=(3, 3)))
    moved = (coords.astype(np.float64) @ q.T + np.array([3.0, -7.0, 11.0]))
    got = c_oracle.we(moved.astype(np.float32), wn, mask)
    for a, b in zip(base, got):
        assert np.abs(a - b).max() < 2e-4          # coordinates re-rounded to float32 after the motion
    perm = rng.permutation(coords.shape[1])
    gotp = c_oracle.we(coords[:, perm], wn, mask[:, perm])
    for a, b in zip(base, gotp):
        assert np.abs(a[:, perm] - b).max() < 1e-11


def test_mask_semantics():
    coords, wn, mask = _random_case(6, Z=1, N=30)
    out, cs, ss = c_oracle.we(coords, wn, mask)
    # a padded observer's rows are zero
    assert (out[0][mask[0]] == 0).all() and (cs[0][mask[0]] == 0).all() and (ss[0][mask[0]] == 0).all()
    # a padded source contributes nothing: same as removing it from the sequence
    keep = ~mask[0]
    out_c, cs_c, ss_c = c_oracle.we(coords[:, keep], wn, None)
    assert np.abs(out[0][keep] - out_c[0]).max() < 1e-12
    assert np.abs(cs[0][keep] - cs_c[0]).max() < 1e-12
    assert np.abs(ss[0][keep] - ss_c[0]).max() < 1e-12


def test_coincident_points_and_self_pair_are_dropped():
    coords = np.array([[[0, 0, 0], [0, 0, 0], [3, 4, 0]]], np.float32)
    wn = np.array([0.5], np.float32)
    out, cs, ss = c_oracle.we(coords, wn)
    # tokens 0 and 1 each see only token 2 (distance 5); token 2 sees both
    assert cs[0, 0, 0] == pytest.approx(math.cos(2.5)) and cs[0, 1, 0] == pytest.approx(math.cos(2.5))
    assert cs[0, 2, 0] == pytest.approx(2 * math.cos(2.5))
    assert out[0, 2, 1] == pytest.approx(2 * math.sin(2.5) / 5)


def test_small_wavenumber_limit():
    coords, _, mask = _random_case(7, Z=1, N=25)
    wn = np.array([1e-7], np.float32)
    out, cs, ss = c_oracle.we(coords, wn, mask)
    keep = ~mask[0]
    nvalid = keep.sum() - 1
    d = np.linalg.norm(coords[0][:, None].astype(np.float64) - coords[0][None].astype(np.float64), axis=-1)
    inv = np.where((d > 0) & keep[None, :], 1 / np.where(d > 0, d, 1), 0).sum(1)
    assert np.abs(cs[0][keep, 0] - nvalid).max() < 1e-9
    assert np.abs(out[0][keep, 0] - inv[keep]).max() < 1e-9
    assert np.abs(ss[0][keep, 0]).max() < 1e-3 and np.abs(out[0][keep, 1]).max() < 1e-4


def test_parity_of_wavenumber_sign():
    coords, wn, mask = _random_case(8)
    a = c_oracle.we(coords, wn, mask)
    b = c_oracle.we(coords, -wn, mask)
    assert np.abs(a[0][..., 0::2] - b[0][..., 0::2]).max() < 1e-12      # cos is even
    assert np.abs(a[0][..., 1::2] + b[0][..., 1::2]).max() < 1e-12      # sin is odd
    assert np.abs(a[1] - b[1]).max() < 1e-12 and np.abs(a[2] + b[2]).max() < 1e-12


def test_sums_are_the_wavenumber_derivative_of_the_embedding():
    # d out[i,2k]/dk = -sin_sums[i,k],  d out[i,2k+1]/dk = +cos_sums[i,k]
    # (the identity the analytical backward rests on, isotropic/cuda/wf_embedding.py:81)
    coords, wn, mask = _random_case(9, Z=1, N=20, K=3)
    wn = np.abs(wn) + 0.2
    _, cs, ss = c_oracle.we(coords, wn, mask)
    h = 1e-3
    hi = c_oracle.we(coords, (wn.astype(np.float64) + h).astype(np.float32), mask)[0]
    lo = c_oracle.we(coords, (wn.astype(np.float64) - h).astype(np.float32), mask)[0]
    step = (wn.astype(np.float64) + h).astype(np.float32).astype(np.float64) - (wn.astype(np.float64) - h).astype(np.float32).astype(np.float64)
    fd = (hi - lo) / np.repeat(step, 2)[None, None, :]
    assert np.abs(fd[..., 0::2] + ss).max() < 2e-3 * max(1, np.abs(ss).max())
    assert np.abs(fd[..., 1::2] - cs).max() < 2e-3 * max(1, np.abs(cs).max())


def test_backward_formula_matches_autograd():
    # what tests/wf_embed/wf_embed.py:60-79 checks: dk from the saved sums == autograd through the dense statement
    coords, wn, mask = _random_case(10, Z=2, N=16, K=5)
    c = torch.from_numpy(coords).double()
    w = torch.from_numpy(wn).double().requires_grad_(True)
    m = torch.from_numpy(mask)
    d = torch.sqrt(((c[:, :, None] - c[:, None]) ** 2).sum(-1))
    bad = m[:, :, None] | m[:, None, :] | (d == 0)
    mag = 1 / torch.where(bad, torch.full_like(d, float("inf")), d)
    ph = d[..., None] * w
    feats = torch.stack([(mag[..., None] * torch.cos(ph)).sum(2), (mag[..., None] * torch.sin(ph)).sum(2)], -1).flatten(2)
    dO = torch.from_numpy(np.random.default_rng(1).normal(size=tuple(feats.shape)))
    (feats * dO).sum().backward()
    _, cs, ss = torch_oracle.we_torch(c, w.detach(), m, dtype=torch.float64)
    dk = torch_oracle.we_backward_torch(dO, cs, ss)
    assert torch.allclose(dk, w.grad, rtol=1e-9, atol=1e-9)


def test_row_subset_equals_full():
    coords, wn, mask = _random_case(11, Z=2, N=50, K=4)
    full = c_oracle.we(coords, wn, mask, precision="f32")
    rows = np.array([0, 7, 49, 23], np.int32)
    sub = c_oracle.we(coords, wn, mask, rows=rows, precision="f32")
    for f, s in zip(full, sub):
        assert np.array_equal(f[:, rows], s)
    t = torch_oracle.we_torch(torch.from_numpy(coords), torch.from_numpy(wn), torch.from_numpy(mask), rows=rows.tolist())
    for f, s in zip(full, t):
        assert np.abs(f[:, rows] - s.numpy()).max() < 1e-4


@pytest.mark.parametrize("mag_type", [0, 2, 3])
def test_other_source_weights(mag_type):
    # two tokens 5 apart: closed form; then, on a random case, the identity the backward rests on for every
    # weight (sums = wavenumber derivative of the embedding), and agreement with the dense statement of
    # tests/wf_embed/wf_embed.py:108-116 written with torch
    weight = {0: lambda d: 1.0, 2: lambda d: 1 / math.log2(d), 3: lambda d: 1 / math.sqrt(d)}[mag_type]
    coords = np.array([[[0, 0, 0], [3, 4, 0]]], np.float32)
    wn = np.array([0.7], np.float32)
    out, cs, ss = c_oracle.we(coords, wn, mag_type=mag_type)
    kk = float(wn[0])
    assert out[0, 0, 0] == pytest.approx(weight(5.0) * math.cos(5 * kk), abs=1e-12)
    assert out[0, 1, 1] == pytest.approx(weight(5.0) * math.sin(5 * kk), abs=1e-12)
    assert cs[0, 0, 0] == pytest.approx(5 * weight(5.0) * math.cos(5 * kk), abs=1e-12)
    assert ss[0, 1, 0] == pytest.approx(5 * weight(5.0) * math.sin(5 * kk), abs=1e-12)

    coords, wn, mask = _random_case(20 + mag_type, Z=2, N=18, K=3)
    coords = coords * 2 + 0.0                     # keeps distances away from 1, where 1/log2 has its pole
    wn = (np.round((np.abs(wn) + 0.2) * 64) / 64).astype(np.float32)
    out, cs, ss = c_oracle.we(coords, wn, mask, mag_type=mag_type)
    h = np.float32(2.0 ** -14)
    fd = (c_oracle.we(coords, wn + h, mask, mag_type=mag_type)[0] - c_oracle.we(coords, wn - h, mask, mag_type=mag_type)[0]) / (2 * float(h))
    scale = max(1.0, np.abs(cs).max())
    assert np.abs(fd[..., 0::2] + ss).max() < 1e-5 * scale
    assert np.abs(fd[..., 1::2] - cs).max() < 1e-5 * scale

    c = torch.from_numpy(coords).double()
    d = torch.sqrt(((c[:, :, None] - c[:, None]) ** 2).sum(-1))
    m = torch.from_numpy(mask)
    bad = m[:, :, None] | m[:, None, :] | (d == 0)
    dd = torch.where(bad, torch.full_like(d, float("inf")), d)
    mag = {0: torch.where(bad, torch.zeros_like(d), torch.ones_like(d)), 2: 1 / torch.log2(dd), 3: 1 / torch.sqrt(dd)}[mag_type]
    ph = d[..., None] * torch.from_numpy(wn).double()
    feats = torch.stack([(mag[..., None] * torch.cos(ph)).sum(2), (mag[..., None] * torch.sin(ph)).sum(2)], -1).flatten(2)
    np.testing.assert_allclose(out, feats.numpy(), rtol=0, atol=1e-11)
