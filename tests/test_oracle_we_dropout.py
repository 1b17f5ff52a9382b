"""Pins the oracle of the WE forward's in-kernel dropout (oracle/we_oracle.c: we_oracle_hash5, we_oracle_dropout_keep,
we_oracle_dropout_f64) on the CPU.

hash5 is the reference's own function (isotropic/cuda/wf_embedding_kernel.cu:27-41: four multiply-add terms xor-ed
into the seed, then a mix that resembles MurmurHash3's 32-bit finalizer but has one more shift-xor before the second
multiply, so that finalizer's published known answers do NOT apply -- the first test shows the difference).  Its
constants and operation order are restated from the source; nothing but the reference's kernel, which is CUDA and does
not run here, could tell a typing slip in them: "parity unpinned" for the hash itself.  What is pinned around it:
  * the 32-bit wrap-around and the order of operations of the C restatement, against a second restatement on
    arbitrary-precision Python integers (masked to 32 bits by hand);
  * the keep test float(h) / float(UINT32_MAX) >= p, against exact rational arithmetic on the rounded float;
  * the sums, against the pinned oracle without dropout (p -> 0, and p so small that nothing is dropped), a pure-Python
    loop, the share of kept terms (a hash that mixes badly would miss it), independence of the four indices."""
import fractions
import math

import numpy as np
import pytest

from oracle import c_oracle

M32 = 0xffffffff
PRE = ((0x85ebca6b, 0x9e3779b9), (0xc2b2ae35, 0x165667b1), (0x27d4eb2f, 0xd6e8feb8), (0x85ebca6b, 0x1b873593))


def fmix32(h):                       # MurmurHash3's finalizer
    h ^= h >> 16
    h = (h * 0x85ebca6b) & M32
    h ^= h >> 13
    h = (h * 0xc2b2ae35) & M32
    h ^= h >> 16
    return h


def final_mix(h):                    # kernel.cu:36-40
    h = ((h ^ (h >> 16)) * 0x85ebca6b) & M32
    h ^= h >> 13
    h = ((h ^ (h >> 16)) * 0xc2b2ae35) & M32
    h ^= h >> 16
    return h


def hash5_python(a, b, c, d, seed):
    h = seed & M32
    for v, (mul, add) in zip((a, b, c, d), PRE):
        h ^= ((v & M32) * mul + add) & M32
    return final_mix(h)


def test_final_mix_is_not_murmur3_fmix32():
    # MurmurHash3_x86_32("", seed) = fmix32(seed): the published verification values hold for fmix32 ...
    assert fmix32(0) == 0 and fmix32(1) == 0x514E28B7 and fmix32(0xffffffff) == 0x81F16F39
    # ... and not for the reference's mix, which xors h >> 16 in once more (kernel.cu:38)
    assert final_mix(0) == 0 and final_mix(1) != 0x514E28B7 and final_mix(0xffffffff) != 0x81F16F39
    cancel = 0
    for _, add in PRE:
        cancel ^= add
    for seed in (0, 1, 0xffffffff, 0x12345678):
        assert c_oracle.we_hash5(0, 0, 0, 0, seed ^ cancel) == final_mix(seed)


def test_hash5_wraps_at_32_bits_like_arbitrary_precision_integers():
    rng = np.random.default_rng(0)
    for _ in range(2000):
        a, b, c, d = (int(x) for x in rng.integers(0, 70000, 4))
        seed = int(rng.integers(0, 2 ** 32))
        assert c_oracle.we_hash5(a, b, c, d, seed) == hash5_python(a, b, c, d, seed)
    # every index matters, and so does the seed
    base = c_oracle.we_hash5(3, 5, 7, 11, 13)
    assert len({base, c_oracle.we_hash5(4, 5, 7, 11, 13), c_oracle.we_hash5(3, 6, 7, 11, 13), c_oracle.we_hash5(3, 5, 8, 11, 13),
                c_oracle.we_hash5(3, 5, 7, 12, 13), c_oracle.we_hash5(3, 5, 7, 11, 14)}) == 6
    assert c_oracle.we_hash5(5, 3, 7, 11, 13) != base          # observer and batch index are not interchangeable


def test_keep_is_the_float_comparison_of_the_reference():
    # float(h): round to nearest even at 24 bits; float(UINT32_MAX) = 2^32; the quotient is exact
    def keep_exact(h, p):
        return fractions.Fraction(float(np.float32(h))) / 2 ** 32 >= fractions.Fraction(float(np.float32(p)))
    rng = np.random.default_rng(1)
    for p in (0.1, 0.25, 0.5, 0.9, 1e-6, 0.999999):
        for _ in range(300):
            z, i, j, k = (int(x) for x in rng.integers(0, 5000, 4))
            h = hash5_python(z, i, j, k, 99)
            assert c_oracle.we_dropout_keep(z, i, j, k, 99, p) == keep_exact(h, p)


def _inputs(seed=0, Z=2, N=37, K=6):
    rng = np.random.default_rng(seed)
    coords = np.cumsum(rng.normal(size=(Z, N, 3)) * 2.0, axis=1).astype(np.float32)
    wn = np.linspace(0.05, 2.0, K).astype(np.float32)
    mask = np.zeros((Z, N), bool)
    if Z > 1:
        mask[1, 29:] = True
    mask[0, 4] = True
    return coords, wn, mask


@pytest.mark.parametrize("mag_type", [0, 1, 2, 3])
def test_sums_against_a_pure_python_loop(mag_type):
    coords, wn, mask = _inputs()
    p, seed = 0.3, 12345
    out, cs, ss = c_oracle.we_dropout(coords, wn, mask, p, seed, mag_type=mag_type)
    Z, N, K = 2, 37, 6
    scale = 1.0 / (1.0 - float(np.float32(p)))
    for z in range(Z):
        for i in (0, 4, 5, 17, 36):
            want = np.zeros(2 * K)
            wc, wsn = np.zeros(K), np.zeros(K)
            if not mask[z, i]:
                for j in range(N):
                    if mask[z, j]:
                        continue
                    r = math.sqrt(sum((float(coords[z, i, c]) - float(coords[z, j, c])) ** 2 for c in range(3)))
                    if r == 0.0:
                        continue
                    m = (1.0, 1.0 / r, 1.0 / math.log2(r), 1.0 / math.sqrt(r))[mag_type]
                    for k in range(K):
                        h = hash5_python(z, i, j, k, seed)
                        if not (fractions.Fraction(float(np.float32(h))) / 2 ** 32 >= fractions.Fraction(float(np.float32(p)))):
                            continue
                        ph = r * float(wn[k])
                        want[2 * k] += math.cos(ph) * m * scale
                        want[2 * k + 1] += math.sin(ph) * m * scale
                        wc[k] += math.cos(ph) * m * r * scale
                        wsn[k] += math.sin(ph) * m * r * scale
            assert np.allclose(out[z, i], want, rtol=1e-12, atol=1e-12)
            assert np.allclose(cs[z, i], wc, rtol=1e-12, atol=1e-12) and np.allclose(ss[z, i], wsn, rtol=1e-12, atol=1e-12)


def test_no_dropout_limit_and_share_of_kept_terms():
    coords, wn, mask = _inputs(seed=3, Z=1, N=300, K=8)
    mask[:] = False
    plain = c_oracle.we(coords, wn, mask)
    # p = 0 and a p below every hash value's quotient (2^-33 rounds the test to "always"): the pinned oracle itself
    for p in (0.0, 2.0 ** -40):
        got = c_oracle.we_dropout(coords, wn, mask, p, 7)
        for a, b in zip(got, plain):
            assert np.allclose(a, b, rtol=1e-12, atol=1e-10)
    # zero wavenumber: cos = 1, so cos_sums / scale counts the kept partners of a row: a share 1 - p of N - 1, and
    # different seeds drop different terms
    w0 = np.zeros(1, np.float32)
    for p in (0.2, 0.5, 0.8):
        _, cs, _ = c_oracle.we_dropout(coords, w0, mask, p, 2024)
        kept = cs[0, :, 0] * (1.0 - float(np.float32(p)))
        assert np.allclose(kept, np.round(kept), atol=1e-9)
        share = kept.sum() / (300 * 299)
        assert abs(share - (1 - p)) < 4 * math.sqrt(p * (1 - p) / (300 * 299)) + 1e-3
        _, cs2, _ = c_oracle.we_dropout(coords, w0, mask, p, 2025)
        assert not np.array_equal(cs, cs2)
    # the expectation over seeds is the embedding without dropout
    ref = c_oracle.we(coords[:, :60], wn, None)[0]
    acc = np.zeros_like(ref)
    n = 200
    for s in range(n):
        acc += c_oracle.we_dropout(coords[:, :60], wn, None, 0.5, 1000 + s)[0]
    assert np.abs(acc / n - ref).max() < 6 * np.abs(ref).max() / math.sqrt(n)
