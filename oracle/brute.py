"""TEST INFRASTRUCTURE. Pure-Python float64 loops for tiny inputs.

Independent of numpy/torch vectorisation and of the C oracle: one scalar
statement per formula, used to pin the other oracles and to write the
fixtures under tests/golden/.
"""
import math


def we_brute(coords, wavenumbers, mask=None):
    """coords: Z x N x 3 nested lists; wavenumbers: list; mask: Z x N of bool.

    out[z][i][2k] = sum_j cos(k r)/r, out[z][i][2k+1] = sum_j sin(k r)/r,
    cs[z][i][k] = sum_j cos(k r), ss[z][i][k] = sum_j sin(k r), over j with
    neither i nor j padded and r != 0 (tests/wf_embed/wf_embed.py:100-127,
    isotropic/cuda/wf_embedding_kernel.cu:187,224-238).
    """
    Z, N, K = len(coords), len(coords[0]), len(wavenumbers)
    out = [[[0.0] * (2 * K) for _ in range(N)] for _ in range(Z)]
    cs = [[[0.0] * K for _ in range(N)] for _ in range(Z)]
    ss = [[[0.0] * K for _ in range(N)] for _ in range(Z)]
    for z in range(Z):
        for i in range(N):
            if mask is not None and mask[z][i]:
                continue
            for j in range(N):
                if mask is not None and mask[z][j]:
                    continue
                r = math.sqrt(sum((coords[z][i][c] - coords[z][j][c]) ** 2 for c in range(3)))
                if r == 0.0:
                    continue
                for k in range(K):
                    ph = r * wavenumbers[k]
                    out[z][i][2 * k] += math.cos(ph) / r
                    out[z][i][2 * k + 1] += math.sin(ph) / r
                    cs[z][i][k] += math.cos(ph)
                    ss[z][i][k] += math.sin(ph)
    return out, cs, ss


def we_aniso_brute(coordsA, coordsB, cb_magnitudes, wavenumbers, mask=None):
    """coordsA, coordsB: Z x N x 3 nested lists; cb_magnitudes, wavenumbers: lists; mask: Z x N of bool.

    Per pair: R = a_i - a_j, r = |R|, A = (b_j . R)/r, u = r - cb_k A, phase = u k_k
    (tests/wf_embed/wf_embed_aniso_learnCB_learnK.py:127-149); out as in we_brute; the partials are
    those of .../cb_scaling/learnable_wavenumbers/cuda/wf_embedding_kernel.cu:187-194.
    Returns (out, d_cb, d_k), each Z x N x 2K.
    """
    Z, N, K = len(coordsA), len(coordsA[0]), len(wavenumbers)
    out = [[[0.0] * (2 * K) for _ in range(N)] for _ in range(Z)]
    d_cb = [[[0.0] * (2 * K) for _ in range(N)] for _ in range(Z)]
    d_k = [[[0.0] * (2 * K) for _ in range(N)] for _ in range(Z)]
    for z in range(Z):
        for i in range(N):
            if mask is not None and mask[z][i]:
                continue
            for j in range(N):
                if mask is not None and mask[z][j]:
                    continue
                R = [coordsA[z][i][c] - coordsA[z][j][c] for c in range(3)]
                r = math.sqrt(sum(x * x for x in R))
                if r == 0.0:
                    continue
                A = sum(R[c] * coordsB[z][j][c] for c in range(3)) / r
                for k in range(K):
                    u = r - cb_magnitudes[k] * A
                    ph = u * wavenumbers[k]
                    real, imag = math.cos(ph) / r, math.sin(ph) / r
                    out[z][i][2 * k] += real
                    out[z][i][2 * k + 1] += imag
                    d_k[z][i][2 * k] += -imag * u
                    d_k[z][i][2 * k + 1] += real * u
                    d_cb[z][i][2 * k] += imag * wavenumbers[k] * A
                    d_cb[z][i][2 * k + 1] += -real * wavenumbers[k] * A
    return out, d_cb, d_k


def geo_attn_brute(Q, K, V, coords, sigma, key_padding_mask=None):
    """Q,K,V: Z x H x N x d nested lists. Returns (O, L) nested lists.

    s_ij = (q_i.k_j)/sqrt(d) * (1 + exp(-|ri-rj|^2/(2 sigma_h^2)))   README.md:40,
    scale before the factor (old/old_scripts/attn/geometric_attn.py:186,201);
    padded query or key -> -inf (:196); empty row -> O = 0, L = -inf (:233-236).
    """
    Z, H, N, d = len(Q), len(Q[0]), len(Q[0][0]), len(Q[0][0][0])
    O = [[[[0.0] * d for _ in range(N)] for _ in range(H)] for _ in range(Z)]
    L = [[[-math.inf] * N for _ in range(H)] for _ in range(Z)]
    for z in range(Z):
        for h in range(H):
            for i in range(N):
                if key_padding_mask is not None and key_padding_mask[z][i]:
                    continue
                s = []
                for j in range(N):
                    if key_padding_mask is not None and key_padding_mask[z][j]:
                        s.append(-math.inf)
                        continue
                    dot = sum(Q[z][h][i][t] * K[z][h][j][t] for t in range(d)) / math.sqrt(d)
                    d2 = sum((coords[z][i][c] - coords[z][j][c]) ** 2 for c in range(3))
                    s.append(dot * (1.0 + math.exp(-d2 / (2.0 * sigma[h] ** 2))))
                mx = max(s)
                if mx == -math.inf:
                    continue
                p = [math.exp(v - mx) if v != -math.inf else 0.0 for v in s]
                l = sum(p)
                for t in range(d):
                    O[z][h][i][t] = sum(p[j] * V[z][h][j][t] for j in range(N)) / l
                L[z][h][i] = mx + math.log(l)
    return O, L
