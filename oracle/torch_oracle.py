"""TEST INFRASTRUCTURE. The reference's CPU PyTorch path, restated and tiled.

Not part of the product.  These are the functions whose time on the host
cores is reported as the CPU baseline, and the fp32 checker of the parity
tests.  Rows (observers / queries) are processed in chunks so temporaries stay
bounded; rows are independent in both algorithms.
"""
import math

import torch


def we_torch(coords, wavenumbers, mask=None, rows=None, row_chunk=None, dtype=torch.float32,
             max_temp_bytes=1 << 30):
    """Isotropic wavefunction embedding, magnitude 1/|r|.

    Follows tests/wf_embed/wf_embed.py:91-129 (wf_embedding_torch, mag_type 1):
    dists = sqrt(sum((ci - cj)^2)); phases = dists*k; masked = mi | mj | dists==0;
    magnitudes = 1/where(masked, inf, dists); real/imag = magnitudes*cos/sin(phases);
    sum over sources; features = stack([real, imag], -1).view(Z, N, 2K).
    The cos/sin sums follow isotropic/cuda/wf_embedding_kernel.cu:224-238
    (warp_sum(real*dists)): sum over unmasked pairs of cos(phase), sin(phase).

    coords [Z,N,3], wavenumbers [K], mask [Z,N] bool (True = padded).
    Returns (out [Z,R,2K], cos_sums [Z,R,K], sin_sums [Z,R,K]).
    """
    coords = coords.to(dtype)
    wavenumbers = wavenumbers.to(dtype)
    Z, N, _ = coords.shape
    K = wavenumbers.shape[0]
    mask = torch.zeros(Z, N, dtype=torch.bool) if mask is None else mask.bool()
    rows_t = torch.arange(N) if rows is None else torch.as_tensor(rows, dtype=torch.long)
    R = rows_t.numel()
    if row_chunk is None:
        per_row = N * K * coords.element_size() * 4
        row_chunk = max(1, min(R, max_temp_bytes // max(per_row, 1)))
    out = torch.zeros(Z, R, 2 * K, dtype=dtype)
    cs = torch.zeros(Z, R, K, dtype=dtype)
    ss = torch.zeros(Z, R, K, dtype=dtype)
    for z in range(Z):
        cz, mz = coords[z], mask[z]
        for a in range(0, R, row_chunk):
            idx = rows_t[a:a + row_chunk]
            ci = cz[idx]                                                     # r x 3
            dists = torch.sqrt(torch.sum((ci[:, None, :] - cz[None, :, :]) ** 2, dim=2))   # r x N
            phases = dists[:, :, None] * wavenumbers[None, None, :]          # r x N x K
            m = mz[idx][:, None] | mz[None, :] | (dists == 0)                # r x N
            mag = 1 / torch.where(m, torch.full_like(dists, float("inf")), dists)
            valid = (~m).to(dtype)
            cosp, sinp = torch.cos(phases), torch.sin(phases)
            real = (mag[:, :, None] * cosp).sum(dim=1)
            imag = (mag[:, :, None] * sinp).sum(dim=1)
            out[z, a:a + idx.numel()] = torch.stack([real, imag], dim=-1).view(idx.numel(), 2 * K)
            cs[z, a:a + idx.numel()] = (valid[:, :, None] * cosp).sum(dim=1)
            ss[z, a:a + idx.numel()] = (valid[:, :, None] * sinp).sum(dim=1)
    return out, cs, ss


def we_aniso_torch(coordsA, coordsB, cb_magnitudes, wavenumbers, mask=None, dtype=torch.float64):
    """Anisotropic (C-beta scaled) wavefunction embedding, dense and differentiable in cb_magnitudes
    and wavenumbers.

    Follows tests/wf_embed/wf_embed_aniso_learnCB_learnK.py:117-163 (wf_embedding_torch):
    R = a_i - a_j; R_unit = R/|R| (0 where |R| = 0); distsB = R_unit . (b_j cb_k);
    phases = (|R| - distsB) k; masked = m_i | m_j | |R| == 0; magnitudes = 1/where(masked, inf, |R|);
    features = stack([sum_j mag cos, sum_j mag sin], -1).view(Z, N, 2K).
    """
    a = coordsA.to(dtype)
    b = coordsB.to(dtype)
    cb = cb_magnitudes.to(dtype)
    wn = wavenumbers.to(dtype)
    Z, N, _ = a.shape
    K = wn.shape[0]
    mask = torch.zeros(Z, N, dtype=torch.bool) if mask is None else mask.bool()
    R = a[:, :, None, :] - a[:, None, :, :]                                   # Z x N x N x 3
    R_norm = torch.linalg.vector_norm(R, dim=3, keepdim=True)                 # Z x N x N x 1
    R_unit = R / torch.where(R_norm == 0, torch.full_like(R_norm, float("inf")), R_norm)
    b_scaled = b[:, :, None, :] * cb[None, None, :, None]                     # Z x N x K x 3
    distsB = torch.sum(R_unit[:, :, :, None, :] * b_scaled[:, None, :, :, :], dim=4)   # Z x N x N x K
    phases = (R_norm - distsB) * wn[None, None, None, :]
    m = mask[:, :, None, None] | mask[:, None, :, None] | (R_norm == 0)
    mag = 1 / torch.where(m, torch.full_like(R_norm, float("inf")), R_norm)
    real = (mag * torch.cos(phases)).sum(dim=2)
    imag = (mag * torch.sin(phases)).sum(dim=2)
    return torch.stack([real, imag], dim=-1).view(Z, N, 2 * K)


def we_aniso_backward_torch(dO, d_cb, d_k):
    """anisotropic/cb_scaling/learnable_wavenumbers/cuda/wf_embedding.py:65-79: contract the per-token
    partial derivatives with dO over batch and tokens, then add the real and imaginary halves."""
    g_cb = (dO * d_cb).sum(dim=(0, 1))
    g_k = (dO * d_k).sum(dim=(0, 1))
    return g_cb[0::2] + g_cb[1::2], g_k[0::2] + g_k[1::2]


def we_backward_torch(dO, cos_sums, sin_sums):
    """d(loss)/d(wavenumbers): isotropic/cuda/wf_embedding.py:64-83."""
    real_dO = dO[:, :, 0::2]
    imag_dO = dO[:, :, 1::2]
    return ((imag_dO * cos_sums) - (real_dO * sin_sums)).sum(dim=(0, 1))


def geo_attn_torch(Q, K, V, coords, sigma, key_padding_mask=None, rows=None, row_chunk=None,
                   dtype=torch.float32, max_temp_bytes=1 << 30):
    """RBF-scaled attention with the multiplier of README.md:40.

    Dense structure of tests/attn/geo_attn.py:194-210 (S = QK^T/sqrt(d); dists;
    rbfs = exp(-d^2/(2 sigma^2)); masked -> -inf; softmax; P V), with the logits
    S*(1+rbf) and the conventions of old/old_scripts/attn/geometric_attn.py:
    both padded queries and padded keys are masked (:196), a row without valid
    keys gives O = 0 (:233) and L = -inf (:236).

    Q,K,V [Z,H,N,d]; coords [Z,N,3]; sigma [H]; key_padding_mask [Z,N] bool.
    Returns (O [Z,H,R,d], L [Z,H,R]).
    """
    Q, K, V = Q.to(dtype), K.to(dtype), V.to(dtype)
    coords, sigma = coords.to(dtype), sigma.to(dtype)
    Z, H, N, d = Q.shape
    mask = torch.zeros(Z, N, dtype=torch.bool) if key_padding_mask is None else key_padding_mask.bool()
    rows_t = torch.arange(N) if rows is None else torch.as_tensor(rows, dtype=torch.long)
    R = rows_t.numel()
    if row_chunk is None:
        per_row = H * N * Q.element_size() * 4
        row_chunk = max(1, min(R, max_temp_bytes // max(per_row, 1)))
    O = torch.zeros(Z, H, R, d, dtype=dtype)
    L = torch.full((Z, H, R), float("-inf"), dtype=dtype)
    for z in range(Z):
        for a in range(0, R, row_chunk):
            idx = rows_t[a:a + row_chunk]
            S = torch.matmul(Q[z][:, idx, :], K[z].transpose(1, 2)) / math.sqrt(d)      # H x r x N
            d2 = torch.sum((coords[z][idx][:, None, :] - coords[z][None, :, :]) ** 2, dim=2)   # r x N
            rbf = torch.exp(-d2[None] / (2 * sigma[:, None, None] ** 2))                # H x r x N
            am = (mask[z][idx][:, None] | mask[z][None, :])[None]                       # 1 x r x N
            S = torch.where(am, torch.full_like(S, float("-inf")), S * (1 + rbf))
            Lz = torch.logsumexp(S, dim=-1)                                             # -inf for empty rows
            P = torch.softmax(S, dim=-1)
            P = torch.where(torch.isnan(P), torch.zeros_like(P), P)                     # empty rows -> 0
            O[z][:, a:a + idx.numel()] = torch.matmul(P, V[z])
            L[z][:, a:a + idx.numel()] = Lz
    return O, L


def geo_attn_legacy_torch(Q, K, V, coords, spreads, b, mask=None, min_rbf=0.0, max_rbf=1.0, dtype=torch.float32):
    """The reference's dense statement of its own kernel, line for line in meaning
    (tests/attn/geo_attn.py:172-212, torch_attn): S = QK^T/sqrt(d); dists; rbfs = exp(-dists^2/(2 spreads^2));
    attn_mask = mask_i | mask_j | rbfs < min_rbf | rbfs > max_rbf; rbfs = 2(rbfs-min)/(max-min) - 1;
    S = where(attn_mask, -inf, S + b*rbfs*|S|); softmax; P V.  Fully masked rows are returned as zeros
    (the kernel's convention, old/old_scripts/attn/geometric_attn.py:233) instead of NaN."""
    Q, K, V = Q.to(dtype), K.to(dtype), V.to(dtype)
    coords, spreads, b = coords.to(dtype), spreads.to(dtype), b.to(dtype)
    Z, H, N, d = Q.shape
    mask = torch.zeros(Z, N, dtype=torch.bool) if mask is None else mask.bool()
    S = torch.matmul(Q, K.transpose(2, 3)) / math.sqrt(d)
    dists = torch.sqrt(torch.sum((coords[:, :, None, :] - coords[:, None, :, :]) ** 2, dim=3))[:, None, :, :]
    rbfs = torch.exp(-(dists ** 2) / (2 * (spreads[None, :, None, None] ** 2)))
    attn_mask = mask[:, None, :, None] | mask[:, None, None, :] | (rbfs < min_rbf) | (rbfs > max_rbf)
    rbfs = (2 * (rbfs - min_rbf) / (max_rbf - min_rbf)) - 1
    S = torch.where(attn_mask, torch.full_like(S, float("-inf")), S + b[None, :, None, None] * rbfs * torch.abs(S))
    P = torch.softmax(S, dim=-1)
    P = torch.where(torch.isnan(P), torch.zeros_like(P), P)
    return torch.matmul(P, V), torch.logsumexp(S, dim=-1)


def geo_attn_autograd_torch(Q, K, V, coords, sigma, key_padding_mask=None, betas=None, min_rbf=0.0, max_rbf=1.0,
                            dtype=torch.float64):
    """The dense statements above in a form torch.autograd can differentiate in Q, K, V, sigma and betas
    (the oracle of the backward kernel: nothing of the hand-derived gradient formulas enters here).
    betas=None: logits S*(1+rbf); otherwise the reference's S + b*rbf_norm*|S| with its pair mask.
    Rows without any unmasked pair give O = 0 and pass no gradient.
    sigma (and betas) may also be given per query row, [Z,H,N]: the gradient with respect to such a tensor is the
    contribution of every query row to the per-head gradient (their sum over Z and N), which tells how much of
    the per-head number is left after cancellation."""
    Q, K, V = Q.to(dtype), K.to(dtype), V.to(dtype)
    coords, sigma = coords.to(dtype), sigma.to(dtype)
    Z, H, N, d = Q.shape
    mask = torch.zeros(Z, N, dtype=torch.bool) if key_padding_mask is None else key_padding_mask.bool()
    S = torch.matmul(Q, K.transpose(2, 3)) / math.sqrt(d)
    d2 = torch.sum((coords[:, :, None, :] - coords[:, None, :, :]) ** 2, dim=3)[:, None, :, :]
    sg = sigma[:, :, :, None] if sigma.dim() == 3 else sigma[None, :, None, None]
    rbf = torch.exp(-d2 / (2 * sg ** 2))
    am = (mask[:, None, :, None] | mask[:, None, None, :]).expand(Z, H, N, N)
    if betas is None:
        T = S * (1 + rbf)
    else:
        am = am | (rbf < min_rbf) | (rbf > max_rbf)
        bt = betas.to(dtype)
        bt = bt[:, :, :, None] if bt.dim() == 3 else bt[None, :, None, None]
        T = S + bt * ((2 * (rbf - min_rbf) / (max_rbf - min_rbf)) - 1) * torch.abs(S)
    T = torch.where(am, torch.full_like(T, float("-inf")), T)
    row_any = (~am).any(dim=-1, keepdim=True)
    T = torch.where(row_any, T, torch.zeros_like(T))
    P = torch.softmax(T, dim=-1) * row_any.to(dtype)
    return torch.matmul(P, V)


def geo_attn_scalar_grad_mass(Q, K, V, dO, coords, sigma, key_padding_mask=None, betas=None, min_rbf=0.0, max_rbf=1.0,
                              dtype=torch.float64):
    """Scale of the rounding error of d_sigma and d_beta: (mass_sigma [H], mass_beta [H] | None, and the same two
    sums with their signs kept, which are the gradients themselves and pin the terms against torch.autograd).

    Both gradients are sums over the pairs of P (dP - D) dT/d(sigma | beta), dP = dO . V, D = sum_j P dP, in which dP
    and D largely cancel (exactly, for a query with one surviving pair).  A kernel whose P, dP or D carry a relative
    error eps leaves about eps times
        mass = sum_pairs P (|dP| + |D|) |dT/d(sigma | beta)|
    however small the gradient itself comes out; tests hold the kernel to a fraction of this mass.  It is a bound on
    magnitudes only; GPU tests take no gradient value from it (tests/test_oracle_attn.py checks the signed sums of the
    same terms against autograd through geo_attn_autograd_torch).
    Logits as in geo_attn_autograd_torch (old/old_scripts/attn/geometric_attn.py:193-201 with betas, README.md:40 without)."""
    Q, K, V, dO = Q.to(dtype), K.to(dtype), V.to(dtype), dO.to(dtype)
    coords, sigma = coords.to(dtype), sigma.to(dtype)
    Z, H, N, d = Q.shape
    mask = torch.zeros(Z, N, dtype=torch.bool) if key_padding_mask is None else key_padding_mask.bool()
    S = torch.matmul(Q, K.transpose(2, 3)) / math.sqrt(d)
    d2 = torch.sum((coords[:, :, None, :] - coords[:, None, :, :]) ** 2, dim=3)[:, None, :, :]
    sg = sigma[None, :, None, None]
    rbf = torch.exp(-d2 / (2 * sg ** 2))
    drbf = rbf * d2 / sg ** 3                                   # d rbf / d sigma
    am = (mask[:, None, :, None] | mask[:, None, None, :]).expand(Z, H, N, N)
    if betas is None:
        T = S * (1 + rbf)
        w_sigma, w_beta = S * drbf, None
    else:
        am = am | (rbf < min_rbf) | (rbf > max_rbf)
        bt = betas.to(dtype)[None, :, None, None]
        rn = (2 * (rbf - min_rbf) / (max_rbf - min_rbf)) - 1
        T = S + bt * rn * S.abs()
        w_sigma, w_beta = bt * (2 / (max_rbf - min_rbf)) * drbf * S.abs(), rn * S.abs()
    T = torch.where(am, torch.full_like(T, float("-inf")), T)
    row_any = (~am).any(dim=-1, keepdim=True)
    T = torch.where(row_any, T, torch.zeros_like(T))
    P = torch.softmax(T, dim=-1) * row_any.to(dtype)
    dP = torch.matmul(dO, V.transpose(2, 3))
    D = (P * dP).sum(dim=-1, keepdim=True)
    spread, signed = P * (dP.abs() + D.abs()), P * (dP - D)
    mass_sigma, total_sigma = (spread * w_sigma.abs()).sum(dim=(0, 2, 3)), (signed * w_sigma).sum(dim=(0, 2, 3))
    if w_beta is None:
        return mass_sigma, None, total_sigma, None
    return mass_sigma, (spread * w_beta.abs()).sum(dim=(0, 2, 3)), total_sigma, (signed * w_beta).sum(dim=(0, 2, 3))


def geo_attn_backward_tiled_torch(Q, K, V, dO, coords, sigma, key_padding_mask=None, row_chunk=2048, dtype=torch.float64):
    """Gradients of the README-logit attention at sizes where the dense N x N statement does not fit: the hand-derived
    formulas of old/old_scripts/attn/geometric_attn.py:448-505 with t = S (1 + rbf), evaluated over chunks of query rows
        P = softmax(t); dP = dO V^T; D = sum_j P dP; dt = P (dP - D); dS = dt (1 + rbf)
        dQ = dS K / sqrt(d); dK = dS^T Q / sqrt(d); dV = P^T dO; d sigma_h = sum dt S rbf d^2 / sigma_h^3
    Not a second source of truth: tests/test_oracle_attn.py pins it to torch.autograd through
    geo_attn_autograd_torch.  Also returns the pair mass of d sigma (see geo_attn_scalar_grad_mass).

    Q, K, V, dO [Z,H,N,d]; coords [Z,N,3]; sigma [H]; mask [Z,N] bool.  Returns (dQ, dK, dV, d_sigma [H], mass_sigma [H])."""
    Q, K, V, dO = Q.to(dtype), K.to(dtype), V.to(dtype), dO.to(dtype)
    coords, sigma = coords.to(dtype), sigma.to(dtype)
    Z, H, N, d = Q.shape
    mask = torch.zeros(Z, N, dtype=torch.bool) if key_padding_mask is None else key_padding_mask.bool()
    dQ, dK, dV = torch.zeros_like(Q), torch.zeros_like(K), torch.zeros_like(V)
    d_sigma, mass = torch.zeros(H, dtype=dtype), torch.zeros(H, dtype=dtype)
    isd = 1.0 / math.sqrt(d)
    sg = sigma[:, None, None]
    for z in range(Z):
        for a in range(0, N, row_chunk):
            r = slice(a, min(a + row_chunk, N))
            S = torch.matmul(Q[z][:, r], K[z].transpose(1, 2)) * isd                        # H x r x N
            d2 = torch.sum((coords[z][r][:, None, :] - coords[z][None, :, :]) ** 2, dim=2)[None]
            rbf = torch.exp(-d2 / (2 * sg ** 2))
            am = (mask[z][r][:, None] | mask[z][None, :])[None].expand_as(S)
            T = torch.where(am, torch.full_like(S, float("-inf")), S * (1 + rbf))
            row_any = (~am).any(dim=-1, keepdim=True)
            T = torch.where(row_any, T, torch.zeros_like(T))
            P = torch.softmax(T, dim=-1) * row_any.to(dtype)
            dP = torch.matmul(dO[z][:, r], V[z].transpose(1, 2))
            Dr = (P * dP).sum(dim=-1, keepdim=True)
            dT = P * (dP - Dr)
            dS = dT * (1 + rbf)
            dQ[z][:, r] = torch.matmul(dS, K[z]) * isd
            dK[z] += torch.matmul(dS.transpose(1, 2), Q[z][:, r]) * isd
            dV[z] += torch.matmul(P.transpose(1, 2), dO[z][:, r])
            w = S * rbf * d2 / sg ** 3
            d_sigma += (dT * w).sum(dim=(1, 2))
            mass += (P * (dP.abs() + Dr.abs()) * w.abs()).sum(dim=(1, 2))
    return dQ, dK, dV, d_sigma, mass


def encoder_forward_torch(params, min_spread, coords, tokens, mask, attention=None):
    """The encoder stack in fp32 on the CPU with the oracles in place of the kernels: WE(coords) + embedding[tokens],
    then per layer geometric multi-head attention on the projections of x (per-head [d_model, d_k] weights and
    [d_k] biases, sigma = min_spread + exp(w)), output projection, residual + LayerNorm, FFN (GELU), residual +
    LayerNorm (old/old_scripts/encoder.py:33-41 and :88-89, old/old_scripts/attn/geometric_attn.py:625-655), and a
    linear head.

    params: state dict of the module (name -> tensor), any dtype; min_spread: float; attention: the attention oracle
    to use, (Q, K, V, coords, sigma, mask) -> O [Z,H,N,d] (default: geo_attn_torch)."""
    import torch.nn.functional as F
    p = {k: v.detach().cpu().float() for k, v in params.items()}
    if attention is None:
        def attention(Q, K, V, c, sg, m):
            return geo_attn_torch(Q, K, V, c, sg, m)[0]
    wf, _, _ = we_torch(coords, torch.exp(p["wf_embedding.wavenumbers"]), mask)
    x = wf + p["aa_embedding.weight"][tokens]
    layers = 1 + max(int(k.split(".")[1]) for k in p if k.startswith("layers."))
    for i in range(layers):
        pre = f"layers.{i}."
        Q, K, V = (torch.matmul(x.unsqueeze(1), p[pre + f"attn.{n}_proj"].unsqueeze(0)) + p[pre + f"attn.{n}_bias"][None, :, None]
                   for n in ("q", "k", "v"))
        O = attention(Q, K, V, coords, min_spread + torch.exp(p[pre + "attn.spread_weights"]), mask)
        Z, H, N, d = O.shape
        a = O.permute(0, 2, 3, 1).reshape(Z, N, H * d) @ p[pre + "attn.out_proj.weight"].T
        x = F.layer_norm(x + a, (x.shape[-1],), p[pre + "attn_norm.weight"], p[pre + "attn_norm.bias"])
        f = F.gelu(x @ p[pre + "ffn.in_proj.weight"].T + p[pre + "ffn.in_proj.bias"]) @ p[pre + "ffn.out_proj.weight"].T \
            + p[pre + "ffn.out_proj.bias"]
        x = F.layer_norm(x + f, (x.shape[-1],), p[pre + "ffn_norm.weight"], p[pre + "ffn_norm.bias"])
    return x @ p["head.weight"].T + p["head.bias"]
