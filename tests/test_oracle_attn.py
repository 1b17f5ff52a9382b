"""Pins the geometric-attention oracles without a GPU: reductions to
torch.nn.functional.scaled_dot_product_attention, brute force, invariants and
the committed golden fixture."""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import brute, c_oracle, torch_oracle


def _case(seed, Z=2, H=3, N=37, d=64, maskfrac=0.0):
    g = torch.Generator().manual_seed(seed)
    Q = torch.randn(Z, H, N, d, generator=g).bfloat16().float()
    K = torch.randn(Z, H, N, d, generator=g).bfloat16().float()
    V = torch.randn(Z, H, N, d, generator=g).bfloat16().float()
    coords = torch.cumsum(torch.randn(Z, N, 3, generator=g) * 2.2, dim=1)
    sigma = torch.linspace(3.0, 25.0, H)
    mask = (torch.rand(Z, N, generator=g) < maskfrac) if maskfrac > 0 else None
    return Q, K, V, coords, sigma, mask


def _both(Q, K, V, coords, sigma, mask):
    o1, l1 = c_oracle.geo_attn(Q.numpy(), K.numpy(), V.numpy(), coords.numpy(), sigma.numpy(), None if mask is None else mask.numpy())
    o2, l2 = torch_oracle.geo_attn_torch(Q, K, V, coords, sigma, mask, dtype=torch.float64)
    o3, l3 = torch_oracle.geo_attn_torch(Q, K, V, coords, sigma, mask, dtype=torch.float32, row_chunk=7)
    return {"c_f64": (o1, l1), "torch_f64": (o2.numpy(), l2.numpy()), "torch_f32": (o3.double().numpy(), l3.double().numpy())}


TOL = {"c_f64": 1e-11, "torch_f64": 1e-11, "torch_f32": 5e-5}


def test_flat_multiplier_reduces_to_sdpa():
    # all coordinates identical, or sigma -> infinity: multiplier == 2 -> plain attention with scale 2/sqrt(d)
    Q, K, V, coords, sigma, _ = _case(1)
    ref = F.scaled_dot_product_attention(Q.double(), K.double(), V.double(), scale=2 / math.sqrt(64)).numpy()
    for variant in ("same_coords", "huge_sigma"):
        c = torch.zeros_like(coords) + 5.0 if variant == "same_coords" else coords
        s = sigma if variant == "same_coords" else torch.full_like(sigma, 1e7)
        for name, (O, L) in _both(Q, K, V, c, s, None).items():
            assert np.abs(O - ref).max() < TOL[name] * 100, (variant, name)


def test_far_apart_small_sigma_reduces_to_diagonal_boost():
    # points >> sigma apart: multiplier 1 off the diagonal, 2 on it -> SDPA with an additive diagonal bias of S_ii
    Q, K, V, coords, sigma, _ = _case(2, Z=1, H=2, N=19)
    coords = (torch.arange(19, dtype=torch.float32)[None, :, None] * torch.tensor([100.0, 0.0, 0.0]))
    sigma = torch.tensor([0.5, 1.0])
    S = torch.matmul(Q.double(), K.double().transpose(2, 3)) / 8
    bias = torch.diag_embed(torch.diagonal(S, dim1=2, dim2=3))
    ref = F.scaled_dot_product_attention(Q.double(), K.double(), V.double(), attn_mask=bias).numpy()
    for name, (O, L) in _both(Q, K, V, coords, sigma, None).items():
        assert np.abs(O - ref).max() < TOL[name] * 100, name


def test_key_mask_reduces_to_sdpa_mask():
    Q, K, V, coords, sigma, mask = _case(3, maskfrac=0.3)
    s = torch.full_like(sigma, 1e7)
    am = (~mask)[:, None, None, :].expand(-1, Q.shape[1], Q.shape[2], -1)
    ref = F.scaled_dot_product_attention(Q.double(), K.double(), V.double(), attn_mask=am, scale=2 / 8).numpy()
    for name, (O, L) in _both(Q, K, V, coords, s, mask).items():
        valid_q = ~mask.numpy()
        for z in range(Q.shape[0]):
            assert np.abs(O[z][:, valid_q[z]] - ref[z][:, valid_q[z]]).max() < TOL[name] * 100, name
            # padded queries: O = 0, L = -inf (old/old_scripts/attn/geometric_attn.py:196,233-236)
            assert (O[z][:, ~valid_q[z]] == 0).all() and np.isneginf(L[z][:, ~valid_q[z]]).all(), name


def test_brute_force_and_golden(golden_dir):
    g = np.load(os.path.join(golden_dir, "geo_attn_small.npz"))
    t = {k: torch.from_numpy(g[k]) for k in ("Q", "K", "V", "coords", "sigma", "mask")}
    for name, (O, L) in _both(t["Q"], t["K"], t["V"], t["coords"], t["sigma"], t["mask"]).items():
        assert np.abs(O - g["O"]).max() < TOL[name] * 100, name
        fin = np.isfinite(g["L"])
        assert (np.isfinite(L) == fin).all() and np.abs(L[fin] - g["L"][fin]).max() < TOL[name] * 100, name
    # an independent brute-force evaluation of a fresh tiny case
    Q, K, V, coords, sigma, mask = _case(4, Z=1, H=2, N=9, maskfrac=0.3)
    Ob, Lb = brute.geo_attn_brute(Q.double().tolist(), K.double().tolist(), V.double().tolist(),
                                  coords.double().tolist(), sigma.double().tolist(), mask.tolist())
    for name, (O, L) in _both(Q, K, V, coords, sigma, mask).items():
        assert np.abs(O - np.array(Ob)).max() < TOL[name] * 100, name


def test_invariants():
    Q, K, V, coords, sigma, mask = _case(5, maskfrac=0.2)
    O, L = c_oracle.geo_attn(Q.numpy(), K.numpy(), V.numpy(), coords.numpy(), sigma.numpy(), mask.numpy())
    # softmax rows sum to one: V = 1 -> O = 1 on valid rows
    O1, _ = c_oracle.geo_attn(Q.numpy(), K.numpy(), np.ones_like(V.numpy()), coords.numpy(), sigma.numpy(), mask.numpy())
    valid = ~mask.numpy()
    for z in range(Q.shape[0]):
        assert np.abs(O1[z][:, valid[z]] - 1).max() < 1e-12
    # rigid motion of the coordinates changes nothing (up to float32 re-rounding of the moved coordinates)
    q, _ = np.linalg.qr(np.random.default_rng(0).normal(size=(3, 3)))
    moved = (coords.double().numpy() @ q.T + np.array([1.0, 2.0, 3.0])).astype(np.float32)
    O2, L2 = c_oracle.geo_attn(Q.numpy(), K.numpy(), V.numpy(), moved, sigma.numpy(), mask.numpy())
    assert np.abs(O - O2).max() < 1e-3
    # key padding == truncation to the unpadded tokens
    z = 0
    keep = valid[z]
    O3, L3 = c_oracle.geo_attn(Q.numpy()[z:z + 1][:, :, keep], K.numpy()[z:z + 1][:, :, keep], V.numpy()[z:z + 1][:, :, keep],
                               coords.numpy()[z:z + 1][:, keep], sigma.numpy(), None)
    assert np.abs(O[z][:, keep] - O3[0]).max() < 1e-12 and np.abs(L[z][:, keep] - L3[0]).max() < 1e-12
    # heads are independent: head h alone with its own sigma
    O4, _ = c_oracle.geo_attn(Q.numpy()[:, 1:2], K.numpy()[:, 1:2], V.numpy()[:, 1:2], coords.numpy(), sigma.numpy()[1:2], mask.numpy())
    assert np.abs(O[:, 1:2] - O4).max() < 1e-12


def test_logsumexp_output():
    Q, K, V, coords, sigma, _ = _case(6, Z=1, H=2, N=15)
    O, L = c_oracle.geo_attn(Q.numpy(), K.numpy(), V.numpy(), coords.numpy(), sigma.numpy())
    S = torch.matmul(Q.double(), K.double().transpose(2, 3)) / 8
    d2 = ((coords[:, :, None].double() - coords[:, None].double()) ** 2).sum(-1)
    S = S * (1 + torch.exp(-d2[:, None] / (2 * sigma.double()[None, :, None, None] ** 2)))
    assert np.abs(L - torch.logsumexp(S, -1).numpy()).max() < 1e-11


def test_row_subset_equals_full():
    Q, K, V, coords, sigma, mask = _case(7, maskfrac=0.2)
    rows = np.array([0, 36, 5], np.int32)
    O, L = c_oracle.geo_attn(Q.numpy(), K.numpy(), V.numpy(), coords.numpy(), sigma.numpy(), mask.numpy())
    Os, Ls = c_oracle.geo_attn(Q.numpy(), K.numpy(), V.numpy(), coords.numpy(), sigma.numpy(), mask.numpy(), rows=rows)
    assert np.array_equal(O[:, :, rows], Os) and np.array_equal(L[:, :, rows], Ls)
    Ot, Lt = torch_oracle.geo_attn_torch(Q, K, V, coords, sigma, mask, rows=rows.tolist(), dtype=torch.float64)
    assert np.abs(Ot.numpy() - Os).max() < 1e-11


def test_legacy_logits_oracles():
    # the reference kernel's own logits: C and torch statements agree, and beta = 0 with the full rbf range is
    # plain scaled-dot-product attention with a key mask
    Q, K, V, coords, sigma, mask = _case(8, maskfrac=0.25)
    beta = torch.tensor([1.0, 0.3, 2.0])
    Oc, Lc = c_oracle.geo_attn_legacy(Q.numpy(), K.numpy(), V.numpy(), coords.numpy(), sigma.numpy(), beta.numpy(), mask.numpy(), 0.001, 0.9)
    Ot, Lt = torch_oracle.geo_attn_legacy_torch(Q, K, V, coords, sigma, beta, mask, 0.001, 0.9, dtype=torch.float64)
    assert np.abs(Oc - Ot.numpy()).max() < 1e-11
    fin = np.isfinite(Lc)
    assert (np.isfinite(Lt.numpy()) == fin).all() and np.abs(Lc[fin] - Lt.numpy()[fin]).max() < 1e-11
    O0, _ = c_oracle.geo_attn_legacy(Q.numpy(), K.numpy(), V.numpy(), coords.numpy(), sigma.numpy(), np.zeros(3, np.float32), mask.numpy(), 0.0, 1.0)
    am = (~mask)[:, None, None, :].expand(-1, Q.shape[1], Q.shape[2], -1)
    ref = F.scaled_dot_product_attention(Q.double(), K.double(), V.double(), attn_mask=am).numpy()
    valid = ~mask.numpy()
    for z in range(Q.shape[0]):
        assert np.abs(O0[z][:, valid[z]] - ref[z][:, valid[z]]).max() < 1e-9
    # identical coordinates: rbf = 1 -> rbf_norm = +1 -> logits S + beta |S|
    same = torch.zeros_like(coords)
    O1, _ = c_oracle.geo_attn_legacy(Q.numpy(), K.numpy(), V.numpy(), same.numpy(), sigma.numpy(), beta.numpy(), None, 0.0, 1.0)
    S = torch.matmul(Q.double(), K.double().transpose(2, 3)) / 8
    S = S + beta.double()[None, :, None, None] * S.abs()
    ref1 = torch.matmul(torch.softmax(S, -1), V.double()).numpy()
    assert np.abs(O1 - ref1).max() < 1e-10


def test_differentiable_statement_equals_the_tiled_ones():
    # the backward tests differentiate geo_attn_autograd_torch with torch.autograd: its forward must be the
    # same function as the oracles pinned above, for both kinds of logits, masks and empty rows included
    g = torch.Generator().manual_seed(11)
    Z, H, N = 2, 3, 37
    Q, K, V = (torch.randn(Z, H, N, 64, generator=g, dtype=torch.float64) for _ in range(3))
    coords = torch.randn(Z, N, 3, generator=g, dtype=torch.float64) * 5
    sigma = torch.tensor([2.0, 5.0, 11.0], dtype=torch.float64)
    mask = torch.rand(Z, N, generator=g) < 0.3
    mask[1] = True
    mask[1, 5] = False
    O1, _ = torch_oracle.geo_attn_torch(Q, K, V, coords, sigma, mask, dtype=torch.float64)
    O2 = torch_oracle.geo_attn_autograd_torch(Q, K, V, coords, sigma, mask)
    torch.testing.assert_close(O2, O1, rtol=1e-12, atol=1e-12)
    betas = torch.tensor([0.5, 1.0, 2.0], dtype=torch.float64)
    O3, _ = torch_oracle.geo_attn_legacy_torch(Q, K, V, coords, sigma, betas, mask, 0.05, 0.9, dtype=torch.float64)
    O4 = torch_oracle.geo_attn_autograd_torch(Q, K, V, coords, sigma, mask, betas, 0.05, 0.9)
    torch.testing.assert_close(O4, O3, rtol=1e-12, atol=1e-12)
    # and it is differentiable without NaNs through masked and empty rows
    q = Q.clone().requires_grad_(True)
    s = sigma.clone().requires_grad_(True)
    torch_oracle.geo_attn_autograd_torch(q, K, V, coords, s, mask).sum().backward()
    assert torch.isfinite(q.grad).all() and torch.isfinite(s.grad).all()
    assert (q.grad[mask[:, None, :].expand(-1, H, -1)] == 0).all()


def test_per_query_sigma_and_beta_split_the_per_head_gradients():
    """sigma / beta given per query row [Z,H,N]: the same output, and gradients that sum over the queries to the
    per-head ones (they are the per-query contributions the GPU tests weigh the per-head numbers against)."""
    g = torch.Generator().manual_seed(12)
    Z, H, N = 2, 3, 37
    Q, K, V, dO = (torch.randn(Z, H, N, 64, generator=g, dtype=torch.float64) for _ in range(4))
    coords = torch.cumsum(torch.randn(Z, N, 3, generator=g, dtype=torch.float64) * 2.2, dim=1)
    mask = torch.rand(Z, N, generator=g) < 0.2
    for betas, lo, hi in ((None, 0.0, 1.0), (torch.tensor([0.3, 1.0, 1.7], dtype=torch.float64), 0.05, 0.9)):
        s_head = torch.tensor([2.0, 5.0, 11.0], dtype=torch.float64, requires_grad=True)
        b_head = None if betas is None else betas.clone().requires_grad_(True)
        O1 = torch_oracle.geo_attn_autograd_torch(Q, K, V, coords, s_head, mask, b_head, lo, hi)
        O1.backward(dO)
        s_rows = s_head.detach()[None, :, None].expand(Z, H, N).clone().requires_grad_(True)
        b_rows = None if betas is None else betas[None, :, None].expand(Z, H, N).clone().requires_grad_(True)
        O2 = torch_oracle.geo_attn_autograd_torch(Q, K, V, coords, s_rows, mask, b_rows, lo, hi)
        O2.backward(dO)
        assert torch.equal(O1.detach(), O2.detach())
        assert torch.allclose(s_rows.grad.sum(dim=(0, 2)), s_head.grad, rtol=1e-10, atol=1e-12)
        assert (s_rows.grad[mask[:, None, :].expand(Z, H, N)] == 0).all()          # a padded query contributes nothing
        if betas is not None:
            assert torch.allclose(b_rows.grad.sum(dim=(0, 2)), b_head.grad, rtol=1e-10, atol=1e-12)
        # the pair-level error scale of the per-head scalars: its terms, signs kept, ARE the gradients (autograd's), and
        # it bounds what survives the cancellation inside a query and between the queries
        m_s, m_b, t_s, t_b = torch_oracle.geo_attn_scalar_grad_mass(Q, K, V, dO, coords, s_head.detach(), mask, betas, lo, hi)
        assert torch.allclose(t_s, s_head.grad, rtol=1e-9, atol=1e-12)
        assert (m_s >= s_rows.grad.abs().sum(dim=(0, 2)) * (1 - 1e-12)).all() and (m_s > 0).all()
        if betas is not None:
            assert torch.allclose(t_b, b_head.grad, rtol=1e-9, atol=1e-12)
            assert (m_b >= b_rows.grad.abs().sum(dim=(0, 2)) * (1 - 1e-12)).all()
        else:
            assert m_b is None and t_b is None


def test_tiled_backward_equals_autograd():
    """The chunked hand-derived gradients (used where N x N does not fit) against torch.autograd through the dense
    differentiable statement: masks, an empty batch item but for one token, chunks that do not divide N."""
    g = torch.Generator().manual_seed(13)
    Z, H, N = 2, 3, 53
    Q, K, V, dO = (torch.randn(Z, H, N, 64, generator=g, dtype=torch.float64) for _ in range(4))
    coords = torch.cumsum(torch.randn(Z, N, 3, generator=g, dtype=torch.float64) * 2.2, dim=1)
    sigma = torch.tensor([2.0, 5.0, 11.0], dtype=torch.float64)
    mask = torch.rand(Z, N, generator=g) < 0.25
    mask[1] = True
    mask[1, 7] = False
    q, k, v = (t.clone().requires_grad_(True) for t in (Q, K, V))
    s = sigma.clone().requires_grad_(True)
    torch_oracle.geo_attn_autograd_torch(q, k, v, coords, s, mask).backward(dO)
    for chunk in (7, 16, 53, 2048):
        dQ, dK, dV, ds, mass = torch_oracle.geo_attn_backward_tiled_torch(Q, K, V, dO, coords, sigma, mask, row_chunk=chunk)
        torch.testing.assert_close(dQ, q.grad, rtol=1e-10, atol=1e-12)
        torch.testing.assert_close(dK, k.grad, rtol=1e-10, atol=1e-12)
        torch.testing.assert_close(dV, v.grad, rtol=1e-10, atol=1e-12)
        torch.testing.assert_close(ds, s.grad, rtol=1e-9, atol=1e-12)
        m_ref, _, t_ref, _ = torch_oracle.geo_attn_scalar_grad_mass(Q, K, V, dO, coords, sigma, mask)
        torch.testing.assert_close(mass, m_ref, rtol=1e-10, atol=1e-14)
        torch.testing.assert_close(ds, t_ref, rtol=1e-9, atol=1e-12)
