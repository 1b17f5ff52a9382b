"""GPU parity tests of the geometric attention at head dimensions 32 and 128 and with fp16 operands, forward and
backward, through the operator API (and so through the C ABI), against the CPU oracles.

The reference's kernel takes any d_k >= 16 and casts Q, K, V to fp16 (old/old_scripts/attn/geometric_attn.py:567-569,
:597); its own test runs Z, H, N, d_k = 1, 4, 128, 32 with collinear coordinates, spreads 3 and betas 1, and compares
the kernel with the dense fp32 statement on the UNROUNDED inputs at atol = 1e-2 (tests/attn/geo_attn.py:15-39,
:172-212).  That test is restated here with a seed; the other tests compare with the oracles on operands rounded to
the kernel's type, at the bars of the d = 64 tests (2e-2 max-abs on O, 1e-2 relative L2 on dQ, dK, dV, the pair-sum
bar on d_sigma and d_beta)."""
import numpy as np
import pytest
import torch

import proteusai_amd as pa
from oracle import c_oracle, torch_oracle
from proteusai_amd import synth

pytestmark = pytest.mark.gpu

MAX_ABS_TOL = 2e-2
REL_L2_TOL = 1e-2
LSE_TOL_BF16 = 4.0e-3          # the row sum is taken over the rounded probabilities: 2^-8 for bf16,
LSE_TOL_F16 = 6.0e-4           # 2^-11 for fp16


def rel_l2(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    nb = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / nb) if nb > 0 else float(np.linalg.norm(a - b))


def make(seed, Z, H, N, d, dtype, qscale=1.0, maskfrac=0.0):
    g = torch.Generator().manual_seed(seed)
    Q = (torch.randn(Z, H, N, d, generator=g) * qscale).to(dtype)
    K = (torch.randn(Z, H, N, d, generator=g) * qscale).to(dtype)
    V = torch.randn(Z, H, N, d, generator=g).to(dtype)
    dO = torch.randn(Z, H, N, d, generator=g).to(dtype)
    coords = torch.stack([synth.random_walk_chain(N, g) for _ in range(Z)])
    sigma = synth.log_spaced_sigma(H)
    mask = (torch.rand(Z, N, generator=g) < maskfrac) if maskfrac > 0 else None
    return Q, K, V, dO, coords, sigma, mask


def check_forward(O, L, Q, K, V, coords, sigma, mask, betas, lo, hi, lse_tol, what):
    m = None if mask is None else mask.numpy()
    if betas is None:
        Or, Lr = c_oracle.geo_attn(Q.float().numpy(), K.float().numpy(), V.float().numpy(), coords.numpy(), sigma.numpy(), m)
    else:
        Or, Lr = c_oracle.geo_attn_legacy(Q.float().numpy(), K.float().numpy(), V.float().numpy(), coords.numpy(), sigma.numpy(),
                                          betas.numpy(), m, lo, hi)
    O, L = O.cpu().numpy().astype(np.float64), L.cpu().numpy().astype(np.float64)
    assert np.isfinite(O).all(), what
    fin = np.isfinite(Lr)
    assert (np.isneginf(L) == ~fin).all(), f"{what}: -inf pattern of L"
    assert np.abs(O - Or).max() <= MAX_ABS_TOL, f"{what}: O {np.abs(O - Or).max():.3e}"
    assert np.abs(L[fin] - Lr[fin]).max() <= lse_tol, f"{what}: L {np.abs(L[fin] - Lr[fin]).max():.3e}"
    assert (O[~fin] == 0).all(), what


@pytest.mark.parametrize("d", [32, 128])
@pytest.mark.parametrize("N", [1, 33, 64, 130, 257, 600])
def test_forward_readme_logits(gpu, d, N):
    Q, K, V, _, coords, sigma, mask = make(500 + N + d, 2, 3, N, d, torch.bfloat16, maskfrac=0.2 if N > 33 else 0.0)
    # automatic; matrix-core / direct distances; one / two query blocks per wave; keys split; at d = 32 also the
    # software-pipelined kernel (with and without the direct-distance workgroups beside it)
    for tuning in (0, 1, 2, 3, 4, 7) + ((5, 6) if d == 32 else ()):
        O, L = pa.geo_attn(Q.to(gpu), K.to(gpu), V.to(gpu), coords.to(gpu), sigma.to(gpu), None if mask is None else mask.to(gpu),
                           return_lse=True, tuning=tuning)
        check_forward(O, L, Q, K, V, coords, sigma, mask, None, 0.0, 1.0, LSE_TOL_BF16, f"d={d} N={N} tuning={tuning}")


@pytest.mark.parametrize("d", [32, 128])
def test_forward_long_ragged_sequence_sampled_rows(gpu, d):
    # N = 5003 (79 tiles, the last one ragged), tail padding, both kinds of logits: the two LDS stages of the directly
    # loaded tiles are reused 39 times; sampled query rows against the torch oracle
    Z, H, N = 1, 2, 5003
    Q, K, V, _, coords, sigma, _ = make(900 + d, Z, H, N, d, torch.bfloat16)
    mask = torch.zeros(Z, N, dtype=torch.bool)
    mask[0, 4700:] = True
    rows = np.sort(np.random.default_rng(d).choice(4700, 48, replace=False))
    betas = torch.tensor([0.6, -0.3])
    # (tuning 5 at d = 32: the software-pipelined kernel, whose K ring is reused 19 times and whose V ring 26 times)
    for bt, lo, hi, tuning in ((None, 0.0, 1.0, 0), (betas, 0.01, 0.97, 0)) + (((None, 0.0, 1.0, 5),) if d == 32 else ()):
        O, L = pa.geo_attn(Q.to(gpu), K.to(gpu), V.to(gpu), coords.to(gpu), sigma.to(gpu), mask.to(gpu), return_lse=True,
                           betas=None if bt is None else bt.to(gpu), min_rbf=lo, max_rbf=hi, tuning=tuning)
        O, L = O.cpu().double(), L.cpu().double()
        assert torch.isfinite(O).all() and (O[0, :, 4700:] == 0).all() and torch.isneginf(L[0, :, 4700:]).all()
        if bt is None:
            Or, Lr = torch_oracle.geo_attn_torch(Q.float(), K.float(), V.float(), coords, sigma, mask, rows=rows, dtype=torch.float64)
        else:
            # (the dense legacy statement has no row subset: two heads of 5003^2 pairs in fp64 fit)
            Or, Lr = torch_oracle.geo_attn_legacy_torch(Q.float(), K.float(), V.float(), coords, sigma, bt, mask, lo, hi, dtype=torch.float64)
            Or, Lr = Or[:, :, rows], Lr[:, :, rows]
        fin = torch.isfinite(Lr)
        assert (torch.isfinite(L[:, :, rows]) == fin).all()
        assert (O[:, :, rows] - Or).abs().max() <= MAX_ABS_TOL, f"d={d} legacy={bt is not None}: O {(O[:, :, rows] - Or).abs().max():.3e}"
        assert (L[:, :, rows][fin] - Lr[fin]).abs().max() <= LSE_TOL_BF16, f"d={d} legacy={bt is not None}: L {(L[:, :, rows][fin] - Lr[fin]).abs().max():.3e}"


@pytest.mark.parametrize("d", [32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_forward_legacy_logits(gpu, d, dtype):
    Q, K, V, _, coords, sigma, mask = make(600 + d, 2, 4, 333, d, dtype, maskfrac=0.15)
    betas = torch.tensor([1.0, 0.5, 2.0, 0.1])
    lse_tol = LSE_TOL_F16 if dtype == torch.float16 else LSE_TOL_BF16
    O, L = pa.geo_attn(Q.to(gpu), K.to(gpu), V.to(gpu), coords.to(gpu), sigma.to(gpu), mask.to(gpu), return_lse=True,
                       betas=betas.to(gpu), operand_dtype=dtype)
    check_forward(O, L, Q, K, V, coords, sigma, mask, betas, 0.0, 1.0, lse_tol, f"legacy d={d} {dtype}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_large_logits_rebase_within_the_operand_range(gpu, dtype):
    # scores that run up by hundreds along the keys: the lazily re-based exponentials must stay below the largest
    # finite value of the operand type (65504 for fp16) before they are packed for the P V product
    Z, H, N, d = 1, 2, 700, 64
    g = torch.Generator().manual_seed(9)
    Q = torch.randn(Z, H, N, d, generator=g)
    K = torch.randn(Z, H, N, d, generator=g)
    Q[..., 0] = 6.0
    K[..., 0] = torch.linspace(-40.0, 40.0, N)[None, None, :]        # S rises by 60 from the first key to the last
    Q, K = Q.to(dtype), K.to(dtype)
    V = torch.randn(Z, H, N, d, generator=g).to(dtype)
    coords = synth.random_walk_chain(N, g)[None]
    sigma = torch.tensor([5.0, 12.0])
    betas = torch.tensor([0.3, 0.8])
    O, L = pa.geo_attn(Q.to(gpu), K.to(gpu), V.to(gpu), coords.to(gpu), sigma.to(gpu), None, return_lse=True,
                       betas=betas.to(gpu), operand_dtype=dtype)
    check_forward(O, L, Q, K, V, coords, sigma, None, betas, 0.0, 1.0, LSE_TOL_F16 if dtype == torch.float16 else LSE_TOL_BF16,
                  f"rising scores {dtype}")


def reference_grads(Q, K, V, dO, coords, sigma, mask, betas, lo, hi):
    Z, H, N, _ = Q.shape
    q, k, v = (t.double().requires_grad_(True) for t in (Q, K, V))
    s = sigma.double()[None, :, None].expand(Z, H, N).clone().requires_grad_(True)
    b = None if betas is None else betas.double()[None, :, None].expand(Z, H, N).clone().requires_grad_(True)
    torch_oracle.geo_attn_autograd_torch(q, k, v, coords, s, mask, b, lo, hi).backward(dO.double())
    mass_s, mass_b, _, _ = torch_oracle.geo_attn_scalar_grad_mass(Q, K, V, dO, coords, sigma, mask, betas, lo, hi)
    return q.grad, k.grad, v.grad, s.grad.sum(dim=(0, 2)), None if b is None else b.grad.sum(dim=(0, 2)), mass_s, mass_b


def check_backward(gpu, Q, K, V, dO, coords, sigma, mask, betas, lo, hi, dtype, scalar_tol, what):
    q, k, v = (t.to(gpu).requires_grad_(True) for t in (Q, K, V))
    s = sigma.to(gpu).requires_grad_(True)
    b = None if betas is None else betas.to(gpu).requires_grad_(True)
    O = pa.geometric_attn(q, k, v, coords.to(gpu), s, b, None if mask is None else mask.to(gpu), lo, hi,
                          operand_dtype=None if betas is None else dtype)
    O.backward(dO.to(gpu).float())
    torch.cuda.synchronize()
    rq, rk, rv, rs, rb, mass_s, mass_b = reference_grads(Q, K, V, dO, coords, sigma, mask, betas, lo, hi)
    for got, ref, name in ((q.grad, rq, "dQ"), (k.grad, rk, "dK"), (v.grad, rv, "dV")):
        got = got.float().cpu()
        assert torch.isfinite(got).all(), f"{what} {name}"
        e = rel_l2(got.numpy(), ref.numpy())
        assert e <= REL_L2_TOL, f"{what} {name}: rel-L2 {e:.3e}"
        if mask is not None:
            assert (got[mask[:, None, :].expand(-1, got.shape[1], -1)] == 0).all(), f"{what} {name}: padded tokens"
    for got, ref, mass, name in ((s.grad, rs, mass_s, "d_sigma"),) + (() if betas is None else ((b.grad, rb, mass_b, "d_beta"),)):
        err = (got.double().cpu() - ref).abs()
        assert (err <= scalar_tol * mass + 1e-30).all(), f"{what} {name}: error / pair mass {(err / mass.clamp_min(1e-300)).max():.3e}"


# (Z, H): a launch of few workgroups (at d <= 64 they own 64 tokens each, two waves per own block) and one of more than
# 256 workgroups of 128 own tokens
@pytest.mark.parametrize("ZH", [(2, 3), (5, 32)])
@pytest.mark.parametrize("d", [32, 128])
@pytest.mark.parametrize("N", [2, 65, 200, 333])
def test_backward_readme_logits(gpu, d, N, ZH):
    a = make(700 + N + d, ZH[0], ZH[1], N, d, torch.bfloat16, maskfrac=0.2 if N > 65 else 0.0)
    check_backward(gpu, *a, None, 0.0, 1.0, torch.bfloat16, 2.0 ** -9, f"d={d} N={N} Z,H={ZH}")


@pytest.mark.parametrize("d", [32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_backward_legacy_logits(gpu, d, dtype):
    a = make(800 + d, 2, 4, 300, d, dtype, maskfrac=0.2)
    betas = torch.tensor([0.5, 1.0, 0.25, 2.0])
    for lo, hi in ((0.0, 1.0), (0.05, 0.9)):
        check_backward(gpu, *a, betas, lo, hi, dtype, 2.0 ** -9, f"legacy d={d} {dtype} [{lo},{hi}]")


def test_the_reference_test_shape_at_its_own_tolerance(gpu):
    """tests/attn/geo_attn.py: batch, nheads, N, d_k = 1, 4, 128, 32; coords = 50 N(0,1) on the line x = y = z;
    spreads 3, betas 1, min_rbf 0, max_rbf 1, no mask; fp32 Q, K, V ~ N(0,1) cast to fp16 by the operator; the dense
    fp32 statement on the unrounded inputs is the reference; forward and the gradients of out.sum() at atol = 1e-2.

    O and dV are held to that, against the unrounded reference, as the reference's test does.  dQ and dK cannot be: the
    logits S + b Rn |S| have a kink at S = 0, so dQ and dK jump where a score changes sign, and rounding Q and K to fp16
    alone (exact arithmetic afterwards) moves them by 7.6e-2 and 9.0e-2 on this very input (3e-3 of that would be the
    smooth part).  They are held to atol = 1e-2 against the same dense statement on the inputs the kernel sees, i.e.
    rounded to its operand type; d_spreads and d_betas likewise."""
    Z, H, N, d = 1, 4, 128, 32
    g = torch.Generator().manual_seed(37)
    coords = (50 * torch.randn(Z, N, 1, generator=g)).expand(Z, N, 3).contiguous()
    spreads, betas = torch.full((H,), 3.0), torch.full((H,), 1.0)
    Q, K, V = (torch.randn(Z, H, N, d, generator=g) for _ in range(3))
    dense, _ = torch_oracle.geo_attn_legacy_torch(Q, K, V, coords, spreads, betas, None, 0.0, 1.0)

    def reference(Qx, Kx, Vx):
        rq, rk, rv = (t.clone().float().requires_grad_(True) for t in (Qx, Kx, Vx))
        rs, rb = spreads.clone().requires_grad_(True), betas.clone().requires_grad_(True)
        ref = torch_oracle.geo_attn_autograd_torch(rq, rk, rv, coords, rs, None, rb, 0.0, 1.0, dtype=torch.float32)
        ref.sum().backward()
        return ref.detach(), rq.grad, rk.grad, rv.grad, rs.grad, rb.grad
    unrounded = reference(Q, K, V)
    assert torch.allclose(unrounded[0], dense, atol=1e-5)            # the differentiable form is the dense statement

    for dtype, atol in ((torch.float16, 1e-2), (torch.bfloat16, 2e-2)):
        q, k, v = (t.to(gpu).requires_grad_(True) for t in (Q, K, V))
        s, b = spreads.to(gpu).requires_grad_(True), betas.to(gpu).requires_grad_(True)
        out = pa.geometric_attn(q, k, v, coords.to(gpu), s, b, None, 0.0, 1.0, operand_dtype=dtype)
        out.sum().backward()
        torch.cuda.synchronize()
        assert torch.allclose(out.detach().cpu(), dense, atol=atol, rtol=0), f"{dtype}: O {(out.detach().cpu() - dense).abs().max():.3e}"
        assert torch.allclose(v.grad.cpu(), unrounded[3], atol=atol, rtol=0), f"{dtype} dV: {(v.grad.cpu() - unrounded[3]).abs().max():.3e}"
        rounded = reference(Q.to(dtype), K.to(dtype), V.to(dtype))
        for got, want, name in ((q.grad, rounded[1], "dQ"), (k.grad, rounded[2], "dK"), (v.grad, rounded[3], "dV"),
                                (s.grad, rounded[4], "d_spreads"), (b.grad, rounded[5], "d_betas")):
            assert torch.allclose(got.cpu(), want, atol=atol, rtol=0), f"{dtype} {name}: {(got.cpu() - want).abs().max():.3e}"


def test_module_at_head_dimension_32_with_fp16_operands(gpu):
    # the reference's module configuration: d_model 128, 4 heads (d_k = 32), beta-weighted logits, fp16 inside the kernel
    torch.manual_seed(3)
    mods = [pa.GeoAttention(d_model=128, heads=4, legacy_logits=True, operand_dtype=dt).to(gpu) for dt in (torch.float16, None)]
    mods[1].load_state_dict(mods[0].state_dict())
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 90, 128, generator=g).to(gpu)
    coords = torch.stack([synth.random_walk_chain(90, g) for _ in range(2)]).to(gpu)
    mask = torch.zeros(2, 90, dtype=torch.bool, device=gpu)
    mask[1, 60:] = True
    outs = []
    for m in mods:
        xi = x.clone().requires_grad_(True)
        y = m(xi, xi, xi, coords, mask)
        y[~mask].square().mean().backward()
        assert torch.isfinite(y[~mask]).all() and torch.isfinite(xi.grad).all()
        assert m.spread_weights.grad.abs().sum() > 0 and m.beta_weights.grad.abs().sum() > 0
        outs.append((y.detach(), xi.grad))
    # the two operand types agree to their rounding
    assert (outs[0][0] - outs[1][0])[~mask].abs().max() <= 2e-2
    assert rel_l2(outs[0][1].cpu().numpy(), outs[1][1].cpu().numpy()) <= 3e-2
    with pytest.raises(NotImplementedError):
        pa.GeoAttention(d_model=128, heads=4, operand_dtype=torch.float16)
