"""GPU parity tests of the RBF-scaled geometric attention forward: the HIP
kernel, called through the C ABI, against the CPU oracles evaluated on the
bf16-rounded operands.

Bar: max |O - O_ref| <= 2e-2 (bf16 operands, fp32 accumulation) on rows the
reference defines; padded / empty rows must be exactly 0 with L = -inf."""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import proteusai_amd as pa
from oracle import c_oracle
from proteusai_amd import _lib, synth

pytestmark = pytest.mark.gpu

MAX_ABS_TOL = 2e-2         # the stated parity bar for bf16 attention
# The kernels sum the bf16-ROUNDED probabilities (the ones the P V product uses), so that the weights of O add up to
# exactly one and rowsum(O dO) cancels against dP in the backward.  Each term is off by at most 2^-8 of itself (bf16
# keeps 8 significant bits), hence so is the sum, and |logsumexp error| <= 2^-8 = 3.9e-3 (measured: up to 3.8e-3 for rows
# that one key dominates, around 1e-3 for rows with many keys).
LSE_TOL = 4.0e-3


def make(seed, Z, H, N, qscale=1.0, maskfrac=0.0, tail=False):
    g = torch.Generator().manual_seed(seed)
    Q = (torch.randn(Z, H, N, 64, generator=g) * qscale).bfloat16()
    K = (torch.randn(Z, H, N, 64, generator=g) * qscale).bfloat16()
    V = torch.randn(Z, H, N, 64, generator=g).bfloat16()
    coords = torch.stack([synth.random_walk_chain(N, g) for _ in range(Z)])
    sigma = synth.log_spaced_sigma(H)
    mask = None
    if maskfrac > 0:
        mask = torch.rand(Z, N, generator=g) < maskfrac
    if tail:
        lens = torch.randint(max(1, N // 2), N + 1, (Z,), generator=g)
        t = torch.arange(N)[None, :] >= lens[:, None]
        mask = t if mask is None else (mask | t)
    return Q, K, V, coords, sigma, mask


# 0: the launcher's choice (small grids take the kernel with one query block per wave); 5: the software-pipelined
# kernel, which large grids take, forced on these small shapes too (its direct-distance fallback beside it)
KERNELS = [0, 3, 5, 7]      # automatic; one query block per wave; the pipelined kernel; a pair of waves per query block (keys split)


def run_gpu(gpu, Q, K, V, coords, sigma, mask, tuning=0):
    O, L = pa.geo_attn(Q.to(gpu), K.to(gpu), V.to(gpu), coords.to(gpu), sigma.to(gpu),
                       None if mask is None else mask.to(gpu), return_lse=True, tuning=tuning)
    torch.cuda.synchronize()
    return O.cpu().numpy(), L.cpu().numpy()



def sample_rows(n, count, seed, tile=256):
    """`count` distinct query rows of 0..n-1: the first and last rows, both sides of the first and last boundaries of
    the 32-query blocks and of the 256-query workgroup tiles and of one in the middle, the rest uniformly at random."""
    edges = {0, 1, 31, 32, 63, 64, tile - 1, tile, n // 2 - 1, n // 2, n - tile - 1, n - tile, n - 65, n - 64, n - 33, n - 32,
             n - 2, n - 1}
    edges = {r for r in edges if 0 <= r < n}
    rest = np.random.default_rng(seed).permutation(n)
    rows = list(edges) + [int(r) for r in rest if int(r) not in edges][:max(0, count - len(edges))]
    return np.sort(np.asarray(rows, dtype=np.int32))


def check(got, Q, K, V, coords, sigma, mask, rows=None, what=""):
    O, L = got
    Or, Lr = c_oracle.geo_attn(Q.float().numpy(), K.float().numpy(), V.float().numpy(), coords.numpy(), sigma.numpy(),
                               None if mask is None else mask.numpy(), rows=rows)
    sel = slice(None) if rows is None else np.asarray(rows)
    O, L = O[:, :, sel].astype(np.float64), L[:, :, sel].astype(np.float64)
    assert np.isfinite(O).all(), f"{what}: non-finite output"
    err = np.abs(O - Or).max()
    assert err <= MAX_ABS_TOL, f"{what}: max abs error {err:.3e}"
    fin = np.isfinite(Lr)
    assert (np.isneginf(L) == ~fin).all(), f"{what}: -inf pattern of L differs"
    if fin.any():
        assert np.abs(L[fin] - Lr[fin]).max() <= LSE_TOL, f"{what}: logsumexp error {np.abs(L[fin] - Lr[fin]).max():.3e}"
    assert (O[~fin] == 0).all(), f"{what}: padded / empty rows must be exactly zero"
    return err


@pytest.mark.parametrize("tuning", KERNELS)
@pytest.mark.parametrize("N", [1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 191, 192, 193, 200, 255, 256, 257, 513])
def test_ragged_lengths(gpu, N, tuning):
    a = make(100 + N, 2, 3, N)
    check(run_gpu(gpu, *a, tuning=tuning), *a, what=f"N={N}")


def test_golden_fixture(gpu, golden_dir):
    g = np.load(os.path.join(golden_dir, "geo_attn_small.npz"))
    t = [torch.from_numpy(g[k]) for k in ("Q", "K", "V", "coords", "sigma", "mask")]
    O, L = run_gpu(gpu, t[0].bfloat16(), t[1].bfloat16(), t[2].bfloat16(), t[3], t[4], t[5])
    assert np.abs(O - g["O"]).max() <= MAX_ABS_TOL
    fin = np.isfinite(g["L"])
    assert (np.isneginf(L) == ~fin).all() and np.abs(L[fin] - g["L"][fin]).max() <= LSE_TOL
    assert (O[~fin] == 0).all()


@pytest.mark.parametrize("tuning", KERNELS)
def test_masks(gpu, tuning):
    N = 300
    Q, K, V, coords, sigma, _ = make(1, 5, 2, N)
    g = torch.Generator().manual_seed(1)
    mask = torch.zeros(5, N, dtype=torch.bool)
    mask[0] = torch.rand(N, generator=g) < 0.5       # scattered
    mask[1, 131:] = True                             # tail padding, not tile aligned
    mask[2] = True                                   # everything padded
    mask[3] = True
    mask[3, 77] = False                              # one valid token
    mask[4, :64] = True                              # a whole leading key tile padded
    check(run_gpu(gpu, Q, K, V, coords, sigma, mask, tuning=tuning), Q, K, V, coords, sigma, mask, what="masks")


@pytest.mark.parametrize("tuning", KERNELS)
def test_large_logits(gpu, tuning):
    # logits of order +-40: the online softmax must not overflow or lose the maximum
    a = make(2, 1, 4, 400, qscale=2.5)
    check(run_gpu(gpu, *a, tuning=tuning), *a, what="large logits")


@pytest.mark.parametrize("profile", ["rising", "falling", "sawtooth", "late_spike", "very_negative_start", "masked_start"])
@pytest.mark.parametrize("near", [False, True])
@pytest.mark.parametrize("tuning", KERNELS)
def test_softmax_reference_is_rebased_when_the_scores_run_away(gpu, profile, near, tuning):
    """Scores that climb, fall or jump by hundreds along the key axis: the kernel keeps a lazy softmax reference
    (no running maximum) and must re-base it exactly when an exponential would run away, whatever the order."""
    N, H = 640, 2
    g = torch.Generator().manual_seed(11)
    j = torch.arange(N, dtype=torch.float32)
    ramp = {"rising": -60 + 120 * j / (N - 1),
            "falling": 60 - 120 * j / (N - 1),
            "sawtooth": 50 * ((j % 97) / 96.0 * 2 - 1) * (1 + j / N),
            "late_spike": torch.where(j == N - 3, torch.tensor(150.0), -20 + 0 * j),
            "very_negative_start": torch.where(j < 200, torch.tensor(-300.0), 5 * torch.sin(j)),
            "masked_start": 10 * torch.cos(j)}[profile]
    # s_ij = q_i . k_j / 8 with q = 8 on one axis and k_j = ramp_j there, plus small noise on the other axes
    Q = 0.05 * torch.randn(1, H, N, 64, generator=g)
    K = 0.05 * torch.randn(1, H, N, 64, generator=g)
    Q[..., 0] = 8.0
    K[..., 0] = ramp
    Q, K = Q.bfloat16(), K.bfloat16()
    V = torch.randn(1, H, N, 64, generator=g).bfloat16()
    coords = synth.random_walk_chain(N, g)[None]
    # near: every pair within reach of the multiplier (it then doubles the scores); far: none but the diagonal
    sigma = torch.tensor([2000.0, 3000.0]) if near else torch.tensor([0.05, 0.08])
    mask = None
    if profile == "masked_start":
        mask = torch.zeros(1, N, dtype=torch.bool)
        mask[0, :130] = True
        mask[0, 300:333] = True
    a = (Q, K, V, coords, sigma, mask)
    check(run_gpu(gpu, *a, tuning=tuning), *a, what=f"{profile}, near={near}")


def test_every_variant_matches_the_oracle(gpu):
    """Distance path (matrix cores / vector ALU) and query blocks per wave (1 / 2) are tuning choices, not semantics."""
    a = make(21, 2, 3, 700, maskfrac=0.1, tail=True)
    Q, K, V, coords, sigma, mask = a
    for t, name in enumerate(_lib.geo_attn_variants()):
        O, L = pa.geo_attn(Q.to(gpu), K.to(gpu), V.to(gpu), coords.to(gpu), sigma.to(gpu), mask.to(gpu),
                           return_lse=True, tuning=t)
        torch.cuda.synchronize()
        check((O.cpu().numpy(), L.cpu().numpy()), *a, what=f"variant {name}")


def test_strided_operands_and_token_major_output_are_read_and_written_in_place(gpu):
    """Q, K, V as slices of one fused [Z,N,3,H,d] buffer (what a fused projection leaves) and O laid out
    [Z,N,H,d]: the same bits as from contiguous [Z,H,N,d] tensors, and nothing written outside O's rows."""
    Z, H, N = 2, 3, 333
    a = make(31, Z, H, N, maskfrac=0.1, tail=True)
    Q, K, V, coords, sigma, mask = a
    fused = torch.stack([t.permute(0, 2, 1, 3) for t in (Q, K, V)], dim=2).contiguous().to(gpu)      # [Z,N,3,H,d]
    Qs, Ks, Vs = (fused[:, :, i].permute(0, 2, 1, 3) for i in range(3))                            # [Z,H,N,d] views
    assert not Qs.is_contiguous() and Qs.stride(2) == 3 * H * 64
    ref_O, ref_L = pa.geo_attn(Q.to(gpu), K.to(gpu), V.to(gpu), coords.to(gpu), sigma.to(gpu), mask.to(gpu), return_lse=True)
    O, L = pa.geo_attn(Qs, Ks, Vs, coords.to(gpu), sigma.to(gpu), mask.to(gpu), return_lse=True, token_major_out=True)
    torch.cuda.synchronize()
    assert O.shape == (Z, H, N, 64) and O.permute(0, 2, 1, 3).is_contiguous()
    assert torch.equal(O, ref_O) and torch.equal(L, ref_L)
    check((O.cpu().numpy(), L.cpu().numpy()), *a, what="strided")
    # head-major batch order [H,Z,N,d] (what a per-head batched projection leaves)
    Qh, Kh, Vh = (t.to(gpu).permute(1, 0, 2, 3).contiguous().permute(1, 0, 2, 3) for t in (Q, K, V))
    O2 = pa.geo_attn(Qh, Kh, Vh, coords.to(gpu), sigma.to(gpu), mask.to(gpu))
    assert torch.equal(O2, ref_O)
    # rows that are not 16-byte aligned cannot be read in place: the wrapper copies, the result is the same
    pad = torch.zeros(Z, H, N, 68, dtype=torch.bfloat16, device=gpu)
    pad[..., 4:] = Q.to(gpu)
    O3 = pa.geo_attn(pad[..., 4:], K.to(gpu), V.to(gpu), coords.to(gpu), sigma.to(gpu), mask.to(gpu))
    assert torch.equal(O3, ref_O)


def test_strided_output_rows_leave_the_gaps_between_them_alone(gpu):
    """Raw C ABI: O with a token stride of 80 floats and L next to canaries: only the 64 floats of each row are
    written, whatever the rows are embedded in."""
    import ctypes
    lib = _lib.load()
    Z, H, N = 1, 2, 150
    Q, K, V, coords, sigma, mask = make(33, Z, H, N, maskfrac=0.1)
    q, k, v, c, s, m = (t.to(gpu) for t in (Q, K, V, coords, sigma, mask.view(torch.uint8)))
    ref = pa.geo_attn(q, k, v, c, s, mask.to(gpu))
    buf = torch.full((Z, H, N, 80), -7.25, device=gpu)
    Lb = torch.full((Z * H * N + 32,), -7.25, device=gpu)
    plain = [H * N * 64, N * 64, 64]
    strides = (ctypes.c_int64 * 12)(*(plain * 3 + [H * N * 80, N * 80, 80]))
    rc = lib.proteus_geo_attn_fwd_strided(q.data_ptr(), k.data_ptr(), v.data_ptr(), strides, c.data_ptr(), s.data_ptr(),
                                          m.data_ptr(), buf.data_ptr(), Lb.data_ptr(), Z, H, N, 64, 0,
                                          torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(buf[..., :64], ref)
    assert (buf[..., 64:] == -7.25).all() and (Lb[Z * H * N:] == -7.25).all()


def test_flat_multiplier_equals_sdpa_on_gpu(gpu):
    # sigma -> infinity: multiplier == 2 -> torch SDPA with scale 2/sqrt(d), evaluated in fp32 on the same bf16 values
    Q, K, V, coords, _, _ = make(3, 2, 4, 777)
    sigma = torch.full((4,), 1e7)
    O, _ = run_gpu(gpu, Q, K, V, coords, sigma, None)
    ref = F.scaled_dot_product_attention(Q.float().to(gpu), K.float().to(gpu), V.float().to(gpu), scale=2 / 8).cpu().numpy()
    assert np.abs(O - ref).max() <= MAX_ABS_TOL


def test_softmax_rows_sum_to_one(gpu):
    Q, K, V, coords, sigma, mask = make(4, 2, 8, 1000, tail=True)
    O, L = run_gpu(gpu, Q, K, torch.ones_like(V), coords, sigma, mask)
    valid = ~mask.numpy()
    for z in range(2):
        assert np.abs(O[z][:, valid[z]] - 1).max() < 1e-2 and (O[z][:, ~valid[z]] == 0).all()


def test_key_padding_equals_truncation(gpu):
    Q, K, V, coords, sigma, _ = make(5, 1, 2, 260)
    mask = torch.zeros(1, 260, dtype=torch.bool)
    mask[0, 200:] = True
    O, L = run_gpu(gpu, Q, K, V, coords, sigma, mask)
    O2, L2 = run_gpu(gpu, Q[:, :, :200].contiguous(), K[:, :, :200].contiguous(), V[:, :, :200].contiguous(),
                     coords[:, :200].contiguous(), sigma, None)
    assert np.array_equal(O[:, :, :200], O2) and np.array_equal(L[:, :, :200], L2)


@pytest.mark.parametrize("tuning", KERNELS)
def test_what_padded_tokens_hold_cannot_reach_valid_rows(gpu, tuning):
    """NaN, Inf and huge values in Q, K, V and the coordinates of padded tokens: the valid rows come out bit for bit as
    with zeros there, padded rows are exactly zero (scattered and tail padding; several key tiles)."""
    Z, H, N = 2, 3, 450
    Q, K, V, coords, sigma, mask = make(41, Z, H, N, maskfrac=0.15, tail=True)
    clean = [t.clone() for t in (Q, K, V, coords)]
    junk = torch.tensor([float("nan"), float("inf"), -float("inf"), 3e38, -1e30])
    g = torch.Generator().manual_seed(41)
    for t, c in zip((Q, K, V), clean[:3]):
        pick = junk[torch.randint(0, 5, (Z, N), generator=g)].to(t.dtype)
        t[:] = torch.where(mask[:, None, :, None], pick[:, None, :, None], t)
        c[:] = torch.where(mask[:, None, :, None], torch.zeros((), dtype=t.dtype), c)
    pick = junk[torch.randint(0, 5, (Z, N), generator=g)]
    coords[:] = torch.where(mask[:, :, None], pick[:, :, None], coords)
    clean[3][:] = torch.where(mask[:, :, None], torch.zeros(()), clean[3])
    O1, L1 = run_gpu(gpu, Q, K, V, coords, sigma, mask, tuning=tuning)
    O0, L0 = run_gpu(gpu, *clean, sigma, mask, tuning=tuning)
    assert np.array_equal(O1, O0) and np.array_equal(L1, L0)
    check((O0, L0), *clean, sigma, mask, what="padded junk")


def test_rigid_motion_of_coordinates(gpu):
    Q, K, V, coords, sigma, _ = make(6, 1, 4, 500)
    O, _ = run_gpu(gpu, Q, K, V, coords, sigma, None)
    g = torch.Generator().manual_seed(6)
    q, _ = torch.linalg.qr(torch.randn(3, 3, generator=g, dtype=torch.float64))
    moved = (coords.double() @ q.T + torch.tensor([10.0, -20.0, 5.0], dtype=torch.float64)).float()
    O2, _ = run_gpu(gpu, Q, K, V, moved, sigma, None)
    assert np.abs(O - O2).max() < 5e-3


def test_raw_c_abi_without_lse_and_canaries(gpu):
    Q, K, V, coords, sigma, _ = make(7, 1, 2, 150)
    lib = _lib.load()
    n, pad = 1 * 2 * 150 * 64, 64
    buf = torch.full((n + 2 * pad,), -777.0, device=gpu)
    buf[pad:pad + n] = float("nan")
    q, k, v, c, s = Q.to(gpu), K.to(gpu), V.to(gpu), coords.to(gpu), sigma.to(gpu)
    rc = lib.proteus_geo_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), c.data_ptr(), s.data_ptr(), None,
                                  buf.data_ptr() + 4 * pad, None, 1, 2, 150, 64, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    h = buf.cpu()
    assert (h[:pad] == -777.0).all() and (h[pad + n:] == -777.0).all()
    O = h[pad:pad + n].view(1, 2, 150, 64).numpy()
    Or, _ = c_oracle.geo_attn(Q.float().numpy(), K.float().numpy(), V.float().numpy(), coords.numpy(), sigma.numpy())
    assert np.abs(O - Or).max() <= MAX_ABS_TOL


def test_deterministic(gpu):
    a = make(8, 2, 4, 900, tail=True)
    x, y = run_gpu(gpu, *a), run_gpu(gpu, *a)
    assert np.array_equal(x[0], y[0]) and np.array_equal(x[1], y[1])


def test_module_forward_matches_composition(gpu):
    # GeoAttention: per-head projections -> op -> (d_k x heads) interleaved concat -> out_proj
    torch.manual_seed(0)
    mod = pa.GeoAttention(d_model=128, heads=2, min_spread=2.0).to(gpu)
    with torch.no_grad():
        mod.spread_weights.copy_(torch.tensor([0.3, 1.2]))
    g = torch.Generator().manual_seed(9)
    x = torch.randn(2, 90, 128, generator=g)
    coords = torch.stack([synth.random_walk_chain(90, g) for _ in range(2)])
    mask = torch.zeros(2, 90, dtype=torch.bool)
    mask[1, 60:] = True
    with torch.no_grad():
        y = mod(x.to(gpu), x.to(gpu), x.to(gpu), coords.to(gpu), mask=mask.to(gpu)).cpu()
        p = {k: v.detach().cpu() for k, v in mod.named_parameters()}
        Qh = torch.matmul(x.unsqueeze(1), p["q_proj"].unsqueeze(0)) + p["q_bias"][None, :, None]
        Kh = torch.matmul(x.unsqueeze(1), p["k_proj"].unsqueeze(0)) + p["k_bias"][None, :, None]
        Vh = torch.matmul(x.unsqueeze(1), p["v_proj"].unsqueeze(0)) + p["v_bias"][None, :, None]
        sig = 2.0 + torch.exp(p["spread_weights"])
        Or, _ = c_oracle.geo_attn(Qh.bfloat16().float().numpy(), Kh.bfloat16().float().numpy(), Vh.bfloat16().float().numpy(),
                                  coords.numpy(), sig.numpy(), mask.numpy())
        ref = torch.from_numpy(Or).float().permute(0, 2, 3, 1).reshape(2, 90, 128) @ p["out_proj.weight"].T
    assert (y - ref).abs().max() < 5e-2


def test_cfg3_sampled_rows(gpu):
    # B=4, N=4096, H=8, d=64, Q,K,V ~ N(0,1)/8, lengths in [2048, 4096]
    Q, K, V, coords, sigma, mask = synth.attn_inputs(4, 8, 4096, 64, seed=3, min_len=2048)
    got = run_gpu(gpu, Q, K, V, coords, sigma, mask)
    # 160 query rows x 8 heads x 4 batch items (padded rows among them: they must be exact zeros), ends of the sequence,
    # of the 32-query blocks and of the 256-query tiles included
    rows = sample_rows(4096, 160, seed=3)
    check(got, Q, K, V, coords, sigma, mask, rows=rows, what="cfg3")


def test_cfg3_shape_with_unit_variance_logits(gpu):
    # same shape, but logits of order one so that the softmax is far from uniform
    Q, K, V, coords, sigma, mask = make(33, 4, 8, 4096, tail=True)
    got = run_gpu(gpu, Q, K, V, coords, sigma, mask)
    rows = np.sort(np.random.default_rng(33).choice(4096, 48, replace=False)).astype(np.int32)
    check(got, Q, K, V, coords, sigma, mask, rows=rows, what="cfg3 unit-variance")


def test_cfg5_sampled_rows(gpu):
    # N=16384, H=8, d=64 on the first 16384 residues of the compacted N=65536 chain
    wc, _ = synth.we_inputs(65536, seed=5, compact=True)
    Q, K, V, coords, sigma, mask = synth.attn_inputs(1, 8, 16384, 64, seed=5, coords=wc[:, :16384].contiguous())
    got = run_gpu(gpu, Q, K, V, coords, sigma, mask)
    rows = sample_rows(16384, 160, seed=5)              # 160 query rows x 8 heads, tile boundaries and both ends included
    check(got, Q, K, V, coords, sigma, mask, rows=rows, what="cfg5")
    # size-independent property at full size: V = 1 -> O = 1
    O1, _ = run_gpu(gpu, Q, K, torch.ones_like(V), coords, sigma, None)
    assert np.abs(O1 - 1).max() < 1e-2


def test_long_ragged_sequence_sampled_rows(gpu):
    # N = 40003 (not a multiple of the key tile, 626 tiles, offsets beyond 5 MB per head) with tail padding, two heads,
    # through the kernel large grids take; the last rows and the rows around the end of the unpadded part included
    N, valid = 40003, 39000
    wc, _ = synth.we_inputs(65536, seed=8, compact=True)
    Q, K, V, coords, sigma, _ = synth.attn_inputs(1, 2, N, 64, seed=8, coords=wc[:, :N].contiguous())
    mask = (torch.arange(N) >= valid)[None, :]
    got = run_gpu(gpu, Q, K, V, coords, sigma, mask)
    rows = np.unique(np.concatenate([np.random.default_rng(8).choice(valid, 24, replace=False),
                                     [0, 63, 64, valid - 1, valid, N - 1]])).astype(np.int32)
    check(got, Q, K, V, coords, sigma, mask, rows=rows, what="N=40003")
    assert (got[0][:, :, valid:] == 0).all() and np.isneginf(got[1][:, :, valid:]).all()


def test_legacy_logits(gpu):
    # the reference kernel's own logits S + beta*rbf_norm*|S| with its [min_rbf, max_rbf] pair mask
    # (old/old_scripts/attn/geometric_attn.py:193-201), against the restated torch_attn oracle
    Q, K, V, coords, sigma, mask = make(21, 2, 4, 333, maskfrac=0.15)
    beta = torch.tensor([1.0, 0.5, 2.0, 0.1])
    for min_rbf, max_rbf in ((0.0, 1.0), (0.001, 1.0)):
        O, L = pa.geo_attn(Q.to(gpu), K.to(gpu), V.to(gpu), coords.to(gpu), sigma.to(gpu), mask.to(gpu), return_lse=True,
                           betas=beta.to(gpu), min_rbf=min_rbf, max_rbf=max_rbf)
        torch.cuda.synchronize()
        Or, Lr = c_oracle.geo_attn_legacy(Q.float().numpy(), K.float().numpy(), V.float().numpy(), coords.numpy(), sigma.numpy(),
                                          beta.numpy(), mask.numpy(), min_rbf, max_rbf)
        O, L = O.cpu().numpy().astype(np.float64), L.cpu().numpy().astype(np.float64)
        # rows holding a pair whose rbf sits within 1e-4 (relative) of a threshold may legitimately flip: leave them out
        d2 = ((coords[:, :, None].double() - coords[:, None].double()) ** 2).sum(-1)
        rbf = torch.exp(-d2[:, None] / (2 * sigma.double()[None, :, None, None] ** 2))
        edge = ((rbf - min_rbf).abs() < 1e-4 * max(min_rbf, 1e-30)).any(-1).numpy() if min_rbf > 0 else np.zeros(L.shape, bool)
        fin = np.isfinite(Lr) & ~edge
        assert (np.isneginf(L) == np.isneginf(Lr))[~edge].all()
        assert np.abs(O - Or)[~edge].max() <= MAX_ABS_TOL
        assert np.abs(L[fin] - Lr[fin]).max() <= LSE_TOL
    # module: the reference's GeoAttention semantics (beta = exp(w), min_rbf default) are available on request
    torch.manual_seed(1)
    mod = pa.GeoAttention(d_model=128, heads=2, legacy_logits=True).to(gpu)
    assert mod.min_rbf == 0.001 and pa.GeoAttention(d_model=128, heads=2).min_rbf == 0.0      # old/old_scripts/encoder.py:57
    x = torch.randn(1, 70, 128)
    with torch.no_grad():
        y = mod(x.to(gpu), x.to(gpu), x.to(gpu), coords[:1, :70].to(gpu))
    assert y.shape == (1, 70, 128) and torch.isfinite(y).all()
