"""GPU parity tests of the Wavefunction Embedding forward: the HIP kernel,
called through the C ABI (via the Python operator layer or raw ctypes), against
the CPU oracles on the same seeded inputs.

Bar: relative L2 error <= 1e-4 for out, cos_sums and sin_sums against the fp32
oracle (checked separately for each tensor)."""
import os

import numpy as np
import pytest
import torch

import proteusai_amd as pa
from oracle import c_oracle, torch_oracle
from proteusai_amd import _lib, synth

pytestmark = pytest.mark.gpu

REL_L2_TOL = 1e-4          # the stated parity bar for fp32 WE


def rel_l2(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    nb = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / nb) if nb > 0 else float(np.linalg.norm(a - b))


def run_gpu(gpu, coords, wn, mask=None, tuning=0):
    out, cs, ss = pa.we_forward(coords.to(gpu), wn.to(gpu), None if mask is None else mask.to(gpu), tuning=tuning)
    torch.cuda.synchronize()
    return out.cpu().numpy(), cs.cpu().numpy(), ss.cpu().numpy()


def check(got, coords, wn, mask=None, rows=None, tol=REL_L2_TOL, what=""):
    c, w = coords.numpy(), wn.numpy()
    m = None if mask is None else mask.numpy()
    ref32 = c_oracle.we(c, w, m, rows=rows, precision="f32")
    ref64 = c_oracle.we(c, w, m, rows=rows, precision="f64")
    sel = slice(None) if rows is None else np.asarray(rows)
    for g, r32, r64, name in zip(got, ref32, ref64, ("out", "cos_sums", "sin_sums")):
        g = g[:, sel]
        e32, e64 = rel_l2(g, r32), rel_l2(g, r64)
        assert e32 <= tol and e64 <= tol, f"{what} {name}: rel-L2 {e32:.3e} (fp32 oracle) {e64:.3e} (fp64 oracle)"
        assert np.isfinite(g).all(), f"{what} {name}: non-finite values"



def sample_rows(n, count, seed, tile=64):
    """`count` distinct rows of 0..n-1: the first and last rows, both sides of the first and last tile boundaries and
    of a boundary in the middle, the rest uniformly at random."""
    edges = {0, 1, tile - 1, tile, 4 * tile - 1, 4 * tile, n // 2 - 1, n // 2, n - 4 * tile - 1, n - 4 * tile,
             n - tile - 1, n - tile, n - 2, n - 1}
    edges = {r for r in edges if 0 <= r < n}
    rest = np.random.default_rng(seed).permutation(n)
    rows = list(edges) + [int(r) for r in rest if int(r) not in edges][:max(0, count - len(edges))]
    return np.sort(np.asarray(rows, dtype=np.int32))


def test_cfg1_full(gpu):
    # B=1, N=512, d_model=512, no mask, uncompacted chain, every row checked
    coords, wn = synth.we_inputs(512, seed=1)
    check(run_gpu(gpu, coords, wn), coords, wn, what="cfg1")


def test_cfg1_against_tiled_torch_path(gpu):
    coords, wn = synth.we_inputs(512, seed=1)
    got = run_gpu(gpu, coords, wn)
    ref = torch_oracle.we_torch(coords, wn)
    for g, r, name in zip(got, ref, ("out", "cos_sums", "sin_sums")):
        assert rel_l2(g, r.numpy()) <= REL_L2_TOL, name


def test_golden_fixture(gpu, golden_dir):
    g = np.load(os.path.join(golden_dir, "we_small.npz"))
    got = run_gpu(gpu, torch.from_numpy(g["coords"]), torch.from_numpy(g["wavenumbers"]), torch.from_numpy(g["mask"]))
    for a, key in zip(got, ("out", "cos_sums", "sin_sums")):
        assert rel_l2(a, g[key]) <= REL_L2_TOL, key
    pad = g["mask"]
    assert (got[0][pad] == 0).all() and (got[1][pad] == 0).all() and (got[2][pad] == 0).all()


@pytest.mark.parametrize("N", [1, 2, 3, 63, 64, 65, 255, 256, 257, 700])
def test_ragged_lengths(gpu, N):
    coords, _ = synth.we_inputs(N, seed=10 + N, batch=2)
    wn = synth.wavenumbers(64)
    got = run_gpu(gpu, coords, wn)
    if N == 1:
        assert all((a == 0).all() for a in got)      # a lone token sees nobody
    else:
        check(got, coords, wn, what=f"N={N}")


@pytest.mark.parametrize("K", [1, 2, 7, 31, 33, 100, 129])
def test_wavenumber_counts(gpu, K):
    coords, _ = synth.we_inputs(150, seed=3)
    g = torch.Generator().manual_seed(K)
    wn = torch.randn(K, generator=g)                  # signed, like the reference test
    check(run_gpu(gpu, coords, wn), coords, wn, what=f"K={K}")


def test_every_variant_gives_the_same_answer(gpu):
    coords, wn = synth.we_inputs(600, seed=4, batch=2, d_model=160)
    g = torch.Generator().manual_seed(4)
    mask = torch.rand(2, 600, generator=g) < 0.2
    for t, name in enumerate(_lib.we_variants()):
        check(run_gpu(gpu, coords, wn, mask, tuning=t), coords, wn, mask, what=f"variant {name}")


def test_without_sums_the_embedding_is_unchanged(gpu):
    """cos_sums = sin_sums = NULL selects kernels that skip the two sums; `out` must not depend on that."""
    for N, Z, d_model in ((600, 2, 160), (1500, 1, 512), (64, 3, 16)):
        coords, wn = synth.we_inputs(N, seed=N, batch=Z, d_model=d_model)
        g = torch.Generator().manual_seed(N)
        mask = torch.rand(Z, N, generator=g) < 0.2
        c, w, m = coords.to(gpu), wn.to(gpu), mask.to(gpu)
        for t, name in enumerate(_lib.we_variants()):
            full, cs, ss = pa.we_forward(c, w, m, tuning=t)
            lean, none_c, none_s = pa.we_forward(c, w, m, tuning=t, need_sums=False)
            assert none_c is None and none_s is None
            assert torch.equal(full, lean), f"variant {name}, N={N}"


def test_operator_computes_the_sums_only_when_a_backward_can_follow(gpu):
    # the autograd operator asks for the sums (what its backward consumes) only when autograd is recording and the
    # wavenumbers want a gradient: not under no_grad / inference_mode, whatever requires_grad says
    import importlib
    wfe = importlib.import_module("proteusai_amd.wf_embedding")       # (the package attribute of that name is the operator)
    coords, wn = synth.we_inputs(200, seed=3, batch=2, d_model=32)
    c, w = coords.to(gpu), wn.to(gpu).requires_grad_(True)
    seen, real = [], wfe.we_forward

    def spy(*args, **kwargs):
        seen.append(kwargs.get("need_sums"))
        return real(*args, **kwargs)
    wfe.we_forward = spy
    try:
        with torch.no_grad():
            y0 = pa.wf_embedding(c, w)
        with torch.inference_mode():
            pa.wf_embedding(c, w)
        y1 = pa.wf_embedding(c, w)
        y2 = pa.wf_embedding(c, w.detach())
    finally:
        wfe.we_forward = real
    assert seen == [False, False, True, False]
    assert y1.requires_grad and not y0.requires_grad and not y2.requires_grad and torch.equal(y0, y1.detach())
    y1.sum().backward()
    assert w.grad is not None and torch.isfinite(w.grad).all()


def test_masks(gpu):
    N = 333
    coords, wn = synth.we_inputs(N, seed=5, batch=4, d_model=64)
    g = torch.Generator().manual_seed(5)
    mask = torch.zeros(4, N, dtype=torch.bool)
    mask[0] = torch.rand(N, generator=g) < 0.5          # scattered
    mask[1, 100:] = True                                # tail padding
    mask[2] = True                                      # everything padded
    mask[3] = True
    mask[3, 17] = False                                 # a single survivor sees nobody
    got = run_gpu(gpu, coords, wn, mask)
    check(got, coords, wn, mask, what="masks")
    for a in got:
        assert (a[mask] == 0).all()
        assert (a[2] == 0).all() and (a[3] == 0).all()
    # padded sources contribute nothing: identical to running on the compacted sequence
    keep = ~mask[0]
    sub = run_gpu(gpu, coords[0:1, keep], wn)
    for a, b in zip(got, sub):
        assert rel_l2(a[0][keep.numpy()], b[0]) < 1e-5
    # what padded positions hold (NaN, Inf, huge) reaches nothing: padded rows stay exact zeros, valid rows keep their values
    junk = torch.tensor([float("nan"), float("inf"), -float("inf"), 3e38, -1e30])
    dirty = coords.clone()
    dirty[mask] = junk[torch.randint(0, 5, (int(mask.sum()), 3), generator=g)]
    for tuning in range(len(_lib.we_variants())):
        bad = run_gpu(gpu, dirty, wn, mask, tuning=tuning)
        for a, b in zip(bad, got):
            assert np.isfinite(a).all(), f"variant {tuning}"
            assert (a[mask.numpy()] == 0).all()
            assert rel_l2(a, b) < 1e-5
    no_sums = pa.we_forward(dirty.to(gpu), wn.to(gpu), mask.to(gpu), need_sums=False)[0].cpu().numpy()
    assert np.isfinite(no_sums).all() and (no_sums[mask.numpy()] == 0).all() and rel_l2(no_sums, got[0]) < 1e-5


def test_coincident_points_and_reference_sentinel(gpu):
    coords, wn = synth.we_inputs(90, seed=6, d_model=32)
    coords[0, 40] = coords[0, 12]                     # coincident pair -> dropped like the self pair
    # the reference's in-band mask value is an ordinary coordinate here: move the chain so that token 50 sits
    # at x == 12345.0 exactly (a lone far-away point would only test fp32's phase rounding at thousands of turns)
    coords[0, :, 0] += 12345.0 - coords[0, 50, 0]
    coords[0, 50, 0] = 12345.0
    check(run_gpu(gpu, coords, wn), coords, wn, what="coincident")


def test_large_phases(gpu):
    # |k r| far beyond 256 revolutions: range reduction must hold (both signs of k)
    g = torch.Generator().manual_seed(7)
    coords = torch.randn(1, 128, 3, generator=g) * 3000.0
    wn = torch.tensor([2.5, -2.5, 0.001, 1.0])
    got = run_gpu(gpu, coords, wn)
    ref = c_oracle.we(coords.numpy(), wn.numpy(), precision="f32")
    # at ~1e4 rad the float32 phase itself carries ~1e-3 rad of rounding: compare loosely, demand sanity
    for a, r in zip(got, ref):
        assert np.isfinite(a).all() and rel_l2(a, r) < 5e-2


def test_soa_layout_through_raw_c_abi(gpu):
    # the layout the reference's wrapper hands its kernel: [Z,3,N]
    coords, wn = synth.we_inputs(200, seed=8, batch=2, d_model=48)
    lib = _lib.load()
    Z, N, K = 2, 200, 24
    c = coords.transpose(1, 2).contiguous().to(gpu)
    w = wn.to(gpu)
    out = torch.full((Z, N, 2 * K), float("nan"), device=gpu)
    cs = torch.full((Z, N, K), float("nan"), device=gpu)
    ss = torch.full((Z, N, K), float("nan"), device=gpu)
    rc = lib.proteus_we_fwd(c.data_ptr(), _lib.COORDS_SOA, w.data_ptr(), None, out.data_ptr(), cs.data_ptr(), ss.data_ptr(),
                            Z, N, K, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    check((out.cpu().numpy(), cs.cpu().numpy(), ss.cpu().numpy()), coords, wn, what="SoA")


def test_outputs_fully_overwritten_and_no_out_of_bounds_writes(gpu):
    # canaries around each output buffer; outputs pre-filled with NaN
    coords, wn = synth.we_inputs(130, seed=9, d_model=70)
    lib = _lib.load()
    Z, N, K, pad = 1, 130, 35, 64
    bufs = []
    for n in (Z * N * 2 * K, Z * N * K, Z * N * K):
        b = torch.full((n + 2 * pad,), -777.0, device=gpu)
        b[pad:pad + n] = float("nan")
        bufs.append(b)
    c, w = coords.to(gpu), wn.to(gpu)
    ptrs = [b.data_ptr() + 4 * pad for b in bufs]
    rc = lib.proteus_we_fwd(c.data_ptr(), _lib.COORDS_AOS, w.data_ptr(), None, ptrs[0], ptrs[1], ptrs[2], Z, N, K, 0,
                            torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    for b, n in zip(bufs, (Z * N * 2 * K, Z * N * K, Z * N * K)):
        h = b.cpu()
        assert (h[:pad] == -777.0).all() and (h[pad + n:] == -777.0).all(), "write outside the output"
        assert torch.isfinite(h[pad:pad + n]).all(), "output not fully overwritten"


def test_deterministic(gpu):
    coords, wn = synth.we_inputs(1024, seed=11, d_model=128)
    a = run_gpu(gpu, coords, wn, tuning=1)
    b = run_gpu(gpu, coords, wn, tuning=1)
    assert all(np.array_equal(x, y) for x, y in zip(a, b))


def test_autograd_function_and_module(gpu):
    # wf_embedding returns only `out`; backward gives dk from the saved sums (isotropic/cuda/wf_embedding.py:64-83)
    coords, _ = synth.we_inputs(96, seed=12, batch=2)
    mask = torch.zeros(2, 96, dtype=torch.bool)
    mask[1, 70:] = True
    mod = pa.WaveFunctionEmbedding(d_wf=64, min_wl=3.7, max_wl=20.0, base_wl=20.0, anisotropic=False, learn_wl=True).to(gpu)
    out = mod(coords.to(gpu), None, key_padding_mask=mask.to(gpu))
    assert out.shape == (2, 96, 64) and out.dtype == torch.float32
    g = torch.Generator().manual_seed(1)
    dO = torch.randn(2, 96, 64, generator=g)
    (out * dO.to(gpu)).sum().backward()
    # autograd through the dense float64 statement, chained through exp(log k)
    logk = mod.wavenumbers.detach().cpu().double().requires_grad_(True)
    k = torch.exp(logk)
    c = coords.double()
    d = torch.sqrt(((c[:, :, None] - c[:, None]) ** 2).sum(-1))
    bad = mask[:, :, None] | mask[:, None, :] | (d == 0)
    mag = 1 / torch.where(bad, torch.full_like(d, float("inf")), d)
    ph = d[..., None] * k
    feats = torch.stack([(mag[..., None] * torch.cos(ph)).sum(2), (mag[..., None] * torch.sin(ph)).sum(2)], -1).flatten(2)
    (feats * dO.double()).sum().backward()
    assert rel_l2(out.detach().cpu().numpy(), feats.detach().numpy()) <= REL_L2_TOL
    assert rel_l2(mod.wavenumbers.grad.cpu().numpy(), logk.grad.numpy()) <= 1e-3


def test_input_dtypes_are_cast_like_the_reference(gpu):
    coords, wn = synth.we_inputs(64, seed=13, d_model=32)
    a = pa.we_forward(coords.double().to(gpu), wn.double().to(gpu))
    b = pa.we_forward(coords.to(gpu), wn.to(gpu))
    assert all(torch.equal(x, y) for x, y in zip(a, b)) and a[0].dtype == torch.float32


def test_cfg2_sampled_rows(gpu):
    # B=1, N=16384, d_model=512, compacted chain: 256 full rows (tile boundaries and ends included) against the oracle
    coords, wn = synth.we_inputs(16384, seed=2, compact=True)
    got = run_gpu(gpu, coords, wn)
    rows = sample_rows(16384, 256, seed=2)
    assert len(rows) == 256
    check(got, coords, wn, rows=rows, what="cfg2")


def test_cfg2_size_independent_properties(gpu):
    coords, wn = synth.we_inputs(16384, seed=2, compact=True)
    out, cs, ss = run_gpu(gpu, coords, wn)
    # (1) rigid motion: the embedding only sees distances
    g = torch.Generator().manual_seed(3)
    q, r = torch.linalg.qr(torch.randn(3, 3, generator=g, dtype=torch.float64))
    moved = (coords.double() @ q.T).float()
    out2, cs2, ss2 = run_gpu(gpu, moved, wn)
    assert rel_l2(out2, out) < 2e-4 and rel_l2(cs2, cs) < 2e-4
    # (2) reversing the chain permutes the rows and nothing else
    out3, cs3, ss3 = run_gpu(gpu, coords.flip(1), wn)
    assert rel_l2(out3[:, ::-1], out) < 1e-5 and rel_l2(ss3[:, ::-1], ss) < 1e-5
    # (3) sum over observers of cos_sums is symmetric in the pair: sum_i cs[i,k] = 2 sum_{i<j} cos(k r_ij);
    #     check through the k -> 0 channel instead: a zero wavenumber counts the valid partners exactly
    o0, c0, s0 = run_gpu(gpu, coords, torch.zeros(1))
    assert np.array_equal(c0[0, :, 0], np.full(16384, 16383.0, np.float32)) and (s0 == 0).all()


def test_cfg5_stress_sampled_rows(gpu):
    # B=1, N=65536, d_model=512: 256 full rows (rows are independent, so each is an exact check), ends and tile boundaries included
    coords, wn = synth.we_inputs(65536, seed=5, compact=True)
    got = run_gpu(gpu, coords, wn)
    rows = sample_rows(65536, 256, seed=5)
    assert len(rows) == 256
    check(got, coords, wn, rows=rows, what="cfg5")


def test_cfg4_batch_with_padding(gpu):
    # the encoder configuration's WE call: B=8, N=1024, lengths in [128, 1024]
    coords, wn = synth.we_inputs(1024, seed=4, batch=8)
    g = torch.Generator().manual_seed(4)
    lens = torch.randint(128, 1025, (8,), generator=g)
    mask = torch.arange(1024)[None, :] >= lens[:, None]
    got = run_gpu(gpu, coords, wn, mask)
    rows = sample_rows(1024, 128, seed=4)
    check(got, coords, wn, mask, rows=rows, what="cfg4")


@pytest.mark.parametrize("N,d_model,kind", [(640, 64, "ties"), (520, 128, "unaligned"), (1024, 512, "many"), (512, 32, "few tiles")])
def test_padded_batches_handed_out_by_their_number_of_sources(gpu, N, d_model, kind):
    # Padded batches of 2 .. 64 items with N >= 512 (up to 4096 workgroups): every workgroup ranks the items by their number
    # of unpadded sources and takes its place in a list laid over the launch as a snake.  Every (item, observer block,
    # wavenumber tile) must still be done exactly once: full rows against the oracle, and exact zeros on padded rows
    # of an output that was filled with NaN.
    g = torch.Generator().manual_seed(N)
    if kind == "ties":          # equal counts, an empty item, lengths on and beside the 64-row block borders, a scattered mask
        lens = [640, 64, 640, 0, 65, 63, 320, 1]
        Z = len(lens)
        mask = torch.arange(N)[None, :] >= torch.tensor(lens)[:, None]
        mask = torch.cat([mask, (torch.rand(1, N, generator=g) < 0.6)], 0)      # fewer sources than its last token says
        mask[-1, 600] = False
        Z += 1
    elif kind == "unaligned":   # rows of the mask that are not multiples of 16 bytes: the byte-wise scan
        Z = 5
        lens = torch.randint(1, N + 1, (Z,), generator=g)
        mask = torch.arange(N)[None, :] >= lens[:, None]
    elif kind == "many":        # 4 items x 16 blocks x 16 wavenumber tiles: several rows of the snake, the last one partial
        Z = 4
        lens = torch.tensor([1024, 130, 777, 512])
        mask = torch.arange(N)[None, :] >= lens[:, None]
    else:                       # 64 items, the most that are ranked
        Z = 64
        lens = torch.randint(0, N + 1, (Z,), generator=g)
        mask = torch.arange(N)[None, :] >= lens[:, None]
    coords, wn = synth.we_inputs(N, seed=N, batch=Z, d_model=d_model)
    K = wn.numel()
    for sums in (True, False):
        c, w, m = coords.to(gpu), wn.to(gpu), mask.to(gpu)
        got = pa.we_forward(c, w, m, need_sums=sums)
        out = got[0].cpu().numpy()
        assert np.isfinite(out).all() and (out[mask.numpy()] == 0).all(), f"{kind} sums={sums}"
        ref = c_oracle.we(coords.numpy(), wn.numpy(), mask.numpy(), precision="f32")
        assert rel_l2(out, ref[0]) <= REL_L2_TOL, f"{kind} sums={sums}: {rel_l2(out, ref[0]):.3e}"
        if sums:
            for a, r, name in zip(got[1:], ref[1:], ("cos_sums", "sin_sums")):
                a = a.cpu().numpy()
                assert (a[mask.numpy()] == 0).all() and rel_l2(a, r) <= REL_L2_TOL, f"{kind} {name}"
    # the anisotropic kernel takes its workgroups in the same order
    gb = torch.Generator().manual_seed(N + 1)
    cb_dir = torch.randn(Z, N, 3, generator=gb)
    cb_dir = cb_dir / cb_dir.norm(dim=-1, keepdim=True)
    cb = torch.rand(K, generator=gb) * 4 - 2
    got = pa.we_aniso_forward(coords.to(gpu), cb_dir.to(gpu), cb.to(gpu), wn.to(gpu), mask.to(gpu))
    ref = c_oracle.we_aniso(coords.numpy(), cb_dir.numpy(), cb.numpy(), wn.numpy(), mask.numpy())
    for a, r, name in zip(got, ref, ("out", "d_cb", "d_k")):
        a = a.cpu().numpy()
        assert np.isfinite(a).all() and (a[mask.numpy()] == 0).all() and rel_l2(a, r) <= REL_L2_TOL, f"{kind} anisotropic {name}: {rel_l2(a, r):.3e}"
    # through the raw entry point into buffers full of NaN, every tile width: nothing left unwritten, nothing written twice differently
    lib = _lib.load()
    c, w, m = coords.to(gpu).contiguous(), wn.to(gpu), mask.to(gpu).view(torch.uint8).contiguous()
    base = None
    for tuning in range(len(_lib.we_variants())):
        bufs = [torch.full((Z, N, 2 * K), float("nan"), device=gpu), torch.full((Z, N, K), float("nan"), device=gpu),
                torch.full((Z, N, K), float("nan"), device=gpu)]
        rc = lib.proteus_we_fwd(c.data_ptr(), 1, w.data_ptr(), m.data_ptr(), bufs[0].data_ptr(), bufs[1].data_ptr(), bufs[2].data_ptr(),
                                Z, N, K, tuning, None)
        assert rc == 0
        torch.cuda.synchronize()
        o = bufs[0].cpu().numpy()
        assert all(torch.isfinite(b).all() for b in bufs), f"{kind} variant {tuning}"
        if base is None:
            base = o
        assert rel_l2(o, base) < 1e-5, f"{kind} variant {tuning}"


def test_hardware_sincos_and_sqrt_error(gpu):
    # the stated fp32 error of the fast path: v_sin_f32 / v_cos_f32 on revolutions, with and without the
    # explicit range reduction, and r = r2*rsq(r2) with one Newton step (measurement probes: their own library)
    from proteusai_amd import _probes
    lib = _probes.load()
    g = torch.Generator().manual_seed(0)
    n = 1 << 20
    x = ((torch.rand(n, generator=g, dtype=torch.float64) - 0.5) * 500.0).float()      # |x| < 250 revolutions
    xd = x.to(gpu)
    s, c, q = torch.empty_like(xd), torch.empty_like(xd), torch.empty_like(xd)
    ph = 2 * np.pi * (x.double().numpy() % 1.0)
    for use_fract in (1, 0):
        rc = lib.proteus_probe_sincos(xd.data_ptr(), s.data_ptr(), c.data_ptr(), q.data_ptr(), n, use_fract, None)
        assert rc == 0
        torch.cuda.synchronize()
        es = np.abs(s.cpu().numpy() - np.sin(ph)).max()
        ec = np.abs(c.cpu().numpy() - np.cos(ph)).max()
        assert es < 5e-7 and ec < 5e-7, (use_fract, es, ec)
    r2 = (torch.rand(n, generator=g, dtype=torch.float64) * 1e6).float()
    rd = r2.to(gpu)
    rc = lib.proteus_probe_sincos(rd.data_ptr(), s.data_ptr(), c.data_ptr(), q.data_ptr(), n, 1, None)
    assert rc == 0
    torch.cuda.synchronize()
    ref = np.sqrt(r2.double().numpy())
    assert (np.abs(q.cpu().numpy() - ref) / np.maximum(ref, 1e-30)).max() < 1.2e-7


@pytest.mark.parametrize("mag_type", [0, 2, 3])
@pytest.mark.parametrize("N,Z,K", [(300, 2, 40), (2048, 1, 256)])
def test_other_source_weights(gpu, mag_type, N, Z, K):
    # the reference's magnitude_type 0 / 2 / 3 (isotropic/cuda/wf_embedding_kernel.cu:192-206), both tilings
    coords, _ = synth.we_inputs(N, seed=40 + mag_type, batch=Z)
    wn = synth.wavenumbers(2 * K)
    mask = torch.rand(Z, N, generator=torch.Generator().manual_seed(N)) < 0.2
    got = pa.we_forward(coords.to(gpu), wn.to(gpu), mask.to(gpu), magnitude_type=mag_type)
    rows = None if N <= 512 else np.arange(0, N, 37)
    ref = c_oracle.we(coords.numpy(), wn.numpy(), mask.numpy(), rows=rows, mag_type=mag_type)
    sel = slice(None) if rows is None else rows
    for g, r, name in zip(got, ref, ("out", "cos_sums", "sin_sums")):
        g = g.cpu().numpy()
        assert (g[mask.numpy()] == 0).all()
        assert rel_l2(g[:, sel], r) <= REL_L2_TOL, f"magnitude_type {mag_type} {name}: {rel_l2(g[:, sel], r):.3e}"
    # and through the autograd function: the backward consumes these sums unchanged
    w = wn.to(gpu).requires_grad_(True)
    out = pa.wf_embedding(coords.to(gpu), w, magnitude_type=mag_type, mask=mask.to(gpu))
    out.sum().backward()
    dk = torch_oracle.we_backward_torch(torch.ones(Z, N if rows is None else len(rows), 2 * K, dtype=torch.float64),
                                        torch.from_numpy(ref[1]), torch.from_numpy(ref[2]))
    if rows is None:
        assert rel_l2(w.grad.cpu().numpy(), dk.numpy()) <= REL_L2_TOL
