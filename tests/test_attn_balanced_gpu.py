"""GPU tests of the two schedules of the attention forward for padded batches (proteus_geo_attn_fwd_ws): the key
tiles of one (batch, head, query tile) item may go to several workgroups, whose partial softmax states meet in a
caller-provided workspace -- as equal shares of all steps over a persistent grid ("balanced") or as equal parts of
the long items, handed out longest first ("split_items", what a padded batch of long sequences gets by itself).
Checked against the CPU oracle at the forward's bars (max |O - O_ref| <= 2e-2, logsumexp <= 4e-3, exact zeros / -inf on
padded rows) and against the plain grid on every row."""
import ctypes

import numpy as np
import pytest
import torch

import proteusai_amd as pa
from oracle import c_oracle
from proteusai_amd import _lib, synth

pytestmark = pytest.mark.gpu

MAX_ABS_TOL = 2e-2
LSE_TOL = 4e-3
BALANCED = 8            # tuning selector: the balanced schedule wherever it is possible
SPLIT = 9               # long items split, longest parts first, wherever it is possible
PLAIN = 5               # the pipelined kernel on the plain grid


@pytest.fixture(params=[BALANCED, SPLIT], ids=["balanced", "split_items"])
def sched(request):
    return request.param


def make(seed, Z, H, N, qscale=1.0):
    g = torch.Generator().manual_seed(seed)
    Q = (torch.randn(Z, H, N, 64, generator=g) * qscale).bfloat16()
    K = (torch.randn(Z, H, N, 64, generator=g) * qscale).bfloat16()
    V = torch.randn(Z, H, N, 64, generator=g).bfloat16()
    coords = torch.stack([synth.random_walk_chain(N, g) for _ in range(Z)])
    return Q, K, V, coords, synth.log_spaced_sigma(H), g


def run(gpu, Q, K, V, coords, sigma, mask, tuning):
    O, L = pa.geo_attn(Q.to(gpu), K.to(gpu), V.to(gpu), coords.to(gpu), sigma.to(gpu), None if mask is None else mask.to(gpu),
                       return_lse=True, tuning=tuning)
    torch.cuda.synchronize()
    return O.cpu().numpy(), L.cpu().numpy()


def check_oracle(got, Q, K, V, coords, sigma, mask, rows, what):
    O, L = got
    Or, Lr = c_oracle.geo_attn(Q.float().numpy(), K.float().numpy(), V.float().numpy(), coords.numpy(), sigma.numpy(),
                               None if mask is None else mask.numpy(), rows=rows)
    sel = slice(None) if rows is None else np.asarray(rows)
    O, L = O[:, :, sel].astype(np.float64), L[:, :, sel].astype(np.float64)
    assert np.isfinite(O).all(), what
    assert np.abs(O - Or).max() <= MAX_ABS_TOL, f"{what}: max abs error {np.abs(O - Or).max():.3e}"
    fin = np.isfinite(Lr)
    assert (np.isneginf(L) == ~fin).all(), f"{what}: -inf pattern of L differs"
    if fin.any():
        assert np.abs(L[fin] - Lr[fin]).max() <= LSE_TOL, f"{what}: logsumexp error {np.abs(L[fin] - Lr[fin]).max():.3e}"
    assert (O[~fin] == 0).all(), f"{what}: padded / empty rows must be exactly zero"


def check_against_plain(bal, plain, what, bar=5e-3):
    # the two schedules differ in where a query's softmax reference was last re-based, i.e. in how single
    # probabilities were rounded to bf16 (2^-9 each, averaged over the keys: more where few keys carry the weight)
    (Ob, Lb), (Op, Lp) = bal, plain
    fin = np.isfinite(Lp)
    assert (np.isneginf(Lb) == ~fin).all(), what
    assert np.abs(Ob - Op).max() <= bar, f"{what}: |O_balanced - O_plain| {np.abs(Ob - Op).max():.3e}"
    assert np.abs(Lb[fin] - Lp[fin]).max() <= 2 * LSE_TOL, what          # each within LSE_TOL of the exact value
    assert (Ob[~fin] == 0).all(), what


def tail_mask(Z, N, g, lo):
    lens = torch.randint(lo, N + 1, (Z,), generator=g)
    return torch.arange(N)[None, :] >= lens[:, None], lens


def test_library_takes_the_balanced_schedule_where_these_tests_expect_it():
    lib = _lib.load()
    assert lib.proteus_geo_attn_fwd_workspace_bytes(4, 8, 4096, 64, 0) > 0        # BASELINE configs[2]: automatic
    assert lib.proteus_geo_attn_fwd_workspace_bytes(8, 8, 1024, 64, 0) == 0       # the encoder's batch: plain grid
    assert lib.proteus_geo_attn_fwd_workspace_bytes(8, 8, 1024, 64, BALANCED) > 0
    assert lib.proteus_geo_attn_fwd_workspace_bytes(3, 2, 700, 32, BALANCED) == 0     # d_head = 64 only
    assert lib.proteus_geo_attn_fwd_workspace_bytes(300, 2, 700, 64, BALANCED) == 0   # at most 256 batch items
    assert lib.proteus_geo_attn_fwd_workspace_bytes(3, 2, 700, 64, PLAIN) == 0
    assert lib.proteus_geo_attn_fwd_workspace_bytes(16, 8, 1024, 64, 0) > 0       # 8192 steps of sequences of 1024 tokens
    assert lib.proteus_geo_attn_fwd_workspace_bytes(8, 8, 1024, 64, SPLIT) > 0
    assert lib.proteus_geo_attn_fwd_workspace_bytes(3, 2, 700, 32, SPLIT) == 0
    assert lib.proteus_geo_attn_fwd_workspace_bytes(300, 2, 700, 64, SPLIT) == 0
    names = _lib.geo_attn_variants()
    assert names[BALANCED] == "balanced" and names[SPLIT] == "split_items" and names[PLAIN] == "pipelined"


@pytest.mark.parametrize("Z,H,N,lo,qscale", [
    (3, 2, 700, 100, 1.0),          # a few steps per item: one step per workgroup (balanced: up to 11 parts per item)
    (2, 3, 1000, 500, 1.0),         # N not a multiple of the key tile or the query tile
    (5, 4, 2600, 300, 1.0),         # shares of a few tiles: parts of two or three items per workgroup
    (1, 4, 8192, 8192, 1.0),        # nothing padded: whole items, nothing to merge but a part per item
    (2, 2, 4100, 1, 4.0),           # lengths from 1 on, large logits (re-based references differ between parts)
    (37, 1, 520, 1, 1.0),           # many short sequences of every length (equal ones too): their ranking, single heads
])
def test_tail_padding_against_oracle_and_plain_grid(gpu, sched, Z, H, N, lo, qscale):
    Q, K, V, coords, sigma, g = make(Z * 1000 + N, Z, H, N, qscale)
    mask, lens = tail_mask(Z, N, g, lo)
    bal = run(gpu, Q, K, V, coords, sigma, mask, sched)
    plain = run(gpu, Q, K, V, coords, sigma, mask, PLAIN)
    what = f"Z={Z} H={H} N={N} lengths {lens.tolist()}"
    check_against_plain(bal, plain, what, bar=5e-3 if qscale <= 1.0 else 1.5e-2)
    rows = None if Z * H * N <= 9000 else np.unique(np.concatenate([
        np.random.default_rng(N).choice(N, 96, replace=False), [0, 63, 64, 255, 256, N - 1],
        np.clip(np.concatenate([lens.numpy() - 1, lens.numpy()]), 0, N - 1)])).astype(np.int32)
    check_oracle(bal, Q, K, V, coords, sigma, mask, rows, what)
    # a second call on the same inputs (fresh workspace, counters zeroed again by the plan): the parts of an item are
    # added in a fixed order, whoever finishes last, so the result is the same to the bit
    again = run(gpu, Q, K, V, coords, sigma, mask, sched)
    assert np.array_equal(bal[0], again[0]) and np.array_equal(bal[1], again[1])


def test_scattered_padding_empty_sequence_and_padded_query_tiles(gpu, sched):
    Z, H, N = 4, 2, 1500
    Q, K, V, coords, sigma, g = make(7, Z, H, N)
    mask = torch.zeros(Z, N, dtype=torch.bool)
    mask[0] = torch.rand(N, generator=g) < 0.4                  # scattered
    mask[1] = True                                              # a whole sequence padded: no item at all
    mask[2, 256:768] = True                                     # two query tiles whose queries are all padded, keys beyond them valid
    mask[2, 1400:] = True
    mask[3, 5:] = True                                          # five tokens
    # what padded tokens hold must not matter
    Qn, Kn, Vn, cn = Q.clone(), K.clone(), V.clone(), coords.clone()
    for t in (Qn, Kn, Vn):
        t.transpose(1, 2)[mask] = float("nan")
    cn[mask] = float("inf")
    bal = run(gpu, Q, K, V, coords, sigma, mask, sched)
    baln = run(gpu, Qn, Kn, Vn, cn, sigma, mask, sched)
    assert np.array_equal(bal[0], baln[0]) and np.array_equal(bal[1], baln[1])
    check_against_plain(bal, run(gpu, Q, K, V, coords, sigma, mask, PLAIN), "scattered")
    check_oracle(bal, Q, K, V, coords, sigma, mask, None, "scattered")
    assert (bal[0][1] == 0).all() and np.isneginf(bal[1][1]).all()


def test_cfg3_shape_takes_the_split_items_schedule_automatically(gpu):
    # BASELINE configs[2]: B=4, H=8, N=4096, lengths in [2048, 4096]; tuning 0 through the operator
    Q, K, V, coords, sigma, mask = synth.attn_inputs(4, 8, 4096, 64, seed=3, min_len=2048)
    auto = run(gpu, Q, K, V, coords, sigma, mask, 0)
    forced = run(gpu, Q, K, V, coords, sigma, mask, SPLIT)
    assert np.array_equal(auto[0], forced[0]) and np.array_equal(auto[1], forced[1])
    check_against_plain(auto, run(gpu, Q, K, V, coords, sigma, mask, PLAIN), "cfg3")
    rows = np.unique(np.concatenate([np.random.default_rng(3).choice(4096, 120, replace=False), [0, 255, 256, 2047, 2048, 4095]])).astype(np.int32)
    check_oracle(auto, Q, K, V, coords, sigma, mask, rows, "cfg3")


def test_unmasked_sequences_that_do_not_fill_the_chip_are_split_by_themselves(gpu):
    # one sequence of 4096 tokens at 4 heads: 64 items for 512 workgroup slots.  Without a mask the operator still
    # brings a workspace, and the library splits every item into parts (tuning 0 = the split-items schedule here).
    lib = _lib.load()
    assert lib.proteus_geo_attn_fwd_workspace_bytes(1, 4, 4096, 64, 0) > 0
    Q, K, V, coords, sigma, g = make(21, 1, 4, 4096)
    auto = run(gpu, Q, K, V, coords, sigma, None, 0)
    forced = run(gpu, Q, K, V, coords, sigma, None, SPLIT)
    assert np.array_equal(auto[0], forced[0]) and np.array_equal(auto[1], forced[1])
    plain = run(gpu, Q, K, V, coords, sigma, None, PLAIN)
    assert not np.array_equal(auto[0], plain[0])                     # (another schedule did run)
    check_against_plain(auto, plain, "unmasked 1x4x4096")
    rows = np.unique(np.concatenate([np.random.default_rng(21).choice(4096, 100, replace=False), [0, 255, 256, 4095]])).astype(np.int32)
    check_oracle(auto, Q, K, V, coords, sigma, None, rows, "unmasked 1x4x4096")
    # the raw entry point with a NULL mask, N not a multiple of any tile
    Z, H, N, d = 2, 3, 2500, 64
    Q, K, V, coords, sigma, g = make(22, Z, H, N)
    want = run(gpu, Q, K, V, coords, sigma, None, PLAIN)
    q, k, v, c, s = (t.to(gpu) for t in (Q, K, V, coords, sigma))
    O = torch.full((Z, H, N, d), float("nan"), device=gpu)
    L = torch.full((Z, H, N), float("nan"), device=gpu)
    nbytes = lib.proteus_geo_attn_fwd_workspace_bytes(Z, H, N, d, 0)
    assert nbytes > 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device=gpu)
    rc = lib.proteus_geo_attn_fwd_ws(q.data_ptr(), k.data_ptr(), v.data_ptr(), None, c.data_ptr(), s.data_ptr(), None,
                                     O.data_ptr(), L.data_ptr(), ws.data_ptr(), nbytes, Z, H, N, d, 0,
                                     ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    check_against_plain((O.cpu().numpy(), L.cpu().numpy()), want, "raw, no mask")


def test_tokens_too_far_apart_for_the_matrix_core_distances_take_direct_distances(gpu, sched):
    # a straight chain: the 256 tokens of a query tile span 970 A, far beyond what the matrix-core distances of the
    # pipelined body resolve at sigma = 3 A.  The plan marks the tiles and the persistent grid runs the direct-distance
    # body over whole items instead.
    Z, H, N = 2, 2, 1300
    Q, K, V, _, sigma, g = make(11, Z, H, N)
    coords = torch.zeros(Z, N, 3)
    coords[:, :, 0] = 3.8 * torch.arange(N)
    mask, lens = tail_mask(Z, N, g, 700)
    bal = run(gpu, Q, K, V, coords, sigma, mask, sched)
    check_against_plain(bal, run(gpu, Q, K, V, coords, sigma, mask, PLAIN), "straight chain")
    direct = run(gpu, Q, K, V, coords, sigma, mask, 2)              # direct distances on the plain grid (the launcher's tile shape)
    assert np.abs(bal[0] - direct[0]).max() <= 2e-3 and np.array_equal(np.isneginf(bal[1]), np.isneginf(direct[1]))
    check_oracle(bal, Q, K, V, coords, sigma, mask, None, "straight chain")
    # more items than persistent workgroups: every workgroup takes several in turn
    Z, H, N = 5, 16, 2100
    Q = (torch.randn(Z, H, N, 64, generator=g)).bfloat16()
    K = (torch.randn(Z, H, N, 64, generator=g)).bfloat16()
    V = torch.randn(Z, H, N, 64, generator=g).bfloat16()
    coords = torch.zeros(Z, N, 3)
    coords[:, :, 1] = 3.8 * torch.arange(N)
    sigma = synth.log_spaced_sigma(H)
    mask, lens = tail_mask(Z, N, g, 900)
    bal = run(gpu, Q, K, V, coords, sigma, mask, sched)
    rows = np.unique(np.concatenate([np.random.default_rng(5).choice(N, 40, replace=False), [0, 255, 256, N - 1]])).astype(np.int32)
    check_oracle(bal, Q, K, V, coords, sigma, mask, rows, "straight chain, 720 items")


def test_raw_c_abi_strided_operands_no_lse_workspace_canary_and_reuse(gpu, sched):
    lib = _lib.load()
    Z, H, N, d = 2, 4, 1800, 64
    Q, K, V, coords, sigma, g = make(13, Z, H, N)
    mask, _ = tail_mask(Z, N, g, 600)
    want = run(gpu, Q, K, V, coords, sigma, mask, PLAIN)
    # operands as slices of a fused projection [Z,N,3,H,d], O token-major
    qkv = torch.stack([t.permute(0, 2, 1, 3) for t in (Q, K, V)], dim=2).contiguous().to(gpu)        # [Z,N,3,H,d]
    q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    O = torch.full((Z, N, H, d), float("nan"), device=gpu).permute(0, 2, 1, 3)
    nbytes = lib.proteus_geo_attn_fwd_workspace_bytes(Z, H, N, d, sched)
    assert nbytes > 0 and nbytes % 256 == 0
    ws = torch.full((nbytes + 4096,), 0xA5, dtype=torch.uint8, device=gpu)
    c, s, m = coords.to(gpu), sigma.to(gpu), mask.to(gpu).view(torch.uint8)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for _ in range(2):                                   # the second call finds the first one's counters and parts
        rc = lib.proteus_geo_attn_fwd_ws(q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.stride_array(q, k, v, O),
                                         c.data_ptr(), s.data_ptr(), m.data_ptr(), O.data_ptr(), None,
                                         ws.data_ptr(), nbytes, Z, H, N, d, sched, stream)
        assert rc == 0, lib.proteus_strerror(rc)
        torch.cuda.synchronize()
        got = O.cpu().numpy()
        assert np.isfinite(got).all()
        check_against_plain((got, want[1]), want, "strided")
        assert (ws[nbytes:] == 0xA5).all()               # nothing written behind the workspace
    # too small a workspace, or none: the call is the plain one
    O2 = torch.full((Z, H, N, d), float("nan"), device=gpu)
    L2 = torch.full((Z, H, N), float("nan"), device=gpu)
    qc, kc, vc = Q.to(gpu), K.to(gpu), V.to(gpu)
    rc = lib.proteus_geo_attn_fwd_ws(qc.data_ptr(), kc.data_ptr(), vc.data_ptr(), None, c.data_ptr(), s.data_ptr(), m.data_ptr(),
                                     O2.data_ptr(), L2.data_ptr(), ws.data_ptr(), 1024, Z, H, N, d, 0, stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert np.array_equal(O2.cpu().numpy(), run(gpu, Q, K, V, coords, sigma, mask, 0)[0])
    # argument errors come back before any launch
    assert lib.proteus_geo_attn_fwd_ws(qc.data_ptr(), kc.data_ptr(), vc.data_ptr(), None, c.data_ptr(), s.data_ptr(), m.data_ptr(),
                                       O2.data_ptr(), None, None, 4096, Z, H, N, d, 0, stream) == -1
    assert lib.proteus_geo_attn_fwd_ws(qc.data_ptr(), kc.data_ptr(), vc.data_ptr(), None, c.data_ptr(), s.data_ptr(), m.data_ptr(),
                                       O2.data_ptr(), None, ws.data_ptr() + 8, nbytes, Z, H, N, d, 0, stream) == -5


def test_padded_schedules_replay_from_a_captured_graph(gpu, sched):
    Z, H, N = 3, 2, 1700
    Q, K, V, coords, sigma, g = make(17, Z, H, N)
    mask, _ = tail_mask(Z, N, g, 400)
    q, k, v, c, s, m = (t.to(gpu) for t in (Q, K, V, coords, sigma, mask))
    eager = pa.geo_attn(q, k, v, c, s, m, tuning=sched).clone()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        pa.geo_attn(q, k, v, c, s, m, tuning=sched)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = pa.geo_attn(q, k, v, c, s, m, tuning=sched, check_sigma=False)
    torch.cuda.synchronize()
    for _ in range(3):
        out.fill_(float("nan"))
        pa.geo_attn(q, k, v, c, s, m, tuning=sched)              # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)


@pytest.mark.parametrize("case", range(12))
def test_random_long_batches_through_the_operator(gpu, case):
    # what the operator does by itself (tuning 0: split items where the shape asks for it, the plain grid otherwise) and
    # both schedules forced, on random shapes with tail padding, scattered padding or none, against the oracle on sampled rows
    rng = np.random.default_rng(1000 + case)
    Z, H = int(rng.integers(1, 6)), int(rng.choice([1, 2, 3, 4, 8]))
    N = int(rng.integers(1024, 4200))
    Q, K, V, coords, sigma, g = make(5000 + case, Z, H, N, qscale=float(rng.choice([0.5, 1.0, 2.0])))
    sigma = torch.exp(torch.empty(H).uniform_(np.log(2.0), np.log(30.0), generator=g))
    kind = case % 3
    if kind == 0:
        mask = None
    elif kind == 1:
        mask, _ = tail_mask(Z, N, g, 1)
    else:
        mask, _ = tail_mask(Z, N, g, N // 3)
        mask |= torch.rand(Z, N, generator=g) < 0.1
    rows = np.unique(np.concatenate([rng.choice(N, 48, replace=False), [0, 255, 256, N - 1]])).astype(np.int32)
    what = f"case {case}: Z={Z} H={H} N={N} mask kind {kind}"
    auto = run(gpu, Q, K, V, coords, sigma, mask, 0)
    check_oracle(auto, Q, K, V, coords, sigma, mask, rows, what + " (automatic)")
    for tuning in (BALANCED, SPLIT):
        got = run(gpu, Q, K, V, coords, sigma, mask, tuning)
        check_oracle(got, Q, K, V, coords, sigma, mask, rows, what + f" (tuning {tuning})")
