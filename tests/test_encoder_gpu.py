"""GPU tests of the encoder stack built around the two kernels (BASELINE configuration 4)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import proteusai_amd as pa
from oracle import c_oracle, torch_oracle
from proteusai_amd import synth

pytestmark = pytest.mark.gpu


def reference_forward(model, coords, tokens, mask):
    """The same stack in fp32 on the CPU, with the oracles in place of the kernels (the C oracle for the attention)."""
    def attention(Q, K, V, c, sg, m):
        return torch.from_numpy(c_oracle.geo_attn(Q.numpy(), K.numpy(), V.numpy(), c.numpy(), sg.numpy(), m.numpy())[0]).float()
    return torch_oracle.encoder_forward_torch(model.state_dict(), model.layers[0].attn.min_spread, coords, tokens, mask, attention)


def test_small_encoder_matches_cpu_composition(gpu):
    torch.manual_seed(0)
    model = pa.ProteusEncoder(d_model=128, heads=2, layers=2, d_hidden=256).eval()
    g = torch.Generator().manual_seed(1)
    coords = torch.stack([synth.random_walk_chain(150, g) for _ in range(2)])
    tokens = torch.randint(0, 33, (2, 150), generator=g)
    mask = torch.zeros(2, 150, dtype=torch.bool)
    mask[1, 100:] = True
    ref = reference_forward(model, coords, tokens, mask)
    with torch.no_grad():
        out = model.to(gpu)(coords.to(gpu), tokens.to(gpu), mask.to(gpu)).cpu()
    valid = ~mask
    assert out.shape == (2, 150, 20) and torch.isfinite(out).all()
    # fp32 weights; the only low-precision step is the bf16 cast of Q, K, V and P inside the attention kernel
    assert (out[valid] - ref[valid]).abs().max() < 5e-2


def test_cfg4_shape_bf16_and_padding_independence(gpu):
    # B=8, N=1024, d_model=512, 4 layers, bf16 weights with fp32 WE, lengths in [128, 1024]
    torch.manual_seed(4)
    model = pa.ProteusEncoder().eval().to(gpu)
    model.aa_embedding.to(torch.bfloat16)
    model.layers.to(torch.bfloat16)
    model.head.to(torch.bfloat16)
    g = torch.Generator().manual_seed(4)
    coords = torch.stack([synth.random_walk_chain(1024, g) for _ in range(8)])
    tokens = torch.randint(0, 33, (8, 1024), generator=g)
    lens = torch.randint(128, 1025, (8,), generator=g)
    mask = torch.arange(1024)[None, :] >= lens[:, None]
    with torch.no_grad():
        out = model(coords.to(gpu), tokens.to(gpu), mask.to(gpu)).float().cpu()
        # what sits in padded positions must not influence the valid ones
        coords2, tokens2 = coords.clone(), tokens.clone()
        coords2[mask] = 777.0
        tokens2[mask] = 0
        out2 = model(coords2.to(gpu), tokens2.to(gpu), mask.to(gpu)).float().cpu()
    valid = ~mask
    assert out.shape == (8, 1024, 20) and torch.isfinite(out[valid]).all()
    assert torch.equal(out[valid], out2[valid])


def test_cfg4_shape_inference_path_equals_the_path_autograd_records(gpu):
    # Without gradients the layer's residual add + LayerNorm is one HIP kernel and the per-head constants are cached;
    # with gradients enabled the torch expressions run.  Same weights, same batch: the two forwards differ only by
    # how a bf16 result was rounded here and there (fp32 weights: by fp32 rounding, which the attention's cast of its
    # operands to bf16 turns into a flipped bf16 rounding now and then: measured 2.3e-4).
    g = torch.Generator().manual_seed(4)
    coords = torch.stack([synth.random_walk_chain(1024, g) for _ in range(8)]).to(gpu)
    tokens = torch.randint(0, 33, (8, 1024), generator=g).to(gpu)
    lens = torch.randint(128, 1025, (8,), generator=g)
    mask = (torch.arange(1024)[None, :] >= lens[:, None]).to(gpu)
    valid = ~mask.cpu()
    for dtype, bar in ((torch.float32, 2e-3), (torch.bfloat16, 3e-2)):
        torch.manual_seed(4)
        model = pa.ProteusEncoder().eval().to(gpu)
        model.aa_embedding.to(dtype)
        model.layers.to(dtype)
        model.head.to(dtype)
        with torch.no_grad():
            fast = model(coords, tokens, mask).float().cpu()
        recorded = model(coords, tokens, mask)                      # parameters require gradients: the torch expressions
        assert recorded.requires_grad
        recorded = recorded.detach().float().cpu()
        err = float((fast[valid] - recorded[valid]).norm() / recorded[valid].norm())
        assert err <= bar, f"{dtype}: rel-L2 {err:.3e}"
        # a second call reuses the cached constants: bit-equal
        with torch.no_grad():
            again = model(coords, tokens, mask).float().cpu()
        assert torch.equal(fast[valid], again[valid])
        # and they follow the parameter: a changed spread must change the result
        with torch.no_grad():
            for layer in model.layers:
                layer.attn.spread_weights.add_(0.5)
            moved = model(coords, tokens, mask).float().cpu()
        assert not torch.equal(fast[valid], moved[valid])
        # a write through `.data` (how EMA weights are swapped in) bumps no version counter: in eval() mode the kept
        # constants are dropped by invalidate_caches() or another eval() call, and then the result follows
        with torch.no_grad():
            for layer in model.layers:
                layer.attn.out_proj.weight.data.mul_(1.5)
                layer.attn.q_proj.data.mul_(0.5)
                layer.attn.invalidate_caches()
            swapped = model(coords, tokens, mask).float().cpu()
            for layer in model.layers:
                layer.attn.spread_weights.data.add_(0.5)
            model.eval()
            swapped2 = model(coords, tokens, mask).float().cpu()
        assert not torch.equal(moved[valid], swapped[valid]) and not torch.equal(swapped[valid], swapped2[valid])
        # in training mode nothing is kept: a `.data` write shows at once, also under no_grad
        model.train()
        with torch.no_grad():
            t1 = model(coords, tokens, mask).float().cpu()
            for layer in model.layers:
                layer.attn.out_proj.weight.data.mul_(1.25)
            t2 = model(coords, tokens, mask).float().cpu()
        assert not torch.equal(t1[valid], t2[valid])


def test_cfg4_shape_embedding_and_first_attention_on_sampled_rows(gpu):
    """At the real shape (B=8, N=1024, d_model=512, H=8, bf16 weights, fp32 WE, lengths in [128, 1024]) the two kernels
    in isolation, held to their own bars: rows are independent in both, so the embedding and the first layer's
    attention (fed with the activations the model itself produces) are checked on sampled rows against the C oracles.
    (The logits of the whole stack are compared with the CPU statement of the stack in
    test_cfg4_shape_logits_match_the_cpu_statement_of_the_whole_stack.)"""
    torch.manual_seed(4)
    model = pa.ProteusEncoder().eval().to(gpu)
    model.aa_embedding.to(torch.bfloat16)
    model.layers.to(torch.bfloat16)
    model.head.to(torch.bfloat16)
    g = torch.Generator().manual_seed(4)
    coords = torch.stack([synth.random_walk_chain(1024, g) for _ in range(8)])
    tokens = torch.randint(0, 33, (8, 1024), generator=g)
    lens = torch.randint(128, 1025, (8,), generator=g)
    mask = torch.arange(1024)[None, :] >= lens[:, None]
    rows = sorted(set(torch.randint(0, 1024, (40,), generator=g).tolist()) | {0, 127, 128, 1023})
    with torch.no_grad():
        wf = model.wf_embedding(coords.to(gpu), None, key_padding_mask=mask.to(gpu))
        wn = torch.exp(model.wf_embedding.wavenumbers.detach()).cpu()
        ref_wf, _, _ = c_oracle.we(coords.numpy(), wn.numpy(), mask.numpy(), rows=rows)
        got_wf = wf.cpu().numpy()[:, rows]
        assert np.isfinite(got_wf).all()
        e = np.linalg.norm(got_wf - ref_wf) / np.linalg.norm(ref_wf)
        assert e <= 1e-4, f"embedding at the encoder's shape: rel-L2 {e:.3e}"
        assert (got_wf[mask.numpy()[:, rows]] == 0).all()

        attn = model.layers[0].attn
        x = (wf + model.aa_embedding(tokens.to(gpu)).to(wf.dtype)).to(torch.bfloat16)
        w, b = attn._fused_qkv()
        qkv = torch.addmm(b, x.reshape(8 * 1024, 512), w).view(8, 1024, 3, 8, 64)
        Q, K, V = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))              # strided [Z,H,N,d] views, read in place
        sigma = attn.get_spreads().detach().float()
        O, L = pa.geo_attn(Q, K, V, coords.to(gpu), sigma, mask.to(gpu), return_lse=True)
        Or, Lr = c_oracle.geo_attn(Q.float().cpu().numpy(), K.float().cpu().numpy(), V.float().cpu().numpy(), coords.numpy(),
                                   sigma.cpu().numpy(), mask.numpy(), rows=rows)
        O, L = O.cpu().numpy()[:, :, rows].astype(np.float64), L.cpu().numpy()[:, :, rows].astype(np.float64)
        fin = np.isfinite(Lr)
        assert np.isfinite(O).all() and (np.isneginf(L) == ~fin).all()
        # O is a convex combination of V rows whose weights are rounded to bf16: the 2e-2 bar of unit-scale values scales
        # with the largest |V| (the projections of WE + embedding reach about 10 here)
        vmax = float(V.float().abs().max())
        assert 1.0 < vmax < 100.0
        assert np.abs(O - Or).max() <= 2e-2 * vmax / 4, f"first-layer attention at the encoder's shape: {np.abs(O - Or).max():.3e} (max |V| {vmax:.2f})"
        assert np.abs(L[fin] - Lr[fin]).max() <= 4e-3
        assert (O[~fin] == 0).all()


def _cfg4_batch():
    g = torch.Generator().manual_seed(4)
    coords = torch.stack([synth.random_walk_chain(1024, g) for _ in range(8)])
    tokens = torch.randint(0, 33, (8, 1024), generator=g)
    lens = torch.randint(128, 1025, (8,), generator=g)
    mask = torch.arange(1024)[None, :] >= lens[:, None]
    return coords, tokens, mask


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32_weights", "bf16_weights"])
def test_cfg4_shape_logits_match_the_cpu_statement_of_the_whole_stack(gpu, dtype):
    """The whole encoder at BASELINE.json configs[3] (B=8, N=1024, d_model=512, H=8, 4 layers, FFN 2048, head to 20
    logits, lengths in [128, 1024]) against the fp32 CPU statement of the same stack with the same weights
    (torch_oracle.encoder_forward_torch: dense torch attention and embedding oracles, pinned in
    tests/test_oracle_encoder.py), on every valid token.

    Bars (about twice what is measured: fp32 weights rel-L2 3.9e-3, worst token 2.5e-2, max-abs 0.85 % of the range;
    bf16 weights 9.2e-3, 4.6e-2, 1.1 %).  fp32 weights: the only low-precision steps are the attention's bf16 operands
    and probabilities (four layers): rel-L2 over all valid logits <= 8e-3, per token <= 5e-2, max-abs <= 2 % of the
    logits' range.  bf16 weights (the
    configuration BASELINE names): every activation between two layers is rounded to bf16 (2^-9 relative, some 30
    roundings from the embedding to the head, which LayerNorm renormalises rather than damps): rel-L2 <= 2e-2, per
    token rel-L2 <= 8e-2 on every token, max-abs <= 4 % of the logits' range, and the arg-max amino acid agrees where
    the reference's top two logits are further apart than that."""
    torch.manual_seed(4)
    model = pa.ProteusEncoder().eval().to(gpu)
    model.aa_embedding.to(dtype)
    model.layers.to(dtype)
    model.head.to(dtype)
    coords, tokens, mask = _cfg4_batch()
    with torch.no_grad():
        out = model(coords.to(gpu), tokens.to(gpu), mask.to(gpu)).float().cpu()
    ref = torch_oracle.encoder_forward_torch(model.state_dict(), model.layers[0].attn.min_spread, coords, tokens, mask)
    valid = ~mask
    got, want = out[valid].double(), ref[valid].double()
    assert got.shape == want.shape and got.shape[1] == 20 and torch.isfinite(got).all()
    rel = float((got - want).norm() / want.norm())
    per_token = ((got - want).norm(dim=1) / want.norm(dim=1))
    span = float(want.max() - want.min())
    max_abs = float((got - want).abs().max())
    print(f"encoder at configs[3], {dtype}: rel-L2 {rel:.3e}, worst token {float(per_token.max()):.3e}, "
          f"max abs {max_abs:.3e} of a logit range of {span:.2f}", flush=True)
    bars = {torch.float32: (8e-3, 5e-2, 0.02), torch.bfloat16: (2e-2, 8e-2, 0.04)}[dtype]
    assert rel <= bars[0], f"rel-L2 {rel:.3e}"
    assert float(per_token.max()) <= bars[1], f"worst token rel-L2 {float(per_token.max()):.3e}"
    assert max_abs <= bars[2] * span, f"max abs {max_abs:.3e}, range {span:.2f}"
    top2 = want.topk(2, dim=1).values
    clear = (top2[:, 0] - top2[:, 1]) > 2 * bars[2] * span
    assert clear.sum() > 0 and torch.equal(got.argmax(dim=1)[clear], want.argmax(dim=1)[clear])


def test_forward_replays_bit_equal_from_a_captured_graph(gpu):
    """Every entry point launches on the caller's stream without allocating or synchronising, so a forward can be
    captured into a graph.  Replays (with eager work and synchronisations between them) must reproduce the eager result."""
    torch.manual_seed(7)
    model = pa.ProteusEncoder(d_model=256, heads=4, layers=2, d_hidden=512).eval().to(gpu)
    g = torch.Generator().manual_seed(7)
    coords = torch.stack([synth.random_walk_chain(300, g) for _ in range(3)]).to(gpu)
    tokens = torch.randint(0, 33, (3, 300), generator=g).to(gpu)
    mask = torch.zeros(3, 300, dtype=torch.bool, device=gpu)
    mask[1, 200:] = True
    mask[2, 77:] = True
    with torch.no_grad():
        eager = model(coords, tokens, mask).clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                model(coords, tokens, mask)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = model(coords, tokens, mask)
        torch.cuda.synchronize()
        for _ in range(3):
            out.fill_(float("nan"))
            model(coords, tokens, mask)                     # eager work between the replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out[~mask], eager[~mask])


def test_operators_forward_and_backward_replay_from_a_captured_graph(gpu):
    """The attention forward and backward and the embedding forward and backward, through their autograd functions,
    captured into one graph: replays (with eager work between them) reproduce the eager gradients, to the bit except
    d_sigma, which is summed with atomic adds.  (A whole training step is not captured here: torch's own many-block
    reductions, the bias gradients' column sums, clear their accumulators with memset nodes that replays do not repeat.)"""
    g = torch.Generator().manual_seed(7)
    Z, H, N, d = 2, 4, 700, 64
    Q, K, V, coords, sigma, _ = synth.attn_inputs(Z, H, N, d, 7)
    mask = torch.zeros(Z, N, dtype=torch.bool)
    mask[1, 500:] = True
    dO = (torch.randn(Z, H, N, d, generator=g) / 8).to(gpu)
    dE = torch.randn(Z, N, 64, generator=g).to(gpu)
    q, k, v = (t.to(gpu).requires_grad_(True) for t in (Q, K, V))
    s = sigma.to(gpu).requires_grad_(True)
    wn = torch.exp(torch.linspace(-1.0, 0.5, 32)).to(gpu).requires_grad_(True)
    c, m = coords.to(gpu), mask.to(gpu)
    leaves = (q, k, v, s, wn)

    def step():
        for t in leaves:
            t.grad.zero_()
        pa.geometric_attn(q, k, v, c, s, None, m, check_spreads=False).backward(dO)      # (the check reads sigma on the host)
        pa.wf_embedding(c, wn, mask=m).backward(dE)

    for t in leaves:
        t.grad = torch.zeros_like(t)
    step()
    torch.cuda.synchronize()
    eager = [t.grad.clone() for t in leaves]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    torch.cuda.synchronize()
    for _ in range(3):
        step()                                              # eager work between the replays
        torch.cuda.synchronize()
        for t in leaves:
            t.grad.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for t, e, name in zip(leaves, eager, ("dQ", "dK", "dV", "d_sigma", "d_wavenumbers")):
            if name == "d_sigma":
                assert torch.allclose(t.grad, e, rtol=1e-5, atol=1e-9), name
            else:
                assert torch.equal(t.grad, e), name


def test_training_step_through_both_kernels(gpu):
    # forward and backward of the whole stack on the HIP kernels (attention backward, wavenumber backward of the
    # embedding), one SGD step, and the loss goes down
    torch.manual_seed(1)
    model = pa.ProteusEncoder(d_model=128, heads=2, layers=2, d_hidden=256).to(gpu)
    model.wf_embedding.wavenumbers.requires_grad_(True)
    g = torch.Generator().manual_seed(2)
    coords = torch.stack([synth.random_walk_chain(120, g) for _ in range(2)]).to(gpu)
    tokens = torch.randint(0, 33, (2, 120), generator=g).to(gpu)
    labels = torch.randint(0, 20, (2, 120), generator=g).to(gpu)
    mask = torch.zeros(2, 120, dtype=torch.bool, device=gpu)
    mask[1, 90:] = True
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    losses = []
    for _ in range(4):
        opt.zero_grad()
        logits = model(coords, tokens, mask)
        loss = F.cross_entropy(logits[~mask], labels[~mask])
        loss.backward()
        for name, p in model.named_parameters():
            if p.requires_grad and "beta_weights" not in name and "aa_magnitudes" not in name:
                assert p.grad is not None and torch.isfinite(p.grad).all(), name
        opt.step()
        losses.append(loss.item())
    assert losses[-1] < losses[0]
    assert model.layers[0].attn.spread_weights.grad.abs().sum() > 0
    assert model.wf_embedding.wavenumbers.grad.abs().sum() > 0
