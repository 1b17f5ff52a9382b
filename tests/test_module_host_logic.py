"""Host-side logic of the modules that needs no GPU: the constants GeoAttention keeps across inference calls, and the
choice between writing the fused projection's gradient in place and through buffers of its own."""
import importlib

import torch

import proteusai_amd as pa

ga = importlib.import_module("proteusai_amd.geometric_attn")


def _attn():
    torch.manual_seed(0)
    return pa.GeoAttention(d_model=64, heads=2)


def test_kept_constants_follow_every_way_the_weights_are_known_to_change():
    m = _attn().eval()
    with torch.no_grad():
        s0, w0, (q0, b0) = m._per_head("spread"), m._out_weight(), m._fused_qkv()
        same = lambda a, b: a.data_ptr() == b.data_ptr()
        assert same(m._per_head("spread"), s0) and same(m._out_weight(), w0) and same(m._fused_qkv()[0], q0)       # kept
        # an in-place update that autograd sees bumps the version counter
        m.spread_weights.add_(0.5)
        m.out_proj.weight.mul_(2.0)
        m.q_proj.mul_(2.0)
        assert torch.allclose(m._per_head("spread"), m.get_spreads()) and not torch.equal(m._per_head("spread"), s0)
        assert torch.equal(m._out_weight().reshape(64, 2, 32).permute(0, 2, 1).reshape(64, 64), m.out_proj.weight)
        assert torch.equal(m._fused_qkv()[0][:, :32], m.q_proj[0])
        # load_state_dict and dtype / device conversions drop them
        sd = {k: v.clone() for k, v in m.state_dict().items()}
        sd["spread_weights"] = sd["spread_weights"] + 1.0
        kept = m._per_head("spread")
        m.load_state_dict(sd)
        assert not torch.equal(m._per_head("spread"), kept) and torch.allclose(m._per_head("spread"), m.get_spreads())
        m.double()
        assert m._fused_qkv()[0].dtype == torch.float64 and m._out_weight().dtype == torch.float64
        m.float()


def test_writes_through_data_need_invalidate_caches_only_in_eval_mode():
    # `p.data.copy_()` (how EMA / SWA weights are swapped in) bumps no version counter
    m = _attn().eval()
    with torch.no_grad():
        s0, w0, q0 = m._per_head("spread").clone(), m._out_weight().clone(), m._fused_qkv()[0].clone()
        v = m.spread_weights._version
        m.spread_weights.data.copy_(m.spread_weights.data + 1.0)
        m.out_proj.weight.data.mul_(3.0)
        m.q_proj.data.mul_(3.0)
        assert m.spread_weights._version == v                    # which is why the module cannot notice by itself
        m.invalidate_caches()
        assert not torch.equal(m._per_head("spread"), s0) and torch.allclose(m._per_head("spread"), m.get_spreads())
        assert not torch.equal(m._out_weight(), w0) and not torch.equal(m._fused_qkv()[0], q0)
        # eval() / train() calls drop the constants too: swap the weights in, then call eval()
        s1 = m._per_head("spread").clone()
        m.spread_weights.data.copy_(m.spread_weights.data + 1.0)
        m.eval()
        assert not torch.equal(m._per_head("spread"), s1)
    # in training mode nothing is kept at all, with or without gradients
    m.train()
    with torch.no_grad():
        s2 = m._per_head("spread").clone()
        m.spread_weights.data.copy_(m.spread_weights.data + 1.0)
        assert not torch.equal(m._per_head("spread"), s2)
        assert getattr(m, "_qkv_cache", None) is None and getattr(m, "_wo_cache", None) is None
    # with gradients enabled the results stay attached to the parameters
    assert m._fused_qkv()[0].requires_grad and m._out_weight().requires_grad and m._per_head("spread").requires_grad


def test_fused_gradient_is_written_in_place_only_where_the_kernels_can_address_it():
    # dQ, dK, dV as views of one [Z,N,3,H,d] fp32 buffer: a sequence must span less than 2 GiB (N*3*H*d*4 bytes)
    for N, ok in ((300000, True), (349000, True), (349600, False), (1 << 20, False)):
        g = torch.empty((1, N, 3, 8, 64), dtype=torch.float32, device="meta")
        grads = tuple(g[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        assert ga._fused_grad_views_ok(grads) == ok, N
