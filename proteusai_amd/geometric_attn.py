"""RBF-scaled geometric attention operator and module on the HIP kernel.

Mirrors the reference's Python surface:
  geometric_attn(...) / _geometric_attn   old/old_scripts/attn/geometric_attn.py:545-607
  GeoAttention                            old/old_scripts/encoder.py:43-121
with the logits of README.md:40, s = (q.k/sqrt(d)) * (1 + exp(-|rq-rk|^2/(2 sigma_h^2))),
plus `geo_attn`, the (Q, K, V, coords, sigma_per_head, key_padding_mask) form.
"""
import functools

import torch
import torch.nn as nn

from . import _lib


@functools.lru_cache(maxsize=1024)
def _layout_ok(size, stride, itemsize):
    per16 = 16 // itemsize
    return (stride[3] == 1 and stride[2] >= size[3]
            and all(st >= 0 and st % per16 == 0 for st in stride[:3])
            and (size[0] == 1 or stride[0] > 0) and (size[1] == 1 or stride[1] > 0)
            and size[2] * stride[2] * itemsize < 2 ** 31)


def _rows_ok(t, itemsize):
    """Can the kernels read / write this [Z,H,N,d] tensor in place?  Rows of d contiguous elements, 16-byte
    aligned, no negative or overlapping-row strides; the batch, head and token strides are otherwise free."""
    if t.data_ptr() % 16 != 0:
        return False
    return t.is_contiguous() or _layout_ok(tuple(t.shape), t.stride(), itemsize)


def _operand(t, dtype=torch.bfloat16):
    """16-bit view of an operand the kernels can read where it lies (a copy only if it has to be cast or its rows
    are not contiguous)."""
    if t.requires_grad:
        t = t.detach()
    if t.dtype != dtype:
        t = t.to(dtype)
    return t if _rows_ok(t, 2) else t.contiguous()


def _f32(t, dev):
    """fp32, contiguous, on `dev`, outside autograd: the tensor itself where it already is all that."""
    if t.dtype == torch.float32 and t.device == dev and not t.requires_grad and t.is_contiguous():
        return t
    return t.detach().to(device=dev, dtype=torch.float32).contiguous()


def _mask_bytes(mask, dev):
    if mask.dtype == torch.bool and mask.device == dev and mask.is_contiguous():
        return mask.view(torch.uint8)
    return mask.to(device=dev, dtype=torch.bool).contiguous().view(torch.uint8)


def _operand_type(operand_dtype, legacy):
    if operand_dtype in (None, torch.bfloat16):
        return torch.bfloat16, _lib.OPERAND_BF16
    if operand_dtype == torch.float16:
        if not legacy:
            raise NotImplementedError("fp16 operands go with the beta-weighted logits (pass betas); the README logits run in bf16")
        return torch.float16, _lib.OPERAND_F16
    raise AssertionError(f"operand_dtype must be torch.bfloat16 or torch.float16, not {operand_dtype}")


def _is_plain(*ts):
    return all(t.is_contiguous() for t in ts)


def geo_attn(Q, K, V, coords, sigma, key_padding_mask=None, return_lse: bool = False, tuning: int = 0,
             betas=None, min_rbf: float = 0.0, max_rbf: float = 1.0, check_sigma: bool = True,
             token_major_out: bool = False, operand_dtype=None):
    """O = geo_attn(Q, K, V [Z,H,N,d], coords [Z,N,3], sigma [H], key_padding_mask [Z,N] bool | None), d = 32, 64 or 128.

    Operands are cast to bf16 (the reference casts to fp16, geometric_attn.py:567-569; with `betas`,
    operand_dtype=torch.float16 does the same here), coords and sigma to fp32; O is fp32 [Z,H,N,d] as in the
    reference (:578).
    key_padding_mask: True = padded.  Padded query rows and rows without a
    valid key give O = 0 and logsumexp = -inf.  With return_lse the
    logsumexp L [Z,H,N] is returned as well.

    Q, K, V may be views with any batch / head / token strides as long as the rows of d elements are
    contiguous and 16-byte aligned (e.g. slices of a fused [Z,N,3,H,d] projection): they are read in place.
    token_major_out=True returns O as a [Z,H,N,d] view of memory laid out [Z,N,H,d] (what a following
    projection over the concatenated heads reads without a copy).

    With `betas` [H] the logits are those of the reference's kernel instead,
    S + beta_h*(2(rbf-min_rbf)/(max_rbf-min_rbf)-1)*|S| with pairs whose rbf lies outside
    [min_rbf, max_rbf] masked (old/old_scripts/attn/geometric_attn.py:193-201).
    """
    if not (Q.shape == K.shape == V.shape):
        raise AssertionError(f"Q, K, and V projection shapes must match, but got {Q.shape=}, {K.shape=}, {V.shape=}")
    if Q.dim() != 4:
        raise AssertionError(f"Q, K, V must be of shape (batch, heads, N, d_k), not {tuple(Q.shape)}")
    Z, H, N, d = Q.shape
    if coords.dim() != 3 or coords.size(2) != 3 or coords.size(0) != Z or coords.size(1) != N:
        raise AssertionError(f"coordinates must be of shape (batch, N, 3), not {tuple(coords.shape)}")
    if sigma.dim() != 1 or sigma.size(0) != H:
        raise AssertionError(f"number of spreads must be equal to nheads, not {tuple(sigma.shape)} and {H=}")
    if not Q.is_cuda:
        raise _lib.ProteusError("geo_attn needs tensors on the GPU (there is no CPU path)")
    # (reading the answer back synchronises with the device: callers whose sigma is positive by construction skip it)
    if check_sigma and not bool(torch.all(sigma > 0)):
        raise AssertionError(f"spreads must be a tensor of positive, non-zero floats, not {sigma}")
    lib = _lib.load()
    dev = Q.device
    legacy = betas is not None
    op_dtype, op_type = _operand_type(operand_dtype, legacy)
    q, k, v = _operand(Q, op_dtype), _operand(K, op_dtype), _operand(V, op_dtype)
    c = _f32(coords, dev)
    s = _f32(sigma, dev)
    m = None
    if key_padding_mask is not None:
        if tuple(key_padding_mask.shape) != (Z, N):
            raise AssertionError(f"mask must be of shape ({Z}, {N}), not {tuple(key_padding_mask.shape)}")
        m = _mask_bytes(key_padding_mask, dev)
    if token_major_out:
        O = torch.empty(Z, N, H, d, dtype=torch.float32, device=dev).permute(0, 2, 1, 3)
    else:
        O = torch.empty(Z, H, N, d, dtype=torch.float32, device=dev)
    L = torch.empty(Z, H, N, dtype=torch.float32, device=dev)
    if Z == 0 or H == 0 or N == 0:
        return (O, L) if return_lse else O
    with _lib.on_device(dev):
        stream = _lib.raw_stream(dev)
        ws_bytes = lib.proteus_geo_attn_fwd_workspace_bytes(Z, H, N, d, int(tuning)) if not legacy else 0
        if ws_bytes:
            # long sequences: with a workspace the library may cut the key loop of a (batch, head, query tile) item into
            # parts -- the long items of a padded batch, or all items of a batch too small to fill the chip -- instead
            # of one workgroup per item (the size is asked for the shape alone; without a use for it the call is the
            # plain one)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
            rc = lib.proteus_geo_attn_fwd_ws(q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                             None if _is_plain(q, k, v, O) else _lib.stride_array(q, k, v, O),
                                             c.data_ptr(), s.data_ptr(), None if m is None else m.data_ptr(), O.data_ptr(), L.data_ptr(),
                                             ws.data_ptr(), ws_bytes, Z, H, N, d, int(tuning), stream)
        elif not legacy and _is_plain(q, k, v, O):
            rc = lib.proteus_geo_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), c.data_ptr(), s.data_ptr(),
                                          None if m is None else m.data_ptr(),
                                          O.data_ptr(), L.data_ptr(), Z, H, N, d, int(tuning), stream)
        elif not legacy:
            rc = lib.proteus_geo_attn_fwd_strided(q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.stride_array(q, k, v, O),
                                                  c.data_ptr(), s.data_ptr(), None if m is None else m.data_ptr(),
                                                  O.data_ptr(), L.data_ptr(), Z, H, N, d, int(tuning), stream)
        else:
            if betas.dim() != 1 or betas.size(0) != H:
                raise AssertionError(f"number of betas must be equal to nheads, not {tuple(betas.shape)} and {H=}")
            bt = _f32(betas, dev)
            if _is_plain(q, k, v, O):
                rc = lib.proteus_geo_attn_legacy_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), c.data_ptr(), s.data_ptr(),
                                                     bt.data_ptr(), None if m is None else m.data_ptr(),
                                                     O.data_ptr(), L.data_ptr(), Z, H, N, d,
                                                     float(min_rbf), float(max_rbf), op_type, int(tuning), stream)
            else:
                rc = lib.proteus_geo_attn_legacy_fwd_strided(q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                                             _lib.stride_array(q, k, v, O), c.data_ptr(), s.data_ptr(),
                                                             bt.data_ptr(), None if m is None else m.data_ptr(),
                                                             O.data_ptr(), L.data_ptr(), Z, H, N, d,
                                                             float(min_rbf), float(max_rbf), op_type, int(tuning), stream)
    _lib.check(rc, "proteus_geo_attn_fwd")
    return (O, L) if return_lse else O


_DELTA_DTYPES = {torch.float32: _lib.DTYPE_F32, torch.bfloat16: _lib.DTYPE_BF16, torch.float16: _lib.DTYPE_F16}


def _delta(O, dO):
    """D = rowsum(O * dO) [Z,H,N] fp32 (old/old_scripts/attn/geometric_attn.py:618), in one pass over both tensors
    where their layout allows (rows of d contiguous, strides multiples of 4 elements); the torch expression otherwise."""
    Z, H, N, d = O.shape
    plain = (O.is_cuda and O.dtype == torch.float32 and dO.dtype in _DELTA_DTYPES and dO.shape == O.shape and d in (32, 64, 128)
             and Z * H * N > 0 and Z * H <= 65535
             and O.stride(3) == 1 and dO.stride(3) == 1 and O.stride(2) >= d and dO.stride(2) >= d
             and all(s % 4 == 0 for s in O.stride()[:3] + dO.stride()[:3])
             and O.data_ptr() % 16 == 0 and dO.data_ptr() % (4 * dO.element_size()) == 0)
    if not plain:
        return torch.sum(O.float() * dO, dim=3).contiguous()       # fp32 by type promotion
    D = torch.empty(Z, H, N, dtype=torch.float32, device=O.device)
    strides = None if (O.is_contiguous() and dO.is_contiguous()) else _lib.stride_array(O, dO)
    with _lib.on_device(O.device):
        rc = _lib.load().proteus_geo_attn_delta(O.data_ptr(), dO.data_ptr(), strides, D.data_ptr(), Z, H, N, d,
                                                _DELTA_DTYPES[dO.dtype], _lib.raw_stream(O.device))
    _lib.check(rc, "proteus_geo_attn_delta")
    return D


def geo_attn_backward(Q, K, V, O, L, dO, coords, sigma, key_padding_mask=None, betas=None,
                      min_rbf: float = 0.0, max_rbf: float = 1.0, operand_dtype=None, grads=None):
    """dQ, dK, dV [Z,H,N,d] f32, d_sigma [H] f32, d_betas [H] f32 | None from the forward's O and logsumexp L.

    What the reference's wrapper does around its backward kernel (geometric_attn.py:609-660):
    D = rowsum(O*dO), dO cast to the operand type (bf16, or fp16 with operand_dtype=torch.float16 and betas), zeroed
    accumulators for the per-head scalars.
    grads: optional (dQ, dK, dV) fp32 [Z,H,N,d] tensors to write into (rows of d contiguous, e.g. views of one
    [Z,N,3,H,d] buffer); allocated here otherwise.
    """
    Z, H, N, d = Q.shape
    if not Q.is_cuda:
        raise _lib.ProteusError("geo_attn_backward needs tensors on the GPU (there is no CPU path)")
    lib = _lib.load()
    dev = Q.device
    op_dtype, op_type = _operand_type(operand_dtype, betas is not None)
    q, k, v = _operand(Q, op_dtype), _operand(K, op_dtype), _operand(V, op_dtype)
    D = _delta(O.detach(), dO.detach())
    do = _operand(dO, op_dtype)
    c = _f32(coords, dev)
    s = _f32(sigma, dev)
    lse = _f32(L, dev)
    m = None if key_padding_mask is None else _mask_bytes(key_padding_mask, dev)
    bt = None if betas is None else _f32(betas, dev)
    # gradients in the memory order of their operands (dense), so that what consumes them needs no reshuffle
    def like(t):
        g = torch.empty_like(t, dtype=torch.float32)
        return g if _rows_ok(g, 4) else torch.empty(Z, H, N, d, dtype=torch.float32, device=dev)
    if grads is None:
        dQ, dK, dV = like(Q), like(K), like(V)
    else:
        dQ, dK, dV = grads
        for g_ in grads:
            if g_.dtype != torch.float32 or tuple(g_.shape) != (Z, H, N, d) or not _rows_ok(g_, 4):
                raise AssertionError("grads must be fp32 [Z,H,N,d] tensors with contiguous, 16-byte aligned rows")
    d_sigma = torch.zeros(H, dtype=torch.float32, device=dev)
    d_beta = None if bt is None else torch.zeros(H, dtype=torch.float32, device=dev)
    if Z == 0 or H == 0 or N == 0:
        return dQ, dK, dV, d_sigma, d_beta
    with _lib.on_device(dev):
        stream = _lib.raw_stream(dev)
        tail = (c.data_ptr(), s.data_ptr(), None if bt is None else bt.data_ptr(), None if m is None else m.data_ptr(),
                lse.data_ptr(), D.data_ptr(), dQ.data_ptr(), dK.data_ptr(), dV.data_ptr(),
                d_sigma.data_ptr(), None if d_beta is None else d_beta.data_ptr(),
                Z, H, N, d, float(min_rbf), float(max_rbf), op_type, stream)
        if _is_plain(q, k, v, do, dQ, dK, dV):
            rc = lib.proteus_geo_attn_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), do.data_ptr(), *tail)
        else:
            rc = lib.proteus_geo_attn_bwd_strided(q.data_ptr(), k.data_ptr(), v.data_ptr(), do.data_ptr(),
                                                  _lib.stride_array(q, k, v, do, dQ, dK, dV), *tail)
    _lib.check(rc, "proteus_geo_attn_bwd")
    return dQ, dK, dV, d_sigma, d_beta


class _geometric_attn(torch.autograd.Function):
    """Forward and backward on the HIP kernels (old/old_scripts/attn/geometric_attn.py:550-660).  No gradient
    flows to the coordinates, as in the reference."""

    @staticmethod
    def forward(ctx, Q, K, V, coords, spreads, betas, key_padding_mask, min_rbf, max_rbf, check_sigma=True,
                token_major_out=False, out_dtype=None, operand_dtype=None):
        O, L = geo_attn(Q, K, V, coords, spreads, key_padding_mask, return_lse=True, betas=betas,
                        min_rbf=min_rbf, max_rbf=max_rbf, check_sigma=check_sigma, token_major_out=token_major_out,
                        operand_dtype=operand_dtype)
        ctx.save_for_backward(Q, K, V, O, L, coords, spreads, betas, key_padding_mask)
        ctx.min_rbf, ctx.max_rbf, ctx.operand_dtype = min_rbf, max_rbf, operand_dtype
        # the fp32 O is what the backward reads; the caller may ask for it in its own working precision
        return O if out_dtype is None or out_dtype == O.dtype else O.to(out_dtype)

    @staticmethod
    def backward(ctx, dO):
        Q, K, V, O, L, coords, spreads, betas, mask = ctx.saved_tensors
        dQ, dK, dV, d_sigma, d_beta = geo_attn_backward(Q, K, V, O, L, dO, coords, spreads, mask, betas,
                                                        ctx.min_rbf, ctx.max_rbf, ctx.operand_dtype)
        return (dQ.to(Q.dtype), dK.to(K.dtype), dV.to(V.dtype), None, d_sigma.to(spreads.dtype),
                None if betas is None else d_beta.to(betas.dtype), None, None, None, None, None, None, None)


def _fused_grad_views_ok(grads):
    """Can the backward kernels write dQ, dK, dV straight into these views of one fused [Z,N,3,H,d] fp32 buffer?"""
    return all(_rows_ok(g_, 4) for g_ in grads)


class _geometric_attn_qkv(torch.autograd.Function):
    """The same operator on a fused projection qkv [Z,N,3,H,d] (self-attention: what one GEMM over the three
    projections leaves).  Forward and backward read Q, K, V in place; the backward writes dQ, dK, dV into one
    [Z,N,3,H,d] buffer, which is the gradient of qkv: no per-slice gradients for autograd to pad and add up."""

    @staticmethod
    def forward(ctx, qkv, coords, spreads, betas, key_padding_mask, min_rbf, max_rbf, check_sigma, out_dtype, operand_dtype):
        Q, K, V = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        O, L = geo_attn(Q, K, V, coords, spreads, key_padding_mask, return_lse=True, betas=betas,
                        min_rbf=min_rbf, max_rbf=max_rbf, check_sigma=check_sigma, token_major_out=True,
                        operand_dtype=operand_dtype)
        ctx.save_for_backward(qkv, O, L, coords, spreads, betas, key_padding_mask)
        ctx.min_rbf, ctx.max_rbf, ctx.operand_dtype = min_rbf, max_rbf, operand_dtype
        return O if out_dtype is None or out_dtype == O.dtype else O.to(out_dtype)

    @staticmethod
    def backward(ctx, dO):
        qkv, O, L, coords, spreads, betas, mask = ctx.saved_tensors
        Q, K, V = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        g = torch.empty(qkv.shape, dtype=torch.float32, device=qkv.device)
        grads = tuple(g[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        if _fused_grad_views_ok(grads):
            _, _, _, d_sigma, d_beta = geo_attn_backward(Q, K, V, O, L, dO, coords, spreads, mask, betas,
                                                         ctx.min_rbf, ctx.max_rbf, ctx.operand_dtype, grads=grads)
        else:
            # a sequence of the fused buffer spans 2 GiB or more: the kernels cannot address it in place, so the
            # gradients go to buffers of their own (as the sliced operator does) and are copied in
            dQ, dK, dV, d_sigma, d_beta = geo_attn_backward(Q, K, V, O, L, dO, coords, spreads, mask, betas,
                                                            ctx.min_rbf, ctx.max_rbf, ctx.operand_dtype)
            for dst, src in zip(grads, (dQ, dK, dV)):
                dst.copy_(src)
        return (g.to(qkv.dtype), None, d_sigma.to(spreads.dtype), None if betas is None else d_beta.to(betas.dtype),
                None, None, None, None, None, None)


def geometric_attn_qkv(qkv, coords, spreads, betas=None, mask=None, min_rbf=0.00, max_rbf=1.00, check_spreads=True,
                       out_dtype=None, operand_dtype=None):
    """geometric_attn for self-attention on a fused projection: qkv [Z,N,3,H,d] (Q, K, V = qkv[:, :, 0 / 1 / 2]).
    Returns O as a [Z,H,N,d] view of memory laid out [Z,N,H,d].  Same arguments otherwise; the gradient of qkv comes
    back as one tensor."""
    if betas is None and (min_rbf > 0.0 or max_rbf < 1.0):
        raise NotImplementedError("the [min_rbf, max_rbf] pair mask belongs to the beta-weighted logits; pass betas")
    if qkv.dim() != 5 or qkv.size(2) != 3:
        raise AssertionError(f"qkv must be of shape (batch, N, 3, heads, d_k), not {tuple(qkv.shape)}")
    if not _rows_ok(qkv[:, :, 0].permute(0, 2, 1, 3), qkv.element_size()):
        qkv = qkv.contiguous()
    if not (torch.is_grad_enabled() and (qkv.requires_grad or spreads.requires_grad or (betas is not None and betas.requires_grad))):
        # nothing to differentiate: the forward alone, without an autograd node
        Q, K, V = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        O = geo_attn(Q, K, V, coords, spreads, mask, betas=betas, min_rbf=min_rbf, max_rbf=max_rbf, check_sigma=check_spreads,
                     token_major_out=True, operand_dtype=operand_dtype)
        return O if out_dtype is None or out_dtype == O.dtype else O.to(out_dtype)
    return _geometric_attn_qkv.apply(qkv, coords, spreads, betas, mask, min_rbf, max_rbf, check_spreads, out_dtype, operand_dtype)


def geometric_attn(Q, K, V, coords, spreads, betas=None, mask=None, min_rbf=0.00, max_rbf=1.00, check_spreads=True,
                   token_major_out=False, out_dtype=None, operand_dtype=None):
    """Same call as the reference's geometric_attn (geometric_attn.py:545-548).

    betas=None selects the README logits S*(1+RBF) (README.md:40; the rbf range must then be the full
    [0, 1]); a betas tensor selects the reference kernel's own logits S + beta*RBF_norm*|S| with its
    [min_rbf, max_rbf] pair mask (geometric_attn.py:193-201).

    Beyond the reference's call: token_major_out lays O out [Z,N,H,d] in memory (returned as a [Z,H,N,d] view),
    out_dtype returns O in another dtype than fp32 (the fp32 result is kept for the backward either way),
    operand_dtype=torch.float16 (with betas) casts Q, K, V and dO to fp16 as the reference does (:567-569) instead of bf16.
    """
    if betas is None and (min_rbf > 0.0 or max_rbf < 1.0):
        raise NotImplementedError("the [min_rbf, max_rbf] pair mask belongs to the beta-weighted logits; pass betas")
    if not (torch.is_grad_enabled() and (Q.requires_grad or K.requires_grad or V.requires_grad or spreads.requires_grad
                                         or (betas is not None and betas.requires_grad))):
        O = geo_attn(Q, K, V, coords, spreads, mask, betas=betas, min_rbf=min_rbf, max_rbf=max_rbf, check_sigma=check_spreads,
                     token_major_out=token_major_out, operand_dtype=operand_dtype)
        return O if out_dtype is None or out_dtype == O.dtype else O.to(out_dtype)
    return _geometric_attn.apply(Q, K, V, coords, spreads, betas, mask, min_rbf, max_rbf, check_spreads,
                                 token_major_out, out_dtype, operand_dtype)


class GeoAttention(nn.Module):
    """Multi-head attention whose logits are scaled per head by 1 + RBF of the
    pairwise C-alpha distance.  Constructor, parameters and forward follow
    old/old_scripts/encoder.py:43-121 (per-head QKV projections with bias,
    sigma = min_spread + exp(w), heads concatenated as a (d_k x heads)
    interleave, bias-free output projection).  With legacy_logits=True the
    logits are the reference module's (beta-weighted bias, [min_rbf, max_rbf]
    pair mask); otherwise beta_weights is kept only so that state dicts line up.
    min_rbf=None takes the reference module's default 0.001 (encoder.py:57) with legacy_logits and 0 without
    (the README logits have no pair mask).  operand_dtype=torch.float16 (legacy_logits only) runs the kernels on fp16
    operands as the reference's do (old/old_scripts/attn/geometric_attn.py:567-569); default bf16.
    d_model / heads must be 32, 64 or 128."""

    def __init__(self, d_model=512, heads=8, min_spread=2.0, min_rbf=None, max_rbf=1.00, learn_spreads=True,
                 legacy_logits=False, operand_dtype=None):
        super().__init__()
        if operand_dtype not in (None, torch.bfloat16) and not legacy_logits:
            raise NotImplementedError("fp16 operands go with legacy_logits=True; the README logits run in bf16")
        self.operand_dtype = operand_dtype
        if min_rbf is None:
            min_rbf = 0.001 if legacy_logits else 0.0
        self.legacy_logits = legacy_logits      # True: the reference module's beta-weighted bias and pair mask
        self.heads = heads
        self.d_model = d_model
        if self.d_model % self.heads != 0:
            raise ValueError(f"number of dimensions ({self.d_model}) must be divisible by number of attention heads ({self.heads})")
        self.d_k = self.d_model // self.heads
        self.spread_weights = nn.Parameter(torch.zeros(heads), requires_grad=learn_spreads)
        self.beta_weights = nn.Parameter(torch.zeros(heads))
        self.min_spread = min_spread
        self.min_rbf = min_rbf
        self.max_rbf = max_rbf
        xavier_scale = (6 / (self.d_k + d_model)) ** 0.5
        self.q_proj = nn.Parameter(-xavier_scale + torch.rand(self.heads, self.d_model, self.d_k) * (2 * xavier_scale))
        self.k_proj = nn.Parameter(-xavier_scale + torch.rand(self.heads, self.d_model, self.d_k) * (2 * xavier_scale))
        self.v_proj = nn.Parameter(-xavier_scale + torch.rand(self.heads, self.d_model, self.d_k) * (2 * xavier_scale))
        self.q_bias = nn.Parameter(torch.zeros(self.heads, self.d_k))
        self.k_bias = nn.Parameter(torch.zeros(self.heads, self.d_k))
        self.v_bias = nn.Parameter(torch.zeros(self.heads, self.d_k))
        self.out_proj = nn.Linear(d_model, d_model, bias=False)

    def get_spreads(self):
        return self.min_spread + torch.exp(self.spread_weights)

    def get_betas(self):
        return torch.exp(self.beta_weights)

    def forward(self, q, k, v, coords, mask=None):
        assert q.shape == k.shape == v.shape
        assert q.dim() == 3
        batch, N, d_model = q.shape
        assert d_model == self.d_model
        # Per-head projections x @ W_h + b_h (encoder.py:99-101) as plain GEMMs against the heads' weights laid
        # side by side, [d_model, heads*d_k] (the broadcast batched matmul of the reference materialises the
        # activations once per head); self-attention takes one GEMM for all three.  The kernels read Q, K, V
        # where the GEMM left them ([Z,N,(3,)H,d_k], as strided [Z,H,N,d_k] views) and write O token-major, so
        # no head split or merge is ever copied.
        H, dk = self.heads, self.d_k

        def heads_first(x):                # [Z, N, H*d_k] -> [Z, H, N, d_k] view
            return x.view(batch, N, H, dk).permute(0, 2, 1, 3)
        qkv = None
        if q is k and k is v:
            w, b = self._fused_qkv()
            qkv = torch.addmm(b, q.reshape(batch * N, d_model), w).view(batch, N, 3, H, dk)
        else:
            def flat(w_):                  # [H, d_model, d_k] -> [d_model, H*d_k]
                return w_.permute(1, 0, 2).reshape(self.d_model, H * dk)
            Q = heads_first(torch.addmm(self.q_bias.reshape(-1), q.reshape(batch * N, d_model), flat(self.q_proj)))
            K = heads_first(torch.addmm(self.k_bias.reshape(-1), k.reshape(batch * N, d_model), flat(self.k_proj)))
            V = heads_first(torch.addmm(self.v_bias.reshape(-1), v.reshape(batch * N, d_model), flat(self.v_proj)))
        # sigma = min_spread + exp(w) is positive by construction: no need to read a check back from the device
        betas = self._per_head("beta") if self.legacy_logits else None
        lo, hi = (self.min_rbf, self.max_rbf) if self.legacy_logits else (0.0, 1.0)
        if qkv is not None:
            out = geometric_attn_qkv(qkv, coords, self._per_head("spread"), betas, mask=mask, min_rbf=lo, max_rbf=hi,
                                     check_spreads=False, out_dtype=q.dtype, operand_dtype=self.operand_dtype)
        else:
            out = geometric_attn(Q, K, V, coords, self._per_head("spread"), betas, mask=mask, min_rbf=lo, max_rbf=hi,
                                 check_spreads=False, token_major_out=True, out_dtype=q.dtype, operand_dtype=self.operand_dtype)
        # The reference concatenates the heads as a (d_k x heads) interleave (encoder.py:114-115) before the output
        # projection.  Token-major O is the (heads x d_k) order; the same product is taken against the projection's
        # input columns in that order instead of reshuffling the activations.
        out = out.permute(0, 2, 1, 3).reshape(batch, N, self.d_model)           # a view when O is token-major
        return torch.nn.functional.linear(out, self._out_weight())

    # ---- constants derived from the parameters, kept across inference calls ----
    # sigma / beta of the heads, the output projection with its columns permuted and the fused projection weight are
    # functions of the parameters.  They are kept across calls only in eval() mode and only where no gradient is
    # needed, keyed on the parameters' version counters and storage, and dropped by anything that is known to change
    # the weights: train() / eval(), .to() / .half() / .cuda() (through _apply), load_state_dict, and
    # invalidate_caches().  A write through `p.data` (e.g. `p.data.copy_(ema)`) bumps no version counter and cannot be
    # seen from here: after such a write in eval() mode call invalidate_caches() (or eval() again).

    def invalidate_caches(self):
        """Drop the constants kept from earlier inference calls.  Needed only after the parameters were changed
        behind autograd's back (writes through `.data`) while the module stayed in eval() mode."""
        self.__dict__.pop("_head_cache", None)
        self._wo_cache = None
        self._qkv_cache = None

    def train(self, mode: bool = True):
        self.invalidate_caches()
        return super().train(mode)

    def _apply(self, fn, *args, **kwargs):
        self.invalidate_caches()
        return super()._apply(fn, *args, **kwargs)

    def _load_from_state_dict(self, *args, **kwargs):
        self.invalidate_caches()
        return super()._load_from_state_dict(*args, **kwargs)

    def _may_keep(self, params):
        return (not self.training) and not (torch.is_grad_enabled() and any(p.requires_grad for p in params))

    def _per_head(self, which):
        """sigma (`spread`) or beta of the heads, as the fp32 tensor the kernel reads (kept across inference calls:
        three small launches per layer otherwise)."""
        p = self.spread_weights if which == "spread" else self.beta_weights
        fn = self.get_spreads if which == "spread" else self.get_betas
        if not self._may_keep((p,)):
            return fn()
        key = (p._version, p.data_ptr(), p.dtype, self.min_spread)
        cache = self.__dict__.setdefault("_head_cache", {})
        if which not in cache or cache[which][0] != key:
            cache[which] = (key, fn().detach().float().contiguous())
        return cache[which][1]

    def _out_weight(self):
        """The output projection's weight with its input columns in (heads x d_k) order."""
        p = self.out_proj.weight
        keep = self._may_keep((p,))
        key = (p._version, p.data_ptr(), p.dtype)
        if keep and getattr(self, "_wo_cache", None) is not None and self._wo_cache[0] == key:
            return self._wo_cache[1]
        w_o = p.view(self.d_model, self.d_k, self.heads).permute(0, 2, 1).reshape(self.d_model, self.d_model)
        self._wo_cache = (key, w_o.detach()) if keep else None
        return w_o

    def _fused_qkv(self):
        """[d_model, 3*H*d_k] weight and [3*H*d_k] bias of the fused self-attention projection, from the per-head
        parameters."""
        params = (self.q_proj, self.k_proj, self.v_proj, self.q_bias, self.k_bias, self.v_bias)
        keep = self._may_keep(params)
        key = tuple((p._version, p.data_ptr(), p.dtype) for p in params)
        if keep and getattr(self, "_qkv_cache", None) is not None and self._qkv_cache[0] == key:
            return self._qkv_cache[1], self._qkv_cache[2]
        H, dk = self.heads, self.d_k
        w = torch.stack((self.q_proj, self.k_proj, self.v_proj)).permute(2, 0, 1, 3).reshape(self.d_model, 3 * H * dk)
        b = torch.stack((self.q_bias, self.k_bias, self.v_bias)).reshape(-1)
        self._qkv_cache = (key, w.detach(), b.detach()) if keep else None
        return w, b
