"""Wavefunction Embedding operators and module on the HIP kernels.

Mirrors the reference's Python surface (paths under utils/model_utils/wf_embedding/):
  wf_embedding(...) / _wf_embedding      isotropic/cuda/wf_embedding.py:18-83
  wf_embedding_learnCB(...)              anisotropic/cb_scaling/learnable_wavenumbers/cuda/wf_embedding.py:16-79
  WaveFunctionEmbedding                  wf_embedding.py:24-49
plus `we_forward` / `we_aniso_forward`, which also return what the kernels save for the backward, and
`we_backward` / `we_aniso_backward`, the reductions the two backward passes consist of.
"""
import torch
import torch.nn as nn

from . import _lib
from .cb_utils import get_coords


def we_forward(coords, wavenumbers, mask=None, tuning: int = 0, magnitude_type: int = 1, need_sums: bool = True,
               dropout_p: float = 0.0, rng_seed=None):
    """out, cos_sums, sin_sums = we_forward(coords [Z,N,3], wavenumbers [K], mask [Z,N] bool | None).

    need_sums=False (weight 1/r only) skips the sums, which only the backward uses: returns (out, None, None).
    dropout_p != 0: the reference kernel's in-kernel dropout (isotropic/cuda/wf_embedding_kernel.cu:27-46, :227-232):
    every (batch item, observer, source, wavenumber) term is kept or dropped by a hash of its four indices and
    rng_seed (a 32-bit integer; None draws a fresh one per call, as isotropic/cuda/wf_embedding.py:48-49 does), what is
    kept is divided by 1 - dropout_p, and the sums carry the same mask.
    magnitude_type: the weight of a source at distance r, 0: 1, 1: 1/r (default), 2: 1/log2(r),
    3: 1/sqrt(r) (isotropic/cuda/wf_embedding_kernel.cu:192-206); the sums carry the weight times r.

    mask: True = padded.  Unlike the reference wrapper (which crashes on
    mask=None at isotropic/cuda/wf_embedding.py:29), None means "nothing padded".
    All outputs are float32 on coords' device: out [Z,N,2K] with cos terms at
    even and sin terms at odd feature indices, cos_sums / sin_sums [Z,N,K].
    """
    if coords.dim() != 3 or coords.size(2) != 3:
        raise ValueError(f"coords must be of shape (batch, N, 3), not {tuple(coords.shape)}")
    if wavenumbers.dim() != 1:
        raise ValueError(f"wavenumbers must be of shape (K,), not {tuple(wavenumbers.shape)}")
    dropout_p = float(dropout_p)
    if not (0.0 <= dropout_p < 1.0):
        raise ValueError(f"dropout_p must be in [0, 1), not {dropout_p}")
    if not coords.is_cuda:
        raise _lib.ProteusError("we_forward needs tensors on the GPU (there is no CPU path)")
    lib = _lib.load()
    dev = coords.device
    # everything in fp32, as isotropic/cuda/wf_embedding.py:32-35
    c = coords.detach().to(torch.float32).contiguous()
    w = wavenumbers.detach().to(device=dev, dtype=torch.float32).contiguous()
    Z, N, _ = c.shape
    K = w.shape[0]
    m = None
    if mask is not None:
        if tuple(mask.shape) != (Z, N):
            raise ValueError(f"mask must be of shape ({Z}, {N}), not {tuple(mask.shape)}")
        m = mask.to(device=dev, dtype=torch.bool).contiguous().view(torch.uint8)
    out = torch.empty(Z, N, 2 * K, dtype=torch.float32, device=dev)
    need_sums = need_sums or magnitude_type != 1 or dropout_p != 0.0
    cos_sums = torch.empty(Z, N, K, dtype=torch.float32, device=dev) if need_sums else None
    sin_sums = torch.empty(Z, N, K, dtype=torch.float32, device=dev) if need_sums else None
    if Z == 0 or N == 0 or K == 0:
        return out, cos_sums, sin_sums
    with _lib.on_device(dev):
        stream = _lib.raw_stream(dev)
        if dropout_p != 0.0:
            if rng_seed is None:
                rng_seed = int(torch.randint(0, 2 ** 32, (1,), dtype=torch.int64).item())
            rc = lib.proteus_we_dropout_fwd(c.data_ptr(), _lib.COORDS_AOS, w.data_ptr(),
                                            None if m is None else m.data_ptr(),
                                            out.data_ptr(), cos_sums.data_ptr(), sin_sums.data_ptr(),
                                            Z, N, K, int(magnitude_type), dropout_p, int(rng_seed) & 0xffffffff, stream)
        elif magnitude_type == 1:
            rc = lib.proteus_we_fwd(c.data_ptr(), _lib.COORDS_AOS, w.data_ptr(),
                                    None if m is None else m.data_ptr(),
                                    out.data_ptr(), cos_sums.data_ptr() if need_sums else None,
                                    sin_sums.data_ptr() if need_sums else None,
                                    Z, N, K, int(tuning), stream)
        else:
            rc = lib.proteus_we_legacy_fwd(c.data_ptr(), _lib.COORDS_AOS, w.data_ptr(),
                                           None if m is None else m.data_ptr(),
                                           out.data_ptr(), cos_sums.data_ptr(), sin_sums.data_ptr(),
                                           Z, N, K, int(magnitude_type), stream)
    _lib.check(rc, "proteus_we_fwd")
    return out, cos_sums, sin_sums


def _bwd_prepare(dO, *saved):
    if not dO.is_cuda:
        raise RuntimeError("the WE backward runs on the HIP kernels only: tensors must be on the GPU")
    Z, N, K2 = dO.shape
    ts = [dO.contiguous().float()] + [None if t is None else t.contiguous().float() for t in saved]
    lib = _lib.load()
    ws = torch.empty(max(1, lib.proteus_we_bwd_workspace_bytes(Z, N, K2 // 2) // 4), dtype=torch.float32, device=dO.device)
    return lib, ts, ws, Z, N, K2 // 2, _lib.raw_stream(dO.device)


def we_backward(dO, cos_sums, sin_sums):
    """d_wavenumbers [K] = sum over tokens of dO_imag * cos_sums - dO_real * sin_sums
    (isotropic/cuda/wf_embedding.py:75-81), as one streaming reduction on the GPU."""
    lib, (g, c, s), ws, Z, N, K, stream = _bwd_prepare(dO, cos_sums, sin_sums)
    dk = torch.empty(K, dtype=torch.float32, device=dO.device)
    if Z == 0 or N == 0 or K == 0:
        return dk.zero_()
    with _lib.on_device(dO.device):
        rc = lib.proteus_we_bwd(g.data_ptr(), c.data_ptr(), s.data_ptr(), dk.data_ptr(), ws.data_ptr(), ws.numel() * 4,
                                Z, N, K, stream)
    _lib.check(rc, "proteus_we_bwd")
    return dk


def we_aniso_backward(dO, d_cb=None, d_k=None):
    """g_cb, g_k [K]: dO contracted with the saved per-token partials over tokens and over each (cos, sin) pair
    (anisotropic/cb_scaling/learnable_wavenumbers/cuda/wf_embedding.py:65-79).  A partial passed as None is
    skipped and its gradient returned as None."""
    if d_cb is None and d_k is None:
        return None, None
    lib, (g, a, b), ws, Z, N, K, stream = _bwd_prepare(dO, d_cb, d_k)
    g_cb = None if a is None else torch.empty(K, dtype=torch.float32, device=dO.device)
    g_k = None if b is None else torch.empty(K, dtype=torch.float32, device=dO.device)
    if Z == 0 or N == 0 or K == 0:
        return (None if g_cb is None else g_cb.zero_()), (None if g_k is None else g_k.zero_())
    ptr = lambda t: None if t is None else t.data_ptr()
    with _lib.on_device(dO.device):
        rc = lib.proteus_we_aniso_bwd(g.data_ptr(), ptr(a), ptr(b), ptr(g_cb), ptr(g_k), ws.data_ptr(), ws.numel() * 4,
                                      Z, N, K, stream)
    _lib.check(rc, "proteus_we_aniso_bwd")
    return g_cb, g_k


class _wf_embedding(torch.autograd.Function):
    """Forward on the HIP kernel; analytical O(N K) backward for the wavenumbers
    (isotropic/cuda/wf_embedding.py:64-83).  No gradient flows to coords, as in
    the reference."""

    @staticmethod
    def forward(ctx, coords, wavenumbers, magnitude_type, dropout_p, mask, recording=True, rng_seed=None):
        if magnitude_type not in (0, 1, 2, 3):
            raise AssertionError("magnitude_type must be one of 0, 1, 2, 3")
        # the sums are what the backward for the wavenumbers consumes: without that gradient they are not computed
        # (`recording`: was autograd recording when the operator was called?  Inside forward() it never is, and
        # needs_input_grad repeats requires_grad whatever the mode: under no_grad / inference_mode no backward follows)
        need = bool(recording and ctx.needs_input_grad[1])
        out, cos_sums, sin_sums = we_forward(coords, wavenumbers, mask, magnitude_type=magnitude_type, need_sums=need,
                                             dropout_p=dropout_p, rng_seed=rng_seed)
        if need:
            ctx.save_for_backward(cos_sums, sin_sums)
        ctx.need = need
        ctx.wn_dtype = wavenumbers.dtype
        return out

    @staticmethod
    def backward(ctx, dO):
        # (autograd also comes here when only another input, e.g. the coordinates, asks for a gradient: there is none to give)
        if not ctx.need:
            return None, None, None, None, None, None, None
        cos_sums, sin_sums = ctx.saved_tensors
        dk = we_backward(dO, cos_sums, sin_sums)
        return None, dk.to(ctx.wn_dtype), None, None, None, None, None


def wf_embedding(coords, wavenumbers, magnitude_type=1, dropout_p=0.0, mask=None, rng_seed=None):
    """Same call as the reference's wf_embedding (isotropic/cuda/wf_embedding.py:18); rng_seed (not in the reference,
    which draws one per call) fixes the dropout mask."""
    return _wf_embedding.apply(coords, wavenumbers, magnitude_type, dropout_p, mask, torch.is_grad_enabled(), rng_seed)


def we_aniso_forward(coordsA, coordsB, cb_magnitudes, wavenumbers, mask=None, tuning: int = 0, partials: bool = True):
    """out, d_cb, d_k = we_aniso_forward(coordsA [Z,N,3], coordsB [Z,N,3], cb_magnitudes [K], wavenumbers [K], mask).

    partials=False: only the embedding is computed (d_cb and d_k come back as None): the kernel keeps two running sums
    per wavenumber instead of six.

    coordsA: token positions; coordsB: per-token C-beta direction vectors (relative to the token);
    mask [Z,N] bool, True = padded (None = nothing padded).  All outputs float32 [Z,N,2K], cos/real
    terms at even and sin/imag terms at odd indices: the embedding and its per-token partial
    derivatives with respect to cb_magnitudes and wavenumbers
    (anisotropic/cb_scaling/learnable_wavenumbers/cuda/wf_embedding_kernel.cu:163-206).
    """
    if coordsA.dim() != 3 or coordsA.size(2) != 3:
        raise ValueError(f"coordsA must be of shape (batch, N, 3), not {tuple(coordsA.shape)}")
    if tuple(coordsB.shape) != tuple(coordsA.shape):
        raise ValueError(f"coordsB must have coordsA's shape {tuple(coordsA.shape)}, not {tuple(coordsB.shape)}")
    if wavenumbers.dim() != 1 or tuple(cb_magnitudes.shape) != tuple(wavenumbers.shape):
        raise ValueError(f"cb_magnitudes and wavenumbers must both be of shape (K,), not "
                         f"{tuple(cb_magnitudes.shape)} and {tuple(wavenumbers.shape)}")
    if not coordsA.is_cuda:
        raise _lib.ProteusError("we_aniso_forward needs tensors on the GPU (there is no CPU path)")
    lib = _lib.load()
    dev = coordsA.device
    a = coordsA.detach().to(torch.float32).contiguous()
    b = coordsB.detach().to(device=dev, dtype=torch.float32).contiguous()
    w = wavenumbers.detach().to(device=dev, dtype=torch.float32).contiguous()
    cb = cb_magnitudes.detach().to(device=dev, dtype=torch.float32).contiguous()
    Z, N, _ = a.shape
    K = w.shape[0]
    m = None
    if mask is not None:
        if tuple(mask.shape) != (Z, N):
            raise ValueError(f"mask must be of shape ({Z}, {N}), not {tuple(mask.shape)}")
        m = mask.to(device=dev, dtype=torch.bool).contiguous().view(torch.uint8)
    out = torch.empty(Z, N, 2 * K, dtype=torch.float32, device=dev)
    d_cb = torch.empty_like(out) if partials else None
    d_k = torch.empty_like(out) if partials else None
    if Z == 0 or N == 0 or K == 0:
        return out, d_cb, d_k
    with _lib.on_device(dev):
        stream = _lib.raw_stream(dev)
        rc = lib.proteus_we_aniso_fwd(a.data_ptr(), b.data_ptr(), _lib.COORDS_AOS, cb.data_ptr(), w.data_ptr(),
                                      None if m is None else m.data_ptr(),
                                      out.data_ptr(), d_cb.data_ptr() if partials else None, d_k.data_ptr() if partials else None,
                                      Z, N, K, int(tuning), stream)
    _lib.check(rc, "proteus_we_aniso_fwd")
    return out, d_cb, d_k


class _wf_embedding_learnCB(torch.autograd.Function):
    """Forward on the HIP kernel; the backward contracts the saved per-token partial derivatives with dO
    (anisotropic/cb_scaling/learnable_wavenumbers/cuda/wf_embedding.py:65-79).  No gradient flows to the
    coordinates, as in the reference."""

    @staticmethod
    def forward(ctx, coordsA, coordsB, cb_magnitudes, wavenumbers, mask, recording=True):
        # the per-token partial derivatives are computed only if autograd will ask for the gradient of one of the two
        # scales: `recording` says whether autograd was recording at the call (inside forward() it never is, and
        # needs_input_grad repeats requires_grad whatever the mode: under no_grad / inference_mode no backward follows)
        ctx.need = bool(recording and (ctx.needs_input_grad[2] or ctx.needs_input_grad[3]))
        out, d_cb, d_k = we_aniso_forward(coordsA, coordsB, cb_magnitudes, wavenumbers, mask, partials=ctx.need)
        if ctx.need:
            ctx.save_for_backward(d_cb, d_k)
        ctx.dtypes = (cb_magnitudes.dtype, wavenumbers.dtype)
        return out.to(coordsA.dtype)

    @staticmethod
    def backward(ctx, dO):
        if not ctx.need:
            return None, None, None, None, None, None
        d_cb, d_k = ctx.saved_tensors
        g_cb, g_k = we_aniso_backward(dO, d_cb if ctx.needs_input_grad[2] else None,
                                      d_k if ctx.needs_input_grad[3] else None)
        return (None, None, None if g_cb is None else g_cb.to(ctx.dtypes[0]),
                None if g_k is None else g_k.to(ctx.dtypes[1]), None, None)


def wf_embedding_learnCB(coordsA, coordsB, cb_magnitudes, wavenumbers, mask=None):
    """Same call as the reference's anisotropic wf_embedding
    (anisotropic/cb_scaling/learnable_wavenumbers/cuda/wf_embedding.py:16)."""
    return _wf_embedding_learnCB.apply(coordsA, coordsB, cb_magnitudes, wavenumbers, mask, torch.is_grad_enabled())


class WaveFunctionEmbedding(nn.Module):
    """Same constructor and forward as utils/model_utils/wf_embedding/wf_embedding.py:24-49.

    The wavelength schedule follows the code (torch.logspace, endpoint
    inclusive), the parameter holds log(wavenumber).  anisotropic=True (the
    reference default) takes the C-beta scaled kernel and needs coords_beta.
    """

    def __init__(self, d_wf=512, min_wl=4.0, max_wl=35.0, base_wl=20.0, anisotropic=True, learn_wl=False, learn_aa=False):
        super().__init__()
        wl = min_wl + (max_wl - min_wl) * ((torch.logspace(0, 1, d_wf // 2, base_wl) - 1) / (base_wl - 1))
        wn = torch.log(torch.pi * 2 / wl)
        self.wavenumbers = nn.Parameter(wn, requires_grad=learn_wl)
        self.aa_magnitudes = nn.Parameter(torch.ones(d_wf // 2), requires_grad=learn_aa)
        self.aniso = anisotropic

    def get_wavenumbers(self):
        return torch.exp(self.wavenumbers)

    def forward(self, coords_alpha, coords_beta=None, key_padding_mask=None):
        if self.aniso:
            if coords_beta is None:
                raise ValueError("the anisotropic embedding needs coords_beta (see get_CaCb_coords)")
            return wf_embedding_learnCB(coords_alpha, coords_beta, self.aa_magnitudes, self.get_wavenumbers(),
                                        mask=key_padding_mask)
        return wf_embedding(coords_alpha, self.get_wavenumbers(), magnitude_type=1, dropout_p=0.0, mask=key_padding_mask)

    def get_CaCb_coords(self, coords, chain_idxs=None, norm=False):
        return get_coords(coords, chain_idxs, norm)
