"""Virtual C-beta direction vectors for the anisotropic embedding.

Same functions as the reference's utils/model_utils/base_modules/Cb_utils.py:3-115
(`get_coords`, `get_Cb_from_Ca`, `get_Cb_from_BB`): the C-beta position relative to
C-alpha is the fixed linear combination of the two backbone bond vectors and their
cross product (the constants of Cb_utils.py:85 and :109).
"""
import torch

# weights of (CA-N), (C-CA) and their cross product
_W_B1, _W_B2, _W_B3 = 0.56802827, -0.58273431, -0.54067466
# ideal N-CA and CA-C bond lengths used when only C-alpha is known (Cb_utils.py:79,81)
_LEN_N_CA, _LEN_CA_C = 1.458, 1.525


def _combine(b1, b2):
    return _W_B1 * b1 + _W_B2 * b2 + _W_B3 * torch.linalg.cross(b1, b2, dim=-1)


def _unit(v, eps=1e-6):
    return v / torch.linalg.vector_norm(v, dim=-1, keepdim=True).clamp(min=eps)


def get_Cb_from_BB(coords, norm=False):
    """coords [Z,N,3(N,CA,C),3] -> (CA [Z,N,3], Cb - CA [Z,N,3]).  Padded tokens with all-zero
    coordinates give a zero vector (Cb_utils.py:94-115)."""
    n, ca, c = coords[:, :, 0, :], coords[:, :, 1, :], coords[:, :, 2, :]
    cb = _combine(ca - n, c - ca)
    return ca, (_unit(cb) if norm else cb)


def get_Cb_from_Ca(coordsA, chain_idxs, norm=True):
    """coordsA [Z,N,3], chain_idxs[z] = [[start, stop), ...] -> (coordsA, Cb - CA [Z,N,3]).

    Inside a chain the previous and next C-alpha stand in for the directions to N and C, with ideal
    bond lengths; the first and last token of a chain, chains shorter than 3 and tokens outside any
    chain get the zero vector (Cb_utils.py:20-92).  With norm=True the vectors are scaled to unit
    length (what Cb_utils.py:90 intends; the reference line names an undefined variable).
    """
    Z, N, _ = coordsA.shape
    interior = torch.zeros(Z, N, dtype=torch.bool)
    for z, chains in enumerate(chain_idxs):
        for start, stop in chains:
            lo, hi = max(int(start) + 1, 0), min(int(stop) - 1, N)
            if hi > lo:
                interior[z, lo:hi] = True
    interior = interior.to(coordsA.device)
    prev = torch.roll(coordsA, 1, dims=1)
    nxt = torch.roll(coordsA, -1, dims=1)
    b1 = _LEN_N_CA * _unit(coordsA - prev)
    b2 = _LEN_CA_C * _unit(nxt - coordsA)
    cb = torch.where(interior.unsqueeze(-1), _combine(b1, b2), torch.zeros_like(coordsA))
    return coordsA, (_unit(cb) if norm else cb)


def get_coords(coords, chain_idxs=None, norm=True):
    """Dispatch on the input rank, as Cb_utils.py:3-18: [Z,N,3] is a C-alpha trace (needs chain_idxs),
    [Z,N,3,3] a backbone."""
    if coords.dim() == 3:
        if chain_idxs is None:
            raise ValueError("chain_idxs must be provided for Ca only model")
        return get_Cb_from_Ca(coords, chain_idxs, norm)
    if coords.dim() == 4:
        return get_Cb_from_BB(coords, norm)
    raise ValueError("invalid input size for coordinates, expected (batch,N,3) for Ca only model or "
                     f"(batch,N,3,3) for backbone model, but got {coords.shape=}")
