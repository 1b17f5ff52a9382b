"""MI355X (gfx950) implementation of proteusAI's two O(N^2) kernels behind the
reference's Python operator API.  The HIP library is loaded lazily on first
use; there is no CPU fallback."""
from .wf_embedding import (WaveFunctionEmbedding, we_aniso_backward, we_aniso_forward, we_backward,  # noqa: F401
                           we_forward, wf_embedding, wf_embedding_learnCB)
from .cb_utils import get_Cb_from_BB, get_Cb_from_Ca, get_coords  # noqa: F401
from .geometric_attn import GeoAttention, geo_attn, geo_attn_backward, geometric_attn, geometric_attn_qkv  # noqa: F401
from .encoder import MLP, Encoder, ProteusEncoder  # noqa: F401
