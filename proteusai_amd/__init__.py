"""MI355X (gfx950) implementation of proteusAI's two O(N^2) kernels behind the
reference's Python operator API.  The HIP library is loaded lazily on first
use; there is no CPU fallback."""
from .wf_embedding import WaveFunctionEmbedding, we_forward, wf_embedding  # noqa: F401
from .geometric_attn import GeoAttention, geo_attn, geometric_attn  # noqa: F401
from .encoder import MLP, Encoder, ProteusEncoder  # noqa: F401
