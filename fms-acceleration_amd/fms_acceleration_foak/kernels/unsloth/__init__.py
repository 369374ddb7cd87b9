from .rms_layernorm import fast_rms_layernorm
from .rope_embedding import fast_rope_embedding
