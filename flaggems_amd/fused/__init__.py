from .fused_add_rms_norm import fused_add_rms_norm
from .reshape_and_cache import reshape_and_cache
from .reshape_and_cache_flash import reshape_and_cache_flash
from .rotary_embedding import apply_rotary_pos_emb
from .silu_and_mul import silu_and_mul, silu_and_mul_out

__all__ = [
    "apply_rotary_pos_emb",
    "fused_add_rms_norm",
    "reshape_and_cache",
    "reshape_and_cache_flash",
    "silu_and_mul",
    "silu_and_mul_out",
]
