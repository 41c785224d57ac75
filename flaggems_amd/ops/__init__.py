from .addmm import addmm, addmm_out
from .attention import flash_attention_forward, flash_attn_varlen_func, scaled_dot_product_attention
from .bmm import bmm
from .log_softmax import log_softmax, log_softmax_backward
from .mm import mm, mm_out
from .rms_norm import rms_norm
from .softmax import softmax, softmax_backward

__all__ = [
    "addmm", "addmm_out", "bmm", "flash_attention_forward", "flash_attn_varlen_func", "log_softmax", "log_softmax_backward",
    "mm", "mm_out", "rms_norm", "scaled_dot_product_attention", "softmax", "softmax_backward",
]
