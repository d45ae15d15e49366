"""MI355X-native attention forward path with the call signatures of
rookie-joe/TritonOps' flash_attn_triton package."""
from .ops import (  # noqa: F401
    LOG2E,
    dense_form,
    flash_attention,
    flash_attention_decoding,
    flash_attention_sparse_decoding,
    flash_attn_sparse_triton,
    flash_attn_triton,
    flash_attn_triton_bwd,
    flash_attn_triton_fwd,
)
from .rms import RMSNormTriton, RMSNormTritonFunction, rmsnorm_bwd, rmsnorm_fwd  # noqa: F401
from .xent import (  # noqa: F401
    CrossEntropyFusedFunction,
    cross_entropy_dlogits,
    cross_entropy_dlogits_,
    cross_entropy_fused_bwd,
    cross_entropy_fused_fwd,
    cross_entropy_fused_triton,
)
from . import masks  # noqa: F401
