"""MI355X-native T5 attention forward: HIP kernels behind the reference's plugin surface."""
from .config import T5Config  # noqa: F401
from .ops import (  # noqa: F401
    block_attention_with_fusing_bias,
    flash_attention_with_fusing_bias,
    flash_attention_with_fusing_bias_varlen,
    flash_attn_v2_fwd,
    flash_decoding_attention,
    local_attention_with_fusing_bias,
    transient_global_attention_with_fusing_bias,
)
from .attentions import (  # noqa: F401
    T5ATTENTION_TYPES,
    T5BlockAttention,
    T5FlashAttention,
    T5LocalAttention,
    T5TransientGlobalAttention,
)
from .modeling import T5EncoderModel, T5Model, T5Stack  # noqa: F401
from .graphs import GraphedForward  # noqa: F401
