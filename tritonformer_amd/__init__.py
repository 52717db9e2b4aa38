"""MI355X-native (gfx950) kernel layer with the operator surface of
fattorib/tritonformer: the aliases below are the ones its ``__init__.py``
exports, backed by hand-written HIP kernels behind a C ABI."""
# The HIP library is loaded on the first kernel call (see _lib.load); if it has
# not been built that call raises: there is no PyTorch or CPU fallback.
from .attention import AttentionBlock as attention_block
from .attention import BiasedCausalAttention as fast_causal_attention_with_bias
from .attention import CausalAttention as fast_causal_attention
from .attention import PackedCausalAttention as fast_causal_attention_qkvpacked
from .crossentropy import CrossEntropyLoss as cross_entropy_loss
from .crossentropy import LMHeadLoss as lm_head_loss
from .crossentropy import ShiftedCrossEntropyLoss as shifted_cross_entropy_loss
from .embedding import EmbeddingSum as embedding_sum
from .layernorm import AddLayerNorm as add_layer_norm
from .layernorm import LayerNorm as layer_norm
from .linear import LinearBias as linear_bias
from .linear import LinearBiasReLU as linear_fused_bias_relu
from .linear import LinearNoBias as linear_no_bias
from .linear import LinearNoBiasReLU as linear_fused_relu
from .linear import MLPReLU as mlp_fused_relu
from .linear import PackedLinearNoBias as linear_no_bias_packed
from .softmax import Softmax
from ._amp import clear_weight_cast_cache, set_weight_cast_cache, weight_cast_cache_enabled
