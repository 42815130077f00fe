"""`models.tilalorn`: a pre-norm decoder-only language model whose layers mix tokens either by grouped-head softmax attention
(biased projections, unit-RMS queries and keys, a query multiplier that grows with the logarithm of the position, capped
scores, one sigmoid gate per head; a layer may read an earlier layer's keys and values) or by latent attention with rotary
positions inside a sliding window (one cached row per token, elementwise sigmoid gate); feed-forwards are dense gated-gelu
layers or group-limited mixtures of silu experts; tied output head.  Same module interface as the other model packages
(ModelConfig / Model / LanguageModel)."""
from .config import LayerConfig, ModelConfig
from .language import LanguageModel
from .tilalorn import Model

__all__ = ["Model", "ModelConfig", "LayerConfig", "LanguageModel"]

# the operator sources (csrc/<name>.hip) the model's step function needs: what a trace replay of a fresh checkout compiles
HIP_SOURCES = ('gemm_bf16', 'gemm256_bf16', 'linear_any', 'stream_f32', 'moe', 'latent_attn', 'window_attn')
