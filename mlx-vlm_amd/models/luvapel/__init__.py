"""`models.luvapel`: a decoder-only language model whose layers read the residual stream un-normed and norm / gate their
results: generalized delta-rule layers, and layers that run sliding-window attention and a gated delta rule side by side;
dense relu^2 feed-forwards; layers may share another layer's weights.  Module contract of the other model packages
(ModelConfig / Model / LanguageModel)."""
from .config import LayerConfig, ModelConfig
from .language import LanguageModel
from .luvapel import Model

__all__ = ["Model", "ModelConfig", "LayerConfig", "LanguageModel"]

# the operator sources (csrc/<name>.hip) the model's step function needs: what a trace replay of a fresh checkout compiles
HIP_SOURCES = ('gemm_bf16', 'gemm256_bf16', 'linear_any', 'stream_f32', 'window_attn', 'delta_rule')
