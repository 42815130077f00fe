"""`models.garesun`: a decoder-only language model of heterogeneous layers - matrix-state recurrences (fixed-decay
retention, gated mLSTM) and latent attention, each in parallel with a mixture-of-experts feed-forward, plus a per-layer
token input - with the module contract of the other model packages (ModelConfig / Model / LanguageModel)."""
from .config import LayerConfig, ModelConfig
from .garesun import Model
from .language import LanguageModel

__all__ = ["Model", "ModelConfig", "LayerConfig", "LanguageModel"]

# the operator sources (csrc/<name>.hip) the model's step function needs: what a trace replay of a fresh checkout compiles
HIP_SOURCES = ('gemm_bf16', 'gemm256_bf16', 'linear_any', 'stream_f32', 'moe', 'latent_attn', 'linear_recurrence')
