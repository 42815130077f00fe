"""`models.dimudra`: a pre-norm decoder-only language model whose norms carry ONE number as their weight and whose mixers read
the normed stream through a short causal convolution with a residual.  A span of layers may run several times in a row with the
same tensors (every run with a cache / state of its own, the embedding output added again before each further pass).  Mixers:
*parallel* - sliding-window softmax attention (biased projections, RMS norm over the whole q / k row, no positions, sigmoid
output gate) side by side with a selective state-space scan; *hgrn2* - a matrix-state recurrence whose lower-bounded forget
gate also decides what is written; *attention* - causal attention with partial rotate-half positions, unit-RMS q / k per head
and a sink in the softmax.  Feed-forwards are mixtures of silu experts routed by sigmoid scores with a choice-only correction
and a group limit, plus a gated shared expert.  Same module interface as the other model packages."""
from .config import LayerConfig, ModelConfig
from .language import LanguageModel
from .dimudra import Model

__all__ = ["Model", "ModelConfig", "LayerConfig", "LanguageModel"]

# the operator sources (csrc/<name>.hip) the model's step function needs: what a trace replay of a fresh checkout compiles
HIP_SOURCES = ('gemm_bf16', 'gemm256_bf16', 'linear_any', 'stream_f32', 'moe', 'window_attn', 'linear_recurrence', 'short_conv',
               'selective_scan')
