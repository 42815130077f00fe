"""Model wrapper of a Dimudra checkpoint: the module interface the generation paths expect from `models.<type>.Model` for a
text-only model.  The language model keeps its residual stream in fp32 and looks the embedding up inside its step
(models/ragged.py, TokenIdModel)."""
from __future__ import annotations

from ..ragged import TokenIdModel
from .config import ModelConfig  # noqa: F401
from .language import LanguageModel


class Model(TokenIdModel):
    NAME = "Dimudra"
    LanguageModel = LanguageModel
