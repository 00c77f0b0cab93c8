"""Model wrapper of a Garesun checkpoint: the module contract the generation paths expect from `models.<type>.Model` for a
text-only model.  The design adds a gated slice of a SECOND embedding table at every layer, so the language model needs the token ids, not
only their embeddings (models/ragged.py, TokenIdModel)."""
from __future__ import annotations

from ..ragged import TokenIdModel
from .config import ModelConfig  # noqa: F401
from .language import LanguageModel


class Model(TokenIdModel):
    NAME = "Garesun"
    LanguageModel = LanguageModel
