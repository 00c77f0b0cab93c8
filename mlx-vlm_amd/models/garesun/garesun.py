"""Model wrapper of a Garesun checkpoint: the module contract the generation paths expect from `models.<type>.Model`
(`language_model`, `get_input_embeddings`, `sanitize`, `load_weights`) for a text-only model.

The design adds a gated slice of a SECOND embedding table at every layer, so the language model needs the token ids, not
only their embeddings: `get_input_embeddings` hands the ids through as the "embeddings" (int32 [1, L, 1]) and the language
model looks both tables up inside its step."""
from __future__ import annotations

import numpy as np
import torch

from ... import _lib
from ..base import InputEmbeddingsFeatures
from .config import ModelConfig
from .language import LanguageModel


class Model:
    def __init__(self, config: ModelConfig, device="cuda", **kwargs):
        self.config = config
        self.model_type = config.model_type
        self.vision_tower = None
        self.language_model = LanguageModel(config, device=device, **kwargs)

    @property
    def layers(self):
        return self.language_model.layers

    def get_input_embeddings(self, input_ids=None, pixel_values=None, **kwargs) -> InputEmbeddingsFeatures:
        if pixel_values is not None:
            raise ValueError("Garesun is a text-only model")
        ids = np.asarray(input_ids.detach().cpu().numpy() if isinstance(input_ids, torch.Tensor) else input_ids, dtype=np.int32)
        if ids.ndim == 1:
            ids = ids[None]
        B, L = ids.shape
        pos = np.broadcast_to(np.arange(L, dtype=np.int64)[None], (B, L)).copy()
        return InputEmbeddingsFeatures(inputs_embeds=_lib.h2d(ids.reshape(B, L, 1), self.language_model.device), position_ids=pos,
                                       rope_deltas=np.zeros((B, 1), dtype=np.int64))

    def sanitize(self, weights):
        return weights

    def load_weights(self, weights):
        self.language_model.load_weights(weights)
        return self

    def __call__(self, input_ids, pixel_values=None, mask=None, cache=None, **kwargs):
        return self.language_model(input_ids, cache=cache, **kwargs)
