"""Token embedding and output head.

stream[t] = E[id[t]] * scale (scale 1 by default), no position term (inference_engine/model.py:96,168);
logits = y W_lm^T * scale with W_lm = E when tied (inference_engine/model.py:112-113,185; the tied
table is used as stored, without the embedding's scale); with ``softcap`` = c the scaled logits pass through
c * tanh(logits / c).  The stream is 32-bit; logits come out in 32-bit.
"""
from __future__ import annotations

import torch

from .base import ParamSpec, Part


class Embedding(Part):
    def __init__(self, vocab_size: int, width: int, weight_name: str, scale: float = 1.0):
        self.vocab_size = int(vocab_size)
        self.width = int(width)
        self.weight_name = weight_name
        self.scale = float(scale)
        self.weight = None

    def params(self):
        return [ParamSpec.single("weight", self.weight_name, (self.vocab_size, self.width))]

    def forward(self, ids, taken_from=None, earlier_tokens=None):
        """``taken_from`` / ``earlier_tokens``: see KernelBackend.embedding (tokens still on the device)."""
        if self.scale != 1.0:
            return self.ops.embedding(ids, self.weight, taken_from, earlier_tokens, scale=self.scale)
        return self.ops.embedding(ids, self.weight, taken_from, earlier_tokens)


class LMHead(Part):
    def __init__(self, vocab_size: int, width: int, weight_name: str, tied_to: Embedding | None = None,
                 scale: float = 1.0, softcap: float | None = None):
        self.scale = float(scale)
        if softcap is not None and not softcap > 0:
            raise ValueError("softcap must be positive or None")
        self.softcap = None if softcap is None else float(softcap)
        self.vocab_size = int(vocab_size)
        self.width = int(width)
        self.weight_name = weight_name
        self.tied_to = tied_to
        self._weight = None

    def params(self):
        if self.tied_to is not None:
            return []
        return [ParamSpec.single("_weight", self.weight_name, (self.vocab_size, self.width))]

    @property
    def weight(self):
        return self.tied_to.weight if self.tied_to is not None else self._weight

    def forward(self, y):
        logits = self.ops.linear(y, self.weight, out_dtype=torch.float32)
        if self.softcap is not None:
            return self.ops.scale_softcap_(logits, self.scale, self.softcap)
        return logits if self.scale == 1.0 else self.ops.scale_(logits, self.scale)
