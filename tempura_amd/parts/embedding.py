"""Token embedding and output head.

``hidden[t] = embed[token[t]]`` with no scaling
(/root/reference/engine/src/model.rs:672-684); logits are
``norm(hidden)[rows] @ lm_head^T`` in float32, and when the checkpoint has no
output matrix the embedding matrix is used for it
(/root/reference/engine/src/weights.rs:156-166).

Two options beyond that: the embedding may add a sinusoidal position vector (``position: "sinusoid"`` with
``position_base`` b: element 2i of position p gets sin(p * b^(-2i / hidden)), element 2i + 1 the cosine), and the
head may multiply its logits by a constant (``scale``).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, WeightInfo, register_part


class TokenEmbedding(Part):
    category = "embedding"

    def __init__(self, spec, hidden_size, dtype, device, vocab_size):
        super().__init__(spec, hidden_size, dtype, device)
        self.vocab_size = vocab_size
        self.weight = None
        kind = spec.params.get("position")
        if kind not in (None, "sinusoid"):
            raise ValueError(f"embedding: position {kind!r} unknown (known: sinusoid)")
        self.inv_freq = None
        if kind == "sinusoid":
            base = float(spec.params.get("position_base", 10000.0))
            i = torch.arange((hidden_size + 1) // 2, dtype=torch.float64)
            # float64 on the host; the kernel forms the angle in float64 too
            self.inv_freq = torch.pow(torch.tensor(base, dtype=torch.float64), -2.0 * i / hidden_size).to(device)

    @classmethod
    def expected_weights(cls, spec, hidden_size, vocab_size):
        return {spec.weights["weight"]: WeightInfo((vocab_size, hidden_size))}

    def load_weights(self, get):
        self.weight = self._to_device(get(self.spec.weights["weight"]))

    def forward(self, tokens, positions=None, streams: int = 1):
        """int32 [tokens] -> float32 [tokens, streams * hidden]: ``streams`` copies of the residual stream."""
        if self.inv_freq is None and streams == 1:
            return ops.embed(tokens, self.weight)
        return ops.embed(tokens, self.weight, positions, self.inv_freq, streams)


class OutputHead(Part):
    category = "lm_head"

    def __init__(self, spec, hidden_size, dtype, device, vocab_size):
        super().__init__(spec, hidden_size, dtype, device)
        self.vocab_size = vocab_size
        self.weight = None
        self.tied = bool(spec.params.get("tied", False))
        self.scale = float(spec.params.get("scale", 1.0))

    @classmethod
    def expected_weights(cls, spec, hidden_size, vocab_size):
        # Tied: the tensor is neither required nor generated, and is ignored if present.
        init = "skip" if spec.params.get("tied", False) else "normal"
        return {spec.weights["weight"]: WeightInfo((vocab_size, hidden_size), init, optional=True)}

    def load_weights(self, get, embedding: TokenEmbedding = None):
        t = None if self.tied else get(self.spec.weights["weight"], optional=True)
        if t is None:
            if embedding is None or embedding.weight is None:
                raise ValueError("output head is tied but no embedding matrix is loaded")
            # The products read tiled weights at nearly twice the rate of row-major ones (the head of the 3B shape,
            # 128256 x 3072: 208 us row-major, 120 us tiled), and the lookup needs the rows as they are: the head
            # takes a tiled copy where the kernels have a tiled form (bfloat16 on the GPU; vocab x hidden x 2 bytes
            # more), else the same buffer.
            self.weight = ops.tile_weight(embedding.weight)
            self.tied = True
        else:
            self.weight = ops.tile_weight(self._to_device(t))

    def forward(self, x):
        """normed rows [m, hidden] -> float32 logits [m, vocab]."""
        logits = ops.linear(x, self.weight, torch.float32)
        return logits if self.scale == 1.0 else ops.scale_(logits, self.scale)


register_part("embedding", "embedding", TokenEmbedding)
register_part("lm_head", "lm_head", OutputHead)
