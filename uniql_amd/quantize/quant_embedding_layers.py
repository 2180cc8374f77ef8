"""int4 embedding table with one fp16 scale per row
(reference: quantize/quant_embedding_layers.py:8-54)."""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import layout, ops


class W4O16Embedding(nn.Module):
    """weight: int32 [V, D/8] Parameter (frozen; a Parameter so that
    next(model.parameters()) works), scales: fp16 [V] buffer."""

    def __init__(self, num_embeddings, embedding_dim, device=None, **kwargs):
        super().__init__()
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        self.num_bits = 4
        self.pack_factor = 32 // self.num_bits
        table = torch.empty((num_embeddings, embedding_dim // self.pack_factor), dtype=torch.int32, device=device)
        self.register_parameter("weight", nn.Parameter(table, requires_grad=False))
        self.register_buffer("scales", torch.empty(num_embeddings, dtype=torch.float16, device=device))

    @classmethod
    def from_fp16(cls, originalLayer: nn.Embedding):
        w = originalLayer.weight.data
        q = cls(originalLayer.num_embeddings, originalLayer.embedding_dim, device=w.device)
        if w.is_cuda and w.dtype == torch.float16 and originalLayer.embedding_dim % 8 == 0:
            # the device kernel: same codes and scales bit for bit, no host round trip
            packed, scales = ops.w4_embedding_quantize(w.contiguous())
        else:
            packed, scales = layout.quantize_embedding(w)
        q.scales = scales.to(w.device)
        q.weight.data = packed.to(w.device)
        return q

    @torch.no_grad()
    def forward(self, x):
        return ops.w4a16_embedding_lookup(x, self.weight, self.scales)

    def __repr__(self):
        return f"W4O16Embedding(num_embeddings={self.num_embeddings}, embedding_dim={self.embedding_dim})"
