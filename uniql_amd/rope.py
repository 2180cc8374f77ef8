"""Rotary position embedding for attention heads pruned to a subset of their columns
(reference: modeling/rope_triton.py, modeling/llama/llama_rope.py:38-96)."""
from __future__ import annotations

from . import ops


def apply_rotary_pos_emb_indices(q, k, cos, sin, indices, unsqueeze_dim=1):
    """Same call as the reference's apply_rotary_pos_emb_indices(_triton): q [b, n_q_heads, s, d]
    and k [b, n_kv_heads, s, d] as the attention blocks hold them (transposed views of the
    projections' token-major outputs), cos / sin [1 or b, s, D], indices [n_kv_heads, d].
    Returns the rotated (q, k) in the same [b, heads, s, d] view.  Like the Triton version it
    works on the token-major storage: in place when the transposed view is contiguous, on a
    contiguous copy otherwise."""
    if unsqueeze_dim != 1:
        raise NotImplementedError("only the [batch, heads, seq, dim] arrangement (unsqueeze_dim=1) is supported")
    qt = q.transpose(1, 2).contiguous()
    kt = k.transpose(1, 2).contiguous()
    if cos.dim() == 2:
        cos, sin = cos.unsqueeze(0), sin.unsqueeze(0)
    ops.rope_indices_(qt, kt, cos.contiguous(), sin.contiguous(), indices.contiguous())
    return qt.transpose(1, 2), kt.transpose(1, 2)


apply_rotary_pos_emb_indices_triton = apply_rotary_pos_emb_indices  # the name the reference's blocks import
