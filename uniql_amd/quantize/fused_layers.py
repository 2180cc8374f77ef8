"""Projections that read the same input, run as one kernel launch.

The reference's blocks call their W4A16B16O16Linear layers one after another:
    q_proj(x), k_proj(x), v_proj(x)              (modeling/llama/llama_qblocks.py:104-106)
    act_fn(gate_proj(x)) * up_proj(x)            (modeling/llama/llama_qblocks.py:48-51)
Every call is a kernel launch plus the tensor operations around it, which at decode sizes cost
as much as the product itself.  The classes here are built from the loaded layers (so the
checkpoint format stays the reference's) and give the same values:

    qkv = W4A16FusedLinear.from_linears([attn.q_proj, attn.k_proj, attn.v_proj])
    q, k, v = qkv(x)
    gate_up = W4A16GateUpSiLU.from_linears(mlp.gate_proj, mlp.up_proj)
    h = gate_up(x)                                # == silu(gate_proj(x)) * up_proj(x)
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import layout, ops
from .quant_linear_layers import W4A16B16O16Linear


def _check_same_input(layers):
    first = layers[0]
    for l in layers:
        if not isinstance(l, W4A16B16O16Linear):
            raise TypeError("expected W4A16B16O16Linear layers")
        if (l.in_features, l.size_k, l.scale.shape[0]) != (first.in_features, first.size_k, first.scale.shape[0]):
            raise ValueError("fused layers must have the same input width and scale grouping")
        if (l.had_block, l.had_scale) != (first.had_block, first.had_scale):
            raise ValueError("fused layers must rotate their input the same way")
        if l.weight.device != first.weight.device:
            raise ValueError("fused layers must live on one device")


class W4A16FusedLinear(nn.Module):
    """Several W4A16 layers over the same input as one product: the packed tensors are laid
    side by side along N, the call returns one tensor per layer (views of one buffer)."""

    def __init__(self, layers):
        super().__init__()
        layers = list(layers)
        _check_same_input(layers)
        first = layers[0]
        self.in_features, self.size_k = first.in_features, first.size_k
        self.had_block, self.had_scale = first.had_block, first.had_scale
        self.out_features = [l.out_features for l in layers]
        self.offsets = [0]
        for l in layers:
            self.offsets.append(self.offsets[-1] + l.size_n)
        self.size_n = self.offsets[-1]
        weight, scale = layout.concat_columns([l.weight for l in layers], [l.scale for l in layers])
        self.register_buffer("weight", weight)
        self.register_buffer("scale", scale)
        self.register_buffer("workspace", torch.zeros((self.size_n // layout.MIN_THREAD_N) * layout.MAX_PARALLEL,
                                                      dtype=torch.int32, device=weight.device))
        if any(l.bias is not None for l in layers):
            bias = torch.zeros(self.size_n, dtype=torch.float16, device=weight.device)
            for l, off in zip(layers, self.offsets):
                if l.bias is not None:
                    bias[off:off + l.out_features] = l.bias.data
            self.register_buffer("bias", bias)
        else:
            self.bias = None

    @classmethod
    def from_linears(cls, layers):
        return cls(layers)

    @torch.no_grad()
    def forward(self, x):
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        if x2.stride(-1) != 1:
            x2 = x2.contiguous()
        y = ops.w4a16_linear(x2, self.weight, self.scale, self.workspace, self.size_n, self.size_k,
                             bias=self.bias, had_block=self.had_block, had_scale=self.had_scale)
        return tuple(y[:, off:off + n].reshape(*lead, n) for off, n in zip(self.offsets, self.out_features))

    def __repr__(self):
        return f"W4A16FusedLinear(in_features={self.in_features}, out_features={self.out_features})"


class W4A16GateUpSiLU(nn.Module):
    """silu(gate_proj(x)) * up_proj(x) in one launch: both projections interleaved in blocks of
    64 columns, the activation and the product applied to the finished sums inside the
    kernel with the reference's fp16 roundings."""

    def __init__(self, gate_proj: W4A16B16O16Linear, up_proj: W4A16B16O16Linear):
        super().__init__()
        _check_same_input([gate_proj, up_proj])
        if gate_proj.out_features != up_proj.out_features:
            raise ValueError("gate and up projections must have the same width")
        self.in_features, self.size_k = gate_proj.in_features, gate_proj.size_k
        self.out_features = gate_proj.out_features
        self.had_block, self.had_scale = gate_proj.had_block, gate_proj.had_scale
        weight, scale = layout.interleave_gate_up(gate_proj.weight, gate_proj.scale, up_proj.weight, up_proj.scale)
        self.size_n = scale.shape[1]
        self.register_buffer("weight", weight)
        self.register_buffer("scale", scale)
        self.register_buffer("workspace", torch.zeros((self.size_n // layout.MIN_THREAD_N) * layout.MAX_PARALLEL,
                                                      dtype=torch.int32, device=weight.device))
        if gate_proj.bias is not None or up_proj.bias is not None:
            bias = torch.zeros(2, self.out_features, dtype=torch.float16, device=weight.device)
            if gate_proj.bias is not None:
                bias[0] = gate_proj.bias.data
            if up_proj.bias is not None:
                bias[1] = up_proj.bias.data
            self.register_buffer("bias", bias.reshape(-1))
        else:
            self.bias = None

    @classmethod
    def from_linears(cls, gate_proj, up_proj):
        return cls(gate_proj, up_proj)

    @torch.no_grad()
    def forward(self, x):
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        if x2.stride(-1) != 1:
            x2 = x2.contiguous()
        y = ops.w4a16_linear(x2, self.weight, self.scale, self.workspace, self.size_n, self.size_k,
                             out_features=self.out_features, bias=self.bias, silu_mul=True,
                             had_block=self.had_block, had_scale=self.had_scale)
        return y.view(*lead, self.out_features)

    def __repr__(self):
        return f"W4A16GateUpSiLU(in_features={self.in_features}, out_features={self.out_features})"
