"""W4A16 linear layer and the Hadamard-fusing calibration layer
(reference: quantize/quant_linear_layers.py)."""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import layout, ops
from .hadamard_helpers import get_had_fn


def _round_up(v: int, to: int) -> int:
    return v + (-v) % to


class W4A16B16O16Linear(nn.Module):
    """y = x . dequant(weight) (+ bias): int4 weights with group-128 fp16 scales,
    fp16 activations and outputs.

    State (all part of the checkpoint format, quant_linear_layers.py:13-48):
      workspace int32 [(N_pad / 64) * 16]  zeros, scratch counters of the kernel
      weight    int32 [K_pad / 16, 2 N_pad]
      scale     fp16  [K_pad / group, N_pad]
      bias      fp16  [out_features] Parameter or None
    with N padded to a multiple of 256 and K to a multiple of the group size.

    Beyond the reference: `had_block` (default 0) rotates the input online with
    a blockwise Walsh-Hadamard transform inside the kernel call.
    """

    def __init__(self, in_features, out_features, bias=False, group_size=128, device=None, **kwargs):
        super().__init__()
        self.in_features, self.out_features = in_features, out_features
        self.size_n = _round_up(out_features, 256)
        self.size_k = _round_up(in_features, group_size)
        self.pad_out = self.size_n - out_features
        self.pad_in = self.size_k - in_features
        self.max_par = layout.MAX_PARALLEL
        self.had_block = 0
        self.had_scale = 1.0
        n_ws = (self.size_n // layout.MIN_THREAD_N) * layout.MAX_PARALLEL
        self.register_buffer("workspace", torch.zeros(n_ws, dtype=torch.int32, device=device))
        self.register_buffer("weight", torch.empty((self.size_k // 16, self.size_n * 2),
                                                   dtype=torch.int32, device=device))
        self.register_buffer("scale", torch.empty((self.size_k // group_size, self.size_n),
                                                  dtype=torch.float16, device=device))
        if bias:
            self.register_parameter("bias", nn.Parameter(torch.empty(out_features, dtype=torch.float16,
                                                                     device=device)))
        else:
            self.bias = None

    @classmethod
    def from_fp16(cls, originalLayer: nn.Linear):
        """Quantises an nn.Linear in fp16 with the reference's arithmetic
        (quant_linear_layers.py:50-89) and packs it for the kernel: on the GPU when the layer's
        weight lives there (same results bit for bit), on the CPU otherwise as the reference
        does."""
        group_size = 128 if originalLayer.in_features > 128 else -1
        given_scale = None
        if getattr(originalLayer, "apply_gptq", False):
            if originalLayer.bits != 4:
                raise AssertionError("Only support 4-bit quantization")
            group_size = originalLayer.group_size
            given_scale = originalLayer.group_scale.to(torch.float16).cpu()
        if group_size not in (-1, 128):
            raise ValueError("Only groupsize -1 and 128 are supported.")
        W = originalLayer.weight
        dev = W.device
        q = cls(originalLayer.in_features, originalLayer.out_features, device=dev)
        if W.is_cuda and group_size == 128:
            w16 = W.detach().to(torch.float16).contiguous()                # [Dout, Din]
            scale_dev = None if given_scale is None else given_scale.to(dev).contiguous()
            q.weight, q.scale = ops.w4a16_quantize(w16, scale_dev, pad_out=q.pad_out)
            q.size_k, q.size_n = q.weight.shape[0] * 16, q.weight.shape[1] // 2
            q.pad_in = q.size_k - originalLayer.in_features
            if originalLayer.bias is not None:
                q.bias = nn.Parameter(originalLayer.bias.data.clone())
            return q
        w_t = W.detach().cpu().to(torch.float16).t().contiguous()      # [Din, Dout]
        w_ref, packed, scale = layout.quantize_and_pack(w_t, group_size, given_scale, pad_out=q.pad_out)
        q.size_k, q.size_n = w_ref.shape
        q.pad_in = q.size_k - w_t.shape[0]
        q.weight = packed.to(dev)
        q.scale = scale.to(dev)
        if originalLayer.bias is not None:
            q.bias = nn.Parameter(originalLayer.bias.data.clone())
        return q

    def set_online_hadamard(self, block: int, scale: float | None = None):
        """Rotate the input with H_block (blockwise along K) before the product."""
        self.had_block = int(block)
        self.had_scale = float(scale) if scale is not None else (block ** -0.5 if block else 1.0)
        return self

    @torch.no_grad()
    def forward(self, x, residual=None, activation=None):
        """Padding of the input, the product, the cut of the padded output columns and the bias
        (quant_linear_layers.py:92-114) happen inside one kernel call.  Beyond the reference:
        `residual` (same shape as the result) is added in the same call, with the rounding of
        the decoder layer's `residual + layer(x)`; `activation="relu2"` applies the squared ReLU
        of the un-gated MLP (nemotron_h_qblocks.py:588: act_fn(up_proj(x))) to the result."""
        if activation not in (None, "relu2"):
            raise ValueError(f"unsupported activation {activation!r} (None or 'relu2')")
        x2 = x if x.dim() == 2 else x.reshape(-1, x.shape[-1])
        if x2.stride(-1) != 1:
            x2 = x2.contiguous()
        y = ops.linear_prepared(self._prepared(), x2,
                                residual=None if residual is None else residual.reshape(-1, self.out_features),
                                relu2=activation == "relu2")
        return y if x.dim() == 2 else y.view(*x.shape[:-1], self.out_features)

    def _prepared(self):
        """The layer's side of the call, validated once and kept until a buffer is replaced
        (load_state_dict copies in place and keeps it; .to(device) or an assignment does not)."""
        buffers = self._buffers
        weight, scale, workspace = buffers["weight"], buffers["scale"], buffers["workspace"]
        bias = self.bias
        key = (weight.data_ptr(), scale.data_ptr(), workspace.data_ptr(), None if bias is None else bias.data_ptr(),
               self.had_block, self.had_scale, self.size_n, self.size_k, self.out_features)
        cached = self.__dict__.get("_prep")
        if cached is None or cached[0] != key:
            prep = ops.prepare_linear(weight, scale, workspace, self.size_n, self.size_k, out_features=self.out_features,
                                      bias=None if bias is None else bias.data, had_block=self.had_block,
                                      had_scale=self.had_scale)
            cached = self.__dict__["_prep"] = (key, prep)
        return cached[1]

    def __repr__(self):
        return (f"W4A16B16O16Linear(in_features={self.in_features}, out_features={self.out_features}, "
                f"bias={self.bias is not None})")


class HadLinear(nn.Linear):
    """nn.Linear whose weight is (or will be) multiplied by Hadamard matrices on
    the input and/or output side; used while calibrating, before quantisation
    (quant_linear_layers.py:122-181).  Weights must live on the GPU."""

    def __init__(self, originalLayer: nn.Linear, input_transform=True, output_transform=False, fuse_had=False):
        assert originalLayer.weight.is_cuda, "Hadamard transform must be on CUDA"
        has_bias = originalLayer.bias is not None
        super().__init__(originalLayer.in_features, originalLayer.out_features, has_bias,
                         originalLayer.weight.device, originalLayer.weight.dtype)
        self.input_transform = input_transform
        self.output_transform = output_transform
        if input_transform:
            self.input_transform_fn, self.Nin, self.had_scale_in = get_had_fn(originalLayer.in_features)
        if output_transform:
            self.output_transform_fn, self.Nout, self.had_scale_out = get_had_fn(originalLayer.out_features)
        self.weight.data = originalLayer.weight.data
        if has_bias:
            assert not output_transform, "Bias is not supported for output_transform"
            self.bias.data = originalLayer.bias.data
        self.fuse_had = False
        if fuse_had:
            self.fuse_hadamard()

    def _rotated(self, w):
        if self.input_transform:
            w = self.input_transform_fn(w, self.had_scale_in)
        if self.output_transform:
            w = self.output_transform_fn(w.t(), self.had_scale_out).t()
        return w

    def fuse_hadamard(self):
        self.weight.data = self._rotated(self.weight.data.clone()).contiguous()
        self.fuse_had = True

    def forward(self, x):
        w = self.weight.clone()
        if not self.fuse_had:
            w = self._rotated(w)
        return F.linear(x, w, self.bias)

    def __repr__(self):
        return (f"HadLinear(in_features={self.in_features}, out_features={self.out_features}, "
                f"bias={self.bias is not None}, input_transform={self.input_transform}, "
                f"output_transform={self.output_transform}, fuse_had={self.fuse_had})")
