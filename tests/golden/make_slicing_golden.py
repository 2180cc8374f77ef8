"""Writes tests/golden/slicing_golden.npz.

Runs in the build container only (needs the reference checkout; the GPU box has none).  It
imports the reference's modeling/modeling_helpers.py (torch, einops, transformers and safetensors
on the CPU; no compiled extension), calls each of its load-time slicing functions
(modeling_helpers.py:361-867) on small seeded layers quantised by the reference's own
w4a16_quantize, and stores inputs and outputs as plain arrays.  No reference text or object is
stored: only numbers.

The vectors pin what uniql_amd/slicing.py must reproduce bit for bit: which columns / rows each cut
keeps, how the kept tensors are padded, and the re-quantisation of the o_proj / out_proj cuts.

    python tests/golden/make_slicing_golden.py [/root/reference]
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    sys.path.insert(0, root)
    import modeling.modeling_helpers as MH
    from quantize.quantize_helpers import w4a16_quantize

    gen = torch.Generator().manual_seed(4321)
    out = {}

    def layer(k, n):
        """a quantised [k -> n] layer as the reference writes it: packed weight, permuted scale, workspace"""
        w = (torch.randn(k, n, generator=gen) * 0.05).to(torch.float16)
        pad_out = (-n) % 256
        _, packed, scale = w4a16_quantize(w, 4, 128, None, pad_out)
        n_pad = n + pad_out
        ws = torch.zeros((n_pad // 64) * 16, dtype=torch.int32)
        return packed.contiguous(), scale.contiguous(), ws

    def put(name, tensors):
        for key, t in tensors.items():
            out[f"{name}.{key}"] = t.detach().cpu().numpy() if torch.is_tensor(t) else np.asarray(t)

    # ---- Llama-style MLP and attention cuts
    hidden, inter, reduced = 256, 768, 600
    w, s, ws = layer(hidden, inter)
    w2, s2, ws2 = MH.slice_w4a16_up_gate_proj(w, s, ws, hidden, inter, reduced, w.shape)
    put("up_gate", dict(w=w, s=s.view(torch.int16), ws=ws, args=[hidden, inter, reduced], w_out=w2, s_out=s2.view(torch.int16),
                        ws_len=[ws2.numel()]))
    w, s, ws = layer(inter, hidden)
    w2, s2, ws2 = MH.slice_w4a16_down_proj(w, s, ws, hidden, inter, reduced, w.shape)
    put("down", dict(w=w, s=s.view(torch.int16), ws=ws, args=[hidden, inter, reduced], w_out=w2, s_out=s2.view(torch.int16),
                     ws_len=[ws2.numel()]))

    nheads, head_dim, red = 6, 64, 40
    w, s, ws = layer(hidden, nheads * head_dim)
    bias = (torch.randn(nheads * head_dim, generator=gen)).to(torch.float16)
    w2, b2, s2, ws2 = MH.slice_w4a16_qk_proj(w, bias, s, ws, hidden, nheads, head_dim, red, w.shape)
    put("qk", dict(w=w, s=s.view(torch.int16), ws=ws, bias=bias.view(torch.int16), args=[hidden, nheads, head_dim, red], w_out=w2,
                   s_out=s2.view(torch.int16), bias_out=b2.view(torch.int16), ws_len=[ws2.numel()]))
    w2, s2, ws2 = MH.slice_w4a16_v_proj(w, s, ws, hidden, nheads, head_dim, red, w.shape)
    put("v", dict(w_out=w2, s_out=s2.view(torch.int16), ws_len=[ws2.numel()]))       # same input layer as "qk"
    w, s, ws = layer(nheads * head_dim, hidden)
    w2, s2, ws2 = MH.slice_w4a16_o_proj(w, s, ws, hidden, nheads, head_dim, red, w.shape)
    put("o", dict(w=w, s=s.view(torch.int16), ws=ws, args=[hidden, nheads, head_dim, red], w_out=w2, s_out=s2.view(torch.int16),
                  ws_len=[ws2.numel()]))
    idx = torch.arange(head_dim, dtype=torch.uint8).repeat(3, 1)
    put("indices", dict(inp=idx, out=MH.slice_indices(idx, head_dim, red), args=[head_dim, red]))

    # ---- Mamba2-style cuts
    n_groups, num_heads, m_inter, state, load_inter, load_state = 2, 8, 512, 64, 384, 48
    proj = 2 * m_inter + 2 * n_groups * state + num_heads
    w, s, ws = layer(hidden, proj)
    w2, s2, ws2 = MH.slice_w4a16_in_proj(w, s, ws, hidden, n_groups, num_heads, m_inter, state, load_inter, load_state, w.shape)
    put("in_proj", dict(w=w, s=s.view(torch.int16), ws=ws, args=[hidden, n_groups, num_heads, m_inter, state, load_inter, load_state],
                        w_out=w2, s_out=s2.view(torch.int16), ws_len=[ws2.numel()]))
    w, s, ws = layer(m_inter, hidden)
    w2, s2, ws2 = MH.slice_w4a16_out_proj(w, s, ws, hidden, n_groups, num_heads, m_inter, load_inter, w.shape)
    put("out_proj", dict(w=w, s=s.view(torch.int16), ws=ws, args=[hidden, n_groups, num_heads, m_inter, load_inter], w_out=w2,
                         s_out=s2.view(torch.int16), ws_len=[ws2.numel()]))
    conv_dim = m_inter + 2 * n_groups * state
    conv_w = torch.randn(conv_dim, 1, 4, generator=gen)
    conv_b = torch.randn(conv_dim, generator=gen)
    cw, cb = MH.slice_conv1d(conv_w, conv_b, n_groups, num_heads, m_inter, state, load_inter, load_state)
    put("conv1d", dict(w=conv_w, b=conv_b, w_out=cw, b_out=cb, args=[n_groups, num_heads, m_inter, state, load_inter, load_state]))
    norm_w = torch.randn(m_inter, generator=gen)
    put("norm", dict(w=norm_w, w_out=MH.slice_norm(norm_w, n_groups, num_heads, m_inter, load_inter),
                     args=[n_groups, num_heads, m_inter, load_inter]))

    path = os.path.join(HERE, "slicing_golden.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
