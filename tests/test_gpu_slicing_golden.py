"""uniql_amd/slicing.py against vectors written by the reference's own load-time slicing functions
(modeling/modeling_helpers.py:361-867, run on the CPU by tests/golden/make_slicing_golden.py):
packed weights, permuted scales, biases, index lists and convolution / norm cuts bit for bit."""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "slicing_golden.npz")


@pytest.fixture(scope="module")
def vec():
    return dict(np.load(PATH))


def dev(vec, name, gpu, dtype=None):
    t = torch.from_numpy(vec[name]).to(gpu)
    return t.view(dtype) if dtype is not None else t


def same(t, want):
    got = t.detach().cpu().contiguous()
    if got.dtype == torch.float16:
        got = got.view(torch.int16)
    assert got.numpy().shape == want.shape, (got.shape, want.shape)
    assert np.array_equal(got.numpy(), want)


def layer(vec, name, gpu):
    return dev(vec, f"{name}.w", gpu), dev(vec, f"{name}.s", gpu, torch.float16), dev(vec, f"{name}.ws", gpu)


def test_up_gate_and_down(vec, gpu):
    from uniql_amd import slicing
    w, s, ws = layer(vec, "up_gate", gpu)
    hidden, inter, reduced = (int(v) for v in vec["up_gate.args"])
    w2, s2, ws2 = slicing.slice_w4a16_up_gate_proj(w, s, ws, hidden, inter, reduced, w.shape)
    same(w2, vec["up_gate.w_out"]); same(s2, vec["up_gate.s_out"]); assert ws2.numel() == int(vec["up_gate.ws_len"][0])
    w, s, ws = layer(vec, "down", gpu)
    w2, s2, ws2 = slicing.slice_w4a16_down_proj(w, s, ws, hidden, inter, reduced, w.shape)
    same(w2, vec["down.w_out"]); same(s2, vec["down.s_out"]); assert ws2.numel() == int(vec["down.ws_len"][0])


def test_attention_projections(vec, gpu):
    from uniql_amd import slicing
    w, s, ws = layer(vec, "qk", gpu)
    bias = dev(vec, "qk.bias", gpu, torch.float16)
    hidden, nheads, head_dim, red = (int(v) for v in vec["qk.args"])
    w2, b2, s2, ws2 = slicing.slice_w4a16_qk_proj(w, bias, s, ws, hidden, nheads, head_dim, red, w.shape)
    same(w2, vec["qk.w_out"]); same(s2, vec["qk.s_out"]); same(b2, vec["qk.bias_out"])
    assert ws2.numel() == int(vec["qk.ws_len"][0])
    w3, s3, ws3 = slicing.slice_w4a16_v_proj(w, s, ws, hidden, nheads, head_dim, red, w.shape)
    same(w3, vec["v.w_out"]); same(s3, vec["v.s_out"]); assert ws3.numel() == int(vec["v.ws_len"][0])
    w, s, ws = layer(vec, "o", gpu)
    w4, s4, ws4 = slicing.slice_w4a16_o_proj(w, s, ws, hidden, nheads, head_dim, red, w.shape)
    same(w4, vec["o.w_out"]); same(s4, vec["o.s_out"]); assert ws4.numel() == int(vec["o.ws_len"][0])
    idx = dev(vec, "indices.inp", gpu)
    same(slicing.slice_indices(idx, *(int(v) for v in vec["indices.args"])), vec["indices.out"])


def test_mamba_block(vec, gpu):
    from uniql_amd import slicing
    w, s, ws = layer(vec, "in_proj", gpu)
    hidden, n_groups, num_heads, inter, state, load_inter, load_state = (int(v) for v in vec["in_proj.args"])
    w2, s2, ws2 = slicing.slice_w4a16_in_proj(w, s, ws, hidden, n_groups, num_heads, inter, state, load_inter, load_state,
                                              w.shape)
    same(w2, vec["in_proj.w_out"]); same(s2, vec["in_proj.s_out"]); assert ws2.numel() == int(vec["in_proj.ws_len"][0])
    w, s, ws = layer(vec, "out_proj", gpu)
    w3, s3, ws3 = slicing.slice_w4a16_out_proj(w, s, ws, hidden, n_groups, num_heads, inter, load_inter, w.shape)
    same(w3, vec["out_proj.w_out"]); same(s3, vec["out_proj.s_out"]); assert ws3.numel() == int(vec["out_proj.ws_len"][0])
    cw, cb = slicing.slice_conv1d(dev(vec, "conv1d.w", gpu), dev(vec, "conv1d.b", gpu),
                                  *(int(v) for v in vec["conv1d.args"]))
    same(cw, vec["conv1d.w_out"]); same(cb, vec["conv1d.b_out"])
    same(slicing.slice_norm(dev(vec, "norm.w", gpu), *(int(v) for v in vec["norm.args"])), vec["norm.w_out"])
