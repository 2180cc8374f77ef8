"""A pruned-Llama style decoder layer assembled twice from the same quantised layers: the
reference's call sequence (one module call per projection, tensor operations in between) and
the fused sequence (q/k/v in one launch, rotary kernel, gate/up with the SiLU epilogue, the residual
additions inside o_proj's and down_proj's calls).  The two
must agree, and the unfused one must agree with the oracle evaluated layer by layer."""
import numpy as np
import pytest
import torch

from oracle import uniql_oracle as O
from tests.helpers import check_layer_output
from tests.test_oracle_fused_rope import rope_tables

pytestmark = pytest.mark.gpu

HIDDEN, HEADS, KV_HEADS, HEAD_DIM, PRUNED_DIM, INTER = 512, 8, 2, 64, 48, 1216   # 1216 = 9.5 x 128: N is padded


def make_layers(dev, bias):
    from uniql_amd.quantize.quant_linear_layers import W4A16B16O16Linear
    gen = torch.Generator().manual_seed(11)

    def layer(i, o, b=False):
        lin = torch.nn.Linear(i, o, bias=b).half()
        lin.weight.data = (torch.randn(o, i, generator=gen) * 0.04).half()
        if b:
            lin.bias.data = (torch.randn(o, generator=gen) * 0.1).half()
        return W4A16B16O16Linear.from_fp16(lin.to(dev))

    return dict(q=layer(HIDDEN, HEADS * PRUNED_DIM, bias), k=layer(HIDDEN, KV_HEADS * PRUNED_DIM, bias),
                v=layer(HIDDEN, KV_HEADS * PRUNED_DIM, bias), o=layer(HEADS * PRUNED_DIM, HIDDEN),
                gate=layer(HIDDEN, INTER), up=layer(HIDDEN, INTER), down=layer(INTER, HIDDEN))


def attention(q, k, v):
    """[b, h, s, d] fp16; grouped-query causal attention with torch's operator"""
    rep = q.shape[1] // k.shape[1]
    k, v = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
    return torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)


def layer_unfused(L, x, cos, sin, idx):
    """the reference's sequence (modeling/llama/llama_uniql_qblocks.py:110-150, llama_qblocks.py:48-51)"""
    b, s, _ = x.shape
    q = L["q"](x).view(b, s, HEADS, PRUNED_DIM).transpose(1, 2)
    k = L["k"](x).view(b, s, KV_HEADS, PRUNED_DIM).transpose(1, 2)
    v = L["v"](x).view(b, s, KV_HEADS, PRUNED_DIM).transpose(1, 2)
    qo, ko = O.rope_indices(q.cpu().numpy(), k.cpu().numpy(), cos.cpu().numpy(), sin.cpu().numpy(),
                            idx.cpu().numpy())
    q, k = torch.from_numpy(qo).to(x.device), torch.from_numpy(ko).to(x.device)
    a = attention(q, k, v).transpose(1, 2).reshape(b, s, HEADS * PRUNED_DIM)
    h = x + L["o"](a)
    mlp = L["down"](torch.nn.functional.silu(L["gate"](h)) * L["up"](h))
    return h + mlp


def layer_fused(F, x, cos, sin, idx):
    from uniql_amd.rope import apply_rotary_pos_emb_indices
    b, s, _ = x.shape
    q, k, v = F["qkv"](x)
    q = q.reshape(b, s, HEADS, PRUNED_DIM).transpose(1, 2)
    k = k.reshape(b, s, KV_HEADS, PRUNED_DIM).transpose(1, 2)
    v = v.reshape(b, s, KV_HEADS, PRUNED_DIM).transpose(1, 2)
    q, k = apply_rotary_pos_emb_indices(q, k, cos, sin, idx)
    a = attention(q, k, v).transpose(1, 2).reshape(b, s, HEADS * PRUNED_DIM)
    h = F["o"](a, residual=x)
    return F["down"](F["gate_up"](h), residual=h)


@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("b,s", [(1, 1), (2, 7), (1, 96)])
def test_fused_layer_equals_the_reference_sequence(gpu, b, s, bias):
    from uniql_amd.quantize.fused_layers import W4A16FusedLinear, W4A16GateUpSiLU
    L = make_layers(gpu, bias)
    F = dict(qkv=W4A16FusedLinear.from_linears([L["q"], L["k"], L["v"]]), o=L["o"],
             gate_up=W4A16GateUpSiLU.from_linears(L["gate"], L["up"]), down=L["down"])
    x = (torch.randn(b, s, HIDDEN, generator=torch.Generator().manual_seed(s)) * 0.5).half().to(gpu)
    cos, sin, _ = rope_tables(s, HEAD_DIM)
    cos, sin = torch.from_numpy(cos).to(gpu), torch.from_numpy(sin).to(gpu)
    first = np.sort(np.random.default_rng(0).choice(HEAD_DIM // 2, PRUNED_DIM // 2, replace=False))
    idx = torch.from_numpy(np.tile(np.concatenate((first, first + HEAD_DIM // 2)), (KV_HEADS, 1))).to(torch.uint8).to(gpu)
    want = layer_unfused(L, x, cos, sin, idx).float().cpu().numpy()
    got = layer_fused(F, x, cos, sin, idx).float().cpu().numpy()
    assert got.shape == want.shape == (b, s, HIDDEN)
    # the same kernels and roundings up to the last bit of a few intermediate sums (other grids),
    # carried through attention and the MLP
    assert np.abs(got - want).max() <= 1e-2
    assert np.abs(got - want).sum() / np.abs(want).sum() <= 1e-3


def test_unfused_projections_equal_the_oracle(gpu):
    """every quantised layer of the block against the oracle's module forward"""
    L = make_layers(gpu, True)
    x = (torch.randn(5, HIDDEN, generator=torch.Generator().manual_seed(1)) * 0.5).half()
    for name in ("q", "k", "gate"):
        layer = L[name]
        y = layer(x.to(gpu)).cpu().numpy()
        ref = O.linear_forward(x.numpy(), layer.weight.cpu().numpy(), layer.scale.cpu().numpy(),
                               in_features=layer.in_features, out_features=layer.out_features,
                               bias=None if layer.bias is None else layer.bias.data.cpu().numpy().astype(np.float64),
                               exact=True)
        check_layer_output(y, ref, max_abs=1.5e-2 if layer.bias is not None else 1e-2)
