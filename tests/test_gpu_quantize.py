"""Producer side on the GPU: quantise + pack (uniql_w4a16_quantize), pack ready codes
(uniql_w4a16_pack) and the unpack -> slice -> repack round trip, against the reference's own
outputs (golden fixtures) and the oracle."""
import numpy as np
import pytest
import torch

from oracle import uniql_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case,pad_out", [("A", 0), ("B", 192), ("C", 0)])
def test_quantize_matches_reference_vectors(gpu, golden, case, pad_out):
    """w4a16_quantize of the reference on seeded matrices: plain, N padded by 192, K padded with
    an all-zero group (the fixtures hold the reference's packed words and permuted scales)."""
    from uniql_amd import ops
    w_kn = torch.from_numpy(golden[f"{case}_w"])                    # [K, N] as the reference takes it
    packed, scale = ops.w4a16_quantize(w_kn.t().contiguous().to(gpu), None, pad_out=pad_out)
    assert np.array_equal(packed.cpu().numpy(), golden[f"{case}_packed"])
    assert np.array_equal(scale.cpu().numpy().view(np.uint16), golden[f"{case}_scale"].view(np.uint16))


def test_quantize_given_scales_matches_reference_vectors(gpu, golden):
    """The GPTQ hand-over: codes re-derived from given scales (quantize_helpers.py:205-218)."""
    from uniql_amd import ops
    w = torch.from_numpy(golden["G_w"]).t().contiguous().to(gpu)
    s_in = torch.from_numpy(golden["G_scale_in"]).to(gpu)
    packed, scale = ops.w4a16_quantize(w, s_in)
    assert np.array_equal(packed.cpu().numpy(), golden["G_packed"])
    assert np.array_equal(scale.cpu().numpy().view(np.uint16), golden["G_scale"].view(np.uint16))


@pytest.mark.parametrize("k,n,pad_out,spread", [(256, 256, 0, 0.05), (384, 320, 192, 1.0), (1000, 256, 0, 0.05),
                                                (4096, 1024, 0, 0.02), (512, 128, 128, 1e-6)])
def test_quantize_matches_oracle_on_random_weights(gpu, k, n, pad_out, spread):
    """Bit for bit against the oracle (itself pinned to the fixtures above), including K that is
    not a multiple of 128, weights small enough for subnormal scales, and exact zeros."""
    from uniql_amd import ops
    g = torch.Generator().manual_seed(k + n)
    w = (torch.randn(n, k, generator=g) * spread).half()
    w[::7, 5:9] = 0
    if k >= 512:
        w[3, 128:256] = 0                                           # an all-zero group
    _, o_packed, o_scale = O.w4a16_quantize(w.t().contiguous(), 128, None, pad_out)
    packed, scale = ops.w4a16_quantize(w.to(gpu), None, pad_out=pad_out)
    assert torch.equal(packed.cpu(), o_packed)
    assert np.array_equal(scale.cpu().numpy().view(np.uint16), o_scale.numpy().view(np.uint16))


def test_quantize_strided_weight(gpu):
    from uniql_amd import ops
    g = torch.Generator().manual_seed(9)
    big = (torch.randn(256, 512, generator=g) * 0.1).half().to(gpu)
    view = big[:, :384]
    a = ops.w4a16_quantize(view)
    b = ops.w4a16_quantize(view.contiguous())
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_pack_matches_reference_vectors(gpu, golden):
    from uniql_amd import ops
    codes = torch.from_numpy(golden["P_codes"]).to(gpu)
    scales = torch.ones((1, codes.shape[1]), dtype=torch.float16, device=gpu)
    packed, _ = ops.w4a16_pack(codes, scales)
    assert np.array_equal(packed.cpu().numpy(), golden["P_packed"])
    for case in ("A", "B", "C"):
        codes = torch.from_numpy(golden[f"{case}_codes"]).to(gpu)
        scales = torch.from_numpy(golden[f"{case}_scale_unperm"]).to(gpu)
        packed, scale = ops.w4a16_pack(codes, scales)
        assert np.array_equal(packed.cpu().numpy(), golden[f"{case}_packed"])
        assert np.array_equal(scale.cpu().numpy().view(np.uint16), golden[f"{case}_scale"].view(np.uint16))


def test_unpack_slice_repack(gpu):
    """The reference's load-time slicing (modeling_helpers.py:235-355) unpacks, cuts columns or
    whole K groups and packs again; the same on the device equals packing the cut tensors."""
    from uniql_amd import ops
    rng = np.random.default_rng(5)
    k, n = 1024, 512
    q = rng.integers(0, 16, size=(k, n)).astype(np.int32)
    s = rng.uniform(0.004, 0.02, size=(k // 128, n)).astype(np.float16)
    packed = torch.from_numpy(O.pack_weights(q)).to(gpu)
    s_perm = torch.from_numpy(O.permute_scales(s, k, n, 128)).to(gpu)
    codes, scales = ops.w4a16_unpack(packed, s_perm, n, k)
    assert np.array_equal(codes.cpu().numpy(), q.astype(np.uint8))
    assert np.array_equal(scales.cpu().numpy().view(np.uint16), s.view(np.uint16))
    # keep 384 of the columns (an up/gate-style cut) ...
    keep_n = np.sort(rng.choice(n, size=384, replace=False))
    idx = torch.from_numpy(keep_n).to(gpu)
    p2, s2 = ops.w4a16_pack(codes[:, idx], scales[:, idx])
    assert np.array_equal(p2.cpu().numpy(), O.pack_weights(q[:, keep_n]))
    assert np.array_equal(s2.cpu().numpy().view(np.uint16),
                          O.permute_scales(s[:, keep_n], k, 384, 128).view(np.uint16))
    # ... and 5 of the 8 K groups (a down-style cut), output columns padded to 256
    groups = [0, 2, 3, 6, 7]
    rows = np.concatenate([np.arange(128 * g, 128 * g + 128) for g in groups])
    ridx = torch.from_numpy(rows).to(gpu)
    gidx = torch.tensor(groups, device=gpu)
    p3, s3 = ops.w4a16_pack(codes[ridx][:, idx], scales[gidx][:, idx], pad_out=128)
    q_cut = np.concatenate([q[rows][:, keep_n], np.zeros((len(rows), 128), np.int32)], axis=1)
    s_cut = np.concatenate([s[groups][:, keep_n], np.zeros((len(groups), 128), np.float16)], axis=1)
    assert np.array_equal(p3.cpu().numpy(), O.pack_weights(q_cut))
    assert np.array_equal(s3.cpu().numpy().view(np.uint16),
                          O.permute_scales(s_cut, len(rows), 512, 128).view(np.uint16))


def test_quantize_errors(gpu):
    from uniql_amd import ops
    with pytest.raises(RuntimeError):
        ops.w4a16_quantize(torch.zeros(256, 128, dtype=torch.float16, device=gpu))      # in_features <= 128
    with pytest.raises(RuntimeError):
        ops.w4a16_quantize(torch.zeros(256, 256, dtype=torch.float32, device=gpu))
    with pytest.raises(RuntimeError):
        ops.w4a16_pack(torch.zeros(100, 128, dtype=torch.uint8, device=gpu),
                       torch.zeros(0, 128, dtype=torch.float16, device=gpu))


def _full_layer(k, n, seed, dev):
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, size=(k, n)).astype(np.int32)
    s = rng.uniform(0.004, 0.02, size=(k // 128, n)).astype(np.float16)
    packed = torch.from_numpy(O.pack_weights(q)).to(dev)
    s_perm = torch.from_numpy(O.permute_scales(s, k, n, 128)).to(dev)
    ws = torch.zeros((n // 64) * 16, dtype=torch.int32, device=dev)
    return q, s, packed, s_perm, ws


def test_slice_up_gate_proj(gpu):
    """modeling_helpers.py:361-408 on the device: cut tensors equal unpack -> cut -> pack of the
    oracle, and the cut layer computes the kept columns of the full layer."""
    from uniql_amd import ops, slicing
    hidden, inter, reduced = 512, 1024, 600          # kept width 600 -> padded to 768
    q, s, packed, s_perm, ws = _full_layer(hidden, inter, 11, gpu)
    w2, s2, ws2 = slicing.slice_w4a16_up_gate_proj(packed, s_perm, ws, hidden, inter, reduced, packed.shape)
    s_cut = s[:, :768].copy()
    s_cut[:, reduced:] = 0
    assert np.array_equal(w2.cpu().numpy(), O.pack_weights(q[:, :768]))
    assert np.array_equal(s2.cpu().numpy().view(np.uint16), O.permute_scales(s_cut, hidden, 768, 128).view(np.uint16))
    assert ws2.numel() == (768 // 64) * 16
    x = torch.randn(3, hidden, generator=torch.Generator().manual_seed(1)).half().to(gpu)
    full = ops.w4a16o16_gemm(x, packed, s_perm, ws, 3, inter, hidden)
    cut = ops.w4a16o16_gemm(x, w2, s2, ws2, 3, 768, hidden)
    assert torch.equal(cut[:, :reduced], full[:, :reduced])
    assert int(cut[:, reduced:].abs().max()) == 0


def test_slice_down_proj(gpu):
    """modeling_helpers.py:411-448 on the device: a prefix of whole K groups; the cut layer on
    the first rows of the activations equals the full layer on activations zeroed past them."""
    from uniql_amd import ops, slicing
    hidden, inter, reduced = 512, 1024, 600          # kept rows 600 -> padded to 640 (5 groups)
    q, s, packed, s_perm, ws = _full_layer(inter, hidden, 12, gpu)
    w2, s2, ws2 = slicing.slice_w4a16_down_proj(packed, s_perm, ws, hidden, inter, reduced, packed.shape)
    assert np.array_equal(w2.cpu().numpy(), O.pack_weights(q[:640]))
    assert np.array_equal(s2.cpu().numpy().view(np.uint16), O.permute_scales(s[:5], 640, hidden, 128).view(np.uint16))
    x = torch.randn(2, inter, generator=torch.Generator().manual_seed(2)).half().to(gpu)
    x[:, reduced:] = 0
    full = ops.w4a16o16_gemm(x, packed, s_perm, ws, 2, hidden, inter)
    cut = ops.w4a16o16_gemm(x[:, :640].contiguous(), w2, s2, ws2, 2, hidden, 640)
    assert torch.allclose(cut.float(), full.float(), atol=2e-3)


def test_slice_qk_and_v_proj(gpu):
    """modeling_helpers.py:451-596 on the device: the cut layers compute exactly the kept
    columns of the full layer (same codes, same scales, same K order), zeros in the padding."""
    from uniql_amd import ops, slicing
    hidden, nheads, head_dim, red = 512, 6, 128, 80           # 768 -> 480 columns, padded to 512
    n_full = nheads * head_dim
    q, s, packed, s_perm, ws = _full_layer(hidden, n_full, 21, gpu)
    x = torch.randn(4, hidden, generator=torch.Generator().manual_seed(3)).half().to(gpu)
    full = ops.w4a16o16_gemm(x, packed, s_perm, ws, 4, n_full, hidden)
    bias = torch.arange(n_full, dtype=torch.float16, device=gpu)
    # q/k: first red/2 columns of each rotary half of every head
    w2, b2, s2, ws2 = slicing.slice_w4a16_qk_proj(packed, bias, s_perm, ws, hidden, nheads, head_dim, red, packed.shape)
    cols = np.concatenate([h * head_dim + np.concatenate([np.arange(red // 2), head_dim // 2 + np.arange(red // 2)])
                           for h in range(nheads)])
    assert tuple(w2.shape) == (hidden // 16, 2 * 512) and ws2.numel() == (512 // 64) * 16
    cut = ops.w4a16o16_gemm(x, w2, s2, ws2, 4, 512, hidden)
    assert torch.equal(cut[:, :len(cols)], full[:, torch.from_numpy(cols).to(gpu)])
    assert int(cut[:, len(cols):].abs().max()) == 0
    assert torch.equal(b2, bias[torch.from_numpy(cols).to(gpu)])
    assert np.array_equal(w2.cpu().numpy(), O.pack_weights(np.concatenate([q[:, cols], np.zeros((hidden, 32), np.int32)], 1)))
    # v: the first `red` columns of every head
    w3, s3, ws3 = slicing.slice_w4a16_v_proj(packed, s_perm, ws, hidden, nheads, head_dim, red, packed.shape)
    vcols = np.concatenate([h * head_dim + np.arange(red) for h in range(nheads)])
    cut = ops.w4a16o16_gemm(x, w3, s3, ws3, 4, 512, hidden)
    assert torch.equal(cut[:, :len(vcols)], full[:, torch.from_numpy(vcols).to(gpu)])


def test_slice_o_proj_requantises(gpu):
    """modeling_helpers.py:600-656 on the device: dequantise, keep every head's first rows,
    quantise again.  Equal to the oracle's quantiser on the oracle's dequantised weights, and
    close to the full layer applied to activations that are zero in the dropped positions."""
    from uniql_amd import ops, slicing
    hidden, nheads, head_dim, red = 512, 6, 128, 80
    k_full = nheads * head_dim
    q, s, packed, s_perm, ws = _full_layer(k_full, hidden, 22, gpu)
    w2, s2, ws2 = slicing.slice_w4a16_o_proj(packed, s_perm, ws, hidden, nheads, head_dim, red, packed.shape)
    rows = np.concatenate([h * head_dim + np.arange(red) for h in range(nheads)])
    w_deq = O.dequant_codes(q, s)                                           # fp16 [k, n]
    _, o_packed, o_scale = O.w4a16_quantize(torch.from_numpy(w_deq[rows]), 128, None, 0)
    assert tuple(w2.shape) == (512 // 16, 2 * hidden)                       # 480 rows -> 512
    assert torch.equal(w2.cpu(), o_packed) and torch.equal(s2.cpu(), o_scale)
    x = torch.randn(2, k_full, generator=torch.Generator().manual_seed(4)).half()
    keep = torch.zeros(k_full, dtype=torch.bool)
    keep[torch.from_numpy(rows)] = True
    x_full = (x * keep).to(gpu)
    x_cut = torch.nn.functional.pad(x[:, torch.from_numpy(rows)], (0, 512 - len(rows))).to(gpu).contiguous()
    full = ops.w4a16o16_gemm(x_full, packed, s_perm, ws, 2, hidden, k_full)
    cut = ops.w4a16o16_gemm(x_cut, w2, s2, ws2, 2, hidden, 512)
    rel = (cut.float() - full.float()).abs().mean() / full.float().abs().mean()
    assert rel < 0.1                                                        # re-quantisation noise only


def test_slice_mamba_in_and_out_proj(gpu):
    """modeling_helpers.py:665-867 on the device, on a small Mamba2-shaped block."""
    from uniql_amd import ops, slicing
    hidden, n_groups, num_heads, inter, state = 256, 2, 8, 512, 64
    load_inter, load_state = 384, 48                      # head_dim 64 -> 48, states 64 -> 48
    proj = 2 * inter + 2 * n_groups * state + num_heads   # 1288 -> padded to 1536
    n_full = proj + (-proj) % 256
    q, s, packed, s_perm, ws = _full_layer(hidden, n_full, 31, gpu)
    w2, s2, ws2 = slicing.slice_w4a16_in_proj(packed, s_perm, ws, hidden, n_groups, num_heads, inter, state,
                                              load_inter, load_state, packed.shape)
    heads = np.concatenate([h * 64 + np.arange(48) for h in range(num_heads)])
    states = np.concatenate([g * state + np.arange(load_state) for g in range(n_groups)])
    cols = np.concatenate([heads, inter + heads, 2 * inter + states, 2 * inter + n_groups * state + states,
                           np.arange(2 * inter + 2 * n_groups * state, proj)])
    red = 2 * load_inter + 2 * n_groups * load_state + num_heads
    assert len(cols) == red
    n_cut = red + (-red) % 256
    assert tuple(w2.shape) == (hidden // 16, 2 * n_cut)
    x = torch.randn(3, hidden, generator=torch.Generator().manual_seed(6)).half().to(gpu)
    full = ops.w4a16o16_gemm(x, packed, s_perm, ws, 3, n_full, hidden)
    cut = ops.w4a16o16_gemm(x, w2, s2, ws2, 3, n_cut, hidden)
    assert torch.equal(cut[:, :red], full[:, torch.from_numpy(cols).to(gpu)])
    assert int(cut[:, red:].abs().max()) == 0
    # out_proj: dequantise, keep head prefixes, quantise again == the oracle's quantiser on the kept rows
    q, s, packed, s_perm, ws = _full_layer(inter, hidden, 32, gpu)
    w3, s3, _ = slicing.slice_w4a16_out_proj(packed, s_perm, ws, hidden, n_groups, num_heads, inter, load_inter,
                                             packed.shape)
    _, o_packed, o_scale = O.w4a16_quantize(torch.from_numpy(O.dequant_codes(q, s)[heads]), 128, None, 0)
    assert torch.equal(w3.cpu(), o_packed) and torch.equal(s3.cpu(), o_scale)
    # the convolution and norm cuts follow the same index lists
    conv_w = torch.arange((inter + 2 * n_groups * state) * 4, dtype=torch.float32, device=gpu).reshape(-1, 1, 4)
    conv_b = torch.arange(inter + 2 * n_groups * state, dtype=torch.float32, device=gpu)
    cw, cb = slicing.slice_conv1d(conv_w, conv_b, n_groups, num_heads, inter, state, load_inter, load_state)
    want = np.concatenate([heads, inter + states, inter + n_groups * state + states])
    assert np.array_equal(cb.cpu().numpy(), want.astype(np.float32)) and cw.shape[0] == len(want)
    nw = slicing.slice_norm(torch.arange(inter, dtype=torch.float32, device=gpu), n_groups, num_heads, inter, load_inter)
    assert np.array_equal(nw.cpu().numpy(), heads.astype(np.float32))


def test_slice_quantized_weights_walks_a_model(gpu):
    """modeling_helpers.py:235-358: the walk over the decoder layers hands every block's tensors to
    the cut that belongs to them, with the block's own sizes, and leaves everything else alone.
    Duck-typed stand-ins for the reference's model and helper objects; the cuts themselves are held
    to the reference's outputs elsewhere."""
    from types import SimpleNamespace as NS
    from uniql_amd import slicing

    hidden, inter, heads, kv_heads, head_dim = 256, 512, 4, 2, 64
    red_inter, red_head = 384, 48
    m_groups, m_heads, m_inter, m_state, m_red_inter, m_red_state = 2, 8, 512, 64, 384, 48

    def packed(k, n, seed):
        _, _, p, sp, ws = _full_layer(k, n, seed, gpu)
        return {"weight": p, "scale": sp, "workspace": ws}

    state, seed = {}, 100
    def add(key, k, n, bias=False):
        nonlocal seed
        seed += 1
        for name, t in packed(k, n, seed).items():
            state[f"{key}.{name}"] = t
        if bias:
            state[f"{key}.bias"] = torch.arange(n, dtype=torch.float16, device=gpu)

    add("L0.mlp.up_proj", hidden, inter)
    add("L0.mlp.gate_proj", hidden, inter)
    add("L0.mlp.down_proj", inter, hidden)
    add("L0.attn.q_proj", hidden, heads * head_dim, bias=True)
    add("L0.attn.k_proj", hidden, 256, bias=True)          # 2 x 64 = 128 columns, padded to 256
    add("L0.attn.v_proj", hidden, 256)
    add("L0.attn.o_proj", heads * head_dim, hidden)
    state["L0.attn.indices"] = torch.arange(head_dim, device=gpu).repeat(heads, 1)
    proj = 2 * m_inter + 2 * m_groups * m_state + m_heads
    add("L1.mixer.in_proj", hidden, proj + (-proj) % 256)
    add("L1.mixer.out_proj", m_inter, hidden)
    conv_ch = m_inter + 2 * m_groups * m_state
    state["L1.mixer.conv1d.weight"] = torch.arange(conv_ch * 4, dtype=torch.float32, device=gpu).reshape(-1, 1, 4)
    state["L1.mixer.conv1d.bias"] = torch.arange(conv_ch, dtype=torch.float32, device=gpu)
    state["L1.mixer.norm.weight"] = torch.arange(m_inter, dtype=torch.float32, device=gpu)
    state["embed.weight"] = torch.ones(4, device=gpu)
    before = {k: v.clone() for k, v in state.items()}

    def shape_of(t):
        return NS(weight=NS(shape=t.shape))

    # what the single cuts return on the untouched tensors (they also give the reduced model's shapes)
    def cut3(fn, key, *args, **kw):
        return fn(before[f"{key}.weight"], before[f"{key}.scale"], before[f"{key}.workspace"], *args, **kw)
    want = {}
    for proj_name in ("up_proj", "gate_proj"):
        want[f"L0.mlp.{proj_name}"] = cut3(slicing.slice_w4a16_up_gate_proj, f"L0.mlp.{proj_name}", hidden, inter, red_inter,
                                            before[f"L0.mlp.{proj_name}.weight"].shape)
    want["L0.mlp.down_proj"] = cut3(slicing.slice_w4a16_down_proj, "L0.mlp.down_proj", hidden, inter, red_inter,
                                    before["L0.mlp.down_proj.weight"].shape)
    qk = {}
    for proj_name, nh in (("q_proj", heads), ("k_proj", kv_heads)):
        key = f"L0.attn.{proj_name}"
        qk[key] = slicing.slice_w4a16_qk_proj(before[f"{key}.weight"], before[f"{key}.bias"], before[f"{key}.scale"],
                                              before[f"{key}.workspace"], hidden, nh, head_dim, red_head,
                                              before[f"{key}.weight"].shape)
    want["L0.attn.v_proj"] = cut3(slicing.slice_w4a16_v_proj, "L0.attn.v_proj", hidden, kv_heads, head_dim, red_head,
                                  before["L0.attn.v_proj.weight"].shape)
    want["L0.attn.o_proj"] = cut3(slicing.slice_w4a16_o_proj, "L0.attn.o_proj", hidden, heads, head_dim, red_head,
                                  before["L0.attn.o_proj.weight"].shape)
    want["L1.mixer.in_proj"] = cut3(slicing.slice_w4a16_in_proj, "L1.mixer.in_proj", hidden_size=hidden, n_groups=m_groups,
                                    num_heads=m_heads, intermediate_size=m_inter, ssm_state_size=m_state,
                                    load_intermediate_size=m_red_inter, load_ssm_state_size=m_red_state,
                                    load_shape=before["L1.mixer.in_proj.weight"].shape)
    want["L1.mixer.out_proj"] = cut3(slicing.slice_w4a16_out_proj, "L1.mixer.out_proj", hidden_size=hidden, n_groups=m_groups,
                                     num_heads=m_heads, intermediate_size=m_inter, load_intermediate_size=m_red_inter,
                                     load_shape=before["L1.mixer.out_proj.weight"].shape)

    class FakeMlp:
        intermediate_size = red_inter
        up_proj = shape_of(before["L0.mlp.up_proj.weight"])
        gate_proj = shape_of(before["L0.mlp.gate_proj.weight"])
        down_proj = shape_of(before["L0.mlp.down_proj.weight"])

    class FakeAttn:
        head_dim = red_head
        q_proj = shape_of(before["L0.attn.q_proj.weight"])
        k_proj = shape_of(before["L0.attn.k_proj.weight"])
        v_proj = shape_of(before["L0.attn.v_proj.weight"])
        o_proj = shape_of(before["L0.attn.o_proj.weight"])

    class FakeMamba:
        n_groups, num_heads, intermediate_size, ssm_state_size = m_groups, m_heads, m_red_inter, m_red_state
        in_proj = shape_of(before["L1.mixer.in_proj.weight"])
        out_proj = shape_of(before["L1.mixer.out_proj.weight"])

    class Other:
        pass

    layers = [NS(named_children=lambda: [("mlp", FakeMlp()), ("self_attn", FakeAttn()), ("norm", Other())]),
              NS(named_children=lambda: [("mixer", FakeMamba())])]
    model = NS(config=NS(hidden_size=hidden, intermediate_size=inter, num_attention_heads=heads,
                         num_key_value_heads=kv_heads, head_dim=head_dim), layers=layers)
    helper = NS(get_layers=lambda m: m.layers, mlp_w4a16_uniql_class_name="FakeMlp",
                attn_w4a16_uniql_class_name="FakeAttn", mamba_w4a16_uniql_class_name="FakeMamba",
                get_mlp_key=lambda i: f"L{i}.mlp", get_attn_key=lambda i: f"L{i}.attn", get_mamba_key=lambda i: f"L{i}.mixer",
                get_mamba_full_intermediate_size=m_inter, get_mamba_full_ssm_state_size=m_state)

    out = slicing.slice_quantized_weights(model, helper, state)
    assert out is state
    for key, (w, s, ws) in want.items():
        assert torch.equal(out[f"{key}.weight"], w) and torch.equal(out[f"{key}.scale"], s), key
        assert torch.equal(out[f"{key}.workspace"], ws), key
    for key, (w, b, s, ws) in qk.items():
        assert torch.equal(out[f"{key}.weight"], w) and torch.equal(out[f"{key}.bias"], b), key
        assert torch.equal(out[f"{key}.scale"], s) and torch.equal(out[f"{key}.workspace"], ws), key
    assert torch.equal(out["L0.attn.indices"], slicing.slice_indices(before["L0.attn.indices"], head_dim, red_head))
    cw, cb = slicing.slice_conv1d(before["L1.mixer.conv1d.weight"], before["L1.mixer.conv1d.bias"], m_groups, m_heads,
                                  m_inter, m_state, m_red_inter, m_red_state)
    assert torch.equal(out["L1.mixer.conv1d.weight"], cw) and torch.equal(out["L1.mixer.conv1d.bias"], cb)
    assert torch.equal(out["L1.mixer.norm.weight"],
                       slicing.slice_norm(before["L1.mixer.norm.weight"], m_groups, m_heads, m_inter, m_red_inter))
    assert torch.equal(out["embed.weight"], before["embed.weight"]) and set(out) == set(before)
    # the cut MLP still computes the kept columns
    assert out["L0.mlp.up_proj.weight"].shape[1] == 2 * 512 and out["L0.mlp.down_proj.weight"].shape[0] == red_inter // 16
