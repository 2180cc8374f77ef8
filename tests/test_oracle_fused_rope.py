"""Pins of the oracle's restatements of the layer glue (bias, SiLU-gated MLP front) and of
the rotary embedding with gathered frequencies, plus the host-side fusing of packed layers."""
import numpy as np
import torch

from oracle import uniql_oracle as O
from uniql_amd import layout


def all_finite_fp16():
    bits = np.arange(0x10000, dtype=np.uint32).astype(np.uint16)
    return bits[(bits & 0x7C00) != 0x7C00].view(np.float16)


# ------------------------------------------------------------------ SiLU, gate * up, bias
def test_silu_fp16_is_torchs_operator_on_every_finite_input():
    """the reference applies torch's nn.SiLU to an fp16 tensor: compare on all 63488 inputs"""
    x = all_finite_fp16()
    want = torch.nn.functional.silu(torch.from_numpy(x.copy())).numpy()
    got = O.silu_fp16(x)
    differ = got.view(np.uint16) != want.view(np.uint16)
    # numpy's and torch's fp32 exp differ in the last bit for a handful of inputs
    assert differ.sum() <= 8
    assert np.abs(got[differ].astype(np.float64) - want[differ].astype(np.float64)).max(initial=0) <= 2.0 ** -10 * \
        np.abs(want[differ].astype(np.float64)).max(initial=1)
    # closed forms: silu(0) = 0, silu(x) -> x for large x, silu(-x) = silu(x) - x
    assert O.silu_fp16(np.array([0.0], np.float16))[0] == 0
    assert O.silu_fp16(np.array([30.0], np.float16))[0] == np.float16(30.0)
    xs = np.linspace(-6, 6, 97).astype(np.float16)
    exact = xs.astype(np.float64) / (1 + np.exp(-xs.astype(np.float64)))
    assert np.abs(O.silu_fp16(xs).astype(np.float64) - exact).max() < 2e-3


def test_relu2_fp16_is_transformers_activation_on_every_finite_input():
    """ACT2FN["relu2"] (relu, then torch.square) on an fp16 tensor, all 63488 finite inputs,
    plus the closed forms: negatives and zeros give +0, 3 -> 9, overflow goes to +inf."""
    from transformers.activations import ACT2FN
    x = all_finite_fp16()
    want = ACT2FN["relu2"](torch.from_numpy(x.copy())).numpy()
    got = O.relu2_fp16(x)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    probe = O.relu2_fp16(np.array([-2.0, -0.0, 0.0, 3.0, 0.5, 300.0], np.float16))
    assert probe.tolist() == [0.0, 0.0, 0.0, 9.0, 0.25, float("inf")]
    assert not np.signbit(probe[:3]).any()


def test_mlp_gate_up_is_torchs_expression():
    g = torch.randn(64, 96, generator=torch.Generator().manual_seed(0)).half() * 3
    u = torch.randn(64, 96, generator=torch.Generator().manual_seed(1)).half() * 3
    want = (torch.nn.functional.silu(g) * u).numpy()
    got = O.mlp_gate_up(g.numpy(), u.numpy())
    assert (got.view(np.uint16) != want.view(np.uint16)).sum() <= 2


def test_linear_forward_fp16_rounds_the_product_then_the_bias_sum():
    rng = np.random.default_rng(3)
    k, n = 256, 256
    q = rng.integers(0, 16, size=(k, n)).astype(np.int32)
    s = rng.uniform(0.004, 0.02, size=(k // 128, n)).astype(np.float16)
    x = rng.standard_normal((5, 200)).astype(np.float16)
    bias = rng.standard_normal(192).astype(np.float16)
    packed, s_perm = O.pack_weights(q), O.permute_scales(s, k, n, 128)
    y = O.linear_forward_fp16(x, packed, s_perm, in_features=200, out_features=192, bias=bias)
    # independent route: torch fp16 tensors, as the module's `y + self.bias`
    prod = O.linear_forward(x, packed, s_perm, in_features=200, out_features=192, exact=True)
    want = (torch.from_numpy(prod.astype(np.float16)) + torch.from_numpy(bias)).numpy()
    assert np.array_equal(y.view(np.uint16), want.view(np.uint16))
    # the padded K rows and the dropped columns do not leak into the result
    w = O.dequant_codes(q, s)
    brute = x.astype(np.float64) @ w[:200, :192].astype(np.float64)
    assert np.abs(prod - brute).max() < 1e-9


# ------------------------------------------------------------------ fusing packed layers
def test_concat_and_interleave_of_packed_layers():
    rng = np.random.default_rng(7)
    k = 256
    qs = [rng.integers(0, 16, size=(k, n)).astype(np.int32) for n in (128, 256, 64)]
    ss = [rng.uniform(0.004, 0.02, size=(k // 128, q.shape[1])).astype(np.float16) for q in qs]
    packed = [torch.from_numpy(O.pack_weights(q)) for q in qs]
    perm = [torch.from_numpy(O.permute_scales(s, k, s.shape[1], 128)) for s in ss]
    w, s = layout.concat_columns(packed, perm)
    n_total = sum(q.shape[1] for q in qs)
    assert np.array_equal(O.unpack_weights(w.numpy(), k, n_total), np.concatenate(qs, axis=1))
    assert np.array_equal(O.unpermute_scales(s.numpy(), k, n_total, 128), np.concatenate(ss, axis=1))
    # gate / up interleaved in blocks of 64 columns
    w, s = layout.interleave_gate_up(packed[1], perm[1], packed[1].flip(0), perm[1].flip(0))
    codes = O.unpack_weights(w.numpy(), k, 512).reshape(k, 4, 2, 64)
    gate, up = qs[1], O.unpack_weights(packed[1].flip(0).numpy(), k, 256)
    assert np.array_equal(codes[:, :, 0].reshape(k, 256), gate)
    assert np.array_equal(codes[:, :, 1].reshape(k, 256), up)
    sc = O.unpermute_scales(s.numpy(), k, 512, 128).reshape(k // 128, 4, 2, 64)
    assert np.array_equal(sc[:, :, 0].reshape(-1, 256), ss[1])
    assert np.array_equal(sc[:, :, 1].reshape(-1, 256), ss[1][::-1])


# ------------------------------------------------------------------ rotary embedding
def rope_tables(seq, dim, batch=1, seed=0):
    """cos / sin as the model builds them: angles t * theta_i, the half-table repeated twice"""
    inv = 1.0 / (10000.0 ** (np.arange(0, dim, 2, dtype=np.float64) / dim))
    pos = np.arange(seq, dtype=np.float64)[None, :, None] + 3.0 * np.arange(batch)[:, None, None]
    ang = pos * inv[None, None, :]
    ang = np.concatenate((ang, ang), axis=-1)
    return np.cos(ang).astype(np.float16), np.sin(ang).astype(np.float16), ang


def test_rope_identity_indices_is_the_complex_rotation():
    rng = np.random.default_rng(1)
    b, hq, hk, s, d = 2, 4, 2, 5, 16
    q = rng.standard_normal((b, hq, s, d)).astype(np.float16)
    k = rng.standard_normal((b, hk, s, d)).astype(np.float16)
    cos, sin, ang = rope_tables(s, d, batch=b)
    idx = np.tile(np.arange(d), (hk, 1))
    qo, ko = O.rope_indices(q, k, cos, sin, idx)
    for x, out in ((q, qo), (k, ko)):
        z = x[..., : d // 2].astype(np.float64) + 1j * x[..., d // 2:].astype(np.float64)
        rot = z * np.exp(1j * ang[:, None, :, : d // 2])
        want = np.concatenate((rot.real, rot.imag), axis=-1)
        # three fp16 roundings of O(1) values and fp16 tables
        assert np.abs(out.astype(np.float64) - want).max() < 6e-3
    # rotations preserve the norm of every (j, j + d/2) pair
    n_in = q[..., : d // 2].astype(np.float64) ** 2 + q[..., d // 2:].astype(np.float64) ** 2
    n_out = qo[..., : d // 2].astype(np.float64) ** 2 + qo[..., d // 2:].astype(np.float64) ** 2
    assert np.abs(n_in - n_out).max() < 2e-2


def test_rope_gather_equals_rotation_with_the_selected_frequencies():
    rng = np.random.default_rng(2)
    b, hq, hk, s, d, D = 1, 6, 3, 7, 8, 32
    q = rng.standard_normal((b, hq, s, d)).astype(np.float16)
    k = rng.standard_normal((b, hk, s, d)).astype(np.float16)
    cos, sin, ang = rope_tables(s, D)
    # every key/value head keeps its own d/2 of the D/2 frequencies (the pruning keeps pairs)
    first = np.stack([np.sort(rng.choice(D // 2, d // 2, replace=False)) for _ in range(hk)])
    idx = np.concatenate((first, first + D // 2), axis=1)
    qo, ko = O.rope_indices(q, k, cos, sin, idx.astype(np.uint8))
    for x, out, rows in ((q, qo, np.arange(hq) // 2), (k, ko, np.arange(hk))):
        for h in range(x.shape[1]):
            a = ang[0][:, first[rows[h]]]                     # [s, d/2] selected angles
            z = x[0, h, :, : d // 2].astype(np.float64) + 1j * x[0, h, :, d // 2:].astype(np.float64)
            rot = z * np.exp(1j * a)
            want = np.concatenate((rot.real, rot.imag), axis=-1)
            assert np.abs(out[0, h].astype(np.float64) - want).max() < 6e-3
    # the second half of the index list is honoured on its own (not assumed equal to the first)
    idx2 = idx.copy()
    idx2[:, d // 2:] = idx[:, : d // 2][:, ::-1] + D // 2
    qo2, _ = O.rope_indices(q, k, cos, sin, idx2)
    assert np.array_equal(qo2[..., : d // 2], qo[..., : d // 2]) and not np.array_equal(qo2[..., d // 2:], qo[..., d // 2:])


def test_rope_roundings_are_those_of_torchs_fp16_tensors():
    """the order of the three roundings against torch evaluating the reference's expression"""
    g = torch.Generator().manual_seed(5)
    b, hq, hk, s, d, D = 2, 4, 2, 9, 12, 20
    q, k = torch.randn(b, hq, s, d, generator=g).half(), torch.randn(b, hk, s, d, generator=g).half()
    cos, sin, _ = rope_tables(s, D, batch=b)
    first = np.stack([np.sort(np.random.default_rng(h).choice(D // 2, d // 2, replace=False)) for h in range(hk)])
    idx = np.concatenate((first, first + D // 2), axis=1)
    ct, st, it = torch.from_numpy(cos), torch.from_numpy(sin), torch.from_numpy(idx)

    def gathered(t, heads, rep):
        rows = it.repeat_interleave(rep, dim=0)                                  # [heads, d]
        e = t.unsqueeze(1).expand(b, heads, s, D)
        return torch.gather(e, 3, rows.view(1, heads, 1, d).expand(b, heads, s, d))

    def rotate_half(x):
        return torch.cat((-x[..., d // 2:], x[..., : d // 2]), dim=-1)

    want_q = q * gathered(ct, hq, 2) + rotate_half(q) * gathered(st, hq, 2)
    want_k = k * gathered(ct, hk, 1) + rotate_half(k) * gathered(st, hk, 1)
    got_q, got_k = O.rope_indices(q.numpy(), k.numpy(), cos, sin, idx)
    assert np.array_equal(got_q.view(np.uint16), want_q.numpy().view(np.uint16))
    assert np.array_equal(got_k.view(np.uint16), want_k.numpy().view(np.uint16))
