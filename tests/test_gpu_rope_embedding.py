"""GPU parity of the rotary embedding with gathered frequencies and of the embedding-table
quantiser (C ABI path), bit-exact against the oracle."""
import numpy as np
import pytest
import torch

from oracle import uniql_oracle as O
from tests.test_oracle_fused_rope import rope_tables

pytestmark = pytest.mark.gpu


def pruned_indices(hk, d, D, seed):
    rng = np.random.default_rng(seed)
    first = np.stack([np.sort(rng.choice(D // 2, d // 2, replace=False)) for _ in range(hk)])
    return np.concatenate((first, first + D // 2), axis=1)


@pytest.mark.parametrize("b,hq,hk,s,d,D", [(1, 32, 8, 1, 128, 128), (2, 32, 8, 17, 108, 128), (1, 4, 4, 33, 64, 64),
                                           (3, 6, 2, 5, 14, 32), (1, 32, 8, 1024, 108, 128), (2, 28, 4, 9, 6, 128),
                                           # 64 rows and more take the kernel that builds the gathered table in LDS
                                           (1, 32, 8, 100, 128, 128), (2, 32, 32, 40, 64, 128), (4, 6, 2, 20, 14, 32),
                                           (1, 16, 2, 64, 96, 256)])
@pytest.mark.parametrize("index_dtype", [torch.uint8, torch.int64, torch.int32])
def test_rope_indices_bit_exact(gpu, b, hq, hk, s, d, D, index_dtype):
    from uniql_amd import ops
    rng = np.random.default_rng(b + s + d)
    q = rng.standard_normal((b, s, hq, d)).astype(np.float16)      # token-major storage
    k = rng.standard_normal((b, s, hk, d)).astype(np.float16)
    cos, sin, _ = rope_tables(s, D, batch=b if b == 2 else 1)
    idx = pruned_indices(hk, d, D, seed=d) if d < D else np.tile(np.arange(D), (hk, 1))
    want_q, want_k = O.rope_indices(q.transpose(0, 2, 1, 3), k.transpose(0, 2, 1, 3), cos, sin, idx)
    qt, kt = torch.from_numpy(q).to(gpu), torch.from_numpy(k).to(gpu)
    ops.rope_indices_(qt, kt, torch.from_numpy(cos).to(gpu), torch.from_numpy(sin).to(gpu),
                      torch.from_numpy(idx).to(index_dtype).to(gpu))
    assert np.array_equal(qt.cpu().numpy().view(np.uint16), want_q.transpose(0, 2, 1, 3).view(np.uint16))
    assert np.array_equal(kt.cpu().numpy().view(np.uint16), want_k.transpose(0, 2, 1, 3).view(np.uint16))


def test_rope_reference_call_shape(gpu):
    """the reference's function signature: [b, heads, s, d] views in, same views out, storage
    updated in place when it is the projections' token-major output"""
    from uniql_amd.rope import apply_rotary_pos_emb_indices, apply_rotary_pos_emb_indices_triton
    assert apply_rotary_pos_emb_indices_triton is apply_rotary_pos_emb_indices
    b, s, hq, hk, d, D = 2, 11, 8, 2, 20, 32
    g = torch.Generator().manual_seed(0)
    q_store = torch.randn(b, s, hq * d, generator=g).half().to(gpu)   # what q_proj returns
    k_store = torch.randn(b, s, hk * d, generator=g).half().to(gpu)
    q = q_store.view(b, s, hq, d).transpose(1, 2)
    k = k_store.view(b, s, hk, d).transpose(1, 2)
    cos, sin, _ = rope_tables(s, D)
    idx = pruned_indices(hk, d, D, seed=1)
    want_q, want_k = O.rope_indices(q.cpu().numpy(), k.cpu().numpy(), cos, sin, idx)
    qo, ko = apply_rotary_pos_emb_indices(q, k, torch.from_numpy(cos).to(gpu), torch.from_numpy(sin).to(gpu),
                                          torch.from_numpy(idx).to(torch.uint8).to(gpu))
    assert qo.shape == q.shape and ko.shape == k.shape
    assert np.array_equal(qo.cpu().numpy().view(np.uint16), want_q.view(np.uint16))
    assert np.array_equal(ko.cpu().numpy().view(np.uint16), want_k.view(np.uint16))
    assert qo.data_ptr() == q_store.data_ptr()      # in place, like the kernel it replaces
    # a [b, heads, s, d]-contiguous input is copied, the caller's tensor stays as it was
    q2 = torch.randn(b, hq, s, d, generator=g).half().to(gpu)
    k2 = torch.randn(b, hk, s, d, generator=g).half().to(gpu)
    keep = q2.clone()
    qo2, _ = apply_rotary_pos_emb_indices(q2, k2, torch.from_numpy(cos).to(gpu), torch.from_numpy(sin).to(gpu),
                                          torch.from_numpy(idx).to(gpu))
    want_q2, _ = O.rope_indices(q2.cpu().numpy(), k2.cpu().numpy(), cos, sin, idx)
    assert torch.equal(q2, keep)
    assert np.array_equal(qo2.cpu().numpy().view(np.uint16), want_q2.view(np.uint16))


def test_rope_errors(gpu):
    from uniql_amd import ops
    q = torch.zeros(1, 4, 8, 16, dtype=torch.float16, device=gpu)
    k = torch.zeros(1, 4, 2, 16, dtype=torch.float16, device=gpu)
    cos = torch.zeros(1, 4, 32, dtype=torch.float16, device=gpu)
    idx = torch.zeros(2, 16, dtype=torch.uint8, device=gpu)
    ops.rope_indices_(q, k, cos, cos, idx)
    with pytest.raises(RuntimeError):
        ops.rope_indices_(q.float(), k, cos, cos, idx)
    with pytest.raises(RuntimeError):
        ops.rope_indices_(q, k, cos, cos, idx[:1])
    with pytest.raises(RuntimeError):
        ops.rope_indices_(q, k, cos[:, :3], cos[:, :3], idx)
    with pytest.raises(RuntimeError):
        ops.rope_indices_(q, k, cos, cos, idx.to(torch.int16))
    with pytest.raises(RuntimeError):
        ops.rope_indices_(q.transpose(1, 2), k, cos, cos, idx)
    with pytest.raises(RuntimeError):   # 3 query heads cannot share 2 key/value heads
        ops.rope_indices_(q[:, :, :3].contiguous(), k, cos, cos, idx)


# ------------------------------------------------------------------ embedding quantiser
@pytest.mark.parametrize("v,d", [(1, 8), (37, 64), (300, 256), (1000, 4096), (5, 2056)])
def test_embedding_quantize_bit_exact(gpu, v, d):
    from uniql_amd import ops
    g = torch.Generator().manual_seed(v + d)
    w = (torch.randn(v, d, generator=g) * 0.05).half()
    if v > 4:
        w[1] = 0                                   # all-zero row: 0/0 -> code 0, scale 0
        w[2] = torch.full((d,), 6e-8).half()       # scale underflows to zero: x/0 = inf -> code 15
        w[3, ::2] = 65504.0                        # largest fp16 values
        w[4] = (torch.arange(d) % 16 - 8).half() * 0.125   # exact multiples of the scale: rounding ties
    packed, scales = ops.w4_embedding_quantize(w.to(gpu))
    o_packed, o_scales = O.embedding_quantize(w)
    assert np.array_equal(scales.cpu().numpy().view(np.uint16), np.asarray(o_scales).view(np.uint16))
    assert np.array_equal(packed.cpu().numpy(), np.asarray(o_packed))


def test_embedding_quantize_hand_computed_ties(gpu):
    """The device quantiser on the rows whose codes are worked out by hand in
    tests/test_oracle_golden.py::test_embedding_quantize_rounding_ties_by_hand (fp16 rounding of
    every step, halves to even, clamp, all-zero row): literal expectations, no oracle call."""
    from uniql_amd import ops
    rows = torch.tensor([[8.0, 0.5, 1.5, -0.5, -1.5, 2.5, 257 / 512, -257 / 512],
                         [7.0, 1341 / 1024, 1340 / 1024, 0.4375, -7.0, 0.0, 0.0, 0.0],
                         [0.0] * 8], dtype=torch.float16)
    packed, scales = ops.w4_embedding_quantize(rows.to(gpu))
    assert scales.cpu().tolist() == [1.0, 0.875, 0.0]
    want = [[15, 8, 10, 8, 6, 10, 8, 8], [15, 10, 9, 8, 0, 8, 8, 8], [0] * 8]
    words = packed.cpu().numpy().view(np.uint32)[:, 0]
    for r in range(3):
        got = [0] * 8
        for i, e in enumerate([0, 2, 4, 6, 1, 3, 5, 7]):      # nibble i holds element e
            got[e] = int(words[r] >> np.uint32(4 * i)) & 15
        assert got == want[r], (r, got)


def test_embedding_module_from_fp16_on_the_device(gpu):
    from uniql_amd.quantize.quant_embedding_layers import W4O16Embedding
    emb = torch.nn.Embedding(500, 512).half()
    emb.weight.data = (torch.randn(500, 512, generator=torch.Generator().manual_seed(2)) * 0.1).half()
    q_dev = W4O16Embedding.from_fp16(emb.to(gpu))
    o_packed, o_scales = O.embedding_quantize(emb.weight.data.cpu())
    assert np.array_equal(q_dev.weight.data.cpu().numpy(), np.asarray(o_packed))
    assert np.array_equal(q_dev.scales.cpu().numpy().view(np.uint16), np.asarray(o_scales).view(np.uint16))
    ids = torch.randint(0, 500, (3, 7), generator=torch.Generator().manual_seed(3))
    out = q_dev(ids.to(gpu))
    want = O.embedding_lookup(ids.numpy(), np.asarray(o_packed), np.asarray(o_scales))
    assert np.array_equal(out.cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_embedding_quantize_errors(gpu):
    from uniql_amd import ops
    with pytest.raises(RuntimeError):
        ops.w4_embedding_quantize(torch.zeros(4, 12, dtype=torch.float16, device=gpu))
    with pytest.raises(RuntimeError):
        ops.w4_embedding_quantize(torch.zeros(4, 16, dtype=torch.float32, device=gpu))
    with pytest.raises(RuntimeError):
        ops.w4_embedding_quantize(torch.zeros(4, 16, dtype=torch.float16))
