"""Host-side layout code of the package (index algebra) against the oracle (table
form) and the reference's golden vectors."""
import numpy as np
import pytest
import torch

from oracle import uniql_oracle as O
from uniql_amd import layout
from uniql_amd.quantize import quantize_helpers as QH


def test_pack_matches_golden_and_oracle(golden):
    codes = torch.from_numpy(golden["P_codes"].astype(np.int32))
    assert np.array_equal(layout.pack_codes(codes).numpy(), golden["P_packed"])
    rng = np.random.default_rng(1)
    q = rng.integers(0, 16, size=(160, 320)).astype(np.int32)
    q[0, 0] = 15; q[9, 8] = 15      # exercise the sign bit of the word (nibble 7)
    assert np.array_equal(layout.pack_codes(torch.from_numpy(q)).numpy(), O.pack_weights(q))


@pytest.mark.parametrize("case", ["A", "B", "C"])
def test_unpack_matches_golden(golden, case):
    packed = torch.from_numpy(golden[f"{case}_packed"])
    kp, np_ = packed.shape[0] * 16, packed.shape[1] // 2
    assert np.array_equal(layout.unpack_codes(packed, kp, np_).numpy(), golden[f"{case}_codes"].astype(np.int32))


def test_scale_permutations(golden):
    ramp = torch.from_numpy(golden["S_ramp"])
    out = layout.permute_scales(ramp, 256, 256, 128)
    assert np.array_equal(out.numpy(), golden["S_grouped"])
    assert torch.equal(layout.unpermute_scales(out, 256, 256, 128), ramp)
    ramp1 = torch.from_numpy(golden["S_ramp1"])
    out1 = layout.permute_scales(ramp1, 128, 256, 128)
    assert np.array_equal(out1.numpy(), golden["S_single"])
    assert torch.equal(layout.unpermute_scales(out1, 128, 256, 128), ramp1)


@pytest.mark.parametrize("case,pad_out", [("A", 0), ("B", 192), ("C", 0)])
def test_quantize_and_pack_matches_golden(golden, case, pad_out):
    w = torch.from_numpy(golden[f"{case}_w"])
    w_ref, packed, scale = layout.quantize_and_pack(w.clone(), 128, None, pad_out)
    assert np.array_equal(packed.numpy(), golden[f"{case}_packed"])
    assert np.array_equal(scale.numpy().view(np.uint16), golden[f"{case}_scale"].view(np.uint16))
    if case == "A":
        assert np.array_equal(w_ref.numpy().view(np.uint16), golden["A_w_ref"].view(np.uint16))


def test_gptq_handover_matches_golden(golden):
    w, s = torch.from_numpy(golden["G_w"]), torch.from_numpy(golden["G_scale_in"])
    _, packed, scale = layout.quantize_and_pack(w.clone(), 128, s.clone(), 0)
    assert np.array_equal(packed.numpy(), golden["G_packed"])
    assert np.array_equal(scale.numpy().view(np.uint16), golden["G_scale"].view(np.uint16))


def test_helper_names_tables(golden):
    assert np.array_equal(QH.get_w4a16_weight_perms().numpy(), golden["weight_perm"])
    g, s = QH.get_scale_perms()
    assert g == golden["scale_perm"].tolist() and s == golden["scale_perm_single"].tolist()
    assert QH.get_pack_factor(4) == 8
    res = QH.w4a16_quantize(torch.from_numpy(golden["A_w"]).clone(), 4, 128, None, pad_out=0)
    assert isinstance(res, list) and np.array_equal(res[1].numpy(), golden["A_packed"])
    q = QH.unpack_w4a16_permute_weights(res[1], 256, 256, 4, QH.get_w4a16_weight_perms(), 128)
    assert np.array_equal(q.numpy(), golden["A_codes"].astype(np.int32))
    assert torch.equal(QH.get_w4a16_permute_weights(q, 256, 256, 4, None, 128), res[1])


def test_embedding_pack_matches_oracle():
    g = torch.Generator().manual_seed(4)
    w = torch.randn(40, 96, generator=g).to(torch.float16)
    packed, scales = layout.quantize_embedding(w)
    o_packed, o_scales = O.embedding_quantize(w)
    assert np.array_equal(packed.numpy(), o_packed)
    assert np.array_equal(scales.numpy().view(np.uint16), o_scales.view(np.uint16))
    assert np.array_equal(layout.unpack_embedding_codes(packed).numpy(), O.embedding_unpack(o_packed))


def test_per_column_quantisation_is_refused():
    with pytest.raises(NotImplementedError):
        layout.quantize_and_pack(torch.zeros(128, 256, dtype=torch.float16), -1)
