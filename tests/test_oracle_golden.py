"""The CPU oracle against vectors written by the reference's own
quantize/quantize_helpers.py (tests/golden/make_golden.py), and against what
the mathematics fixes independently of any restatement."""
import numpy as np
import pytest
import scipy.linalg
import torch

from oracle import uniql_oracle as O


# ---------------------------------------------------------------- tables
def test_weight_perm_table_equals_reference(golden):
    assert np.array_equal(O.weight_perm_table(), golden["weight_perm"])


def test_weight_perm_is_bijection_and_hand_values():
    t = O.weight_perm_table()
    assert sorted(t.tolist()) == list(range(1024))
    # lane 0, tile 0: rows 0,1,8,9 of column 0 then of column 8, interleaved [0,2,4,6,1,3,5,7]
    assert t[:8].tolist() == [0, 128, 8, 136, 16, 144, 24, 152]


def test_scale_perm_tables_equal_reference(golden):
    g, s = O.scale_perm_tables()
    assert np.array_equal(g, golden["scale_perm"])
    assert np.array_equal(s, golden["scale_perm_single"])


def test_weight_perm_closed_form():
    """Independent derivation: word w of a 16x64 row block, nibble p, holds
    K-row [2a, 2a+1, 2a+8, 2a+9][rr] and column 16 j + c8 + 8 blk, where
    lane = w // 4, j = w % 4, a = lane % 4, c8 = lane // 4,
    orig = [0,2,4,6,1,3,5,7][p], blk = orig // 4, rr = orig % 4."""
    t = O.weight_perm_table()
    for w in range(128):
        lane, j = divmod(w, 4)
        a, c8 = lane % 4, lane // 4
        for p in range(8):
            orig = [0, 2, 4, 6, 1, 3, 5, 7][p]
            blk, rr = divmod(orig, 4)
            krow = [2 * a, 2 * a + 1, 2 * a + 8, 2 * a + 9][rr]
            ncol = c8 + 8 * blk
            assert t[8 * w + p] == 256 * j + 16 * krow + ncol


# ---------------------------------------------------------------- pack / unpack
def test_pack_equals_reference(golden):
    codes = golden["P_codes"].astype(np.int32)
    assert np.array_equal(O.pack_weights(codes), golden["P_packed"])


@pytest.mark.parametrize("case", ["A", "B", "C"])
def test_unpack_equals_reference(golden, case):
    packed = golden[f"{case}_packed"]
    kp, np_ = packed.shape[0] * 16, packed.shape[1] // 2
    assert np.array_equal(O.unpack_weights(packed, kp, np_), golden[f"{case}_codes"].astype(np.int32))


def test_pack_unpack_roundtrip_random():
    rng = np.random.default_rng(7)
    q = rng.integers(0, 16, size=(48, 192)).astype(np.int32)
    assert np.array_equal(O.unpack_weights(O.pack_weights(q), 48, 192), q)


def test_pack_bruteforce_tiny():
    """Every nibble of a one-tile-row matrix located by the closed form."""
    rng = np.random.default_rng(3)
    q = rng.integers(0, 16, size=(16, 64)).astype(np.int32)
    packed = O.pack_weights(q).view(np.uint32)
    for w in range(128):
        lane, j = divmod(w, 4)
        a, c8 = lane % 4, lane // 4
        for p in range(8):
            orig = [0, 2, 4, 6, 1, 3, 5, 7][p]
            blk, rr = divmod(orig, 4)
            k = [2 * a, 2 * a + 1, 2 * a + 8, 2 * a + 9][rr]
            n = 16 * j + c8 + 8 * blk
            assert (int(packed[0, w]) >> (4 * p)) & 15 == q[k, n]


# ---------------------------------------------------------------- scales
def test_scale_permutes_equal_reference(golden):
    out = O.permute_scales(golden["S_ramp"], 256, 256, 128)
    assert np.array_equal(out, golden["S_grouped"])
    out1 = O.permute_scales(golden["S_ramp1"], 128, 256, 128)
    assert np.array_equal(out1, golden["S_single"])
    assert np.array_equal(O.unpermute_scales(out, 256, 256, 128), golden["S_ramp"])
    assert np.array_equal(O.unpermute_scales(out1, 128, 256, 128), golden["S_ramp1"])


@pytest.mark.parametrize("case", ["A", "B", "C"])
def test_unpermute_scales_equal_reference(golden, case):
    s = golden[f"{case}_scale"]
    kp = s.shape[0] * 128
    assert np.array_equal(O.unpermute_scales(s, kp, s.shape[1], 128), golden[f"{case}_scale_unperm"])


# ---------------------------------------------------------------- quantiser
@pytest.mark.parametrize("case,pad_out", [("A", 0), ("B", 192), ("C", 0)])
def test_quantizer_equals_reference(golden, case, pad_out):
    w = torch.from_numpy(golden[f"{case}_w"])
    w_ref, packed, scale = O.w4a16_quantize(w.clone(), 128, None, pad_out)
    assert np.array_equal(packed.numpy(), golden[f"{case}_packed"])
    assert np.array_equal(scale.numpy().view(np.uint16), golden[f"{case}_scale"].view(np.uint16))
    if case == "A":
        assert np.array_equal(w_ref.numpy().view(np.uint16), golden["A_w_ref"].view(np.uint16))


def test_quantizer_zero_group_and_k_padding(golden):
    # case C has an all-zero (group, column): scale 0, 0/0 = NaN.  What NaN becomes in
    # .int() is the platform's float->int conversion; on x86 (where the vectors were
    # written) it is INT_MIN, so +8 and the clamp leave code 0.  With scale 0 the
    # dequantised weight is -0.0 either way.
    codes = golden["C_codes"]
    assert (codes[:128, 7] == 0).all()
    assert (golden["C_scale_unperm"][0, 7] == 0)
    # rows appended to reach a multiple of 128 are zero weights in a non-zero group -> code 8
    assert (codes[200:256, :] == 8).all()


def test_gptq_branch_equals_reference(golden):
    w = torch.from_numpy(golden["G_w"])
    s = torch.from_numpy(golden["G_scale_in"])
    _, packed, scale = O.w4a16_quantize(w.clone(), 128, s.clone(), 0)
    assert np.array_equal(packed.numpy(), golden["G_packed"])
    assert np.array_equal(scale.numpy().view(np.uint16), golden["G_scale"].view(np.uint16))


# ---------------------------------------------------------------- dequant
def test_dequant_equals_reference_w_ref(golden):
    """w_ref of the reference == fp16((q-8)*s) of the oracle, bit for bit."""
    w = O.dequant_packed(golden["A_packed"], golden["A_scale"], 256, 256)
    assert np.array_equal(w.view(np.uint16), golden["A_w_ref"].view(np.uint16))


def test_dequant_closed_form_exhaustive_scales():
    """All 16 codes x a sweep of fp16 scale bit patterns against exact rational rounding."""
    bits = np.arange(0x0001, 0x7C00, 37, dtype=np.uint16)        # positive finite, incl. subnormals
    s = bits.view(np.float16)
    q = np.arange(16, dtype=np.int32)
    got = O.dequant_codes(np.repeat(q[:, None], s.size, 1), s[None, :], group_size=16)
    exact = (q[:, None].astype(np.float64) - 8.0) * s[None, :].astype(np.float64)
    want = exact.astype(np.float16)      # float64 -> fp16 is a single correctly rounded step
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_gemm_bruteforce_tiny():
    rng = np.random.default_rng(5)
    q = rng.integers(0, 16, size=(128, 256)).astype(np.int32)
    s = rng.uniform(0.004, 0.02, size=(1, 256)).astype(np.float16)
    x = rng.standard_normal((3, 128)).astype(np.float16)
    packed = O.pack_weights(q)
    s_perm = O.permute_scales(s, 128, 256, 128)
    y = O.linear_forward(x, packed, s_perm, in_features=128, out_features=256, exact=True)
    # explicit loops, no library product
    w = [[float(np.float16((int(q[k, n]) - 8) * np.float32(s[0, n]))) for n in range(256)] for k in range(128)]
    for m in range(3):
        for n in (0, 1, 17, 128, 255):
            acc = 0.0
            for k in range(128):
                acc += float(x[m, k]) * w[k][n]
            assert abs(acc - y[m, n]) < 1e-9


def test_linear_forward_padding_and_bias():
    rng = np.random.default_rng(11)
    in_f, out_f = 200, 300
    geo = O.linear_geometry(in_f, out_f)
    assert (geo["size_k"], geo["size_n"], geo["pad_in"], geo["pad_out"]) == (256, 512, 56, 212)
    assert geo["workspace"] == 512 // 64 * 16 and geo["weight"] == (16, 1024) and geo["scale"] == (2, 512)
    w = torch.from_numpy((rng.standard_normal((in_f, out_f)) * 0.05).astype(np.float16))
    _, packed, scale = O.w4a16_quantize(w, 128, None, geo["pad_out"])
    x = rng.standard_normal((2, 5, in_f)).astype(np.float16)
    b = rng.standard_normal(out_f).astype(np.float16)
    y = O.linear_forward(x, packed.numpy(), scale.numpy(), in_features=in_f, out_features=out_f, bias=b)
    assert y.shape == (2, 5, out_f)
    w_ref, _, _ = O.fake_quantize_grouped(w)
    want = x.reshape(-1, in_f).astype(np.float64) @ w_ref.numpy()[:in_f].astype(np.float64) + b.astype(np.float64)
    assert np.allclose(y.reshape(-1, out_f), want, atol=1e-4)


# ---------------------------------------------------------------- embedding
def test_embedding_hand_case():
    # one row: max |w| = 8 -> scale 1; values k -> code k + 8
    row = torch.tensor([[-8.0, -3.0, 0.0, 7.0, 1.0, 2.0, -1.0, 8.0]], dtype=torch.float16)
    packed, scales = O.embedding_quantize(row)
    assert scales.tolist() == [1.0]
    codes = [0, 5, 8, 15, 9, 10, 7, 15]          # 8 + w, clamped to 15
    # nibble i holds element [0,2,4,6,1,3,5,7][i]
    word = sum(codes[e] << (4 * i) for i, e in enumerate([0, 2, 4, 6, 1, 3, 5, 7]))
    assert int(packed.view(np.uint32)[0, 0]) == word
    out = O.embedding_lookup(np.array([0]), packed, scales)
    assert out[0].tolist() == [-8.0, -3.0, 0.0, 7.0, 1.0, 2.0, -1.0, 7.0]


def _emb_codes(row, dtype):
    packed, scales = O.embedding_quantize(torch.tensor([row], dtype=dtype))
    return O.embedding_unpack(packed)[0].tolist(), scales.tolist()


def test_embedding_quantize_rounding_ties_by_hand():
    """Code selection of W4O16Embedding.from_fp16 (quant_embedding_layers.py:35-37) where the
    rounding steps decide, worked out by hand (not by running the oracle's formula again):
    every operation rounds in the WEIGHT's dtype, and torch.round rounds halves to even.

    Row A, max |w| = 8 -> scale 1 (division exact), fp16:
      0.5 -> 8.5 -> 8;  1.5 -> 9.5 -> 10;  -0.5 -> 7.5 -> 8;  -1.5 -> 6.5 -> 6;  2.5 -> 10.5 -> 10
      257/512 = 0.501953125: the sum 8.501953125 lies between the fp16 neighbours 8.5 and 8.5078125
      (spacing 2^-7 in [8, 16)) and rounds to 8.5, a tie that appears only in fp16 -> 8; in
      float32 the sum is exact and rounds to 9.  -257/512: 7.498046875 -> fp16 7.5 -> 8; float32 -> 7.
      8.0 -> 16 -> clamped to 15.
    Row B, max |w| = 7 -> scale 0.875, fp16: 1341/1024 / 0.875 = 1.496652 rounds to the fp16
      quotient 1533/1024 = 1.4970703 (neighbour 1532/1024 is farther: 0.000558 against 0.000418);
      + 8 = 9.4970703 lies between 9.4921875 and 9.5 and rounds to 9.5 (0.0029 against 0.0049)
      -> 10, while exact arithmetic gives round(9.496652) = 9 (float32 does).
      1340/1024: quotient 1.4955357 -> 1531/1024 = 1.4951172; + 8 -> 9.4921875 -> 9 in both.
      0.4375 / 0.875 = 0.5 exactly -> 8.5 -> 8;  -7 -> -8 + 8 = 0.
    Row C, all zero: scale 0, 0/0 = NaN, NaN survives round and clamp, the int32 conversion
      gives 0x80000000 whose low nibble is 0 -> code 0 (and the lookup returns -0.0 = -8 * 0)."""
    row_a = [8.0, 0.5, 1.5, -0.5, -1.5, 2.5, 257 / 512, -257 / 512]
    codes, scales = _emb_codes(row_a, torch.float16)
    assert scales == [1.0] and codes == [15, 8, 10, 8, 6, 10, 8, 8]
    codes, _ = _emb_codes(row_a, torch.float32)
    assert codes == [15, 8, 10, 8, 6, 10, 9, 7]
    row_b = [7.0, 1341 / 1024, 1340 / 1024, 0.4375, -7.0, 0.0, 0.0, 0.0]
    codes, scales = _emb_codes(row_b, torch.float16)
    assert scales == [0.875] and codes == [15, 10, 9, 8, 0, 8, 8, 8]
    codes, _ = _emb_codes(row_b, torch.float32)
    assert codes == [15, 9, 9, 8, 0, 8, 8, 8]
    packed, scales = O.embedding_quantize(torch.zeros(1, 16, dtype=torch.float16))
    assert scales.tolist() == [0.0] and O.embedding_unpack(packed)[0].tolist() == [0] * 16
    out = O.embedding_lookup(np.array([0]), packed, scales)
    assert np.array_equal(out.view(np.uint16), np.full((1, 16), 0x8000, dtype=np.uint16))


def test_embedding_roundtrip_and_gather():
    g = torch.Generator().manual_seed(2)
    w = torch.randn(50, 64, generator=g).to(torch.float16)
    packed, scales = O.embedding_quantize(w)
    codes = O.embedding_unpack(packed)
    want_codes = torch.round(w / (w.abs().amax(-1, keepdim=True) / 8) + 8).clamp(0, 15).int().numpy()
    assert np.array_equal(codes, want_codes)
    ids = np.array([[3, 49, 0], [7, 7, 21]])
    out = O.embedding_lookup(ids, packed, scales)
    assert out.shape == (2, 3, 64) and out.dtype == np.float16
    for b in range(2):
        for t in range(3):
            i = ids[b, t]
            want = ((codes[i].astype(np.float32) - 8) * np.float32(scales[i])).astype(np.float16)
            assert np.array_equal(out[b, t], want)


# ---------------------------------------------------------------- Hadamard
@pytest.mark.parametrize("n", [2, 8, 128, 1024])
def test_fwht_matches_scipy_hadamard(n):
    rng = np.random.default_rng(n)
    x = rng.standard_normal((3, n)).astype(np.float32)
    got = O.fwht(x, 1.0 / np.sqrt(n), acc=np.float64)
    want = (x.astype(np.float64) @ scipy.linalg.hadamard(n).astype(np.float64)) / np.sqrt(n)
    assert np.allclose(got, want.astype(np.float32), atol=1e-5)


def test_fwht_involution_parseval_and_blocks():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((4, 512)).astype(np.float32)
    y = O.fwht(x, 512 ** -0.5)
    assert np.allclose(O.fwht(y, 512 ** -0.5), x, atol=1e-5)
    assert np.allclose((y ** 2).sum(-1), (x ** 2).sum(-1), rtol=1e-5)
    yb = O.fwht(x, 128 ** -0.5, block=128)
    h = scipy.linalg.hadamard(128) / np.sqrt(128)
    want = np.concatenate([x[:, i:i + 128] @ h for i in range(0, 512, 128)], axis=1)
    assert np.allclose(yb, want, atol=1e-5)


def test_had_variant_selection():
    assert O.had_variant(4096) == (2, 1 / 64)
    assert O.had_variant(14336)[0] == 28       # 28 * 512
    assert O.had_variant(5120)[0] == 40        # 40 * 128
    assert O.had_variant(3584)[0] == 28        # 28 * 128
    assert O.had_variant(12288)[0] == 12
    with pytest.raises(AssertionError):
        O.had_variant(12160)                   # 95 * 128: the reference asserts


def test_hadlinear_identity():
    """Rotating the weight's input side and the activation by the same orthogonal H leaves x W^T unchanged."""
    rng = np.random.default_rng(9)
    w = rng.standard_normal((24, 64)).astype(np.float32)
    x = rng.standard_normal((5, 64)).astype(np.float32)
    wh = O.hadlinear_fused_weight(w, True, False)
    xh = O.fwht(x, 64 ** -0.5)
    assert np.allclose(xh @ wh.T, x @ w.T, atol=1e-4)
    h = scipy.linalg.hadamard(64) / 8.0
    assert np.allclose(wh, w @ h, atol=1e-5)
    who = O.hadlinear_fused_weight(np.ascontiguousarray(w.T), False, True)   # [64, 24] output side
    assert np.allclose(who, h @ w.T, atol=1e-5)


@pytest.mark.parametrize("base", [12, 20, 28, 40])
def test_hadamard_base_matrices_are_hadamard(base):
    """Entries +-1, H H^T = H^T H = n I; the 12 is Sloane's had.12 written out."""
    h = O.hadamard_base_matrix(base)
    assert h.shape == (base, base) and set(np.unique(h)) == {-1, 1}
    assert np.array_equal(h @ h.T, base * np.eye(base, dtype=np.int64))
    assert np.array_equal(h.T @ h, base * np.eye(base, dtype=np.int64))
    if base == 12:
        rows = ["+-----------", "++-+---+++-+", "+++-+---+++-", "+-++-+---+++", "++-++-+---++", "+++-++-+---+",
                "++++-++-+---", "+-+++-++-+--", "+--+++-++-+-", "+---+++-++-+", "++---+++-++-", "+-+---+++-++"]
        assert np.array_equal(h, np.array([[1 if c == "+" else -1 for c in r] for r in rows]))
    if base == 40:
        h20 = O.hadamard_base_matrix(20)
        assert np.array_equal(h[:20, 20:], h20) and np.array_equal(h[20:, 20:], -h20)


@pytest.mark.parametrize("dim", [12, 96, 160, 448, 1280])
def test_composite_transform_is_the_kronecker_product(dim):
    """fwht_composite(x) = x @ kron(H_base, H_P) (float64 matmul with scipy's Sylvester matrix), its rows are
    orthogonal (x -> transform -> transform with the transposed matrix gives dim * x)."""
    from scipy.linalg import hadamard
    base = O.had_variant(dim)[0]
    p = dim // base
    big = np.kron(O.hadamard_base_matrix(base), hadamard(p) if p > 1 else np.ones((1, 1)))
    x = np.random.default_rng(dim).standard_normal((5, dim))
    got = O.fwht_composite(x, 1.0, base, acc=np.float64)
    assert np.allclose(got, x @ big, rtol=0, atol=1e-9)
    assert np.allclose(got @ big.T, dim * x, rtol=0, atol=1e-8)
    x16 = x.astype(np.float16)
    y16 = O.fwht_composite(x16, dim ** -0.5, base)
    assert y16.dtype == np.float16 and np.abs(y16.astype(np.float64) - (x16.astype(np.float64) @ big) * dim ** -0.5).max() < 4e-3
