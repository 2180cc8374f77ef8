"""A lane-by-lane numpy model of the streaming kernel's addressing
(uniql_amd/csrc/w4a16_stream.hip), checked against the oracle.  It pins, on the
CPU, which packed bytes, scales and activations each lane combines and where
each accumulator lands; the MFMA itself is modelled as the dot product it is."""
import numpy as np

from oracle import uniql_oracle as O


def single_scale_pos(n):
    blk, c = n & ~31, n & 31
    return blk + 8 * ((c & 7) >> 1) + 2 * (c >> 3) + (c & 1)


def stream_kernel_model(x, packed, s_perm, n, k):
    """x fp16 [M<=16, K]; returns float64 [M, N] following the kernel's index math."""
    m_rows = x.shape[0]
    groups = s_perm.shape[0]
    words = packed.view(np.uint32).reshape(k // 16, n // 2, 4)       # [row][piece][word]
    y = np.zeros((m_rows, n))
    for strip in range(n // 128):
        for g in range(k // 128):
            for lane in range(64):
                slot, kq = lane & 15, lane >> 4
                c8 = slot & 7
                chunk = 2 * strip + (slot >> 3)
                if groups > 1:
                    sc = s_perm[g, chunk * 64 + 8 * c8: chunk * 64 + 8 * c8 + 8].astype(np.float32)
                else:
                    sc = np.array([s_perm[0, single_scale_pos(chunk * 64 + c8 + 8 * jb)] for jb in range(8)],
                                  dtype=np.float32)
                for rr in range(8):
                    row = 8 * g + rr
                    piece = words[row, chunk * 32 + 4 * c8 + kq]
                    kbase = 16 * row + 2 * kq
                    ks = [kbase, kbase + 1, kbase + 8, kbase + 9]
                    for j in range(4):
                        for blk in range(2):
                            q = int(piece[j]) >> (8 * blk)
                            codes = [q & 15, (q >> 16) & 15, (q >> 4) & 15, (q >> 20) & 15]
                            jb = 2 * j + blk
                            ncol = 128 * strip + 64 * (slot >> 3) + 16 * (jb >> 1) + 8 * (jb & 1) + c8
                            wv = [float(np.float16(np.float32(c - 8) * sc[jb])) for c in codes]
                            # this lane's B-operand values meet the A-operand values of every row m
                            for m in range(m_rows):
                                y[m, ncol] += sum(float(x[m, kk]) * w for kk, w in zip(ks, wv))
    return y


def _case(groups_mode, n=256, k=256, m=2, seed=0):
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, size=(k, n)).astype(np.int32)
    g = k // 128 if groups_mode == "grouped" else 1
    s = rng.uniform(0.004, 0.02, size=(g, n)).astype(np.float16)
    x = rng.standard_normal((m, k)).astype(np.float16)
    packed = O.pack_weights(q)
    s_perm = O.permute_scales(s, k, n, 128 if g > 1 else k)
    want = O.gemm_fp64(x, O.dequant_codes(q, s, 128 if g > 1 else k))
    return x, packed, s_perm, want


def test_stream_model_grouped():
    x, packed, s_perm, want = _case("grouped")
    got = stream_kernel_model(x, packed, s_perm, 256, 256)
    assert np.allclose(got, want, atol=1e-9)


def test_stream_model_per_column():
    x, packed, s_perm, want = _case("single", n=128, k=128, m=1, seed=3)
    got = stream_kernel_model(x, packed, s_perm, 128, 128)
    assert np.allclose(got, want, atol=1e-9)
