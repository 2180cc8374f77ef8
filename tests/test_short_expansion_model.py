"""The arithmetic of the streaming kernel's short expansion (uniql_amd/csrc/w4a16_stream.hip,
process()), restated in numpy and held, for every scale of its range and all 16 codes, to the
reference's dequantised weight fp16_rn((code - 8) * scale) (csrc/linear/marlin_gemm_kernel.cuh:118-146).
An fp16 fused multiply-add is modelled as the exact float64 value (an 11-bit by 11-bit product plus
an 11-bit addend fits) rounded once to fp16."""
import numpy as np

LOW, HIGH = 0x1400, 0x2C00   # bit patterns of 2^-10 and 2^-4: the range is [LOW, HIGH)


def fp16_fma(a, b, c):
    with np.errstate(over="ignore", invalid="ignore"):   # scales past the range overflow on purpose (inf * 0 -> NaN is the point of one test)
        return (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(np.float16)


def short_expansion(codes, scale_bits):
    """codes [C], scale_bits [S] (uint16 patterns) -> (high form, low form * 16) as float64 [S, C]."""
    s = scale_bits.view(np.float16)
    with np.errstate(over="ignore"):
        big = (scale_bits + np.uint16(0x5000)).view(np.float16)              # s * 2^20 by an add on the exponent field
    c_high = (s * np.float16(-8.0)).astype(np.float16)
    c_low = (s * np.float16(-0.5)).astype(np.float16)
    high_in = (codes.astype(np.uint16) << 4).view(np.float16)               # the code in bits 4..7: c * 2^-20
    low_in = codes.astype(np.uint16).view(np.float16)                       # the code in bits 0..3: c * 2^-24
    high = fp16_fma(high_in[None, :], big[:, None], c_high[:, None])
    low = fp16_fma(low_in[None, :], big[:, None], c_low[:, None])
    return high.astype(np.float64), low.astype(np.float64) * 16.0


def reference(codes, scale_bits):
    s = scale_bits.view(np.float16)
    return ((codes.astype(np.float16) - np.float16(8.0))[None, :] * s[:, None]).astype(np.float16).astype(np.float64)


def test_short_expansion_is_exact_on_its_whole_range():
    codes = np.arange(16)
    scale_bits = np.arange(LOW, HIGH, dtype=np.uint16)
    high, low = short_expansion(codes, scale_bits)
    want = reference(codes, scale_bits)
    assert np.array_equal(high, want)
    assert np.array_equal(low, want)


def test_the_range_is_as_wide_as_the_arithmetic_allows():
    codes = np.arange(16)
    # one step below 2^-10 the low form's result (divided by 16) can be subnormal and lose a bit
    below = np.arange(LOW - 0x400, LOW, dtype=np.uint16)
    _, low = short_expansion(codes, below)
    assert not np.array_equal(low, reference(codes, below))
    # from 2^-4 on s * 2^20 is not an fp16 number any more (the exponent add runs into inf / NaN patterns)
    above = np.arange(HIGH, HIGH + 0x400, dtype=np.uint16)
    high, _ = short_expansion(codes, above)
    assert not np.array_equal(high, reference(codes, above))


def test_range_check_of_the_kernel():
    """The kernel's test on a word of two scales: t = bits - 0x14001400; a half is in range iff neither t nor
    t + 0x0800 has one of its three top bits set.  Exhaustive over one half, with the other half in range."""
    bits = np.arange(0x10000, dtype=np.uint32)
    for other_shift, this_shift in ((16, 0), (0, 16)):
        word = (bits << this_shift) | (np.uint32(0x2000) << other_shift)
        t = word - np.uint32(0x14001400)
        bad = ((t | (t + np.uint32(0x08000800))) & np.uint32(0xE000E000)) != 0
        assert np.array_equal(~bad, (bits >= LOW) & (bits < HIGH))
