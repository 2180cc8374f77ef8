// Base Hadamard matrices of the composite widths 12 * 2^k, 20 * 2^k, 28 * 2^k, 40 * 2^k
// (quantize/hadamard_helpers.py:20-31 of the reference selects fast_hadamard_transform_{12,20,28,40}N of a
// third-party package whose tables are not part of the reference tree).  Built here as:
//   12: the 12 x 12 matrix of N. J. A. Sloane's library of Hadamard matrices ("had.12": first row + - - ... -,
//       rows 1..11 the cyclic shifts of + + - + - - - + + + - +)
//   20: Paley's first construction over GF(19), I + S with S = [[0, 1^T], [-1, Q]], Q[i][j] = chi(i - j)
//   28: Paley's second construction over GF(13), [[S + I, S - I], [S - I, -S - I]], S = [[0, 1^T], [1, Q]]
//   40: [[H20, H20], [H20, -H20]]
// Each satisfies H H^T = n I.  y = x . H: word c of a table has bit c' set where H[c'][c] is -1.
#pragma once

#include <stdint.h>

namespace uniql {

__device__ constexpr uint64_t kHadamard12[12] = {
    0x00000000000ull, 0x00000000b89ull, 0x00000000713ull, 0x00000000e25ull,
    0x00000000c4bull, 0x00000000897ull, 0x0000000012full, 0x0000000025dull,
    0x000000004b9ull, 0x00000000971ull, 0x000000002e3ull, 0x000000005c5ull};

__device__ constexpr uint64_t kHadamard20[20] = {
    0x000000ffffeull, 0x0000009ea18ull, 0x0000003d432ull, 0x0000007a864ull,
    0x000000f50c8ull, 0x000000ea192ull, 0x000000d4326ull, 0x000000a864eull,
    0x00000050c9eull, 0x000000a193cull, 0x0000004327aull, 0x000000864f4ull,
    0x0000000c9eaull, 0x000000193d4ull, 0x000000327a8ull, 0x00000064f50ull,
    0x000000c9ea0ull, 0x00000093d42ull, 0x00000027a86ull, 0x0000004f50cull};

__device__ constexpr uint64_t kHadamard28[28] = {
    0x00000004000ull, 0x00004f293c8ull, 0x00009e52790ull, 0x00003ca8f22ull,
    0x00007951e44ull, 0x0000f2a3c88ull, 0x0000e54b912ull, 0x0000ca9b226ull,
    0x0000953a44eull, 0x00002a7889eull, 0x000054f113cull, 0x0000a9e2278ull,
    0x000053c84f2ull, 0x0000a7909e4ull, 0x0000fffc001ull, 0x0000b0dd3caull,
    0x000061be794ull, 0x0000c374f2aull, 0x000086ede54ull, 0x00000ddfca8ull,
    0x00001bb7952ull, 0x000037672a6ull, 0x00006ec654eull, 0x0000dd84a9eull,
    0x0000bb0d53cull, 0x0000761ea78ull, 0x0000ec354f2ull, 0x0000d86e9e4ull};

__device__ constexpr uint64_t kHadamard40[40] = {
    0x0ffffeffffeull, 0x09ea189ea18ull, 0x03d4323d432ull, 0x07a8647a864ull,
    0x0f50c8f50c8ull, 0x0ea192ea192ull, 0x0d4326d4326ull, 0x0a864ea864eull,
    0x050c9e50c9eull, 0x0a193ca193cull, 0x04327a4327aull, 0x0864f4864f4ull,
    0x00c9ea0c9eaull, 0x0193d4193d4ull, 0x0327a8327a8ull, 0x064f5064f50ull,
    0x0c9ea0c9ea0ull, 0x093d4293d42ull, 0x027a8627a86ull, 0x04f50c4f50cull,
    0x000001ffffeull, 0x0615e79ea18ull, 0x0c2bcd3d432ull, 0x08579b7a864ull,
    0x00af37f50c8ull, 0x015e6dea192ull, 0x02bcd9d4326ull, 0x0579b1a864eull,
    0x0af36150c9eull, 0x05e6c3a193cull, 0x0bcd854327aull, 0x079b0b864f4ull,
    0x0f36150c9eaull, 0x0e6c2b193d4ull, 0x0cd857327a8ull, 0x09b0af64f50ull,
    0x03615fc9ea0ull, 0x06c2bd93d42ull, 0x0d857927a86ull, 0x0b0af34f50cull};

}  // namespace uniql
