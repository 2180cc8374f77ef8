/*
 * uniql_amd_diag.h - test hooks and measurement aids of libuniql_amd.so.
 *
 * Nothing here is needed to run a model: the flag bits force a kernel or a plan that the library
 * would not choose by itself (parity tests run both kernels on the same call, benchmarks sweep
 * plans), the entry points time parts of the machine.  None has a counterpart in the reference.
 * Conventions as in uniql_amd.h.
 */
#ifndef UNIQL_AMD_DIAG_H
#define UNIQL_AMD_DIAG_H

#include "uniql_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* more bits of the `flags` argument of uniql_w4a16_gemm / uniql_w4a16_linear / uniql_w4a16_gemm_static */
enum {
    UNIQL_F_FORCE_SKINNY = 1 << 1, /* use the weight-streaming kernel (default for m <= 16) whatever m is */
    UNIQL_F_FORCE_TILED = 1 << 2,  /* use the tiled MFMA kernel (default for m > 16) whatever m is */
    UNIQL_F_SEPARATE_ROTATION = 1 << 4 /* run a whole-row rotation as its own transform kernel into `temp` even
                                      where the streaming kernel could apply it itself (both ways give the
                                      same values bit for bit) */
    /* tuning fields, 0 = choose.  Streaming kernel: bits 8..15 K-groups per wavefront,
       bits 16..20 wavefronts per workgroup (4 or 8).
       Tiled kernels: bits 8..15 number of K splits over workgroups, bits 16..19 row tiles of 32
       per workgroup (1, 2 or 4: the 128-column kernel; 8: the 256 x 256 kernel for long prefill,
       which needs n % 256 == 0, k >= 256 and grouped scales and otherwise leaves the call to the
       128-column kernel), bits 20..21 wave quartets per workgroup (1 or 2). */
};

/*
 * Launches a kernel that only READS what the
 * streaming kernel (m <= 16) of uniql_w4a16_gemm reads for this shape - every packed weight and
 * scale once, with the same grid, waves per workgroup, walk over the K groups and 16-byte loads -
 * and computes nothing.  Its duration is the floor the memory system and the launch set for that
 * plan; bench.py reports it beside the product kernel's.
 *   sink    device, uniql_w4a16_read_floor_sink_bytes(m, n, k, flags) bytes: practically never written
 *   flags   the streaming kernel's tuning fields (bits 8..15, 16..20) choose the same plan;
 *           bits 21..23: units a wave requests before it consumes the first (0 or 1: one, as the
 *           product kernel does per register set; 2 or 4: deeper)
 */
size_t uniql_w4a16_read_floor_sink_bytes(int m, int n, int k, unsigned flags);
int uniql_w4a16_read_floor(const void* B, const void* S, void* sink, size_t sink_bytes, int m, int n, int k,
                           unsigned flags, void* stream);

/*
 * What the matrix pipe alone sustains: 256 workgroups of four waves, each wave issuing `iters` times
 * eight independent v_mfma_f32_32x32x16_f16 on operands loaded once - no loads, LDS reads or weight
 * expansion in the loop.  2 * 32 * 32 * 16 * 8 * iters * 1024 flops per launch.  The operands decide
 * the switching activity, and with it the clock the chip settles at, so the caller provides them.
 *   operands  device, 512 x 16 bytes: fp16 A operand of thread t at 16 t, B operand at 16 (256 + t)
 *   out       device, 256 x 256 floats, written once at the end
 */
int uniql_diag_mfma_loop(const void* operands, void* out, int iters, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* UNIQL_AMD_DIAG_H */
