/*
 * Diagnostics of libflashtensor_diag: hardware probes for benchmark context.  Not part of the product ABI
 * (include/ft_abi.h) and without a counterpart in the reference (monellz/FlashTensor); no product call uses them.
 * Functions return 0 or -1; ft_diag_last_error() then holds a thread-local message.
 */
#ifndef FT_DIAG_H
#define FT_DIAG_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FT_DIAG_PROBE_OPERAND_BYTES 65536 /* the probe reads 4096 x 16 bytes of operands */
#define FT_DIAG_PROBE_MAX_ITERS 4000000   /* about 0.4 s of kernel time */

const char* ft_diag_last_error(void);

/* What the matrix pipe sustains on given operand values.  `workgroups` workgroups of 8 waves each issue
 * 4 * iters v_mfma_f32_32x32x16_f16 (32768 FLOP each) on fp16 fragments read from `operands` (operand_bytes >=
 * FT_DIAG_PROBE_OPERAND_BYTES, 16-byte aligned, any values) and nothing else; time the launch with events on the
 * stream.  clocks (optional, 2 x int64): shader-clock ticks and 100 MHz ticks one wave counted over its loop.
 * The chip is power-limited, so the rate depends on the bit patterns of the operands.  sink: >= 4 bytes, unused. */
int ft_diag_probe_mfma(const void* operands, size_t operand_bytes, int32_t workgroups, int32_t iters, float* sink,
                       int64_t* clocks, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FT_DIAG_H */
