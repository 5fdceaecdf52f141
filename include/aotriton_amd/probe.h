/*
 * Measurement aid of the benchmark, kept apart from the operator interface in flash.h: it stands in for
 * no interface of the reference and no caller of the operators needs it.
 */
#ifndef AOTRITON_AMD_PROBE_H
#define AOTRITON_AMD_PROBE_H

#include <stdint.h>

#include "aotriton_amd/flash.h"

#ifdef __cplusplus
extern "C" {
#endif

/* A register-only loop of v_mfma_f32_32x32x16_bf16 (num_workgroups x 4 waves x iters x 32 MFMAs), on
 * constant operands or on operands with random mantissas: what the matrix pipe sustains under the power
 * limit.  out: num_workgroups * 256 floats (device); clocks: 2 x uint64 (device) = shader cycles and
 * 100 MHz reference ticks of workgroup 0.  Timed by the caller; FLOP per launch =
 * num_workgroups * 4 * iters * 32 * 32768. */
FA_API int fa_probe_mfma_rate(int32_t random_operands, int32_t num_workgroups, int32_t iters,
                              float* out, uint64_t* clocks, void* hip_stream);

#ifdef __cplusplus
}
#endif

#endif
