/*
 * pa_probe.h -- measuring tools for the decode kernels, in a library of their own (libpa_probe.so, built from
 * tests/native/pa_probe.hip).  They are not part of the operator and not of its ABI (include/pa_decode.h);
 * bench.py loads them for its two probe workloads.  Both return 0 or a negative PA_ERR_* code of pa_decode.h.
 */
#ifndef PA_PROBE_H_
#define PA_PROBE_H_

#include <stdint.h>

#include "../../include/pa_decode.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * A read-only probe of the memory access pattern of stage 1.  For the same arguments it reads the K and V bytes
 * that the partition kernel for up to 16 query rows reads (FP8 cache, plain V layout, any power-of-two block size;
 * anything else is PA_ERR_UNSUPPORTED), with the same workgroup decomposition, load width and cache policy, and does no
 * arithmetic: its duration is what the memory system gives the gather pattern.  sink: at least 64 int32 of device
 * memory (written only in a case that does not occur; it keeps the loads alive).
 */
int pa_probe_gather(const PaDecodeArgs* args, int32_t* sink, void* hip_stream);

/*
 * The same pages read by workgroups whose four waves share every 64-token step: wave w loads K of the step's tile
 * w, head dims 32 w .. 32 w + 31 of V and the tile's per-token scales (when the arguments have them), `depth` steps
 * ahead in registers, with one workgroup barrier per step, `workgroups_per_cu` workgroups per CU: depth 2 or 4 with
 * 2, 3 or 4, depth 6 with 2 (what fits the registers).  variant: bit 0 = no barrier, bit 1 = the per-token scales
 * are not read (what each of the two costs), bit 2 = wave w reads all of V for tile w, as the waves of
 * pa_partition_shared_kernel do.  Same restrictions and sink as pa_probe_gather.
 */
int pa_probe_stream(const PaDecodeArgs* args, int32_t depth, int32_t workgroups_per_cu, int32_t variant, int32_t* sink,
                    void* hip_stream);

/*
 * The issue cost of the instructions the decode step is made of.  Launches `workgroups` workgroups of four waves
 * (one per SIMD; 256 x n workgroups put n waves on every SIMD of a 256-CU GPU) that each run `iterations` x 128
 * instructions of one kind: mode 0 v_fma_f32 (the full-rate yardstick), 3 v_exp_f32, 4 v_cvt_pk_fp8_f32,
 * 5 v_permlane32_swap; mode 1 runs iterations x 16 v_mfma_f32_16x16x128_f8f6f4, mode 2 the same 16 MFMAs with
 * eight independent v_fma_f32 behind each (how far the matrix pipe runs beside the vector ALU).  sink: at least
 * 64 int32 of device memory (not written in practice).  Time it with events on the stream.
 */
int pa_probe_issue(int32_t mode, int32_t iterations, int32_t workgroups, int32_t* sink, void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* PA_PROBE_H_ */
