/*
 * flashoptim_hip_diag.h -- measurement and diagnostic entry points.
 *
 * Nothing here is part of the optimizer path and none of it has a counterpart in the reference
 * (/root/reference/flashoptim/optimizers.py): the symbols exist for the benchmark and the tests.  They are exported by
 * the diagnostics build of the library only (libflashoptim_hip_diag.so: the product's sources compiled with
 * -DFO_DIAG, so it also exports everything in flashoptim_hip.h and its step kernels are the product's, from the same
 * text with the same flags); libflashoptim_hip.so holds product kernels only.
 */
#ifndef FLASHOPTIM_HIP_DIAG_H
#define FLASHOPTIM_HIP_DIAG_H

#include <stdint.h>

#include "flashoptim_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * A plain device-to-device copy kernel (128-bit loads and stores, same launch geometry and store policy as the
 * step kernels) used to calibrate hardware byte counters and to show the attainable HBM rate next to the step
 * kernels.  n_bytes must be a multiple of 16 and both pointers 16-byte aligned.
 */
int fo_copy_bytes(void *dst, const void *src, int64_t n_bytes, void *stream);

/*
 * The Adam step's memory accesses without its arithmetic: every tensor of the table is read (parameters, gradients,
 * ECC, both moments and their group scales) and written back unchanged (everything but the gradients) by the step
 * kernels' own load / store code, launch geometry and residency mechanism.  Arguments as fo_multi_adam_step's
 * (flashoptim_hip.h) without the scalars.  The rate it reaches is the ceiling of the step's access mix on the
 * device, to be read next to the step's own rate and to fo_copy_bytes' (one load and one store stream).
 */
int fo_multi_adam_streams_copy(const fo_tensor_desc *descs, int64_t n_tensors, const fo_chunk *chunks, int64_t n_chunks,
                               int dtype, int ecc_bytes, int quantized, void *stream);
/* The same for the momentum kernels' streams (parameters, gradients, ECC, one moment's codes and scales). */
int fo_multi_momentum_streams_copy(const fo_tensor_desc *descs, int64_t n_tensors, const fo_chunk *chunks,
                                   int64_t n_chunks, int dtype, int ecc_bytes, int quantized, void *stream);

/*
 * Residency plan of a step kernel on the current device: the workgroups per compute unit the kernel family asks
 * for (`target`), what the dynamic LDS request that enforces it, the runtime's occupancy query and the kernel's cap
 * of wavefronts per SIMD allow together (`achieved`) and that request in bytes (`dynamic_lds`).  Any output pointer
 * may be NULL.
 *   multi: 0 = the single-tensor kernel, 1 = the multi-tensor kernel, 2 = the multi-tensor kernel launched over a list
 *          of many short tensors (the momentum kernels keep more wavefronts resident there).
 *   kind (momentum): 0 = SGD / SGDW / Nesterov, 1 = Lion, 2 = momentum-free SGD.
 */
int fo_adam_step_residency(int dtype, int ecc_bytes, int quantized, int decoupled, int multi, int *target,
                           int *achieved, int *dynamic_lds);
int fo_momentum_step_residency(int dtype, int ecc_bytes, int quantized, int kind, int multi, int *target,
                               int *achieved, int *dynamic_lds);

/*
 * Measures how many one-wavefront workgroups that request `dynamic_lds_bytes` of LDS a compute unit really holds at
 * once: a probe kernel whose workgroups register on their compute unit (named by the hardware id registers), linger
 * for 20 us and sign off; `most_resident` receives the largest count any unit reached.  The step kernels bound their
 * residency through such requests (fo_adam_step_residency above reports the plan); this shows what the device makes
 * of a request, independent of the runtime's occupancy query and of the allocation unit the plan assumes.
 * `counters`: 32 KiB of device memory (scratch).  Synchronises the stream.
 */
int fo_probe_residency(int dynamic_lds_bytes, void *counters, int64_t counters_bytes, int *most_resident, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASHOPTIM_HIP_DIAG_H */
