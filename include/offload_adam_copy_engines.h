/* liboffload_adam_copy_engines.so: an HSA tools library (loaded by the ROCr
 * runtime through HSA_TOOLS_LIB, before the first HIP call) that gives the
 * host->device and the device->host copies of the optimizer's pinned buffers
 * (of the whole process until a range is registered) one fixed SDMA engine each.  It has no counterpart in the reference, whose copies go
 * through torch's non_blocking copies on two CUDA streams
 * (src/offload_adam/offload_adam.py:346-358 and :362-372) and rely on the CUDA
 * driver's copy engines; on MI355X the HIP runtime's per-copy engine choice has
 * to be taken out of the picture to get a full-duplex host link.
 *
 * OnLoad / OnUnload are the entry points the ROCr runtime calls (tools
 * interface of hsa_api_trace.h).  The functions below only report state; they
 * may be called at any time, from any thread, by whoever dlopen()s the same
 * file.
 *
 * Environment, read once when the runtime loads the library:
 *   OFFLOAD_ADAM_COPY_ENGINES="<h2d mask>,<d2h mask>"  one bit each, values of
 *       hsa_amd_sdma_engine_id_t; default "0x1,0x2" (SDMA engines 0 and 1)
 *   OFFLOAD_ADAM_COPY_ENGINES=off                      rewrite nothing
 */
#ifndef OFFLOAD_ADAM_COPY_ENGINES_H
#define OFFLOAD_ADAM_COPY_ENGINES_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 1 once the ROCr runtime has called OnLoad in this process, else 0. */
int oa_copy_engines_loaded(void);

/* 1 while copies are being rewritten; 0 when switched off by configuration or
 * after eight rewritten calls in a row were rejected by the runtime. */
int oa_copy_engines_active(void);

/* The engine masks in use (hsa_amd_sdma_engine_id_t values). */
void oa_copy_engines_config(unsigned* h2d_mask, unsigned* d2h_mask);

/* Copies issued on the fixed engines so far, per direction, and rewritten
 * calls the runtime rejected (each of those was re-issued unchanged). */
void oa_copy_engines_stats(unsigned long long* h2d_copies, unsigned long long* d2h_copies,
                           unsigned long long* rejected);

/* Host<->device copies that reached the runtime through the call that names no
 * engine (hsa_amd_memory_async_copy) and were sent to the fixed engines as well;
 * they are included in the per-direction counts above. */
unsigned long long oa_copy_engines_unpinned_calls(void);

/* Scope of the rewrite.  Until the first registration every pinned host<->device
 * copy of the process is rewritten; from then on only copies whose host side
 * lies inside a registered range [base, base + bytes) are, and all others keep
 * the engine the HIP runtime chose.  The package's pinned allocator registers
 * what it hands out and unregisters it on release.  Both return 0, or -1 for a
 * null / empty range or a base that was never registered.  Thread-safe. */
int oa_copy_engines_register_range(const void* base, size_t bytes);
int oa_copy_engines_unregister_range(const void* base);

/* 1 once a range has been registered in this process (the rewrite is limited
 * to registered ranges), else 0. */
int oa_copy_engines_scoped(void);

/* Host<->device copies left to the runtime because their host side was outside
 * every registered range. */
unsigned long long oa_copy_engines_passed_by(void);

#ifdef __cplusplus
}
#endif

#endif /* OFFLOAD_ADAM_COPY_ENGINES_H */
