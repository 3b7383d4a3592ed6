/*
 * offload_adam_hip.h -- C ABI of liboffload_adam_hip.so (HIP, gfx950 / MI355X).
 *
 * The library is the MI355X-native replacement for the leaf callees of
 * tascj/offload_adam's optimizer hot path.  The reference has no FFI for its
 * kernels: its plug-in surface is the table of Python callables in
 * src/offload_adam/offload_adam.py:76-112 (OffloadAdam.supported_modes) and
 * src/offload_adam/adam.py:17-49 (Adam.configs), the per-format codec helpers
 * of the src/offload_adam/qweight/ modules and the ctypes binding of
 * src/offload_adam/pinned_alloc.py.  Every entry point below names the
 * reference callable it stands in for.
 *
 * Conventions (all entry points):
 *   - plain pointers and sizes only; the caller owns every buffer;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *     work is enqueued on it and the call returns without synchronising;
 *   - the kernels run on the calling thread's current HIP device;
 *   - return value: 0 on success, a positive hipError_t from the HIP runtime,
 *     or a negative OA_E* code for an argument the library rejects; nothing is
 *     launched when the return value is non-zero;
 *   - re-entrant, no global mutable state, never throws.
 *
 * Element types: "bf16" = bfloat16 stored as uint16_t, "f32" = IEEE binary32,
 * "i16" = int16_t.  Scalars are binary32 because the reference's Triton
 * kernels receive their Python floats as fp32 arguments.
 */
#ifndef OFFLOAD_ADAM_HIP_H
#define OFFLOAD_ADAM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OA_ABI_VERSION 1

/* negative = rejected by the library before any launch */
#define OA_EINVAL   (-1) /* null pointer, negative size, bad enum */
#define OA_EALIGN   (-2) /* pointer not aligned to its element type */
#define OA_ERANGE   (-3) /* size beyond what the entry point supports */
#define OA_EOVERLAP (-4) /* buffers that must be distinct alias each other */

/* ABI version of the loaded library (== OA_ABI_VERSION it was built with). */
int oa_abi_version(void);

/* Text for a return code of any entry point (OA_E* or hipError_t). Never NULL. */
const char* oa_error_string(int code);

/* ------------------------------------------------------------------------
 * A. Fused AdamW update -- one pass over HBM, one launch per parameter.
 *
 * Shared argument meaning (reference kernels take the same list, e.g.
 * src/offload_adam/kernels/fp32_master.py:19-33):
 *   n            number of elements of the flat, contiguous buffers
 *   lr, weight_decay, eps          fp32 hyper-parameters
 *   beta1_hat, beta2_hat           folded bias correction
 *                                  (beta^t - beta) / (beta^t - 1), computed by
 *                                  the caller in double and rounded to fp32
 *                                  (fp32_master.py:74-75)
 *   decoupled    non-zero: M -= (lr*wd)*M ; zero: g += wd*M   (fp32_master.py:46-49)
 *   clip_coef    NULL, or device pointer to ONE bf16 scalar c; the kernel then
 *                uses g' = bf16_rne(float(g) * float(c)) in place of g, which is
 *                what the reference's separate `grad.mul_(clip_coef)` pass
 *                (offload_adam.py:450-451, 464-465) leaves in the grad buffer.
 *                `grad` itself is never written.
 * The update (fp32, one rounding per operation, no FMA contraction):
 *   m += (1-beta1_hat)*(g-m); v += (1-beta2_hat)*(g*g-v);
 *   M -= (lr*m) / (sqrt(v)+eps)          sqrt and divide correctly rounded
 * m and v are stored back as bf16 (round-to-nearest-even).
 * ---------------------------------------------------------------------- */

/* Replaces adam_step_fp32_master (src/offload_adam/kernels/fp32_master.py:62-94)
 * without its trailing device-wide synchronize.
 *   param_out  bf16[n], write-only: bf16_rne(master)   (may alias `grad`; the
 *              reference passes the grad buffer as a sink for quantised
 *              params, offload_adam.py:427-431)
 *   master     f32[n], read-write */
int oa_adam_fp32_master(void* param_out, const void* grad, void* exp_avg,
                        void* exp_avg_sq, void* master, int64_t n, float lr,
                        float weight_decay, float beta1_hat, float beta2_hat,
                        float eps, int decoupled, const void* clip_coef,
                        void* stream);

/* Random-bit layouts of oa_adam_stochastic_rounding. */
#define OA_RNG_TRITON 0 /* element i uses the low 16 bits of word 0 of
                           Philox4x32-10(counter=(i_lo,i_hi,0,0), key=(seed_lo,seed_hi)):
                           the bits tl.randint(seed, offsets) & 0xFFFF gives in
                           stochastic_rounding.py:77 */
#define OA_RNG_X8     1 /* one Philox4x32-10 block per 8 consecutive elements:
                           counter=(j_lo,j_hi,1,0) with j=i/8, element i takes
                           16 bits: word (i%8)/2, low half if i even else high */
#define OA_RNG_BUFFER 2 /* element i uses rand16[i] (caller-supplied bits) */

/* Replaces adam_step_stochastic_rounding
 * (src/offload_adam/kernels/stochastic_rounding.py:82-116).
 *   param      bf16[n], read-write; written with the stochastic rounding of
 *              stochastic_rounding.py:25-34 (round the magnitude up iff r < low
 *              16 bits of the fp32 result)
 *   seed       64-bit seed (layouts TRITON and X8)
 *   rng        one of OA_RNG_*
 *   rand16     device uint16_t[n] when rng == OA_RNG_BUFFER, else ignored */
int oa_adam_stochastic_rounding(void* param, const void* grad, void* exp_avg,
                                void* exp_avg_sq, int64_t n, float lr,
                                float weight_decay, float beta1_hat,
                                float beta2_hat, float eps, int decoupled,
                                uint64_t seed, int rng, const void* rand16,
                                const void* clip_coef, void* stream);

/* Replaces adam_step_fp31_master (src/offload_adam/kernels/fp31_master.py:103-136).
 *   param           bf16[n], read-write
 *   rounding_error  i16[n], read-write; master bits = bits(float(param)) + (err<<1),
 *                   result rounded to 31 bits (ties to even on bit 0) and split
 *                   again (fp31_master.py:26-54) */
int oa_adam_fp31_master(void* param, const void* grad, void* exp_avg,
                        void* exp_avg_sq, void* rounding_error, int64_t n,
                        float lr, float weight_decay, float beta1_hat,
                        float beta2_hat, float eps, int decoupled,
                        const void* clip_coef, void* stream);

/* Replaces adam_step_fp32_master_custom_rounding
 * (src/offload_adam/kernels/fp32_master_custom_rounding.py:103-136).
 *   param = bf16 bits (master_bits + 0x8000) >> 16, rounding_error = the low
 *   16 bits of the difference as int16; the pair always reconstructs the full
 *   32-bit master (fp32_master_custom_rounding.py:33-54). */
int oa_adam_fp32_master_custom_rounding(void* param, const void* grad,
                                        void* exp_avg, void* exp_avg_sq,
                                        void* rounding_error, int64_t n,
                                        float lr, float weight_decay,
                                        float beta1_hat, float beta2_hat,
                                        float eps, int decoupled,
                                        const void* clip_coef, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* OFFLOAD_ADAM_HIP_H */
