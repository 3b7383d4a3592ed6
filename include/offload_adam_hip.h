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
 *   - re-entrant and never throws; no global mutable state, with two exceptions:
 *     oa_grad_norm_bf16_static keeps its partial sums in a device array inside
 *     the library (one per GPU) and caches that array's address per device, and
 *     oa_h2d_async / oa_d2h_async keep a ring of signals per GPU.
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
#define OA_EOS      (-5) /* an operating-system call failed; errno is reported
                            through the entry point's os_errno argument */
#define OA_EUNAVAILABLE (-6) /* oa_h2d_async / oa_d2h_async: fixed-engine copies cannot be
                                set up on this GPU; oa_link_copy_status says why */
#define OA_ELINKTIMEOUT (-7) /* a fixed-engine copy issued earlier had not completed after
                                about a minute: its stream went on without it */

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
 *              params, offload_adam.py:427-431).  NULL: no bf16 copy is written
 *              (18 instead of 20 bytes per element), for callers that re-encode
 *              the parameter from `master` anyway.
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

/* Multi-tensor form of the four step functions: what a loop over parameters
 * such as Adam.step (src/offload_adam/adam.py:111-152) or the in-place branch
 * of OffloadAdam.step (src/offload_adam/offload_adam.py:563-571) does with one
 * step_fn call per parameter, done with one launch per 36 parameters (tensor
 * descriptors travel as kernel arguments; nothing is allocated).
 *   mode        OA_MODE_*
 *   count       number of parameters; every array below has `count` entries
 *   params, grads, exp_avgs, exp_avg_sqs   device pointers, as in the
 *               single-tensor entry points (for OA_MODE_FP32_MASTER params[i] is
 *               the write-only bf16 sink and may equal grads[i])
 *   aux         f32 masters (FP32_MASTER) or i16 rounding errors (FP31, CUSTOM);
 *               ignored (may be NULL) for STOCHASTIC_ROUNDING
 *   numels      element counts
 *   beta1_hats, beta2_hats   per parameter (their step counts may differ)
 *   seeds       per parameter, STOCHASTIC_ROUNDING only (else may be NULL)
 *   rng         OA_RNG_TRITON or OA_RNG_X8 (STOCHASTIC_ROUNDING only)
 * Every argument is validated before the first launch.  Results are identical
 * to `count` single-tensor calls. */
#define OA_MODE_FP32_MASTER         0
#define OA_MODE_STOCHASTIC_ROUNDING 1
#define OA_MODE_FP31_MASTER         2
#define OA_MODE_CUSTOM_ROUNDING     3
int oa_adam_multi(int mode, int count, void* const* params, const void* const* grads,
                  void* const* exp_avgs, void* const* exp_avg_sqs, void* const* aux,
                  const int64_t* numels, const float* beta1_hats,
                  const float* beta2_hats, const uint64_t* seeds, float lr,
                  float weight_decay, float eps, int decoupled, int rng,
                  const void* clip_coef, void* stream);

/* ------------------------------------------------------------------------
 * B. Gradient L2 norm per parameter and the global clip coefficient.
 * ---------------------------------------------------------------------- */

/* Bytes of device scratch oa_grad_norm_bf16 and oa_quant_nvfp4 need (per-block
 * partial results between their two launches).  The caller allocates it
 * (64-byte aligned) and may reuse it for every later call on the same stream;
 * its contents need no initialisation.  Launches that may overlap (different
 * streams) need separate workspaces. */
size_t oa_norm_workspace_bytes(void);

/* Replaces `torch.norm(grad, 2.0)` on the accumulated bf16 gradient
 * (src/offload_adam/offload_adam.py:504-505, 531-532).
 *   grad       bf16[n], any 2-byte alignment
 *   norm_out   ONE bf16: bf16_rne(sqrt(sum g^2)), fp32 accumulation in a fixed
 *              order (bit-reproducible run to run)
 *   sumsq_out  NULL or ONE f32 receiving the unrounded sum of squares */
int oa_grad_norm_bf16(const void* grad, int64_t n, void* norm_out, void* sumsq_out,
                      void* workspace, void* stream);

/* oa_grad_norm_bf16 for callers that cannot allocate device memory or pass a
 * workspace: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  No counterpart in the reference.  The partial sums live in
 * a device array inside the library (OA_NORM_STATIC_PARTIALS floats = 64 KiB per
 * GPU the library runs on, held until the process ends); the call allocates and
 * frees nothing.  Same kernels and same results, bit for bit, as
 * oa_grad_norm_bf16.  n > OA_NORM_STATIC_MAX_ELEMS returns OA_ERANGE and
 * launches nothing.  All calls on one GPU share that GPU's array: calls that
 * may overlap on one GPU (different streams, several threads) race on it -
 * serialise them, or use oa_grad_norm_bf16 with one workspace per stream.  The
 * first call on a GPU looks the array's address up (hipGetSymbolAddress): make
 * that call outside graph capture. */
#define OA_NORM_STATIC_PARTIALS  16384
#define OA_NORM_STATIC_MAX_ELEMS ((int64_t)1 << 31)  /* a 4 GiB bf16 gradient */
int oa_grad_norm_bf16_static(const void* grad, int64_t n, void* norm_out,
                             void* sumsq_out, void* stream);

/* Per-parameter norms of a whole list of gradients: what the loop of
 * `torch.norm(grad, 2.0)` calls over the parameters amounts to on the last
 * micro-batch (src/offload_adam/offload_adam.py:504-505, 531-532, read back by
 * step() at :553-561), done with two launches per 36 gradients instead of one or
 * two per gradient (tensor descriptors travel as kernel arguments).
 *   count       number of gradients; every array below has `count` entries
 *   grads       device pointers to bf16 gradients, any 2-byte alignment
 *   numels      element counts (0 gives a norm of 0)
 *   norm_outs   device pointers, ONE bf16 each (e.g. the slots of one buffer)
 *   sumsq_outs  NULL, or device pointers to ONE f32 each (entries may be NULL)
 *   workspace   device scratch for the partial sums, 64-byte aligned,
 *               `workspace_bytes` long: at least oa_norm_workspace_bytes();
 *               oa_norm_multi_workspace_bytes() lets every launch take its 36
 *               gradients whatever their sizes.  Contents need no initialisation;
 *               launches that may overlap need separate workspaces.
 * Every argument is validated before the first launch.  Results are identical,
 * bit for bit, to `count` calls of oa_grad_norm_bf16. */
size_t oa_norm_multi_workspace_bytes(void);
int oa_grad_norm_multi(int count, const void* const* grads, const int64_t* numels,
                       void* const* norm_outs, void* const* sumsq_outs, void* workspace,
                       size_t workspace_bytes, void* stream);

/* Replaces the global-norm and clip-coefficient arithmetic of
 * OffloadAdam.step (src/offload_adam/offload_adam.py:553-561):
 *   total = vector_norm(stack(norms), 2)                        (bf16)
 *   coef  = clamp(max_norm / (total + 1e-6), max=1.0)           (bf16)
 * with torch's evaluation of `float / tensor` as reciprocal()*float, every
 * step rounded to bf16 like the 0-dim bf16 tensor ops do.  No host sync.
 *   norms      bf16[count] (the per-parameter norms, contiguous)
 *   total_out  NULL or ONE bf16;  coef_out  ONE bf16 */
int oa_clip_coef_bf16(const void* norms, int64_t count, float max_norm,
                      void* total_out, void* coef_out, void* stream);

/* ------------------------------------------------------------------------
 * C. Weight-only quantisation codecs for (rows = out_features, cols =
 *    in_features) matrices.  `src`/`out` are row-major with unit column stride
 *    and a row stride given in ELEMENTS; packed payloads are contiguous.
 *    Element types of float operands: */
#define OA_F32  0
#define OA_BF16 1
#define OA_F16  2
/*    Quantise entry points read the source once per output (the amax passes
 *    hit the same data again through L2 / registers) and write straight into
 *    the payload buffers of the quantised weight.  Results are bit-identical
 *    to the reference's pure-torch functions named at each entry point. */

/* int8, per-row symmetric.  Replaces _quantize_int8_triton
 * (src/offload_adam/qweight/int8.py:202-232; spec: quantize_int8_per_channel,
 * int8.py:30-49).  q: int8[rows*cols]; scales: [rows] of scale_dtype
 * (scale = absmax/127 rounded to scale_dtype; the codes use the fp32 scale). */
int oa_quant_int8(const void* src, int src_dtype, int64_t src_row_stride,
                  int64_t rows, int64_t cols, void* q, void* scales,
                  int scale_dtype, void* stream);

/* Replaces _dequant_int8_triton (int8.py:107-126; spec:
 * dequantize_int8_per_channel, int8.py:52-57): out = round(q * scale) in
 * out_dtype, with the stored scale widened from scale_dtype. */
int oa_dequant_int8(const void* q, const void* scales, int scale_dtype,
                    int64_t rows, int64_t cols, void* out, int out_dtype,
                    int64_t out_row_stride, void* stream);

/* int4, symmetric, groups of `group` columns, GPTQ storage.  Replaces
 * _quantize_pack_int4_triton (src/offload_adam/qweight/int4.py:258-296; spec:
 * quantize_int4_groupwise + pack_int4_gptq, int4.py:30-48, 61-92).
 * qweight: int32[(cols/8) * rows], word (k, r) packs columns 8k..8k+7 of row r
 * LSB first as (code + 8); scales: [(cols/group) * rows] of scale_dtype.
 * cols % group == 0, group % 8 == 0. */
int oa_quant_int4(const void* src, int src_dtype, int64_t src_row_stride,
                  int64_t rows, int64_t cols, int64_t group, void* qweight,
                  void* scales, int scale_dtype, void* stream);

/* Replaces _dequant_int4_triton (int4.py:155-183). */
int oa_dequant_int4(const void* qweight, const void* scales, int scale_dtype,
                    int64_t rows, int64_t cols, int64_t group, void* out,
                    int out_dtype, int64_t out_row_stride, void* stream);

/* NF4, blocks of `block` columns, bitsandbytes storage.  Replaces
 * _quantize_nf4_triton (src/offload_adam/qweight/nf4.py:334-372; spec:
 * quantize_nf4_blockwise + pack_nf4, nf4.py:74-83, 102-135).
 * packed: uint8[rows * cols/2], even column in the HIGH nibble;
 * absmax: f32[rows * cols/block].  cols % block == 0, block % 2 == 0. */
int oa_quant_nf4(const void* src, int src_dtype, int64_t src_row_stride,
                 int64_t rows, int64_t cols, int64_t block, void* packed,
                 void* absmax, void* stream);

/* Replaces _dequant_nf4_triton (nf4.py:230-260): fp32 codebook value times
 * fp32 absmax, rounded once to out_dtype. */
int oa_dequant_nf4(const void* packed, const void* absmax, int64_t rows,
                   int64_t cols, int64_t block, void* out, int out_dtype,
                   int64_t out_row_stride, void* stream);

/* NVFP4: e2m1 codes in blocks of 16 with float8_e4m3fn block scales and one
 * fp32 tensor scale.  Replaces _quantize_nvfp4_triton
 * (src/offload_adam/qweight/nvfp4.py:660-732; spec: quantize_nvfp4_blockwise +
 * pack_fp4, nvfp4.py:72-81, 133-173).  Three launches: per-block amax, global
 * scale, encode.
 *   packed        uint8[rows * cols/2], even column in the LOW nibble
 *   block_scale   uint8[rows * cols/16], float8_e4m3fn bit patterns
 *   global_scale  ONE f32 (device), written: max(amax,1e-12) / (448*6)
 *   workspace     as for oa_grad_norm_bf16 (oa_norm_workspace_bytes() bytes)
 * cols % 16 == 0. */
int oa_quant_nvfp4(const void* src, int src_dtype, int64_t src_row_stride,
                   int64_t rows, int64_t cols, void* packed, void* block_scale,
                   void* global_scale, void* workspace, void* stream);

/* Replaces _dequant_nvfp4_triton (nvfp4.py:411-461, soft path): e2m1 value
 * times (e4m3 scale * global scale) in fp32, rounded once to out_dtype. */
int oa_dequant_nvfp4(const void* packed, const void* block_scale,
                     const void* global_scale, int64_t rows, int64_t cols,
                     void* out, int out_dtype, int64_t out_row_stride,
                     void* stream);

/* fp32_master AdamW step and re-encoding of a quantised weight in one pass.
 * Replaces, for a quantised parameter, the pair the reference runs per step:
 * adam_step_fp32_master with the gradient buffer as a dummy bf16 sink
 * (src/offload_adam/offload_adam.py:427-442, src/offload_adam/adam.py:139-149)
 * followed by `p.data.copy_(master)` -> _quantize_*_triton
 * (offload_adam.py:443-444; int8.py:430-442, int4.py:499-515, nf4.py:604-616,
 * nvfp4.py:952-966).  The encoder's read of each element is the AdamW update of
 * that element: grad/exp_avg/exp_avg_sq (bf16) and master (f32), all
 * [rows*cols] contiguous, are updated exactly as oa_adam_fp32_master does
 * (clip_coef as there; no bf16 copy of the master is written) and the payload is
 * written exactly as oa_quant_* would write it from the new master.
 * 18 + payload bytes per element instead of 20 + 4 + payload.
 * Requirements (else OA_EINVAL / OA_EALIGN, and the caller runs the two calls
 * separately): cols % 8 == 0, 16-byte aligned arrays; int4: group a power of two
 * <= 512; nf4: block/8 a power of two, block <= 512; nvfp4: cols % 16 == 0
 * (three launches: step + per-block amax, global scale, encode from master). */
int oa_adam_requant_int8(const void* grad, void* exp_avg, void* exp_avg_sq,
                         void* master, int64_t rows, int64_t cols, float lr,
                         float weight_decay, float beta1_hat, float beta2_hat,
                         float eps, int decoupled, const void* clip_coef, void* q,
                         void* scales, int scale_dtype, void* stream);
int oa_adam_requant_int4(const void* grad, void* exp_avg, void* exp_avg_sq,
                         void* master, int64_t rows, int64_t cols, float lr,
                         float weight_decay, float beta1_hat, float beta2_hat,
                         float eps, int decoupled, const void* clip_coef,
                         int64_t group, void* qweight, void* scales,
                         int scale_dtype, void* stream);
int oa_adam_requant_nf4(const void* grad, void* exp_avg, void* exp_avg_sq,
                        void* master, int64_t rows, int64_t cols, float lr,
                        float weight_decay, float beta1_hat, float beta2_hat,
                        float eps, int decoupled, const void* clip_coef,
                        int64_t block, void* packed, void* absmax, void* stream);
int oa_adam_requant_nvfp4(const void* grad, void* exp_avg, void* exp_avg_sq,
                          void* master, int64_t rows, int64_t cols, float lr,
                          float weight_decay, float beta1_hat, float beta2_hat,
                          float eps, int decoupled, const void* clip_coef,
                          void* packed, void* block_scale, void* global_scale,
                          void* workspace, void* stream);

/* ------------------------------------------------------------------------
 * D. Pinned host memory and host<->device streaming.
 * ---------------------------------------------------------------------- */

/* Replaces the mmap / mbind / memset / cudaHostRegister sequence of
 * pinned_alloc._alloc (src/offload_adam/pinned_alloc.py:177-235).
 * Allocates `bytes` rounded up to 4 KiB pages of zero-filled, page-locked host
 * memory.  numa_node >= 0 prefers that node softly (MPOL_PREFERRED: spills to
 * other nodes when it is full); -1 leaves placement to the HIP runtime.
 * Returns 0 and the address in *out; OA_EOS with the OS errno in *os_errno
 * when the memory-policy call fails; a positive hipError_t when the runtime
 * cannot allocate or pin. */
int oa_pinned_alloc(size_t bytes, int numa_node, void** out, int* os_errno);

/* Releases memory obtained from oa_pinned_alloc (the cleanup closure of
 * pinned_alloc.py:222-232). */
int oa_pinned_free(void* ptr);

/* Pre-flight of a large request (the reference discovers a refusal only inside
 * pinned_alloc._alloc, src/offload_adam/pinned_alloc.py:204-221, one mapping at a
 * time): 0 when the runtime would grant `bytes` of page-locked memory right now,
 * else the hipError_t it gives.  The block is released before returning and is
 * never written, so the call costs no page faults and no zero-fill. */
int oa_pinned_probe(size_t bytes);

/* Replaces pinned_alloc.gpu_numa_node (src/offload_adam/pinned_alloc.py:113-128):
 * NUMA node of the PCI device behind HIP device `device`, -1 when the kernel
 * reports none. */
int oa_gpu_numa_node(int device, int* node_out);

/* Asynchronous copy on `stream`; stands in for the `Tensor.to(non_blocking)` /
 * `copy_(non_blocking)` calls of OffloadAdam._issue_h2d / _issue_d2h
 * (src/offload_adam/offload_adam.py:347-372).  The host side must be
 * page-locked for the copy to be asynchronous.  Ordering against other streams
 * is the caller's job (events). */
#define OA_COPY_H2D 0
#define OA_COPY_D2H 1
#define OA_COPY_D2D 2
int oa_memcpy_async(void* dst, const void* src, size_t bytes, int kind, void* stream);

/* Host<->device copy of `bytes` on `stream`, on a fixed SDMA engine per direction.
 * Stands in for the same calls as oa_memcpy_async (`host.to(device,
 * non_blocking=True)` in OffloadAdam._issue_h2d, `host.copy_(dev, non_blocking=True)`
 * in _issue_d2h, src/offload_adam/offload_adam.py:347-372) with the semantics of
 * hipMemcpyAsync on `stream`: the copy starts after the work the stream was given
 * before, work given afterwards starts after the copy.  What differs is who picks
 * the SDMA engine: hipMemcpyAsync leaves it to the HIP runtime per copy (a saturated
 * stream walks up to engines that run at a fifth of the link's rate, or onto the
 * other direction's engine); here host->device copies always use one engine and
 * device->host copies another (engines 0 and 1; OFFLOAD_ADAM_COPY_ENGINES="<h2d
 * mask>,<d2h mask>" picks others, "off" disables the entry points).  The copy is
 * handed to the ROCr runtime directly and fenced inside the stream by two one-lane
 * kernels (one releases the copy when the stream reaches it, one holds the stream
 * until the engine has finished), so nothing depends on the process environment or
 * on when the library was loaded, and profilers that trace HSA copies see it.
 *   dst, src       one of them page-locked host memory, the other device memory
 *   wait_event     NULL, or a hipEvent_t the stream waits for before the copy
 *   record_event   NULL, or a hipEvent_t recorded on the stream after the copy
 * Returns OA_EUNAVAILABLE, having enqueued nothing, when the GPU or the runtime
 * lacks what this needs (the caller then uses oa_memcpy_async); a positive
 * hipError_t when a HIP call fails.  Holds per-GPU state inside the library (a ring
 * of 1024 signal pairs, set up at the first call on a GPU); safe to call from
 * several threads; at most 1024 copies may be outstanding per GPU before a call
 * waits for the oldest.  Not for use under stream capture. */
int oa_h2d_async(void* dst, const void* src, size_t bytes, void* stream, void* wait_event,
                 void* record_event);
int oa_d2h_async(void* dst, const void* src, size_t bytes, void* stream, void* wait_event,
                 void* record_event);

/* `count` copies of one direction (kind = OA_COPY_H2D or OA_COPY_D2H) as one unit in
 * the order of `stream` - what the loops over a parameter's states in
 * OffloadAdam._issue_h2d / _issue_d2h (src/offload_adam/offload_adam.py:352-357,
 * 366-371) amount to.  All of them start after the work the stream was given before
 * the call; they run back to back on the direction's engine, without the stream
 * coming round between two of them; the stream observes the completions in order
 * and records record_events[i] (NULL array, or NULL entries, for none) behind copy
 * i; work given to the stream after the call starts after the last copy.  Same
 * availability, state and limits as oa_h2d_async. */
int oa_link_copy_batch(int count, void* const* dsts, const void* const* srcs,
                       const size_t* bytes, int kind, void* stream,
                       void* const* record_events);

/* State of the fixed-engine copies on the current GPU (sets them up if no copy has
 * yet): 0 = in effect, else the reason they are not.  Any out pointer may be NULL:
 * the engine masks in use, the copies issued per direction, and the copies the ROCr
 * runtime declined, which went through hipMemcpyAsync instead. */
#define OA_LINK_OFF                 (-10) /* OFFLOAD_ADAM_COPY_ENGINES=off */
#define OA_LINK_NO_RUNTIME          (-11) /* libhsa-runtime64 or one of its entry points not found */
#define OA_LINK_NO_AGENT            (-13) /* the HIP device was not found among the HSA agents */
#define OA_LINK_NO_SIGNALS          (-14) /* signal memory (hipMallocSignalMemory) could not be obtained or verified */
int oa_link_copy_status(unsigned* h2d_engine, unsigned* d2h_engine,
                        unsigned long long* h2d_copies, unsigned long long* d2h_copies,
                        unsigned long long* runtime_copies);

/* Bound of the stream-side waits issued from now on on the current GPU, in polls of
 * about 3 us each (0 = the default, about a minute; at most 2^32 - 1), and the way
 * out of a timeout.  A wait that reaches its bound lets its stream go on with the
 * copy still outstanding and marks the GPU's link: every later copy call returns
 * OA_ELINKTIMEOUT, as does this call (after applying `max_polls`).  With
 * `clear_timeout` non-zero the mark is taken off: only for a caller that has made
 * sure, by its own means, that no copy is outstanding any more (the data of the copies
 * issued since the timeout must be taken as undefined).  No counterpart in the
 * reference (hipMemcpyAsync has no such bound). */
int oa_link_wait_limit(unsigned long long max_polls, int clear_timeout);

/* The same copy done by a small grid-stride kernel (`workgroups` blocks of 1024
 * lanes, 128-bit accesses, 4 loads in flight per lane; 8 blocks fill a PCIe
 * Gen5 x16 link) instead of the DMA engine.  Either pointer may be
 * page-locked host memory from oa_pinned_alloc: the lanes read or write it
 * across the host link.  Used for one direction of the streaming path so that
 * H2D (DMA engine) and D2H (this kernel) never queue behind each other on one
 * engine.  Both pointers must be 16-byte aligned.  No counterpart in the
 * reference (its copies all go through `Tensor.to` / `copy_`,
 * src/offload_adam/offload_adam.py:347-372). */
int oa_copy_kernel_async(void* dst, const void* src, size_t bytes, int workgroups,
                         void* stream);

#ifdef __cplusplus
}
#endif
#endif /* OFFLOAD_ADAM_HIP_H */
