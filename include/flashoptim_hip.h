/*
 * flashoptim_hip.h -- C ABI of libflashoptim_hip.so, the gfx950 (MI355X) implementation of FlashOptim's
 * fused optimizer-step hot path.
 *
 * Every entry point takes raw device pointers, sizes, fp32 scalars and a HIP stream (as void*); none takes
 * a torch type, allocates tensor memory or synchronises with the host.  All work is enqueued on `stream`
 * and mutates the caller's buffers in place, exactly as the reference's Triton launch wrappers do.
 * Return value: 0 on success, otherwise a negative FO_ERR_* code or a positive hipError_t; the text of the
 * last failure on the calling thread is available from fo_last_error().  Nothing throws across the ABI.
 *
 * "ref:" cites /root/reference/flashoptim/optimizers.py, the interface each symbol replaces.
 *
 * Layout contract shared by all entry points (ref:2476-2484, 1625-1646):
 *   - tensors are flat and contiguous; element i of the parameter pairs with element i of grad, ecc, codes;
 *   - a quantisation group is 32 consecutive elements counted from element 0 of the tensor; scales are
 *     fp16, one per group, ceil(n/32) entries; a short last group is scaled by its own absmax;
 *   - first-moment codes are int8 (softsign companding), second-moment codes uint8 (of sqrt(v));
 *   - ECC is int8 (24-bit master) or int16 (32-bit master), absent for fp32 parameters.
 */
#ifndef FLASHOPTIM_HIP_H
#define FLASHOPTIM_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* parameter / gradient element type (ref:60-64 _TORCH_DTYPE_TO_TRITON_DTYPE) */
enum fo_dtype { FO_F32 = 0, FO_BF16 = 1, FO_F16 = 2 };

enum fo_error {
    FO_OK = 0,
    FO_ERR_INVALID_ARGUMENT = -1, /* bad enum, null pointer, negative size, misaligned scale pointer ... */
    FO_ERR_UNSUPPORTED = -2,      /* e.g. ECC requested for an fp32 parameter */
    FO_ERR_NO_DEVICE = -3
};

/* Library / device identification. */
int fo_version(void);                    /* 100*major + minor */
const char *fo_last_error(void);         /* thread-local, never NULL */
int fo_device_compute_units(int device); /* multiprocessor count, <0 on error (ref:2976-2980 _get_sm_count) */

/*
 * Fused Adam / AdamW step on one tensor.  Replaces _fused_adam_step + _triton_adam_kernel
 * (ref:2203-2251, 2255-2438).
 *   mom, var        : quantized != 0 -> int8 / uint8 codes; else tensors of the parameter dtype
 *   mom_scales,
 *   var_scales      : fp16[ceil(n/32)] when quantized, ignored otherwise (may be NULL)
 *   param, grad     : `dtype` elements; grad is read only
 *   ecc             : int8 (ecc_bytes 1) / int16 (ecc_bytes 2) / NULL (ecc_bytes 0)
 *   weight_decay    : what the reference launcher passes: already multiplied by lr (or lr/initial_lr) for the
 *                     decoupled optimizers, the raw L2 coefficient otherwise (ref:1894-1898)
 *   step            : 1-based step count used for bias correction (ref:2368-2369)
 */
int fo_adam_step(void *mom, void *mom_scales, void *var, void *var_scales, void *param, const void *grad,
                 void *ecc, int64_t n, int dtype, int ecc_bytes, int quantized, float lr, float beta1,
                 float beta2, float eps, float weight_decay, int decoupled, int step, void *stream);

/*
 * Fused SGD / SGDW / Nesterov / Lion step on one tensor.  Replaces _fused_momentum_step +
 * _triton_momentum_kernel (ref:1535-1579, 1586-1719).  Lion: mom_coef = beta2, update_coef = beta1,
 * do_lion = 1 (ref:1313-1317); SGD: mom_coef = momentum, update_coef = 1 - dampening (ref:1432-1433).
 */
int fo_momentum_step(void *mom, void *mom_scales, void *param, const void *grad, void *ecc, int64_t n,
                     int dtype, int ecc_bytes, int quantized, float lr, float mom_coef, float update_coef,
                     float weight_decay, int decoupled, int nesterov, int do_lion, void *stream);

/*
 * Momentum-free SGD step (no state tensor).  Replaces the eager branch the reference takes when
 * momentum == 0 (ref:1447-1465): both decays are skipped when weight_decay == 0.
 */
int fo_sgd_plain_step(void *param, const void *grad, void *ecc, int64_t n, int dtype, int ecc_bytes, float lr,
                      float weight_decay, int decoupled, void *stream);

/*
 * Multi-tensor launch: one grid over many tensors of ragged sizes (no counterpart in the reference, which
 * launches once per tensor from FlashOptimizer.step, ref:770-785; results are bit-identical to calling the
 * single-tensor entry point on every tensor).
 *
 * `descs` is a DEVICE array of n_tensors descriptors; `chunks` is a DEVICE array of n_chunks work items
 * produced by fo_build_chunks (host) and copied by the caller.  All tensors of one call share dtype,
 * ecc_bytes, quantized and the scalar hyper-parameters (callers bucket by those).
 */
typedef struct fo_tensor_desc {
    void *param;
    const void *grad;
    void *ecc;        /* NULL when ecc_bytes == 0 */
    void *mom;        /* first-moment state (codes or plain values) */
    void *mom_scales; /* NULL when not quantized */
    void *var;        /* Adam only */
    void *var_scales; /* Adam only, NULL when not quantized */
    int64_t n;        /* elements in this tensor */
} fo_tensor_desc;

typedef struct fo_chunk {
    int32_t tensor;     /* index into descs */
    int32_t first_tile; /* first 4096-element tile of the tensor covered by this chunk */
    int32_t n_tiles;    /* tiles covered (>= 1) */
    int32_t reserved;
} fo_chunk;

#ifndef FO_TILE_ELEMS
#define FO_TILE_ELEMS 4096
#endif

/* Host helper: number of chunks fo_build_chunks will emit for these tensor lengths (0-length tensors emit
 * none).  tiles_per_chunk <= 0 selects the library default. */
int64_t fo_count_chunks(const int64_t *numels, int64_t n_tensors, int tiles_per_chunk);
/* Host helper: fills `out` (host memory, capacity >= fo_count_chunks) and returns the count, <0 on error. */
int64_t fo_build_chunks(const int64_t *numels, int64_t n_tensors, int tiles_per_chunk, fo_chunk *out,
                        int64_t capacity);

int fo_multi_adam_step(const fo_tensor_desc *descs, int64_t n_tensors, const fo_chunk *chunks, int64_t n_chunks,
                       int dtype, int ecc_bytes, int quantized, float lr, float beta1, float beta2, float eps,
                       float weight_decay, int decoupled, int step, void *stream);

int fo_multi_momentum_step(const fo_tensor_desc *descs, int64_t n_tensors, const fo_chunk *chunks,
                           int64_t n_chunks, int dtype, int ecc_bytes, int quantized, float lr, float mom_coef,
                           float update_coef, float weight_decay, int decoupled, int nesterov, int do_lion,
                           void *stream);

/*
 * fo_multi_adam_step for callers that cannot allocate device memory or copy tables to it (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * The caller passes the descriptors as a HOST array; the library keeps the descriptor and chunk tables in a static
 * device array of its own (FO_STATIC_MAX_TENSORS descriptors + FO_STATIC_MAX_CHUNKS chunk entries, 1.06 MiB per
 * device, held until the process ends), fills them with small kernels whose arguments carry the descriptors, and
 * launches the same step kernel.  It calls no hipMalloc / hipFree / hipMemcpy.  Lists with more than
 * FO_STATIC_MAX_TENSORS tensors are refused; lists with more than FO_STATIC_MAX_CHUNKS tiles are covered with
 * several 4096-element tiles per work item.  Results are bit-identical to fo_multi_adam_step.  All calls on one
 * device share the one array: calls that overlap in time on a device (different streams or threads) race.
 * The first call on a device, and the first call of each kernel variant (dtype, ecc_bytes, quantized, decoupled)
 * there, takes the array's address and plans the kernel's residency through host API calls that must not run while
 * the stream is capturing: make one eager call per variant before capturing.  After that a call enqueues kernel
 * launches only.  There is no `_exact` twin of this entry point: it runs what fo_multi_adam_step runs.
 */
#define FO_STATIC_MAX_TENSORS 1024
#define FO_STATIC_MAX_CHUNKS 65536
int fo_multi_adam_step_static(const fo_tensor_desc *host_descs, int64_t n_tensors, int dtype, int ecc_bytes,
                              int quantized, float lr, float beta1, float beta2, float eps, float weight_decay,
                              int decoupled, int step, void *stream);

/*
 * fo_adam_step / fo_multi_adam_step with the update evaluated operation by operation as the reference writes it,
 *     p -= (lr * (m / bc1)) / (sqrt(v / bc2) + eps)          (ref:2368-2375)
 * with correctly rounded quotients and roots, on every element and for every parameter dtype: every output bit
 * then equals an IEEE evaluation of the reference's formulas.
 * The plain entry points already do this wherever nothing else meets one unit of master precision: fp32
 * parameters, 2-byte parameters with a 2-byte ECC (32-bit masters), fp16 parameters with a 1-byte ECC.  For bf16
 * parameters with a 1-byte ECC (24-bit masters) and 2-byte parameters without ECC they fold the bias corrections
 * and the learning rate into two constants (one reciprocal per element) and redo operation by operation only the
 * elements whose update all but cancels the weight; moment codes and scales are then still bit-identical and
 * every master weight lies within one unit of master precision, but the correction code may differ by one step.
 * Same arguments and errors as the plain entry points.  The reference has one kernel and no such choice; these
 * are for callers who want every bit.
 */
int fo_adam_step_exact(void *mom, void *mom_scales, void *var, void *var_scales, void *param, const void *grad,
                       void *ecc, int64_t n, int dtype, int ecc_bytes, int quantized, float lr, float beta1,
                       float beta2, float eps, float weight_decay, int decoupled, int step, void *stream);
int fo_multi_adam_step_exact(const fo_tensor_desc *descs, int64_t n_tensors, const fo_chunk *chunks,
                             int64_t n_chunks, int dtype, int ecc_bytes, int quantized, float lr, float beta1,
                             float beta2, float eps, float weight_decay, int decoupled, int step, void *stream);

/* Momentum-free SGD over many tensors: the multi-tensor form of fo_sgd_plain_step (descs use param, grad, ecc, n). */
int fo_multi_sgd_plain_step(const fo_tensor_desc *descs, int64_t n_tensors, const fo_chunk *chunks,
                            int64_t n_chunks, int dtype, int ecc_bytes, float lr, float weight_decay,
                            int decoupled, void *stream);

/*
 * Largest magnitude of every tensor of a list in one launch.  Replaces the per-tensor
 * tensor.abs().max().item() behind check_numerics / recompute_param_stats (ref:656-673), which costs one device
 * synchronisation per tensor.  descs use `param` (the data, `dtype` elements) and `n`; `out` is fp32[n_tensors],
 * zeroed by the caller; out[i] receives max |x| of tensor i (NaN if it holds a NaN).  Chunks from
 * fo_build_chunks with any tiles_per_chunk (larger chunks mean fewer atomic merges).
 */
int fo_multi_absmax(const fo_tensor_desc *descs, int64_t n_tensors, const fo_chunk *chunks, int64_t n_chunks,
                    int dtype, float *out, void *stream);

/*
 * Standalone group codec.  Replaces quantize / dequantize and their kernels (ref:2446-2538, 2541-2676).
 *   x            : `x_dtype` elements
 *   codes        : int8 when is_signed, uint8 otherwise
 *   scales       : fp16[ceil(n/32)]
 */
int fo_quantize(const void *x, int x_dtype, void *codes, void *scales, int64_t n, int is_signed, int do_sqrt,
                int softsign, void *stream);
int fo_dequantize(const void *codes, const void *scales, float *out, int64_t n, int is_signed, int do_sqrt,
                  int softsign, void *stream);

/*
 * Standalone ECC.  fo_ecc_join replaces reconstruct_fp32_param (ref:2835-2892, kernel 2779-2803);
 * fo_ecc_split replaces compute_ecc_bits (ref:2895-2970, kernel 2806-2832).  narrow_dtype is FO_BF16 or
 * FO_F16; ecc_bytes is 1 or 2.
 */
int fo_ecc_join(const void *narrow, int narrow_dtype, const void *ecc, int ecc_bytes, float *out, int64_t n,
                void *stream);
int fo_ecc_split(const float *x, const void *narrow, int narrow_dtype, void *ecc, int ecc_bytes, int64_t n,
                 void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASHOPTIM_HIP_H */
