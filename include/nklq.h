/*
 * nklq.h — C-ABI of the MI355X (gfx950) 2-bit gradient quantizer.
 *
 * This is the boundary a binding of necklace's quantizer would load
 * (dlopen / ctypes / cgo / JNI): plain pointers and sizes, no torch or numba
 * types.  Every pointer marked "device" must be memory the current HIP device
 * can address; `stream` is a hipStream_t passed as an opaque pointer (NULL =
 * the device's default stream).  All entry points are asynchronous on
 * `stream`, allocate no device memory and keep no state between calls other
 * than the nklq_tune knobs.  They may be called from several host threads at
 * once, also while another thread changes a knob: the knobs are atomics and a
 * call works from the one snapshot it takes on entry.  The int return value
 * of a launch is that launch's own status, not the runtime's sticky
 * "last error".
 *
 * Bit layout (necklace/cuda/quantize.py:8-13, :34-51): codes are 2 bits,
 * 01 = value >= t, 10 = value <= -t, 00 = in between, 16 codes per 32-bit
 * word, the code of row 16*x + i of column y sits in bits [2i+1 : 2i] of
 * word (x, y); bits of rows past the end are 0.  A flat vector of N elements
 * is the matrix (N, 1): word w holds elements 16w .. 16w+15.
 *
 * Return value of the int entry points: 0 = success, < 0 = one of the
 * NKLQ_E* argument errors below, > 0 = a hipError_t from the launch.
 */
#ifndef NKLQ_H
#define NKLQ_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NKLQ_VERSION 100          /* 1.0.0 */
#define NKLQ_CODES_PER_WORD 16    /* CMP_RATIO, necklace/cuda/quantize.py:8 */
#define NKLQ_MAX_PAYLOADS_PER_LAUNCH 16

#define NKLQ_OK 0
#define NKLQ_ENULL (-1)   /* a required pointer is NULL */
#define NKLQ_EALIGN (-2)  /* a pointer is not 4-byte aligned */
#define NKLQ_ERANGE (-3)  /* a size or count is out of range */
#define NKLQ_EALIAS (-4)  /* the byte range of an output overlaps another buffer of the call; only an
                             output that coincides exactly with an input (r_out == r_in, r_out == g)
                             is allowed.  Checked over the full extents, across all vectors of the
                             *_multi_* calls, before anything is launched */

/*
 * Threshold-quantize an fp32 matrix to 2-bit codes and write the residual.
 * Replaces the kernel cu_knl_matrix_quantize_e (necklace/cuda/quantize.py:16-51)
 * and its launch wrapper cu_fn_matrix_quantize_e (:96-115).
 *
 *   g      device, fp32 [n_rows, n_cols] row-major and contiguous (row i starts
 *          n_cols floats after row i-1: there is no leading dimension): the
 *          matrix A of the reference
 *   r_in   device, fp32 same shape: residual carried from the previous step;
 *          read only when add_residual != 0 (may be NULL otherwise)
 *   r_out  device, fp32 same shape: the matrix R of the reference (every
 *          element is written).  May be the same pointer as r_in (in-place
 *          error feedback) or as g; any other overlap returns NKLQ_EALIAS.
 *          (A matrix whose rows do not start on 128-byte lines is fastest
 *          when r_out overlaps neither input: the kernel can then write
 *          whole lines.)
 *   c      device, uint32 [ceil(n_rows/16), n_cols] row-major: the matrix C
 *          (every word is overwritten, whatever it held)
 *   thrd   the threshold; it crosses as C float, i.e. rounded to fp32 exactly
 *          like the jit signature '(..., float32)' at quantize.py:16 does
 *   add_residual  0: a = g (the reference kernel as is)
 *                 1: a = fl32(g + r_in) (error-feedback step), then as above
 *
 * Per element: a >= t -> code 01, r_out = fl32(a - t); else a <= -t -> code 10,
 * r_out = fl32(a + t); else code 00, r_out = a (same bits).  NaN takes the
 * last branch.  The column guard is y < n_cols (the reference tests y against
 * n_rows, quantize.py:29-31, which is the same thing on the square inputs it
 * is defined for).  n_rows == 0 or n_cols == 0 is a successful no-op.
 */
int nklq_quantize_f32(const float* g, const float* r_in, float* r_out, uint32_t* c,
                      uint64_t n_rows, uint64_t n_cols, float thrd, int add_residual,
                      void* stream);

/*
 * Unpack 2-bit codes to {+t, -t, 0.0f}, overwriting `out`.
 * Replaces cu_knl_matrix_dequantize_e (necklace/cuda/quantize.py:56-87) and
 * cu_fn_matrix_dequantize_e (:118-134).  Code 11 decodes to +0.0f (the
 * reference's `else` branch, :86-87); bits of rows >= n_rows are never used.
 * The reference's third argument R is unused by its kernel and has no
 * counterpart here.
 *
 *   out  device, fp32 [n_rows, n_cols]     c  device, uint32 [ceil(n_rows/16), n_cols]
 */
int nklq_dequantize_f32(float* out, const uint32_t* c, uint64_t n_rows, uint64_t n_cols,
                        float thrd, void* stream);

/*
 * Receive side: unpack k_payloads flat code vectors and sum them, in payload
 * order, into one fp32 vector:
 *     s = accumulate ? acc[j] : +0.0f;
 *     for p = 0 .. k_payloads-1:  s = fl32(s + decode(payloads[p], j));
 *     acc[j] = s;
 * The order is part of the contract (fp32 sums of {0, +t, -t} depend on it).
 * This is the "decompress and sum over workers" step that necklace's trainer
 * hands to mxprms.grads_do_nccl(..., grad_comp_cfg=...) (call site
 * necklace/trainer/tnopmx.py:334-337; that module is not in the reference
 * tree), built on the decode of quantize.py:80-87.
 *
 *   acc       device, fp32 [n]
 *   payloads  HOST array of k_payloads device pointers, each uint32 [ceil(n/16)];
 *             read during the call only (the pointers travel as kernel
 *             arguments; nothing is copied to or allocated on the device).
 *             More than NKLQ_MAX_PAYLOADS_PER_LAUNCH payloads are processed
 *             by consecutive launches that continue the same running sum.
 *   k_payloads >= 1;  n == 0 is a successful no-op.
 */
int nklq_dequant_accumulate_f32(float* acc, const uint32_t* const* payloads, int k_payloads,
                                uint64_t n, float thrd, int accumulate, void* stream);

/*
 * The two flat operations above on MANY vectors with one launch per 96 of them: a model's
 * gradients are a list of separate tensors, and the per-parameter lists grd_resi / grd_comp /
 * grd_recv that necklace's trainer keeps (necklace/trainer/tnopmx.py:140-149) are lists of
 * separate buffers.  All array arguments are HOST arrays of `count` entries, read during the
 * call only.  Vectors with n[i] == 0 are skipped.  A host thread that passes the same tables
 * again (same addresses and sizes, as a training loop does) is not charged the overlap check
 * a second time.
 *
 * nklq_quantize_multi_f32: for every i the flat quantize of g[i] (n[i] elements) into c[i]
 * (ceil(n[i]/16) words); the residual r[i] is updated in place when add_residual != 0
 * (a = g + r) and only written otherwise.
 *
 * nklq_dequant_accumulate_multi_f32: for every i the fixed-order sum of nklq_dequant_accumulate_f32
 * into acc[i], where vector i's code words start at word_offset[i] inside each of the
 * k_payloads payload buffers payload_base[p] (one contiguous message per peer).  Unless
 * divisor == 1 the sum is divided by `divisor` before it is stored (the correctly rounded IEEE
 * quotient): the `/ kn` that follows the all-reduce at necklace/frmwrk/pytorch/ptprms.py:294.
 */
int nklq_quantize_multi_f32(int count, const float* const* g, float* const* r, uint32_t* const* c,
                            const uint64_t* n, float thrd, int add_residual, void* stream);
int nklq_dequant_accumulate_multi_f32(int count, float* const* acc, const uint64_t* n,
                                      const uint64_t* word_offset,
                                      const uint32_t* const* payload_base, int k_payloads,
                                      float thrd, int accumulate, float divisor, void* stream);

/*
 * Number of uint32 words of the packed matrix: ceil(n_rows/16) * n_cols
 * (the `m` of necklace/cuda/quantize.py:145-147 times the column count).
 */
uint64_t nklq_packed_words(uint64_t n_rows, uint64_t n_cols);

/* Text for a return value of the entry points above (static storage). */
const char* nklq_strerror(int code);

/* NKLQ_VERSION the library was built from. */
int nklq_version(void);

/*
 * Launch-geometry knobs, the counterpart of the reference wrapper's bpg/tpb
 * keyword arguments (necklace/cuda/quantize.py:98,120).  Results never depend
 * on them; they apply to the flat kernels of every later call in the process
 * (the sum over payloads only has its interleave knob).  Returns the previous
 * value, or NKLQ_ERANGE for an unknown knob or a value outside its set.
 * value < 0 only queries.  Safe to call while other threads launch.
 *
 * libnklq.so is built with ONE workgroup shape and the non-temporal forms
 * only: there the first three knobs accept just the value in brackets.  The
 * full sets belong to the measurement build of the same source
 * (libnklq_tuning.so, include/nklq_tuning.h).
 */
#define NKLQ_TUNE_CHUNKS_PER_WAVE 0      /* 256-element chunks per wave: [1], 2 or 4 */
#define NKLQ_TUNE_WORKGROUP_SIZE 1       /* threads per workgroup: 64, 128, [256], 512 or 1024 */
#define NKLQ_TUNE_NONTEMPORAL 2          /* non-temporal loads and stores of the fp32 streams: 0 or [1] */
#define NKLQ_TUNE_XCD_INTERLEAVE_LOG2 3  /* quantize: neighbouring chunks are dealt to 2^v consecutive
                                            workgroups (which run on different XCDs): 0..6 */
#define NKLQ_TUNE_XCD_INTERLEAVE_LOG2_DECODE 4  /* the same for dequantize */
#define NKLQ_TUNE_XCD_INTERLEAVE_LOG2_ACCUMULATE 5  /* the same for the tiles (1024 elements) of the sum over payloads */
#define NKLQ_TUNE_DECODE_PREFETCH 6      /* dequantize with code words that are not in the 256 MB memory-side
                                            cache.  Flat: extra workgroups read the words ahead of the decoding
                                            ones; matrix: ranges of bands, each behind a pass over its words.
                                            Pays when the words come from HBM (0.6 -> 0.85-0.9 of the HBM
                                            peak), costs 6 % when they are in that cache anyway (just written
                                            or read).  0: only for inputs whose words exceed the cache (2^30
                                            elements and more); 1: always; 2: never */
int nklq_tune(int which, int value);

#ifdef __cplusplus
}
#endif
#endif /* NKLQ_H */
