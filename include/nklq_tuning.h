/*
 * nklq_tuning.h — what the measurement build of the quantizer exports on top of nklq.h.
 *
 * libnklq_tuning.so is csrc/nklq.hip compiled with -DNKLQ_TUNING_BUILD=1: every entry point of
 * nklq.h with the same kernels, plus
 *   - the launch geometries and cached-access forms that nklq_tune can switch to (1, 2 or 4 chunks
 *     per wave, workgroups of 64 .. 1024 threads, non-temporal on or off), which the product
 *     library leaves out;
 *   - the two entry points below.
 * Nothing here has a counterpart in the reference and nothing in the package's product path loads
 * this library: it serves the launch-geometry sweeps, the HBM counter calibration and the parity
 * tests that run every geometry.
 */
#ifndef NKLQ_TUNING_H
#define NKLQ_TUNING_H

#include "nklq.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * dst[i] = src[i] for n fp32 elements with the same 128-bit access pattern and workgroup -> chunk
 * map as the flat quantizer.  Calibrates the HBM byte counters (a copy's traffic is known) and gives
 * a copy bandwidth to quote beside the kernels.  dst, src: device, 16-byte aligned, not overlapping.
 */
int nklq_copy_f32(float* dst, const float* src, uint64_t n, void* stream);

/*
 * The fixed-order sum of nklq_dequant_accumulate_f32 (accumulate = 0) over payloads that are not
 * k_payloads separate arrays but alternate inside ONE array in runs of 2^run_words_log2 words:
 * run j of payload p starts at word (j * k_payloads + p) << run_words_log2 of `words`.  Same words,
 * bytes and arithmetic as the separate form; only the distance in memory between the k reads of
 * one 1024-element tile changes (run of 64 words: the k reads are one contiguous piece of
 * k * 256 bytes; run >= a whole payload: k streams a payload apart, the separate form).  Answers
 * whether the sum is slowed by the NUMBER of distinct read streams or by reading beside writing.
 *   acc    device, fp32 [n], 16-byte aligned; n a multiple of 1024
 *   words  device, uint32 [ceil(n/16 / run) * k_payloads * run], run = 2^run_words_log2, 6 <= log2 <= 40
 *   thrd   finite, >= 0 (the fast form of the sum only)
 */
int nklq_tuning_sum_interleaved_f32(float* acc, const uint32_t* words, int k_payloads, uint64_t n,
                                    int run_words_log2, float thrd, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NKLQ_TUNING_H */
