/*
 * A caller of libnklq.so that knows nothing of Python or torch: plain C, the HIP runtime's C
 * API for memory, and the declarations of include/nklq.h.
 *
 *   abi_client host   checks what needs no GPU (version, sizes, error codes)
 *   abi_client gpu    quantizes the 19-element known-answer vector of
 *                     tests/golden/kat_vectors.json (codes 0x92499009, 0x00000009), decodes it and
 *                     sums three payloads, comparing bit for bit; then the hand-worked
 *                     error-feedback vector (codes 0x60590850, 0x00000006) and the
 *                     sum-into-an-existing-buffer vector of the same file through the many-vectors
 *                     entry points
 *
 * Exit status 0 = all checks passed.
 */
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <hip/hip_runtime_api.h>

#include "nklq.h"

static int failures = 0;
#define CHECK(cond)                                                          \
    do {                                                                     \
        if (!(cond)) {                                                       \
            fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            ++failures;                                                      \
        }                                                                    \
    } while (0)

static void host_checks(void)
{
    CHECK(nklq_version() == NKLQ_VERSION);
    CHECK(nklq_packed_words(19, 1) == 2);
    CHECK(nklq_packed_words(224, 224) == 14 * 224);
    CHECK(nklq_packed_words(2800000000ull, 1) == 175000000ull);
    CHECK(nklq_quantize_f32(NULL, NULL, NULL, NULL, 0, 1, 0.5f, 0, NULL) == NKLQ_OK);
    CHECK(nklq_quantize_f32(NULL, NULL, (float*)0x1000, (uint32_t*)0x2000, 4, 1, 0.5f, 0, NULL) == NKLQ_ENULL);
    CHECK(nklq_dequantize_f32((float*)0x1002, (const uint32_t*)0x2000, 4, 1, 0.5f, NULL) == NKLQ_EALIGN);
    CHECK(nklq_dequant_accumulate_f32((float*)0x1000, NULL, 0, 4, 0.5f, 0, NULL) == NKLQ_ERANGE);
    CHECK(strlen(nklq_strerror(NKLQ_EALIGN)) > 0);
    CHECK(nklq_tune(NKLQ_TUNE_WORKGROUP_SIZE, -1) > 0);
    CHECK(nklq_tune(99, 1) == NKLQ_ERANGE);
    /* overlapping buffers are refused before anything is launched: code words that start inside
       the residual, and two vectors of one many-vectors call that write the same residual */
    CHECK(nklq_quantize_f32((const float*)0x10000, NULL, (float*)0x20000, (uint32_t*)0x20100, 1024, 1, 0.5f, 0, NULL)
          == NKLQ_EALIAS);
    {
        const float* g[2] = {(const float*)0x10000, (const float*)0x30000};
        float* r[2] = {(float*)0x50000, (float*)0x50800};
        uint32_t* c[2] = {(uint32_t*)0x70000, (uint32_t*)0x80000};
        const uint64_t n[2] = {1024, 1024};
        CHECK(nklq_quantize_multi_f32(2, g, r, c, n, 0.5f, 1, NULL) == NKLQ_EALIAS);
    }
}

static uint32_t bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, sizeof u);
    return u;
}

static void gpu_checks(void)
{
    static const uint32_t a_bits[19] = {
        0x3F000000, 0xBF000000, 0x3EFFFFFF, 0xBEFFFFFF, 0x00000000, 0x80000000, 0x3F800000,
        0xBF800000, 0x7F800000, 0xFF800000, 0x7FC00000, 0x3F400000, 0xBF400000, 0x3E800000,
        0x40000000, 0xC0000000, 0x3F000000, 0xC0400000, 0x3DCCCCCD};
    static const uint32_t r_bits[19] = {
        0x00000000, 0x00000000, 0x3EFFFFFF, 0xBEFFFFFF, 0x00000000, 0x80000000, 0x3F000000,
        0xBF000000, 0x7F800000, 0xFF800000, 0x7FC00000, 0x3E800000, 0xBE800000, 0x3E800000,
        0x3FC00000, 0xBFC00000, 0x00000000, 0xC0200000, 0x3DCCCCCD};
    const int n = 19;
    float *dA = NULL, *dR = NULL, *dB = NULL;
    uint32_t* dC = NULL;
    CHECK(hipMalloc((void**)&dA, n * 4) == hipSuccess);
    CHECK(hipMalloc((void**)&dR, n * 4) == hipSuccess);
    CHECK(hipMalloc((void**)&dB, n * 4) == hipSuccess);
    CHECK(hipMalloc((void**)&dC, 2 * 4) == hipSuccess);
    if (failures) return;
    CHECK(hipMemcpy(dA, a_bits, n * 4, hipMemcpyHostToDevice) == hipSuccess);
    CHECK(hipMemset(dC, 0xFF, 8) == hipSuccess);

    CHECK(nklq_quantize_f32(dA, NULL, dR, dC, n, 1, 0.5f, 0, NULL) == NKLQ_OK);
    CHECK(hipDeviceSynchronize() == hipSuccess);
    uint32_t c[2], r[19];
    CHECK(hipMemcpy(c, dC, 8, hipMemcpyDeviceToHost) == hipSuccess);
    CHECK(hipMemcpy(r, dR, n * 4, hipMemcpyDeviceToHost) == hipSuccess);
    CHECK(c[0] == 0x92499009u && c[1] == 0x00000009u);
    for (int i = 0; i < n; ++i) {
        if (i == 10) CHECK((r[i] & 0x7F800000u) == 0x7F800000u && (r[i] & 0x007FFFFFu) != 0); /* NaN */
        else CHECK(r[i] == r_bits[i]);
    }

    CHECK(nklq_dequantize_f32(dB, dC, n, 1, 0.5f, NULL) == NKLQ_OK);
    CHECK(hipDeviceSynchronize() == hipSuccess);
    float b[19];
    CHECK(hipMemcpy(b, dB, n * 4, hipMemcpyDeviceToHost) == hipSuccess);
    static const float want[19] = {.5f, -.5f, 0, 0, 0, 0, .5f, -.5f, .5f, -.5f, 0, .5f, -.5f, 0, .5f, -.5f, .5f, -.5f, 0};
    for (int i = 0; i < n; ++i) CHECK(bits(b[i]) == bits(want[i]));

    /* three times the same payload, summed in order: 3 x decode, exact for 0.5 */
    const uint32_t* payloads[3] = {dC, dC, dC};
    CHECK(nklq_dequant_accumulate_f32(dB, payloads, 3, n, 0.5f, 0, NULL) == NKLQ_OK);
    CHECK(hipDeviceSynchronize() == hipSuccess);
    CHECK(hipMemcpy(b, dB, n * 4, hipMemcpyDeviceToHost) == hipSuccess);
    for (int i = 0; i < n; ++i) CHECK(bits(b[i]) == bits(3.0f * want[i] + 0.0f));

    hipFree(dA); hipFree(dR); hipFree(dB); hipFree(dC);
}

/* tests/golden/kat_vectors.json, "fused" / error_feedback_t0.5 and "accumulate" /
   into_existing_buffer_t_1e-3, through nklq_quantize_multi_f32 / nklq_dequant_accumulate_multi_f32 */
static void gpu_checks_many_vectors(void)
{
    static const uint32_t g_bits[18] = {
        0x80000000, 0x80000000, 0x3E800000, 0x3E800000, 0x3E800000, 0xBE800000, 0xBE800000, 0x3F800000, 0x3F800000,
        0xC0400000, 0x3F400000, 0x7F800000, 0x7F800000, 0x3DCCCCCD, 0xBF000000, 0x3F000000, 0xBF800000, 0x3E99999A};
    static const uint32_t rin_bits[18] = {
        0x00000000, 0x80000000, 0x3E800000, 0x3E7FFFFF, 0x3E7FFFFE, 0xBE7FFFFF, 0xBE7FFFFE, 0x7FC00000, 0x3F400000,
        0x3F000000, 0xBE800000, 0xBF800000, 0xFF800000, 0x3E4CCCCD, 0x00000000, 0x80000000, 0x3E800000, 0x3E4CCCCD};
    static const uint32_t rout_bits[18] = { /* 0 where the result is NaN (elements 7 and 12) */
        0x00000000, 0x80000000, 0x00000000, 0x00000000, 0x3EFFFFFF, 0x00000000, 0xBEFFFFFF, 0, 0x3FA00000,
        0xC0000000, 0x00000000, 0x7F800000, 0, 0x3E99999A, 0x00000000, 0x00000000, 0xBE800000, 0x00000000};
    float *dG = NULL, *dR = NULL, *dAcc = NULL;
    uint32_t *dC = NULL, *dMsg = NULL;
    CHECK(hipMalloc((void**)&dG, 18 * 4) == hipSuccess);
    CHECK(hipMalloc((void**)&dR, 18 * 4) == hipSuccess);
    CHECK(hipMalloc((void**)&dC, 2 * 4) == hipSuccess);
    CHECK(hipMalloc((void**)&dAcc, 8 * 4) == hipSuccess);
    CHECK(hipMalloc((void**)&dMsg, 2 * 4) == hipSuccess);
    if (failures) return;
    CHECK(hipMemcpy(dG, g_bits, 18 * 4, hipMemcpyHostToDevice) == hipSuccess);
    CHECK(hipMemcpy(dR, rin_bits, 18 * 4, hipMemcpyHostToDevice) == hipSuccess);
    CHECK(hipMemset(dC, 0xFF, 8) == hipSuccess);
    {
        const float* g[1] = {dG};
        float* r[1] = {dR};
        uint32_t* c[1] = {dC};
        const uint64_t n[1] = {18};
        CHECK(nklq_quantize_multi_f32(1, g, r, c, n, 0.5f, 1, NULL) == NKLQ_OK);
    }
    CHECK(hipDeviceSynchronize() == hipSuccess);
    uint32_t c[2], r[18];
    CHECK(hipMemcpy(c, dC, 8, hipMemcpyDeviceToHost) == hipSuccess);
    CHECK(hipMemcpy(r, dR, 18 * 4, hipMemcpyDeviceToHost) == hipSuccess);
    CHECK(c[0] == 0x60590850u && c[1] == 0x00000006u);
    for (int i = 0; i < 18; ++i) {
        if (i == 7 || i == 12) CHECK((r[i] & 0x7F800000u) == 0x7F800000u && (r[i] & 0x007FFFFFu) != 0); /* NaN */
        else CHECK(r[i] == rout_bits[i]);
    }

    /* two one-word messages summed, in order, into a buffer that already holds values; t = 1e-3 */
    static const uint32_t acc_in[8] = {0x80000000, 0x80000000, 0x80000000, 0x3B03126F,
                                       0x3B449BA6, 0x3F800000, 0xBA83126F, 0x7FC00000};
    static const uint32_t acc_out[8] = {0x00000000, 0x00000000, 0x00000000, 0x3B449BA6,
                                        0x3B03126E, 0x3F80418A, 0xBA83126F, 0 /* NaN */};
    static const uint32_t msgs[2] = {0x0000566C, 0x00002410};
    const uint32_t t_bits = 0x3A83126F;
    float t;
    memcpy(&t, &t_bits, sizeof t);
    CHECK(hipMemcpy(dAcc, acc_in, 8 * 4, hipMemcpyHostToDevice) == hipSuccess);
    CHECK(hipMemcpy(dMsg, msgs, 2 * 4, hipMemcpyHostToDevice) == hipSuccess);
    {
        float* acc[1] = {dAcc};
        const uint64_t n[1] = {8};
        const uint64_t word_offset[1] = {0};
        const uint32_t* base[2] = {dMsg, dMsg + 1};
        CHECK(nklq_dequant_accumulate_multi_f32(1, acc, n, word_offset, base, 2, t, 1, 1.0f, NULL) == NKLQ_OK);
    }
    CHECK(hipDeviceSynchronize() == hipSuccess);
    uint32_t a[8];
    CHECK(hipMemcpy(a, dAcc, 8 * 4, hipMemcpyDeviceToHost) == hipSuccess);
    for (int i = 0; i < 8; ++i) {
        if (i == 7) CHECK((a[i] & 0x7F800000u) == 0x7F800000u && (a[i] & 0x007FFFFFu) != 0);
        else CHECK(a[i] == acc_out[i]);
    }
    hipFree(dG); hipFree(dR); hipFree(dC); hipFree(dAcc); hipFree(dMsg);
}

int main(int argc, char** argv)
{
    host_checks();
    if (argc > 1 && strcmp(argv[1], "gpu") == 0) {
        gpu_checks();
        gpu_checks_many_vectors();
    }
    if (failures) {
        fprintf(stderr, "%d check(s) failed\n", failures);
        return 1;
    }
    printf("abi_client %s: ok\n", argc > 1 ? argv[1] : "host");
    return 0;
}
