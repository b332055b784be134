/* TEST INFRASTRUCTURE ONLY - scalar C restatement of the FP8 block-scaled GEMM, independent of torch.
 *
 * Built into oracle/libfp8bs_oracle.so by oracle/Makefile; loaded only by tests/, the smoke check and
 * bench.py's cpu_baseline leg.  It takes HOST pointers in the reference's storage order
 * (1-amd-fp8-mm/amd-fp8-mm-submission.py:66-75):
 *     a[kk*M + i], b[kk*N + j], as[(kk/128)*M + i], bs[(kk/128)*NB + j/128] with NB = (N+127)/128,
 *     c[i*N + j] bf16 bits.
 * Arithmetic: dequantise each element (1-amd-fp8-mm/0-amd-fp8-mm-new-begins.py:17-25, 34-42), sum the
 * products over K in double, round once to fp32 and then to bf16 with round-to-nearest-even
 * (amd-fp8-mm-submission.py:364).  Decode is the OCP e4m3fn closed form.
 *
 * Pinned by tests/test_oracle.py: the decoder against torch's float8_e4m3fn conversion over all 256
 * codes, the bf16 rounding against torch's, the GEMM against the torch restatement
 * (oracle/fp8bs_oracle.py) and against the committed power-of-two fixture.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

float fp8bs_ref_e4m3fn_to_float(uint8_t code) {
    int s = code >> 7, e = (code >> 3) & 15, m = code & 7;
    float v;
    if (e == 0) v = ldexpf((float)m, -9);
    else if (e == 15 && m == 7) v = NAN;
    else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return s ? -v : v;
}

uint16_t fp8bs_ref_float_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);   /* quiet NaN */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;                                                             /* RNE */
    return (uint16_t)(u >> 16);
}

/* rows [row_begin, row_end) of C = dequant(A) * dequant(B)^T ; lda = total rows of a / a_scale. */
static void gemm_rows(const uint8_t* a, const uint8_t* b, const float* as, const float* bs, uint16_t* c,
                      int lda, int n, int k, int row_begin, int row_end) {
    float lut[256];
    for (int i = 0; i < 256; i++) lut[i] = fp8bs_ref_e4m3fn_to_float((uint8_t)i);
    int nb = (n + 127) / 128;
#pragma omp parallel for schedule(static)
    for (int i = row_begin; i < row_end; i++) {
        for (int j = 0; j < n; j++) {
            double acc = 0.0;
            for (int kk = 0; kk < k; kk++) {
                float av = lut[a[(size_t)kk * lda + i]] * as[(size_t)(kk / 128) * lda + i];
                float bv = lut[b[(size_t)kk * n + j]] * bs[(size_t)(kk / 128) * nb + j / 128];
                acc += (double)av * (double)bv;
            }
            c[(size_t)i * n + j] = fp8bs_ref_float_to_bf16((float)acc);
        }
    }
}

int fp8bs_ref_gemm(const uint8_t* a, const uint8_t* b, const float* as, const float* bs, uint16_t* c,
                   int m, int n, int k) {
    if (m < 0 || n < 0 || k < 0 || k % 128) return 2;
    gemm_rows(a, b, as, bs, c, m, n, k, 0, m);
    return 0;
}

/* Grouped: expert e owns rows [row_offsets[e], row_offsets[e+1]) and weight b + e*K*N
 * (2-amd-moe/3-amd-fp8-moe-hip-myhgemm.py:328-336). */
int fp8bs_ref_gemm_grouped(const uint8_t* a, const uint8_t* b, const float* as, const float* bs, uint16_t* c,
                           const int32_t* row_offsets, int num_experts, int total_rows, int n, int k) {
    if (total_rows < 0 || n < 0 || k < 0 || k % 128 || num_experts <= 0) return 2;
    int nb = (n + 127) / 128;
    for (int e = 0; e < num_experts; e++)
        gemm_rows(a, b + (size_t)e * k * n, as, bs + (size_t)e * (k / 128) * nb, c, total_rows, n, k,
                  row_offsets[e], row_offsets[e + 1]);
    return 0;
}
