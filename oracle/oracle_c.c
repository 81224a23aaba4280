/*
 * Plain-C restatement of the same arithmetic as oracle/oracle.py, written
 * independently (explicit scalar loops, own bf16 conversion) so that the two
 * can check each other bit for bit.  TEST INFRASTRUCTURE ONLY: loaded through
 * ctypes by tests/ (and nothing else).  bf16 values travel as uint16_t.
 *
 *   orc_reduce:   kraken/fused/one_shot_all_reduce_bias.py:80-93 (bias first)
 *                 kraken/fused/two_shot_all_reduce_bias.py:71-83 (bias last)
 *   orc_rmsnorm:  kraken/fused/rms_norm.py:34-43
 *   orc_reduce_rmsnorm: kraken/fused/one_shot_all_reduce_bias_rms_norm.py:73-91
 *   orc_gemm:     kraken/fused/gemm_one_shot_all_reduce_fused.py:56-64,85-92
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even, NaN kept quiet */
static uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* out[i] = bf16([bias] + sum_r stack[r*stride + i]); bias_numel is numel or D (or 0) */
void orc_reduce(const uint16_t* stack, int W, int64_t stride, int64_t numel, const uint16_t* bias,
                int64_t bias_numel, int bias_first, uint16_t* out) {
    for (int64_t i = 0; i < numel; ++i) {
        float b = 0.0f;
        if (bias) b = bf16_to_f32(bias[bias_numel == numel ? i : i % bias_numel]);
        volatile float acc = (bias && bias_first) ? b : 0.0f;
        for (int r = 0; r < W; ++r) acc = acc + bf16_to_f32(stack[(int64_t)r * stride + i]);
        if (bias && !bias_first) acc = acc + b;
        out[i] = f32_to_bf16(acc);
    }
}

/* y = bf16(x * rsqrt(mean(x^2)+eps) * w), sum of squares in double as an
 * accuracy yardstick for the fp32 formulas */
void orc_rmsnorm_f32row(const float* row, const uint16_t* w, float eps, int64_t D, uint16_t* y) {
    double ss = 0.0;
    for (int64_t c = 0; c < D; ++c) ss += (double)row[c] * (double)row[c];
    float rstd = (float)(1.0 / sqrt(ss / (double)D + (double)eps));
    for (int64_t c = 0; c < D; ++c) y[c] = f32_to_bf16(row[c] * rstd * bf16_to_f32(w[c]));
}

void orc_reduce_rmsnorm(const uint16_t* stack, int W, int64_t stride, int64_t rows, int64_t D,
                        const uint16_t* bias, int bias_is_vector, const uint16_t* w, float eps,
                        uint16_t* y, float* scratch_row) {
    for (int64_t r0 = 0; r0 < rows; ++r0) {
        for (int64_t c = 0; c < D; ++c) {
            volatile float acc = 0.0f;
            if (bias) acc = bf16_to_f32(bias[bias_is_vector ? c : r0 * D + c]);
            for (int r = 0; r < W; ++r) acc = acc + bf16_to_f32(stack[(int64_t)r * stride + r0 * D + c]);
            scratch_row[c] = acc;
        }
        orc_rmsnorm_f32row(scratch_row, w, eps, D, y + r0 * D);
    }
}

/* C[M,N] (fp32) = A[M,K] @ B[K,N] + sum_p peers[p] + bias, triple loop, double accumulate */
void orc_gemm(const uint16_t* A, const uint16_t* B, int64_t M, int64_t N, int64_t K, const uint16_t* peers,
              int n_peers, const uint16_t* bias, float* C) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k)
                acc += (double)bf16_to_f32(A[m * K + k]) * (double)bf16_to_f32(B[k * N + n]);
            for (int p = 0; p < n_peers; ++p) acc += (double)bf16_to_f32(peers[((int64_t)p * M + m) * N + n]);
            if (bias) acc += (double)bf16_to_f32(bias[n]);
            C[m * N + n] = (float)acc;
        }
}
