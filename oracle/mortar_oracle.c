/* CPU oracle for the MORTAR sparse-MLP path, plain C (TEST INFRASTRUCTURE, not product).
 *
 * Blockwise restatement of the carved block-sparse ternary forward, used (a) as a second,
 * independently written checker next to the numpy oracle and (b) as the timed CPU baseline
 * ("port") of the benchmark.  Only tests, the smoke check and the benchmark's cpu_baseline
 * leg may load the library built from this file.
 *
 * Reference semantics followed (paths relative to the reference checkout):
 *   out[m, r*blk+n] = sum_{j in row r} sum_c x[m, col_j*blk+c] * data[j, n, c]
 *       morph/sparse/stk/backend/triton_kernels.py:170-230 (trans_B), bf16 operands, fp32
 *       accumulate, output stored in the activation dtype (custom_ops.py:49)
 *   data = bf16(code) * bf16(scale)          morph/inference/deploy_quant.py:367-369
 *   h = silu(gate) * up, per-cluster gates   morph/model/transformer.py:402-431
 *   kth / relu / normalise / gates > 0       morph/model/routing.py:232-284
 *
 * Pinned by tests against the numpy oracle's dense-scatter + float64 matmul.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline float bf16_to_f32(uint16_t b) {
    uint32_t u = ((uint32_t)b) << 16; float f; memcpy(&f, &u, 4); return f;
}
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u; memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static inline float bf16r(float f) { return bf16_to_f32(f32_to_bf16(f)); }

/* y[M, Rb*16] (bf16 bits) = x[M, K] (bf16 bits) @ W^T ; codes int8 [nnz,16,16]; scale fp32 [nnz]. */
int oracle_bcsr_spmm_bf16(const uint16_t *x, int M, int K, const int8_t *codes, const float *scale,
                          const int16_t *col_idx, const int32_t *offsets, int Rb, uint16_t *y) {
    const int N = Rb * 16;
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m) {
        float xr[16];
        for (int r = 0; r < Rb; ++r) {
            float acc[16];
            for (int n = 0; n < 16; ++n) acc[n] = 0.f;
            for (int j = offsets[r]; j < offsets[r + 1]; ++j) {
                const uint16_t *xp = x + (size_t)m * K + (size_t)col_idx[j] * 16;
                for (int c = 0; c < 16; ++c) xr[c] = bf16_to_f32(xp[c]);
                const float s = bf16r(scale[j]);
                const int8_t *q = codes + (size_t)j * 256;
                for (int n = 0; n < 16; ++n) {
                    float p = 0.f;
                    for (int c = 0; c < 16; ++c) p += xr[c] * (float)q[n * 16 + c];
                    acc[n] += p * s;   /* +-s*x summed per block; differs from per-term only in rounding order */
                }
            }
            for (int n = 0; n < 16; ++n) y[(size_t)m * N + r * 16 + n] = f32_to_bf16(acc[n]);
        }
    }
    return 0;
}

/* h[M, d_ff] = bf16(bf16(silu(g)) * u) [* bf16(gate[m, n/cls])] from gu[M, 2*d_ff] (all bf16 bits). */
int oracle_swiglu_bf16(const uint16_t *gu, int M, int d_ff, const float *gates, int n_clusters, uint16_t *h) {
    const int cls = gates ? d_ff / n_clusters : 1;
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < d_ff; ++n) {
            float g = bf16_to_f32(gu[(size_t)m * 2 * d_ff + n]);
            float u = bf16_to_f32(gu[(size_t)m * 2 * d_ff + d_ff + n]);
            float s = bf16r(g / (1.0f + expf(-g)));
            float v = bf16r(s * u);
            if (gates) v = bf16r(v * bf16r(gates[(size_t)m * n_clusters + n / cls]));
            h[(size_t)m * d_ff + n] = f32_to_bf16(v);
        }
    return 0;
}

static int cmp_desc(const void *a, const void *b) {
    float fa = *(const float *)a, fb = *(const float *)b;
    return (fa < fb) - (fa > fb);
}

/* gates[M,n] fp32, active[M,n] uint8 from logits[M,n]; threshold = k-th largest value (strict >). */
int oracle_remoe_gates(const float *logits, int M, int n, int k, float *gates, uint8_t *active) {
#pragma omp parallel
    {
        float *tmp = (float *)malloc(sizeof(float) * (size_t)n);
#pragma omp for schedule(static)
        for (int m = 0; m < M; ++m) {
            const float *l = logits + (size_t)m * n;
            float kth = 0.f;
            if (k < n) {
                memcpy(tmp, l, sizeof(float) * (size_t)n);
                qsort(tmp, (size_t)n, sizeof(float), cmp_desc);
                kth = tmp[k - 1];
            }
            float sum = 0.f;
            for (int i = 0; i < n; ++i) {
                float g = (k < n) ? l[i] - kth : l[i];
                g = g > 0.f ? g : 0.f;
                gates[(size_t)m * n + i] = g;
                sum += g;
            }
            if (sum < 1e-6f) sum = 1e-6f;
            const float t = (float)k / sum;
            for (int i = 0; i < n; ++i) {
                float g = gates[(size_t)m * n + i] * t;
                gates[(size_t)m * n + i] = g;
                active[(size_t)m * n + i] = g > 0.f;
            }
        }
        free(tmp);
    }
    return 0;
}

/* Whole MLP: x[M,d_model] -> y[M,d_model]; gu and h are caller-provided scratch (bf16 bits). */
int oracle_mlp_bf16(const uint16_t *x, int M, int d_model, int d_ff,
                    const int8_t *gu_codes, const float *gu_scale, const int16_t *gu_col, const int32_t *gu_off,
                    const int8_t *dn_codes, const float *dn_scale, const int16_t *dn_col, const int32_t *dn_off,
                    const float *gates, int n_clusters, uint16_t *gu, uint16_t *h, uint16_t *y) {
    oracle_bcsr_spmm_bf16(x, M, d_model, gu_codes, gu_scale, gu_col, gu_off, 2 * d_ff / 16, gu);
    oracle_swiglu_bf16(gu, M, d_ff, gates, n_clusters, h);
    oracle_bcsr_spmm_bf16(h, M, d_ff, dn_codes, dn_scale, dn_col, dn_off, d_model / 16, y);
    return 0;
}

int oracle_num_threads(void) {
#ifdef _OPENMP
    extern int omp_get_max_threads(void);
    return omp_get_max_threads();
#else
    return 1;
#endif
}
