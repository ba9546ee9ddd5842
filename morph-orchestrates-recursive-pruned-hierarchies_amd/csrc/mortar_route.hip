// ReMoE gating tail, active-token compaction, decode gather flags and RMSNorm.
//
//   mortar_remoe_gates   TileRouter.forward steps 5-8 (morph/model/routing.py:232-284; single-token
//                        form morph/kernels/triton/fused_router.py:88-97)
//   mortar_remoe_route   per (token tile, cluster) compacted list of active tokens (wavefront ballot)
//   mortar_route_flags   morph/kernels/triton/fused_decode_step.py:1883-1927
//   mortar_rmsnorm_bf16  morph/model/attention.py:133-141
#include "mortar_device.h"
#include "mortar_internal.h"

namespace {

constexpr int MAXPL_LIMIT = 16;   // logits per lane -> n <= 1024

__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t u = __builtin_bit_cast(uint32_t, f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);   // unsigned order == float order (-0 < +0)
}
__device__ __forceinline__ float key_to_float(uint32_t k) {
    const uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    return __builtin_bit_cast(float, u);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// Sum over the wavefront with DPP adds only (no LDS crossbar): quads, half rows, rows, then the row broadcasts; the total
// arrives in the last row and is read from lane 63.  Adds in another order than wave_sum, so not for results that have
// to match a kernel built on wave_sum bit for bit.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_f32(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ float wave_sum_dpp(float v) {
    v += dpp_f32<0xB1, 0xf>(v);     // quad_perm [1,0,3,2]
    v += dpp_f32<0x4E, 0xf>(v);     // quad_perm [2,3,0,1]
    v += dpp_f32<0x141, 0xf>(v);    // row_half_mirror
    v += dpp_f32<0x140, 0xf>(v);    // row_mirror
    v += dpp_f32<0x142, 0xa>(v);    // row_bcast:15 into rows 1 and 3
    v += dpp_f32<0x143, 0xc>(v);    // row_bcast:31 into rows 2 and 3
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Sum of a per-lane count over the wavefront with DPP adds only (quads, half rows, rows, then the row broadcasts): the
// total arrives in the lanes of the last row and is read from lane 63.
__device__ __forceinline__ int wave_count_total(uint32_t v) {
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xf, 0xf, false);    // quad_perm [1,0,3,2]
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xf, 0xf, false);    // quad_perm [2,3,0,1]
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xf, 0xf, false);   // row_half_mirror
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xf, 0xf, false);   // row_mirror
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false);   // row_bcast:15 into rows 1 and 3
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false);   // row_bcast:31 into rows 2 and 3
    return __builtin_amdgcn_readlane((int)v, 63);
}

// Gating tail of one token on one wavefront.  The k-th largest logit is found exactly by an MSB-first radix
// select on order-preserving keys: for each bit the wave counts the keys >= the candidate prefix.  Ties need no special care: the result is a VALUE, and the gate rule is `logit > kth`.
// `lp` may point to global memory or LDS; gates / active are this token's output rows.
template <int MAXPL>      // logits per lane this instantiation holds: n <= 64 * MAXPL
__device__ __forceinline__ void remoe_gates_wave(const float *lp, int n, int k, float *gates, uint8_t *active, int lane) {
    float v[MAXPL];
    uint32_t key[MAXPL];
#pragma unroll
    for (int i = 0; i < MAXPL; ++i) {
        const int idx = i * 64 + lane;
        v[i] = idx < n ? lp[idx] : 0.f;
        key[i] = idx < n ? order_key(v[i] == 0.f ? 0.f : v[i]) : 0u;   // -0 and +0 compare equal, as in topk
    }
    float kth = 0.f;
    const bool thresh = k < n;
    if (thresh) {
        // [prefix, prefix + 2^(bit+1)) is the bucket that holds the k-th largest key: c_lo keys are >= its lower end, c_hi keys
        // >= its upper end.  Once the bucket holds ONE key that key is the answer and the remaining bits need no counting
        // (distinct logits get there after about log2(n) + the exponent bits they share; exact ties walk all 32 bits).
        uint32_t prefix = 0;
        int c_lo = 64 * MAXPL, c_hi = 0, bit = 31;
        for (; bit >= 0 && c_lo - c_hi > 1; --bit) {
            const uint32_t cand = prefix | (1u << bit);
            // counted on the vector ALU: a ballot + scalar popcount per key would queue on the one scalar ALU that the
            // sixteen waves of a CU share
            uint32_t own = 0;
#pragma unroll
            for (int i = 0; i < MAXPL; ++i) own += key[i] >= cand ? 1u : 0u;             // padding keys are 0 < cand
            const int c = wave_count_total(own);
            if (c >= k) { prefix = cand; c_lo = c; } else { c_hi = c; }
        }
        if (bit >= 0) {                       // left early: the bucket's one key (bits 0..bit of it were never looked at)
            uint32_t m = 0;
#pragma unroll
            for (int i = 0; i < MAXPL; ++i) m = (key[i] >> (bit + 1)) == (prefix >> (bit + 1)) && key[i] > m ? key[i] : m;
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                const uint32_t t = (uint32_t)__shfl_xor((int)m, o, 64);
                m = t > m ? t : m;
            }
            prefix = m;
        }
        kth = key_to_float(prefix);
    }
    float g0[MAXPL];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < MAXPL; ++i) {
        const int idx = i * 64 + lane;
        float d = thresh ? v[i] - kth : v[i];
        d = d > 0.f ? d : (d != d ? d : 0.f);     // relu that lets NaN through, as torch.relu does
        g0[i] = idx < n ? d : 0.f;
        s += g0[i];
    }
    s = wave_sum(s);
    s = s < 1e-6f ? 1e-6f : s;                     // clamp(min=1e-6)
    const float t = (float)k / s;
#pragma unroll
    for (int i = 0; i < MAXPL; ++i) {
        const int idx = i * 64 + lane;
        if (idx < n) {
            const float gv = g0[i] * t;
            gates[idx] = gv;
            if (active) active[idx] = gv > 0.f;
        }
    }
}

template <int MAXPL>
__global__ void __launch_bounds__(256) remoe_gates_kernel(const float *logits, int64_t M, int n, int k,
                                                           float *gates, uint8_t *active) {
    const int64_t tok = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tok >= M) return;
    remoe_gates_wave<MAXPL>(logits + tok * n, n, k, gates + tok * n, active ? active + tok * n : nullptr, threadIdx.x & 63);
}

// ---- decode-side router front end (TileRouter.forward steps 1-4 in front of the gating tail) -------------------
// Launch 1: qv[b, o] = sum_i x[b, i] * Wq[o, i] + iter_vec[o].  One wavefront per output row o; the row of Wq is
// read once per group of TB tokens (16-byte loads, fp32), x comes from L2.
template <int TB, bool XF32>
__global__ void __launch_bounds__(256) router_project_kernel(const void *xv, int B, int d, int64_t ldx, const float *wq,
                                                              const float *iter_vec, float *qv) {
    const int lane = threadIdx.x & 63;
    const int o = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (o >= d) return;
    const float4 *wr = reinterpret_cast<const float4 *>(wq + (int64_t)o * d);
    const float bias = iter_vec ? iter_vec[o] : 0.f;
    const int n4 = d / 4;
    for (int b0 = 0; b0 < B; b0 += TB) {
        float acc[TB];
#pragma unroll
        for (int t = 0; t < TB; ++t) acc[t] = 0.f;
        // four 16-byte loads of the weight row in flight per lane (the row is read from HBM exactly once per token
        // group; the loop is latency-bound otherwise)
        for (int i0 = lane; i0 < n4; i0 += 256) {
            float4 w[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i4 = i0 + 64 * u;
                w[u] = i4 < n4 ? wr[i4] : float4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i4 = i0 + 64 * u < n4 ? i0 + 64 * u : n4 - 1;
#pragma unroll
                for (int t = 0; t < TB; ++t) {
                    const int b = b0 + t < B ? b0 + t : B - 1;
                    float x0, x1, x2, x3;
                    if (XF32) {
                        const float4 xx = reinterpret_cast<const float4 *>(static_cast<const float *>(xv) + (int64_t)b * ldx)[i4];
                        x0 = xx.x; x1 = xx.y; x2 = xx.z; x3 = xx.w;
                    } else {
                        const uint2 xx = reinterpret_cast<const uint2 *>(static_cast<const uint16_t *>(xv) + (int64_t)b * ldx)[i4];
                        x0 = __builtin_bit_cast(float, xx.x << 16); x1 = __builtin_bit_cast(float, xx.x & 0xffff0000u);
                        x2 = __builtin_bit_cast(float, xx.y << 16); x3 = __builtin_bit_cast(float, xx.y & 0xffff0000u);
                    }
                    acc[t] = __builtin_fmaf(x3, w[u].w, __builtin_fmaf(x2, w[u].z, __builtin_fmaf(x1, w[u].y, __builtin_fmaf(x0, w[u].x, acc[t]))));
                }
            }
        }
#pragma unroll
        for (int t = 0; t < TB; ++t) {
            const float s = wave_sum(acc[t]);
            if (lane == 0 && b0 + t < B) qv[(int64_t)(b0 + t) * d + o] = s + bias;
        }
    }
}

__device__ __forceinline__ float block_sum256(float v, float *red) {      // red: 4 floats of LDS; all 256 threads call
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return red[0] + red[1] + red[2] + red[3];
}

// Descending bitonic sort of 64 * KPL keys held KPL per lane (element lane * KPL + r in register r): steps between
// elements of one lane are register compare-exchanges, steps between lanes one shuffle per register.  No LDS, no barrier.
template <int KPL>
__device__ __forceinline__ void wave_sort_desc(uint32_t (&key)[KPL], int lane) {
    for (int k2 = 2; k2 <= 64 * KPL; k2 <<= 1) {
        const bool lane_desc = ((lane * KPL) & k2) == 0;       // direction of this lane's elements once k2 >= KPL
        for (int lj = k2 / (2 * KPL); lj >= 1; lj >>= 1) {       // partners in other lanes (distance j = lj * KPL)
            const bool keep_max = ((lane & lj) == 0) == lane_desc;
#pragma unroll
            for (int r = 0; r < KPL; ++r) {
                const uint32_t a = key[r], o = (uint32_t)__shfl_xor((int)a, lj, 64);
                key[r] = keep_max ? (a > o ? a : o) : (a > o ? o : a);
            }
        }
#pragma unroll
        for (int j = KPL / 2; j > 0; j >>= 1) {                  // partners in this lane's registers (distance j < k2)
            if (j < k2) {
#pragma unroll
                for (int r = 0; r < KPL; ++r) {
                    if ((r & j) == 0) {
                        const bool desc = k2 < KPL ? (r & k2) == 0 : lane_desc;
                        const uint32_t a = key[r], c = key[r | j];
                        const uint32_t hi = a > c ? a : c, lo = a > c ? c : a;
                        key[r] = desc ? hi : lo;
                        key[r | j] = desc ? lo : hi;
                    }
                }
            }
        }
    }
}

// The n largest of the P = nsk * nsk product scores of one token in descending order (+ bias) -> lgt[0 .. n), on one wave.
template <int KPL>
__device__ __attribute__((noinline)) void ranked_logits(const float *sct, int nsk, int P, const float *bias, int n, float *lgt,
                                              float *logits_row, int lane) {
    uint32_t key[KPL];
#pragma unroll
    for (int r = 0; r < KPL; ++r) {
        const int i = lane * KPL + r;
        uint32_t kk = 0u;                                    // padding: the smallest key
        if (i < P) {
            const uint32_t u = __float_as_uint(sct[i / nsk] + sct[nsk + i % nsk]);
            kk = (u & 0x80000000u) ? ~u : (u | 0x80000000u);   // NaN ranks above +inf, as torch.topk has it
        }
        key[r] = kk;
    }
    wave_sort_desc<KPL>(key, lane);
#pragma unroll
    for (int r = 0; r < KPL; ++r) {
        const int g = lane * KPL + r;
        if (g < n) {
            const float l = __uint_as_float((key[r] & 0x80000000u) ? (key[r] & 0x7fffffffu) : ~key[r]) + bias[g];
            lgt[g] = l;
            if (logits_row) logits_row[g] = l;
        }
    }
}

// Launch 2, one workgroup per token: LayerNorm(qv) -> sub-key scores of the two query halves -> product-key logits
// (+ group bias) -> gating tail.  P = nsk * nsk products map to the n groups one to one (P == n), wrap (P < n), or are
// ranked and the n largest kept (P > n).
// PRE > 0 (d <= 2048; PRE = sub-key rows per wave: 2 for nsk <= 4, 10 for nsk <= 20): every parameter a thread needs
// (LayerNorm weights, its slices of the sub-key rows of its wave) is fetched into registers before the first reduction,
// so the kernel pays one memory round trip instead of one per phase and key row.
template <int MAXPL, int PRE>
__global__ void __launch_bounds__(256) router_tail_kernel(const float *qv, int d, const float *ln_w, const float *ln_b,
                                                           float ln_eps, const float *ka, const float *kb, int nsk,
                                                           const float *bias, int n, int k, float *logits_out,
                                                           float *gates, uint8_t *active) {
    extern __shared__ __attribute__((aligned(16))) float sm[];       // qn[d] | s[2 * nsk] | logits[n] | red[4] | sort keys
    float *qn = sm, *sc = sm + d, *lg = sc + 2 * nsk, *red = lg + n;
    const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *q = qv + (int64_t)b * d;
    const int d2 = d / 2, n4 = d2 / 4;          // d % 8 == 0: both halves are whole float4 runs
    constexpr int QE = 8, DPW = PRE > 0 ? PRE : 1, KU = 4;      // PRE: entries per thread, sub-key dots per wave, float4 per lane and dot
    float qe[QE], lw[QE], lbv[QE];
    float4 kreg[DPW][KU];
    if (PRE) {
#pragma unroll
        for (int j = 0; j < QE; ++j) {
            const int i = tid + 256 * j, ic = i < d ? i : d - 1;
            qe[j] = q[ic]; lw[j] = ln_w[ic]; lbv[j] = ln_b[ic];
        }
#pragma unroll
        for (int cc = 0; cc < DPW; ++cc) {
            int c = wave + 4 * cc;
            c = c < 2 * nsk ? c : 2 * nsk - 1;
            const float4 *kr = reinterpret_cast<const float4 *>(c < nsk ? ka + (int64_t)c * d2 : kb + (int64_t)(c - nsk) * d2);
#pragma unroll
            for (int u = 0; u < KU; ++u) kreg[cc][u] = lane + 64 * u < n4 ? kr[lane + 64 * u] : float4{0.f, 0.f, 0.f, 0.f};
        }
    }
    float s = 0.f;
    if (PRE) {
#pragma unroll
        for (int j = 0; j < QE; ++j) s += tid + 256 * j < d ? qe[j] : 0.f;
    } else {
        for (int i = tid; i < d; i += 256) { const float t = q[i]; qn[i] = t; s += t; }      // a thread re-reads its own entries
    }
    const float mean = block_sum256(s, red) / (float)d;
    float v = 0.f;
    if (PRE) {
#pragma unroll
        for (int j = 0; j < QE; ++j) { const float c = tid + 256 * j < d ? qe[j] - mean : 0.f; v = __builtin_fmaf(c, c, v); }
    } else {
        for (int i = tid; i < d; i += 256) { const float c = qn[i] - mean; v = __builtin_fmaf(c, c, v); }
    }
    const float rstd = 1.0f / sqrtf(block_sum256(v, red) / (float)d + ln_eps);
    if (PRE) {
#pragma unroll
        for (int j = 0; j < QE; ++j)
            if (tid + 256 * j < d) qn[tid + 256 * j] = (qe[j] - mean) * rstd * lw[j] + lbv[j];
    } else {
        for (int i = tid; i < d; i += 256) qn[i] = (qn[i] - mean) * rstd * ln_w[i] + ln_b[i];
    }
    __syncthreads();
    if (PRE) {
#pragma unroll
        for (int cc = 0; cc < DPW; ++cc) {
            const int c = wave + 4 * cc;
            const float4 *qh = reinterpret_cast<const float4 *>(c < nsk ? qn : qn + d2);
            float a = 0.f;
#pragma unroll
            for (int u = 0; u < KU; ++u) {
                const float4 qq = qh[lane + 64 * u < n4 ? lane + 64 * u : n4 - 1];
                a = __builtin_fmaf(qq.w, kreg[cc][u].w, __builtin_fmaf(qq.z, kreg[cc][u].z, __builtin_fmaf(qq.y, kreg[cc][u].y, __builtin_fmaf(qq.x, kreg[cc][u].x, a))));
            }
            a = wave_sum(a);
            if (lane == 0 && c < 2 * nsk) sc[c] = a;
        }
    } else {
        for (int c = wave; c < 2 * nsk; c += 4) {
            const float4 *kr = reinterpret_cast<const float4 *>(c < nsk ? ka + (int64_t)c * d2 : kb + (int64_t)(c - nsk) * d2);
            const float4 *qh = reinterpret_cast<const float4 *>(c < nsk ? qn : qn + d2);
            float a = 0.f;
            for (int i0 = lane; i0 < n4; i0 += 256) {
                float4 kv[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) kv[u] = i0 + 64 * u < n4 ? kr[i0 + 64 * u] : float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const float4 qq = qh[i0 + 64 * u < n4 ? i0 + 64 * u : n4 - 1];
                    a = __builtin_fmaf(qq.w, kv[u].w, __builtin_fmaf(qq.z, kv[u].z, __builtin_fmaf(qq.y, kv[u].y, __builtin_fmaf(qq.x, kv[u].x, a))));
                }
            }
            a = wave_sum(a);
            if (lane == 0) sc[c] = a;
        }
    }
    __syncthreads();
    const int P = nsk * nsk;
    if (P > n) {
        // more product keys than groups: the group logits are the n largest product scores in descending order
        // (torch.topk(product_scores, n).values, morph/model/routing.py:212-222).  Bitonic sort of order-preserving
        // integer keys (NaN ranks above +inf, as torch.topk has it), padded with the smallest key: in one wave's registers
        // up to 1024 products, through LDS by the whole workgroup beyond.
        if (P <= 1024) {           // one wave ranks them in its registers (no LDS traffic, no barrier per step)
            float *lrow = logits_out ? logits_out + (int64_t)b * n : nullptr;
            if (wave == 0) {
                if (P <= 512) ranked_logits<8>(sc, nsk, P, bias, n, lg, lrow, lane);
                else ranked_logits<16>(sc, nsk, P, bias, n, lg, lrow, lane);
            }
        } else {
            uint32_t *sk = reinterpret_cast<uint32_t *>(red + 4);
            int P2 = 1;
            while (P2 < P) P2 <<= 1;
            for (int i = tid; i < P2; i += 256) {
                uint32_t key = 0u;
                if (i < P) {
                    const uint32_t u = __float_as_uint(sc[i / nsk] + sc[nsk + i % nsk]);
                    key = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
                }
                sk[i] = key;
            }
            __syncthreads();
            for (int k2 = 2; k2 <= P2; k2 <<= 1) {
                for (int j = k2 >> 1; j > 0; j >>= 1) {
                    for (int t = tid; t < P2 / 2; t += 256) {
                        const int i = ((t & ~(j - 1)) << 1) | (t & (j - 1)), l = i | j;
                        const uint32_t a = sk[i], c = sk[l];
                        const bool desc = (i & k2) == 0;
                        if (desc ? a < c : a > c) { sk[i] = c; sk[l] = a; }
                    }
                    __syncthreads();
                }
            }
            for (int g = tid; g < n; g += 256) {
                const uint32_t key = sk[g];
                const float l = __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key) + bias[g];
                lg[g] = l;
                if (logits_out) logits_out[(int64_t)b * n + g] = l;
            }
        }
    } else {
        for (int g = tid; g < n; g += 256) {
            const int pr = g % P;
            const float l = (sc[pr / nsk] + sc[nsk + pr % nsk]) + bias[g];
            lg[g] = l;
            if (logits_out) logits_out[(int64_t)b * n + g] = l;
        }
    }
    __syncthreads();
    if (wave == 0)
        remoe_gates_wave<MAXPL>(lg, n, k, gates + (int64_t)b * n, active ? active + (int64_t)b * n : nullptr, lane);
}

// ---- router tail for prefill-sized calls (TileRouter.forward steps 2-8 behind a library GEMM for the projection) ----

// A workgroup of four waves takes groups of up to TT = 4 tokens (a loop over its share of the groups), so the sub-key
// rows are read from L2 once per group instead of once per token.
//   1. LayerNorm by the whole workgroup: every thread holds its float4 pieces of all rows of the group, the iteration
//      vector and the LayerNorm parameters from ONE round of loads; the sums meet through LDS; normalised rows -> LDS.
//   2. the 2 * nsk sub-key dot products, one key row per wave at a time against all tokens of the group; the next row's
//      piece is requested before the current one is multiplied.
//   3. per token (one wave each): product-key logits (+ bias) -> LDS, ranked first when nsk^2 > n (a bitonic network
//      in the wave's registers), then the gating tail.
// Same arithmetic as router_tail_kernel; the sums are ordered differently.  A group is a chain of latencies (about 3 us of
// loads, 2 us of LayerNorm, 1.3 us per key row and wave, 2-10 us of logits and gating), so throughput comes from the
// groups in flight: three workgroups per CU (two for rows wider than 4096 values) at this register count, with the
// sort kept out of line (inlined, its registers add to the whole kernel's).
constexpr int TAIL_TT = 4;

template <int MAXPL, int J>      // J: float4 pieces of a row per thread (d <= 1024 * J); tokens per group tt = min(4, 8 / J)
__global__ void __launch_bounds__(256, J == 8 ? 2 : 3) router_tail_group_kernel(const float *qv, int64_t N, int d, int64_t ldq, const float *iter_vec,
                                                                 const float *ln_w, const float *ln_b, float ln_eps,
                                                                 const float *ka, const float *kb, int nsk, const float *bias,
                                                                 int n, int k, int tt, float *logits_out, float *gates,
                                                                 uint8_t *active) {
    extern __shared__ __attribute__((aligned(16))) float sm[];       // qn[tt][d] | sc[tt][2 nsk] | lg[tt][n] | red[16]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int d2 = d / 2, d4 = d / 4, n4 = d2 / 4;
    const int P = nsk * nsk;
    float *qn = sm, *sc = qn + (size_t)tt * d, *lg = sc + tt * 2 * nsk, *red = lg + (size_t)tt * n;
    const float4 *iv4 = reinterpret_cast<const float4 *>(iter_vec);
    const float4 *lw4 = reinterpret_cast<const float4 *>(ln_w), *lb4 = reinterpret_cast<const float4 *>(ln_b);
    const float4 zero4 = float4{0.f, 0.f, 0.f, 0.f};
    for (int64_t g0 = (int64_t)blockIdx.x * tt; g0 < N; g0 += (int64_t)gridDim.x * tt) {
        const int nt = N - g0 < tt ? (int)(N - g0) : tt;
        {
            // LayerNorm of the group's tokens by the whole workgroup: thread tid holds the float4 pieces tid + 256 * j of every
            // token (tt * pieces <= 8), so all rows, the iteration vector and the LayerNorm parameters are one round of
            // loads; sums meet through LDS (red: [4 waves][4 tokens]).
            constexpr int TT = 8 / J < TAIL_TT ? 8 / J : TAIL_TT, E = TT * J;
            float4 v[E], w[J], b[J];
#pragma unroll
            for (int jj = 0; jj < J; ++jj) {
                const int i = tid + 256 * jj, ic = i < d4 ? i : d4 - 1;
                if (J < 4) {              // wide rows fetch the LayerNorm parameters when they are used (registers)
                    w[jj] = lw4[ic];
                    b[jj] = lb4[ic];
                }
#pragma unroll
                for (int t = 0; t < TT; ++t) {
                    const bool on = t < nt && i < d4;
                    float4 a = reinterpret_cast<const float4 *>(qv + (g0 + (t < nt ? t : 0)) * ldq)[ic];
                    if (iter_vec) { const float4 c = iv4[ic]; a.x += c.x; a.y += c.y; a.z += c.z; a.w += c.w; }
                    v[t * J + jj] = on ? a : zero4;
                }
            }
            float s[TT], mean[TT], rstd[TT];
#pragma unroll
            for (int t = 0; t < TT; ++t) {
                s[t] = 0.f;
#pragma unroll
                for (int jj = 0; jj < J; ++jj) { const float4 a = v[t * J + jj]; s[t] += (a.x + a.y) + (a.z + a.w); }
                const float a = wave_sum_dpp(s[t]);
                if (lane == 0) red[wave * TAIL_TT + t] = a;
            }
            __syncthreads();
#pragma unroll
            for (int t = 0; t < TT; ++t) mean[t] = (red[t] + red[TAIL_TT + t] + red[2 * TAIL_TT + t] + red[3 * TAIL_TT + t]) / (float)d;
            __syncthreads();
#pragma unroll
            for (int t = 0; t < TT; ++t) {
                s[t] = 0.f;
#pragma unroll
                for (int jj = 0; jj < J; ++jj) {
                    if (tid + 256 * jj < d4) {
                        const float4 q = v[t * J + jj];
                        const float a = q.x - mean[t], c = q.y - mean[t], f = q.z - mean[t], h = q.w - mean[t];
                        s[t] = __builtin_fmaf(h, h, __builtin_fmaf(f, f, __builtin_fmaf(c, c, __builtin_fmaf(a, a, s[t]))));
                    }
                }
                const float a = wave_sum_dpp(s[t]);
                if (lane == 0) red[wave * TAIL_TT + t] = a;
            }
            __syncthreads();
#pragma unroll
            for (int t = 0; t < TT; ++t) {
                rstd[t] = 1.0f / sqrtf((red[t] + red[TAIL_TT + t] + red[2 * TAIL_TT + t] + red[3 * TAIL_TT + t]) / (float)d + ln_eps);
#pragma unroll
                for (int jj = 0; jj < J; ++jj) {
                    const int i = tid + 256 * jj;
                    if (J >= 4) {
                        w[jj] = lw4[i < d4 ? i : d4 - 1];
                        b[jj] = lb4[i < d4 ? i : d4 - 1];
                    }
                    if (t < nt && i < d4) {
                        const float4 q = v[t * J + jj];
                        const float m = mean[t], r = rstd[t];
                        reinterpret_cast<float4 *>(qn + (size_t)t * d)[i] =
                            float4{(q.x - m) * r * w[jj].x + b[jj].x, (q.y - m) * r * w[jj].y + b[jj].y,
                                   (q.z - m) * r * w[jj].z + b[jj].z, (q.w - m) * r * w[jj].w + b[jj].w};
                    }
                }
            }
        }
        __syncthreads();
        {
            // items of this wave: (key row c = wave + 4 * row, piece of 256 float4); the next item's piece is loaded first
            const int chunks = (n4 + 255) / 256;
            const int rows = (2 * nsk - wave + 3) / 4;
            const int items = rows * chunks;
            auto load_item = [&](int it, float4 (&kv)[4]) {
                const int itc = it < items ? it : items - 1;
                const int c = wave + 4 * (itc / chunks), i0 = lane + 256 * (itc % chunks);
                const float4 *kr = reinterpret_cast<const float4 *>(c < nsk ? ka + (int64_t)c * d2 : kb + (int64_t)(c - nsk) * d2);
#pragma unroll
                for (int u = 0; u < 4; ++u) kv[u] = kr[i0 + 64 * u < n4 ? i0 + 64 * u : n4 - 1];
            };
            float4 kv[4];
            if (items > 0) load_item(0, kv);
            float acc[TAIL_TT];
#pragma unroll
            for (int t = 0; t < TAIL_TT; ++t) acc[t] = 0.f;
            for (int it = 0; it < items; ++it) {
                float4 kn[4];
                load_item(it + 1, kn);
                const int c = wave + 4 * (it / chunks), i0 = lane + 256 * (it % chunks);
                const int off4 = c < nsk ? 0 : n4;
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    if (i0 + 64 * u >= n4) kv[u] = zero4;
#pragma unroll
                for (int t = 0; t < TAIL_TT; ++t) {
                    if (t < nt) {
                        const float4 *qh = reinterpret_cast<const float4 *>(qn + (size_t)t * d) + off4;
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const float4 qq = qh[i0 + 64 * u < n4 ? i0 + 64 * u : n4 - 1];
                            acc[t] = __builtin_fmaf(qq.w, kv[u].w, __builtin_fmaf(qq.z, kv[u].z, __builtin_fmaf(qq.y, kv[u].y, __builtin_fmaf(qq.x, kv[u].x, acc[t]))));
                        }
                    }
                }
                if (it % chunks == chunks - 1) {
#pragma unroll
                    for (int t = 0; t < TAIL_TT; ++t) {
                        const float a = wave_sum_dpp(acc[t]);
                        if (lane == 0 && t < nt) sc[t * 2 * nsk + c] = a;
                        acc[t] = 0.f;
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) kv[u] = kn[u];
            }
        }
        __syncthreads();
        if (wave < nt) {                             // tt <= 4: one token per wave, nothing shared between waves from here on
            const int t = wave;
            const float *sct = sc + t * 2 * nsk;
            float *lgt = lg + (size_t)t * n;
            float *lrow = logits_out ? logits_out + (g0 + t) * n : nullptr;
            if (P > n) {
                // more product keys than groups: the n largest product scores in descending order (routing.py:212-222)
                if (P <= 512) ranked_logits<8>(sct, nsk, P, bias, n, lgt, lrow, lane);
                else ranked_logits<16>(sct, nsk, P, bias, n, lgt, lrow, lane);        // the host admits P <= 1024
            } else {
                for (int g = lane; g < n; g += 64) {
                    const int pr = g % P;
                    const float l = (sct[pr / nsk] + sct[nsk + pr % nsk]) + bias[g];
                    lgt[g] = l;
                    if (lrow) lrow[g] = l;
                }
            }
            // the wave reads logits that other lanes of it wrote: LDS serves a wave's accesses in order, the fence keeps
            // the compiler from moving the reads up
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            remoe_gates_wave<MAXPL>(lgt, n, k, gates + (g0 + t) * n, active ? active + (g0 + t) * n : nullptr, lane);
        }
        __syncthreads();
    }
}

// Workgroup = (token tile, chunk of 64 clusters).  The tile's active bytes for the chunk are staged in LDS
// with coalesced reads; then every wave compacts whole clusters: lanes = tokens, ballot -> prefix popcount.
__global__ void __launch_bounds__(256) remoe_route_kernel(const uint8_t *active, int64_t M, int n, int tile,
                                                           int32_t *tok_cnt, uint8_t *tok_list) {
    __shared__ uint8_t a[256][64 + 4];
    const int t = blockIdx.x, cc = blockIdx.y * 64;
    const int ncl = (n - cc) < 64 ? (n - cc) : 64;
    const int64_t m0 = (int64_t)t * tile;
    for (int i = threadIdx.x; i < tile * 64; i += 256) {
        const int r = i >> 6, c = i & 63;
        const int64_t m = m0 + r;
        a[r][c] = (m < M && c < ncl) ? active[m * n + cc + c] : 0;
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int c = wave; c < ncl; c += 4) {
        const int64_t e = (int64_t)t * n + cc + c;
        int base = 0;
        for (int r0 = 0; r0 < tile; r0 += 64) {
            const int r = r0 + lane;
            const bool on = r < tile && a[r][c] != 0;
            const unsigned long long mask = __ballot(on);
            const int pos = base + __popcll(mask & ((1ull << lane) - 1ull));
            if (on) tok_list[e * tile + pos] = (uint8_t)r;
            base += __popcll(mask);
        }
        if (lane == 0) tok_cnt[e] = base;
    }
}

__global__ void __launch_bounds__(256) route_flags_kernel(const float *gates, int64_t B, int ncls, int64_t ldg,
                                                           int d_ff, int32_t *row_act, int64_t ldr,
                                                           int32_t *col_act, int64_t ldc) {
    const int nc = d_ff / 16, cls = d_ff / ncls;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= B * nc) return;
    const int64_t b = i / nc;
    const int r = (int)(i % nc);
    const int lo = (r * 16) / cls, hi = (r * 16 + 15) / cls;
    const int f = (gates[b * ldg + lo] > 0.f) || (gates[b * ldg + hi] > 0.f);
    if (col_act) col_act[b * ldc + r] = f;
    if (row_act) {
        row_act[b * ldr + r] = f;
        row_act[b * ldr + nc + r] = f;
    }
}

// One wavefront per row, in 16-byte units, with the summation order and rounding steps of the fused form in
// the gate_up staging (rms_* in mortar_device.h): both give the same bits.
__global__ void __launch_bounds__(256) rmsnorm_rows_kernel(const uint16_t *x, int64_t M, int d, int64_t ldx,
                                                            const uint16_t *w, float eps, uint16_t *y, int64_t ldy) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= M) return;
    const u32x4_t *xp = reinterpret_cast<const u32x4_t *>(x + row * ldx);
    const u32x4_t *wp = reinterpret_cast<const u32x4_t *>(w);
    u32x4_t *yp = reinterpret_cast<u32x4_t *>(y + row * ldy);
    const int nch = d / 8;
    float ss = 0.f;
    for (int ch = lane; ch < nch; ch += 64) ss = rms_sumsq8(xp[ch], ss);
    const float r = rms_scale(rms_wave_sum(ss), d, eps);
    for (int ch = lane; ch < nch; ch += 64)
        yp[ch] = rms_apply8(xp[ch], r, w ? wp[ch] : u32x4_t{0u, 0u, 0u, 0u}, w != nullptr);
}

// Any d / alignment: element-wise (its sums are ordered differently; no fused counterpart exists for such rows).
__global__ void __launch_bounds__(256) rmsnorm_kernel(const uint16_t *x, int64_t M, int d, int64_t ldx,
                                                       const uint16_t *w, float eps, uint16_t *y, int64_t ldy) {
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const uint16_t *xp = x + row * ldx;
    float s = 0.f;
    for (int i = threadIdx.x; i < d; i += 256) {
        const float v = bf16_to_f32(xp[i]);
        s += v * v;
    }
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    const float tot = red[0] + red[1] + red[2] + red[3];
    const float r = 1.0f / sqrtf(tot / (float)d + eps);
    for (int i = threadIdx.x; i < d; i += 256) {
        float v = bf16r(bf16_to_f32(xp[i]) * r);
        if (w) v = bf16r(v * bf16_to_f32(w[i]));
        y[row * ldy + i] = (uint16_t)bf16_bits_rne(v);
    }
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "%s launch: %s", what, hipGetErrorString(e));
    return MORTAR_OK;
}

}  // namespace

extern "C" int mortar_remoe_gates(const float *logits, int64_t M, int32_t n, int32_t k, float *gates,
                                  uint8_t *active, void *stream) {
    if (!logits || !gates) return mortar_fail(MORTAR_ERR_ARG, "remoe_gates: null pointer");
    if (M <= 0 || n <= 0 || k <= 0) return mortar_fail(MORTAR_ERR_ARG, "remoe_gates: M, n, k must be positive");
    if (n > 64 * MAXPL_LIMIT) return mortar_fail(MORTAR_ERR_LIMIT, "remoe_gates: n=%d exceeds %d clusters", n, 64 * MAXPL_LIMIT);
    const dim3 grid((unsigned)((M + 3) / 4)), block(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int npl = (n + 63) / 64;
    if (npl <= 1) hipLaunchKernelGGL(remoe_gates_kernel<1>, grid, block, 0, st, logits, M, n, k, gates, active);
    else if (npl <= 2) hipLaunchKernelGGL(remoe_gates_kernel<2>, grid, block, 0, st, logits, M, n, k, gates, active);
    else if (npl <= 4) hipLaunchKernelGGL(remoe_gates_kernel<4>, grid, block, 0, st, logits, M, n, k, gates, active);
    else if (npl <= 6) hipLaunchKernelGGL(remoe_gates_kernel<6>, grid, block, 0, st, logits, M, n, k, gates, active);
    else if (npl <= 8) hipLaunchKernelGGL(remoe_gates_kernel<8>, grid, block, 0, st, logits, M, n, k, gates, active);
    else hipLaunchKernelGGL(remoe_gates_kernel<16>, grid, block, 0, st, logits, M, n, k, gates, active);
    return check_launch("remoe_gates");
}

extern "C" int mortar_router_bf16(const void *x, int32_t x_is_f32, int64_t B, int32_t d, int64_t ldx, const float *wq,
                                  const float *iter_vec, const float *ln_w, const float *ln_b, float ln_eps,
                                  const float *ka, const float *kb, int32_t nsk, const float *bias, int32_t n,
                                  int32_t k, float *qv, float *logits_out, float *gates, uint8_t *active,
                                  void *stream) {
    if (!x || !wq || !ln_w || !ln_b || !ka || !kb || !bias || !qv || !gates)
        return mortar_fail(MORTAR_ERR_ARG, "router: null pointer");
    if (B <= 0 || B > 64) return mortar_fail(MORTAR_ERR_LIMIT, "router: the fused front end serves 1..64 tokens (got %lld)", (long long)B);
    if (d <= 0 || d % 8 || d > 8192 || ldx < d || ldx % (x_is_f32 ? 4 : 8))
        return mortar_fail(MORTAR_ERR_ARG, "router: d must be a multiple of 8 up to 8192 and ldx >= d, 16-byte aligned rows");
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(wq) | reinterpret_cast<uintptr_t>(ka) | reinterpret_cast<uintptr_t>(kb)) & 15)
        return mortar_fail(MORTAR_ERR_ARG, "router: x, wq, ka and kb must be 16-byte aligned");
    if (n <= 0 || k <= 0 || nsk <= 0) return mortar_fail(MORTAR_ERR_ARG, "router: n, k, nsk must be positive");
    if (n > 64 * MAXPL_LIMIT) return mortar_fail(MORTAR_ERR_LIMIT, "router: n=%d exceeds %d clusters", n, 64 * MAXPL_LIMIT);
    if ((int64_t)nsk * nsk > 2048)
        return mortar_fail(MORTAR_ERR_LIMIT, "router: %d x %d product keys exceed the 2048 the fused front end ranks", nsk, nsk);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 pg((unsigned)((d + 3) / 4)), blk(256);
#define MORTAR_PROJ(TB, F) hipLaunchKernelGGL((router_project_kernel<TB, F>), pg, blk, 0, st, x, (int)B, d, ldx, wq, iter_vec, qv)
    if (x_is_f32) { if (B == 1) MORTAR_PROJ(1, true); else if (B <= 4) MORTAR_PROJ(4, true); else if (B <= 8) MORTAR_PROJ(8, true); else MORTAR_PROJ(16, true); }
    else { if (B == 1) MORTAR_PROJ(1, false); else if (B <= 4) MORTAR_PROJ(4, false); else if (B <= 8) MORTAR_PROJ(8, false); else MORTAR_PROJ(16, false); }
#undef MORTAR_PROJ
    int rc = check_launch("router projection");
    if (rc) return rc;
    size_t sort_keys = 0;                          // nsk^2 > n: room for the product scores, padded to a power of two
    if ((int64_t)nsk * nsk > n) { sort_keys = 1; while (sort_keys < (size_t)nsk * nsk) sort_keys <<= 1; }
    const size_t smem = (size_t)(d + 2 * nsk + n + 4 + sort_keys) * sizeof(float);
    const dim3 tg((unsigned)B);
    const int npl = (n + 63) / 64;
    const int pre = d > 2048 ? 0 : nsk <= 4 ? 2 : nsk <= 20 ? 10 : 0;      // sub-key dots per wave with their rows in registers
#define MORTAR_TAILP(PL, PR) hipLaunchKernelGGL((router_tail_kernel<PL, PR>), tg, blk, smem, st, qv, d, ln_w, ln_b, ln_eps, \
                                               ka, kb, nsk, bias, n, k, logits_out, gates, active)
#define MORTAR_TAIL(PL) do { if (pre == 2) MORTAR_TAILP(PL, 2); else if (pre == 10) MORTAR_TAILP(PL, 10); else MORTAR_TAILP(PL, 0); } while (0)
    if (npl <= 1) MORTAR_TAIL(1);
    else if (npl <= 2) MORTAR_TAIL(2);
    else if (npl <= 4) MORTAR_TAIL(4);
    else if (npl <= 6) MORTAR_TAIL(6);
    else if (npl <= 8) MORTAR_TAIL(8);
    else MORTAR_TAIL(16);
#undef MORTAR_TAILP
#undef MORTAR_TAIL
    return check_launch("router tail");
}

extern "C" int mortar_router_tail_f32(const float *qv, int64_t N, int32_t d, int64_t ldq, const float *iter_vec,
                                      const float *ln_w, const float *ln_b, float ln_eps, const float *ka, const float *kb,
                                      int32_t nsk, const float *bias, int32_t n, int32_t k, float *logits_out, float *gates,
                                      uint8_t *active, void *stream) {
    if (!qv || !ln_w || !ln_b || !ka || !kb || !bias || !gates) return mortar_fail(MORTAR_ERR_ARG, "router tail: null pointer");
    if (N <= 0 || N > ((int64_t)1 << 31) / (n > 0 ? n : 1)) return mortar_fail(MORTAR_ERR_ARG, "router tail: N=%lld out of range", (long long)N);
    if (d <= 0 || d % 8 || d > 8192 || ldq < d || ldq % 4)
        return mortar_fail(MORTAR_ERR_ARG, "router tail: d must be a multiple of 8 up to 8192 and ldq >= d, 16-byte aligned rows");
    if ((reinterpret_cast<uintptr_t>(qv) | reinterpret_cast<uintptr_t>(iter_vec) | reinterpret_cast<uintptr_t>(ln_w) |
         reinterpret_cast<uintptr_t>(ln_b) | reinterpret_cast<uintptr_t>(ka) | reinterpret_cast<uintptr_t>(kb)) & 15)
        return mortar_fail(MORTAR_ERR_ARG, "router tail: qv, iter_vec, ln_w, ln_b, ka and kb must be 16-byte aligned");
    if (n <= 0 || k <= 0 || nsk <= 0) return mortar_fail(MORTAR_ERR_ARG, "router tail: n, k, nsk must be positive");
    if (n > 64 * MAXPL_LIMIT) return mortar_fail(MORTAR_ERR_LIMIT, "router tail: n=%d exceeds %d clusters", n, 64 * MAXPL_LIMIT);
    if ((int64_t)nsk * nsk > n && (int64_t)nsk * nsk > 1024)
        return mortar_fail(MORTAR_ERR_LIMIT, "router tail: %d x %d product keys for %d groups exceed the 1024 the kernel ranks", nsk, nsk, n);
    hipStream_t st = static_cast<hipStream_t>(stream);
    // a thread holds J float4 pieces of every row of its group (J = 1, 2, 4 or 8 for d <= 1024 J) and tt = min(4, 8 / J)
    // tokens share a group, so the normalised rows take at most 32 KB of LDS
    const int J = d <= 1024 ? 1 : d <= 2048 ? 2 : d <= 4096 ? 4 : 8;
    const int tt = 8 / J < TAIL_TT ? 8 / J : TAIL_TT;
    const size_t smem = ((size_t)tt * d + (size_t)tt * 2 * nsk + (size_t)tt * n + 16) * sizeof(float);
    const int64_t groups = (N + tt - 1) / tt;
    const dim3 grid((unsigned)(groups < 3072 ? groups : 3072)), blk(256);
    const int npl = (n + 63) / 64;
#define MORTAR_TAILG(PL, JJ) hipLaunchKernelGGL((router_tail_group_kernel<PL, JJ>), grid, blk, smem, st, qv, N, d, ldq, iter_vec, ln_w, \
                                               ln_b, ln_eps, ka, kb, nsk, bias, n, k, tt, logits_out, gates, active)
#define MORTAR_TAILJ(PL) do { if (J == 1) MORTAR_TAILG(PL, 1); else if (J == 2) MORTAR_TAILG(PL, 2); else if (J == 4) MORTAR_TAILG(PL, 4); \
                              else MORTAR_TAILG(PL, 8); } while (0)
    if (npl <= 2) MORTAR_TAILJ(2);
    else if (npl <= 6) MORTAR_TAILJ(6);
    else MORTAR_TAILJ(16);
#undef MORTAR_TAILJ
#undef MORTAR_TAILG
    return check_launch("router tail");
}

extern "C" int mortar_remoe_route(const uint8_t *active, int64_t M, int32_t n, int32_t tile, int32_t *tok_cnt,
                                  uint8_t *tok_list, void *stream) {
    if (!active || !tok_cnt || !tok_list) return mortar_fail(MORTAR_ERR_ARG, "remoe_route: null pointer");
    if (M <= 0 || n <= 0) return mortar_fail(MORTAR_ERR_ARG, "remoe_route: M and n must be positive");
    if (tile <= 0 || tile > 256 || (tile % 16 && tile != 4)) return mortar_fail(MORTAR_ERR_LIMIT, "remoe_route: tile must be 4 or a multiple of 16, at most 256");
    const unsigned nt = (unsigned)((M + tile - 1) / tile);
    hipLaunchKernelGGL(remoe_route_kernel, dim3(nt, (unsigned)((n + 63) / 64)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), active, M, n, tile, tok_cnt, tok_list);
    return check_launch("remoe_route");
}

extern "C" int mortar_route_flags(const float *gates, int64_t B, int32_t n_clusters, int64_t ldg, int32_t d_ff,
                                  int32_t *row_act, int64_t ldr, int32_t *col_act, int64_t ldc, void *stream) {
    if (!gates || (!row_act && !col_act)) return mortar_fail(MORTAR_ERR_ARG, "route_flags: null pointer");
    if (B <= 0 || n_clusters <= 0 || d_ff <= 0 || d_ff % 16 || d_ff % n_clusters)
        return mortar_fail(MORTAR_ERR_ARG, "route_flags: d_ff must be a multiple of 16 and of n_clusters");
    const int64_t total = B * (d_ff / 16);
    hipLaunchKernelGGL(route_flags_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), gates, B, n_clusters, ldg, d_ff, row_act, ldr, col_act, ldc);
    return check_launch("route_flags");
}

extern "C" int mortar_rmsnorm_bf16(const uint16_t *x, int64_t M, int32_t d, int64_t ldx, const uint16_t *w,
                                   float eps, uint16_t *y, int64_t ldy, void *stream) {
    if (!x || !y) return mortar_fail(MORTAR_ERR_ARG, "rmsnorm: null pointer");
    if (M <= 0 || d <= 0 || ldx < d || ldy < d) return mortar_fail(MORTAR_ERR_ARG, "rmsnorm: bad shape");
    const bool units = d % 8 == 0 && ldx % 8 == 0 && ldy % 8 == 0 &&
                       ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(w)) & 15) == 0;
    if (units)
        hipLaunchKernelGGL(rmsnorm_rows_kernel, dim3((unsigned)((M + 3) / 4)), dim3(256), 0, static_cast<hipStream_t>(stream),
                           x, M, d, ldx, w, eps, y, ldy);
    else
        hipLaunchKernelGGL(rmsnorm_kernel, dim3((unsigned)M), dim3(256), 0, static_cast<hipStream_t>(stream), x, M, d,
                           ldx, w, eps, y, ldy);
    return check_launch("rmsnorm");
}
