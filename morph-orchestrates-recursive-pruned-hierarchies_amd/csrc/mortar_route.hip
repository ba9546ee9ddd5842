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

// One wavefront per token.  The k-th largest logit is found exactly by an MSB-first radix select on
// order-preserving keys: for each bit the wave counts (ballot + popcount) the keys >= the candidate
// prefix.  Ties need no special care: the result is a VALUE, and the gate rule is `logit > kth`.
template <int MAXPL>      // logits per lane this instantiation holds: n <= 64 * MAXPL
__global__ void __launch_bounds__(256) remoe_gates_kernel(const float *logits, int64_t M, int n, int k,
                                                           float *gates, uint8_t *active) {
    const int lane = threadIdx.x & 63;
    const int64_t tok = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tok >= M) return;
    const float *lp = logits + tok * n;
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
        uint32_t prefix = 0;
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = prefix | (1u << bit);
            int c = 0;
#pragma unroll
            for (int i = 0; i < MAXPL; ++i) c += __popcll(__ballot(key[i] >= cand));     // padding keys are 0 < cand
            if (c >= k) prefix = cand;
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
            gates[tok * n + idx] = gv;
            if (active) active[tok * n + idx] = gv > 0.f;
        }
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
