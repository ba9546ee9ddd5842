// Device-side re-pack: ternarise block values and rewrite a matrix's code and scale arrays in place.
//
// The reference ternarises carved blocks in torch (deploy_quant.py:81-95 for the deploy pack,
// block_sparse.py:909-919 on every QAT forward: scale = mean|w|, q = sign(w/s) * (|w/s| > threshold)) and keeps the
// transposed topology for the dX product as index arrays over the same data (stk matrix.py:107-125).  Here the
// topology of a pack (columns, offsets, octet positions) is fixed once on the host, and this kernel refreshes the
// values: one wavefront per block reads the 256 values (optionally of another block, transposed: the dX pack),
// forms the scale, and writes the row dwords into `codes`, the octet stream and its 4-bit copy.
#include <hip/hip_runtime.h>

#include "mortar_internal.h"

namespace {

constexpr int PARTIALS = 256;           // workgroups of the |w| reduction; the workspace holds one double each

__device__ __forceinline__ float load_val(const void *v, int64_t i, bool f32) {
    if (f32) return reinterpret_cast<const float *>(v)[i];
    return __uint_as_float((uint32_t) reinterpret_cast<const uint16_t *>(v)[i] << 16);
}

__device__ __forceinline__ double wave_sum(double x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
    return x;
}

// sum |w| over all values -> partial[blockIdx] (fixed order: the result does not depend on timing).  n is a multiple
// of 256 (whole blocks) and the array is 16-byte aligned, so every thread reads 16-byte pieces.
__global__ __launch_bounds__(256) void abs_sum_kernel(const void *values, int64_t n, int f32, double *partial) {
    __shared__ double wsum[4];
    double s = 0.0;
    const int per = f32 ? 4 : 8;                                     // values per 16-byte piece
    const uint4 *v = reinterpret_cast<const uint4 *>(values);
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n / per; i += (int64_t)PARTIALS * 256) {
        const uint4 q = v[i];
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (f32) {
                s += (double)fabsf(__uint_as_float(w[e]));
            } else {
                s += (double)fabsf(__uint_as_float(w[e] << 16));
                s += (double)fabsf(__uint_as_float(w[e] & 0xffff0000u));
            }
        }
    }
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) partial[blockIdx.x] = (wsum[0] + wsum[1]) + (wsum[2] + wsum[3]);
}

__global__ void clear_status_kernel(int32_t *status) {
    if (threadIdx.x < 2) status[threadIdx.x] = 0;
}

struct RequantArgs {
    uint32_t *codes, *sdup, *codes_o, *sd_o, *codes4_o;
    const void *values;
    const int32_t *pos, *src_block;
    const float *scale_in;
    float *scale_out;
    int32_t *status;
    const double *partial;
    int32_t nnz, f32, transpose, mode;
    float threshold;
    float ternary_tol;      // > 0: with a given scale, flag values that are neither 0 nor +-s within this relative bound
};

// mode 0: one scale per matrix from the partial sums, 1: one per block, 2: scale_in[0], 3: scale_in[source block]
__global__ __launch_bounds__(256) void requant_kernel(RequantArgs a) {
    __shared__ float tr[4][16][17];                     // per wavefront: one block, for the transposed read
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int j = blockIdx.x * 4 + wv;
    if (j >= a.nnz) return;
    const int src = a.src_block ? a.src_block[j] : j;
    const int n = lane >> 2, q = lane & 3;
    // the lane's four consecutive values of row n of the source block, in one load
    float w[4];
    if (a.f32) {
        const float4 v = reinterpret_cast<const float4 *>(a.values)[(int64_t)src * 64 + lane];
        w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
    } else {
        const uint2 v = reinterpret_cast<const uint2 *>(a.values)[(int64_t)src * 64 + lane];
        w[0] = __uint_as_float(v.x << 16); w[1] = __uint_as_float(v.x & 0xffff0000u);
        w[2] = __uint_as_float(v.y << 16); w[3] = __uint_as_float(v.y & 0xffff0000u);
    }
    if (a.transpose) {                                  // element (n, 4q + e) of the result is element (4q + e, n) of the source
#pragma unroll
        for (int e = 0; e < 4; ++e) tr[wv][n][4 * q + e] = w[e];
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = tr[wv][4 * q + e][n];
    }
    float s;
    if (a.mode == 0) {
        const double t = wave_sum((a.partial[lane] + a.partial[lane + 64]) + (a.partial[lane + 128] + a.partial[lane + 192]));
        s = fmaxf((float)(t / ((double)a.nnz * 256.0)), 1e-8f);
    } else if (a.mode == 1) {
        const double t = wave_sum(((double)fabsf(w[0]) + (double)fabsf(w[1])) + ((double)fabsf(w[2]) + (double)fabsf(w[3])));
        s = fmaxf((float)(t * (1.0 / 256.0)), 1e-6f);
    } else {
        s = a.scale_in[a.mode == 2 ? 0 : src];
    }
    // scale pattern: bf16(s) one exponent step down, in both halves (0 zeroes the block)
    uint32_t u = __float_as_uint(s);
    uint32_t sb = (u & 0x7fffffffu) > 0x7f800000u ? 0x7fc0u : ((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
    uint32_t sd = 0;
    if ((sb & 0x7fffu) != 0) {
        const uint32_t e8 = (sb >> 7) & 0xffu;
        if (e8 < 27 || e8 > 227) {
            if (lane == 0 && a.status) a.status[0] = 1;
        } else {
            const uint32_t adj = sb - 0x0400u;
            sd = adj | (adj << 16);
        }
    }
    if (a.ternary_tol > 0.f && a.status) {
        // every value must be 0 or +-s up to the bound (a bf16 cast of +-s(1 + rounding) may land one step beside bf16(s))
        bool bad = false;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float m = fabsf(w[e]);
            bad = bad || !(m <= a.ternary_tol * s || fabsf(m - s) <= a.ternary_tol * s);
        }
        if (bad) a.status[1] = 1;
    }
    uint32_t row = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int c = 4 * q + e;
        const float wn = w[e] / s;
        const uint32_t enc = (fabsf(wn) > a.threshold && wn != 0.f && sd != 0) ? (wn < 0.f ? 3u : 1u) : 0u;
        row |= enc << (2 * (c < 8 ? 2 * c + 1 : 2 * (c - 8)));
    }
    row |= __shfl_xor(row, 1);
    row |= __shfl_xor(row, 2);
    const int P = a.pos[j];
    if (q == 0) {
        a.codes[(int64_t)j * 16 + n] = row;
    } else if (q == 1) {
        a.codes_o[(int64_t)(P >> 2) * 64 + n * 4 + (P & 3)] = row;
    } else if (a.codes4_o) {
        const int h = q - 2;
        const int64_t g = P >> 3, s2 = (P >> 2) & 1;
        a.codes4_o[((g * 4 + 2 * s2 + h) * 16 + n) * 4 + (P & 3)] = (row << (2 * h)) & 0xCCCCCCCCu;
    }
    if (lane == 0) {
        a.sdup[j] = sd;
        a.sd_o[P] = sd;
        if (a.scale_out) a.scale_out[(a.mode == 0 || a.mode == 2) ? 0 : j] = s;
    }
}

// Overwrites out[0..ndw) with quiet-NaN patterns (0x7FC07FC0: NaN as two bf16 and as one fp32) when a status word is set.
// Every thread reads the two words; the usual case (both 0) ends after that one load.
__global__ __launch_bounds__(256) void poison_kernel(uint32_t *out, int64_t ndw, const int32_t *status) {
    if ((status[0] | status[1]) == 0) return;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < ndw; i += (int64_t)gridDim.x * 256) out[i] = 0x7FC07FC0u;
}

}  // namespace

extern "C" int mortar_poison_on_status(void *out, int64_t bytes, const int32_t *status, void *stream) {
    if (!out || !status) return mortar_fail(MORTAR_ERR_ARG, "poison_on_status: null pointer");
    if (bytes < 0 || (bytes & 3) || (reinterpret_cast<uintptr_t>(out) & 3))
        return mortar_fail(MORTAR_ERR_ARG, "poison_on_status: out must be 4-byte aligned and a multiple of 4 bytes long");
    if (bytes == 0) return MORTAR_OK;
    const int64_t ndw = bytes / 4;
    const int grid = (int)(ndw / 256 < 1 ? 1 : (ndw / 256 > 1024 ? 1024 : ndw / 256));
    hipLaunchKernelGGL(poison_kernel, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<uint32_t *>(out), ndw, status);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "poison_on_status: %s", hipGetErrorString(e));
    return MORTAR_OK;
}

extern "C" int64_t mortar_requantize_workspace_bytes(void) { return (int64_t)PARTIALS * sizeof(double); }

extern "C" int mortar_requantize(const mortar_bcsr_t *W, const void *values, int32_t values_f32, const int32_t *pos,
                                 const int32_t *src_block, int32_t transpose, int32_t scale_mode, float threshold,
                                 const float *scale_in, float *scale_out, int32_t *status, int32_t flags,
                                 float ternary_tol, void *workspace, void *stream) {
    if (!W || !values || !pos) return mortar_fail(MORTAR_ERR_ARG, "requantize: null pointer");
    if (!W->codes || !W->sdup || !W->codes_o || !W->sd_o || W->nnz <= 0)
        return mortar_fail(MORTAR_ERR_ARG, "requantize: incomplete matrix");
    if (scale_mode < 0 || scale_mode > 3) return mortar_fail(MORTAR_ERR_ARG, "requantize: scale_mode %d not in 0..3", scale_mode);
    if (scale_mode >= 2 && !scale_in) return mortar_fail(MORTAR_ERR_ARG, "requantize: scale_mode %d needs scale_in", scale_mode);
    if (scale_mode == 0 && !workspace) return mortar_fail(MORTAR_ERR_ARG, "requantize: scale_mode 0 needs the workspace");
    if (!(threshold >= 0.f)) return mortar_fail(MORTAR_ERR_ARG, "requantize: threshold must be >= 0");
    if (flags & ~1) return mortar_fail(MORTAR_ERR_ARG, "requantize: unknown flags 0x%x", flags);
    if (!(ternary_tol >= 0.f) || (ternary_tol > 0.f && (scale_mode < 2 || !status)))
        return mortar_fail(MORTAR_ERR_ARG, "requantize: ternary_tol needs a given scale (scale_mode 2 or 3) and a status word");
    if (reinterpret_cast<uintptr_t>(values) & 15) return mortar_fail(MORTAR_ERR_ARG, "requantize: values must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (status && !(flags & 1)) hipLaunchKernelGGL(clear_status_kernel, dim3(1), dim3(64), 0, st, status);
    if (scale_mode == 0)
        hipLaunchKernelGGL(abs_sum_kernel, dim3(PARTIALS), dim3(256), 0, st, values, (int64_t)W->nnz * 256, values_f32,
                           static_cast<double *>(workspace));
    RequantArgs a;
    a.codes = const_cast<uint32_t *>(W->codes);
    a.sdup = const_cast<uint32_t *>(W->sdup);
    a.codes_o = const_cast<uint32_t *>(W->codes_o);
    a.sd_o = const_cast<uint32_t *>(W->sd_o);
    a.codes4_o = const_cast<uint32_t *>(W->codes4_o);
    a.values = values;
    a.pos = pos;
    a.src_block = src_block;
    a.scale_in = scale_in;
    a.scale_out = scale_out;
    a.status = status;
    a.partial = static_cast<const double *>(workspace);
    a.nnz = W->nnz;
    a.f32 = values_f32;
    a.transpose = transpose;
    a.mode = scale_mode;
    a.threshold = threshold;
    a.ternary_tol = ternary_tol;
    hipLaunchKernelGGL(requant_kernel, dim3((W->nnz + 3) / 4), dim3(256), 0, st, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "requantize: %s", hipGetErrorString(e));
    return MORTAR_OK;
}
