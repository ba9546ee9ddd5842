// SwiGLU between the two carved matrices, for the training step: h = silu(gate) * up from a stored gate_up output, and
// its derivative.  Inference never runs these (the gate_up kernel applies SwiGLU in its epilogue); training keeps the
// gate_up output for the backward, as the reference's eager path does (morph/model/transformer.py:411-413:
// gate, up = gu.chunk(2); h = F.silu(gate) * up, differentiated by torch autograd).
//
// Rounding follows the tensors that path materialises in bf16: silu(gate), the product; in the backward
// d_up = dh * silu(gate), d(silu) = dh * up, d_gate = d(silu) * sigmoid(g) * (1 + g * (1 - sigmoid(g))).
// Plain HBM-bound streaming kernels: 16 bytes (8 features) per lane.
#include <hip/hip_runtime.h>

#include "mortar_device.h"
#include "mortar_internal.h"

namespace {

__device__ __forceinline__ float lo16(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float hi16(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }

__global__ __launch_bounds__(256) void swiglu_fwd_kernel(const uint16_t *gu, int64_t ldg, uint16_t *h, int64_t ldh,
                                                         int64_t M, int32_t d_ff) {
    const int per_row = d_ff >> 3;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= M * per_row) return;
    const int64_t m = i / per_row;
    const int c = (int)(i - m * per_row) * 8;
    const u32x4_t g = *reinterpret_cast<const u32x4_t *>(gu + m * ldg + c);
    const u32x4_t u = *reinterpret_cast<const u32x4_t *>(gu + m * ldg + d_ff + c);
    u32x4_t o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t s = bf16_pack2(silu_f32(lo16(g[j])), silu_f32(hi16(g[j])));
        o[j] = bf16_pack2(lo16(s) * lo16(u[j]), hi16(s) * hi16(u[j]));
    }
    *reinterpret_cast<u32x4_t *>(h + m * ldh + c) = o;
}

__device__ __forceinline__ float dsilu_f32(float g) {
    const float sg = __builtin_amdgcn_rcpf(1.0f + __expf(-g));
    return sg * (1.0f + g * (1.0f - sg));
}

__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const uint16_t *gu, int64_t ldg, const uint16_t *dh,
                                                         int64_t ldh, uint16_t *dgu, int64_t ldo, int64_t M,
                                                         int32_t d_ff) {
    const int per_row = d_ff >> 3;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= M * per_row) return;
    const int64_t m = i / per_row;
    const int c = (int)(i - m * per_row) * 8;
    const u32x4_t g = *reinterpret_cast<const u32x4_t *>(gu + m * ldg + c);
    const u32x4_t u = *reinterpret_cast<const u32x4_t *>(gu + m * ldg + d_ff + c);
    const u32x4_t d = *reinterpret_cast<const u32x4_t *>(dh + m * ldh + c);
    u32x4_t og, ou;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float g0 = lo16(g[j]), g1 = hi16(g[j]);
        const uint32_t s = bf16_pack2(silu_f32(g0), silu_f32(g1));              // silu(gate) as the forward stored it
        ou[j] = bf16_pack2(lo16(d[j]) * lo16(s), hi16(d[j]) * hi16(s));          // d_up
        const uint32_t ds = bf16_pack2(lo16(d[j]) * lo16(u[j]), hi16(d[j]) * hi16(u[j]));    // d(silu), a bf16 tensor
        og[j] = bf16_pack2(lo16(ds) * dsilu_f32(g0), hi16(ds) * dsilu_f32(g1));  // d_gate
    }
    *reinterpret_cast<u32x4_t *>(dgu + m * ldo + c) = og;
    *reinterpret_cast<u32x4_t *>(dgu + m * ldo + d_ff + c) = ou;
}

int check(const void *gu, int64_t ldg, const void *h, int64_t ldh, int64_t M, int32_t d_ff, const char *what) {
    if (!gu || !h || M < 0 || d_ff <= 0) return mortar_fail(MORTAR_ERR_ARG, "%s: null pointer or bad shape", what);
    if (d_ff % 8 || ldg < 2 * (int64_t)d_ff || ldh < d_ff || (ldg & 7) || (ldh & 7) ||
        (reinterpret_cast<uintptr_t>(gu) & 15) || (reinterpret_cast<uintptr_t>(h) & 15))
        return mortar_fail(MORTAR_ERR_ARG, "%s: d_ff and the leading dimensions must be multiples of 8, rows 16-byte aligned", what);
    return MORTAR_OK;
}

}  // namespace

extern "C" int mortar_swiglu_bf16(const uint16_t *gu, int64_t ldg, int64_t M, int32_t d_ff, uint16_t *h, int64_t ldh,
                                  void *stream) {
    const int rc = check(gu, ldg, h, ldh, M, d_ff, "swiglu");
    if (rc) return rc;
    const int64_t n = M * (d_ff >> 3);
    if (n == 0) return MORTAR_OK;
    hipLaunchKernelGGL(swiglu_fwd_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       gu, ldg, h, ldh, M, d_ff);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "swiglu: %s", hipGetErrorString(e));
    return MORTAR_OK;
}

extern "C" int mortar_swiglu_backward_bf16(const uint16_t *gu, int64_t ldg, const uint16_t *dh, int64_t ldh, int64_t M,
                                           int32_t d_ff, uint16_t *dgu, int64_t ldo, void *stream) {
    int rc = check(gu, ldg, dh, ldh, M, d_ff, "swiglu_backward");
    if (rc) return rc;
    rc = check(dgu, ldo, dh, ldh, M, d_ff, "swiglu_backward");
    if (rc) return rc;
    const int64_t n = M * (d_ff >> 3);
    if (n == 0) return MORTAR_OK;
    hipLaunchKernelGGL(swiglu_bwd_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       gu, ldg, dh, ldh, dgu, ldo, M, d_ff);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "swiglu_backward: %s", hipGetErrorString(e));
    return MORTAR_OK;
}
