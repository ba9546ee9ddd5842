// Microbenchmark behind the kernels' cost model: how a gfx950 SIMD shares its issue between MFMA and vector ALU work.
// Every wave of a workgroup (4, 2 or 1 waves per SIMD) runs rounds of NM 16x16x32 bf16 MFMAs followed by NV independent
// vector instructions of one kind; clock64 per wave and a HIP-event time per launch give the cost of one round per SIMD.
// Reading of the numbers: a round costs max(16 * NM, 8 * NM + c * NV) cycles with c = 4.3 for v_pk_mul_f16, the FP4
// conversion and DPP moves, c = 3 for plain 32-bit integer ops: an MFMA takes two issue slots of four cycles, the
// matrix pipe itself is busy for 16, and every other vector instruction takes one slot.
// Build and run (MI355X):  hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops -Wno-unused-result -o /tmp/issue_port issue_port.hip && /tmp/issue_port

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
#define MF(acc, x, y) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, x), __builtin_bit_cast(bf16x8_t, y), acc, 0, 0, 0)

template <int KIND> __device__ __forceinline__ void valu1(uint32_t& v0, uint32_t& v1, uint32_t& v2, uint32_t& v3, int i) {
    // independent of the MFMA operands; rotating destination so that consecutive ops do not depend on each other
    uint32_t &d = (i & 3) == 0 ? v0 : (i & 3) == 1 ? v1 : (i & 3) == 2 ? v2 : v3;
    uint32_t &s = (i & 3) == 0 ? v2 : (i & 3) == 1 ? v3 : (i & 3) == 2 ? v0 : v1;
    if (KIND == 1) asm volatile("v_and_b32 %0, %0, %1" : "+v"(d) : "v"(s));
    else if (KIND == 2) asm volatile("v_pk_mul_f16 %0, %0, %1" : "+v"(d) : "v"(s));
    else if (KIND == 3) asm volatile("v_cvt_scalef32_pk_bf16_fp4 %0, %1, 1.0" : "+v"(d) : "v"(s));
    else if (KIND == 4) asm volatile("v_mov_b32_dpp %0, %1 row_newbcast:3 row_mask:0xf bank_mask:0xf bound_ctrl:1" : "+v"(d) : "v"(s));
    else if (KIND == 5) asm volatile("v_lshlrev_b32 %0, 2, %1" : "+v"(d) : "v"(s));
    else if (KIND == 6) asm volatile("v_add_u32 %0, %0, %1" : "+v"(d) : "v"(s));
    else if (KIND == 7) asm volatile("v_perm_b32 %0, %0, %1, %1" : "+v"(d) : "v"(s));
    else if (KIND == 8) asm volatile("v_and_or_b32 %0, %0, %1, %1" : "+v"(d) : "v"(s));
    else if (KIND == 9) asm volatile("v_fma_f32 %0, %0, %1, %1" : "+v"(d) : "v"(s));
}

template <int KIND, int NV, int NM>
__global__ void __launch_bounds__(1024) k(uint32_t* out, int iters, uint32_t seed, long long* clk) {
    u32x4_t a = {seed + threadIdx.x, seed * 3u, seed ^ 77u, seed + 5u}, b = {seed, seed + 1u, seed + 2u, seed + 3u};
    f32x4_t acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};
    uint32_t v0 = threadIdx.x, v1 = seed, v2 = seed * 7u, v3 = 11u;
    __syncthreads();
    long long c0 = clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            if (NM >= 1) { if (r & 1) MF(acc1, b, a); else MF(acc0, a, b); }
            if (NM >= 2) { if (r & 1) MF(acc0, b, a); else MF(acc1, a, b); }
#pragma unroll
            for (int i = 0; i < NV; ++i) valu1<KIND>(v0, v1, v2, v3, i);
        }
    }
    long long c1 = clock64();
    if (blockIdx.x == 0 && (threadIdx.x & 63) == 0) clk[threadIdx.x >> 6] = c1 - c0;
    out[blockIdx.x * 1024 + threadIdx.x] = v0 ^ v1 ^ v2 ^ v3 ^ __builtin_bit_cast(uint32_t, acc0[0] + acc1[1]);
}

static long long* clk; static uint32_t* d;
template <int KIND, int NV, int NM> void run(int threads) {
    const int iters = 4000;
    hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
    hipLaunchKernelGGL((k<KIND, NV, NM>), dim3(256), dim3(threads), 0, 0, d, 100, 1u, clk);
    hipEventRecord(e0);
    hipLaunchKernelGGL((k<KIND, NV, NM>), dim3(256), dim3(threads), 0, 0, d, iters, 1u, clk);
    hipEventRecord(e1); hipEventSynchronize(e1);
    float ms; hipEventElapsedTime(&ms, e0, e1);
    long long mx = 0; for (int w = 0; w < threads / 64; ++w) mx = clk[w] > mx ? clk[w] : mx;
    const double rounds = iters * 8.0;
    // per SIMD: waves/SIMD * rounds rounds; ticks per round of one wave (all waves run concurrently, so ticks per round per SIMD =
    // ticks / rounds; divide by waves per SIMD to get ticks per wave-round of issue)
    const int wps = threads / 256;
    printf("kind %d NM %d NV %d waves/SIMD %d: ticks per wave-round %.1f  per SIMD per (NM mfma + NV valu) %.2f   event %.3f ms -> %.2f ns per SIMD-round\n",
           KIND, NM, NV, wps, mx / rounds, mx / rounds / wps, ms, ms * 1e6 / rounds / wps);
}
template <int KIND> void sweep(int threads) {
    run<KIND, 0, 1>(threads); run<KIND, 1, 1>(threads); run<KIND, 2, 1>(threads); run<KIND, 3, 1>(threads); run<KIND, 4, 1>(threads);
    run<KIND, 5, 1>(threads); run<KIND, 6, 1>(threads); run<KIND, 8, 1>(threads); run<KIND, 12, 1>(threads);
    run<KIND, 4, 0>(threads); run<KIND, 8, 0>(threads);
}
int main() {
    hipMalloc(&d, 256 * 1024 * 4); hipHostMalloc(&clk, 16 * 8);
    for (int threads : {1024, 512, 256}) {
        printf("==== %d threads per CU\n", threads);
        sweep<1>(threads); sweep<2>(threads); sweep<3>(threads); sweep<4>(threads);
        if (threads == 1024) { sweep<5>(threads); sweep<6>(threads); sweep<7>(threads); sweep<8>(threads); sweep<9>(threads); }
    }
    // the kernel's own mix per pair: 2 MFMA + (1 dpp + 4 cvt + 4 pkmul + 1 dpp-add) = approximated by kinds separately above
    return 0;
}
