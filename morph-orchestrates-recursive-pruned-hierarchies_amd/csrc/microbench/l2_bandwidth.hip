// Microbenchmark behind the weight-stream design: aggregate bandwidth into the CUs when all 256 workgroups (one per CU)
// stream the SAME region with 16-byte loads (the pattern of the packed weights, which every token tile re-reads from
// L2), for several region sizes, and when every CU streams its own tile.
// Build and run (MI355X):  hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops -Wno-unused-result -o /tmp/l2_bandwidth l2_bandwidth.hip && /tmp/l2_bandwidth

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// every workgroup reads `len` bytes starting at (blockIdx.x / share) * len, `reps` times; wave w takes 4 KB chunks w, w+W, ...
template <int INFLIGHT>
__global__ void __launch_bounds__(1024) rd(const u32x4_t* __restrict__ a, size_t len, int share, int reps, uint32_t* out) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, W = blockDim.x >> 6;
    const u32x4_t* base = a + (size_t)(blockIdx.x / share) * (len / 16);
    const size_t nchunk = len / (1024 * INFLIGHT);
    uint32_t acc = 0;
    for (int r = 0; r < reps; ++r) {
        for (size_t c = wave; c < nchunk; c += W) {
            u32x4_t v[INFLIGHT];
#pragma unroll
            for (int i = 0; i < INFLIGHT; ++i) v[i] = base[(c * INFLIGHT + i) * 64 + lane];
#pragma unroll
            for (int i = 0; i < INFLIGHT; ++i) acc += v[i][0] ^ v[i][1] ^ v[i][2] ^ v[i][3];
        }
    }
    if (acc == 0x12345678u) out[0] = acc;
}

int main() {
    const size_t total = (size_t)64 << 20;
    u32x4_t* a; uint32_t* out;
    hipMalloc(&a, total); hipMalloc(&out, 4); hipMemset(a, 1, total);
    hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
    struct { size_t len; int share; const char* what; } cases[] = {
        {(size_t)720 << 10, 256, "all CUs read one 0.72 MB region"},
        {(size_t)1440 << 10, 256, "all CUs read one 1.44 MB region"},
        {(size_t)2880 << 10, 256, "all CUs read one 2.88 MB region"},
        {(size_t)5760 << 10, 256, "all CUs read one 5.76 MB region"},
        {(size_t)11520 << 10, 256, "all CUs read one 11.5 MB region"},
        {(size_t)128 << 10, 2, "pairs of CUs read their own 128 KB tile"},
        {(size_t)128 << 10, 1, "every CU reads its own 128 KB tile"},
    };
    for (auto& cs : cases) {
        for (int threads : {1024, 512}) {
            const int reps = (int)(((size_t)24 << 20) / cs.len) + 1;
            hipLaunchKernelGGL((rd<4>), dim3(256), dim3(threads), 0, 0, a, cs.len, cs.share, 1, out);
            hipEventRecord(e0);
            hipLaunchKernelGGL((rd<4>), dim3(256), dim3(threads), 0, 0, a, cs.len, cs.share, reps, out);
            hipEventRecord(e1); hipEventSynchronize(e1);
            float ms; hipEventElapsedTime(&ms, e0, e1);
            const double bytes = 256.0 * cs.len * reps;
            printf("%-45s threads %4d inflight 4: %.2f TB/s into the CUs (%.1f B/clk/CU at 2.4 GHz), %.3f ms\n", cs.what, threads,
                   bytes / (ms * 1e-3) / 1e12, bytes / (ms * 1e-3) / 256 / 2.4e9, ms);
            hipEventRecord(e0);
            hipLaunchKernelGGL((rd<8>), dim3(256), dim3(threads), 0, 0, a, cs.len, cs.share, reps, out);
            hipEventRecord(e1); hipEventSynchronize(e1);
            hipEventElapsedTime(&ms, e0, e1);
            printf("%-45s threads %4d inflight 8: %.2f TB/s\n", cs.what, threads, bytes / (ms * 1e-3) / 1e12);
        }
    }
    return 0;
}
