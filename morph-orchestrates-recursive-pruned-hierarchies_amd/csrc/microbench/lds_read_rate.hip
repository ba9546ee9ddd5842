// Microbenchmark behind the LDS tile layout: ds_read_b128 rate per CU for the per-lane address patterns of candidate
// layouts of the activation tile (lane = token n + 16 * (column half + 2 * block of the pair)).  No vector ALU work in
// the loop (asm reads with immediate offsets, results left unused), 16 or 8 waves per CU.
// Build and run (MI355X):  hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops -Wno-unused-result -o /tmp/lds_read_rate lds_read_rate.hip && /tmp/lds_read_rate

#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdint>
#include <vector>
#include <string>
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(1024) probe(const int* offs, uint32_t* out, int iters) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    for (int i = threadIdx.x; i < 16384; i += blockDim.x) reinterpret_cast<uint32_t*>(lds)[i] = i;
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const uint32_t a = (uint32_t)offs[lane];
    u32x4_t v0, v1, v2, v3, v4, v5, v6, v7;
    for (int it = 0; it < iters; ++it) {
        asm volatile("ds_read_b128 %0, %8\n ds_read_b128 %1, %8 offset:4096\n ds_read_b128 %2, %8 offset:8192\n ds_read_b128 %3, %8 offset:12288\n"
                     "ds_read_b128 %4, %8 offset:16384\n ds_read_b128 %5, %8 offset:20480\n ds_read_b128 %6, %8 offset:24576\n ds_read_b128 %7, %8 offset:28672\n"
                     "s_waitcnt lgkmcnt(0)"
                     : "=v"(v0), "=v"(v1), "=v"(v2), "=v"(v3), "=v"(v4), "=v"(v5), "=v"(v6), "=v"(v7) : "v"(a));
    }
    out[blockIdx.x * blockDim.x + threadIdx.x] = v0[0] ^ v1[1] ^ v2[2] ^ v3[3] ^ v4[0] ^ v5[1] ^ v6[2] ^ v7[3];
}
int main() {
    int* d_offs; uint32_t* d_out;
    hipMalloc(&d_offs, 256); hipMalloc(&d_out, 256 * 1024 * 4);
    hipFuncSetAttribute((const void*)probe, hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
    hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
    struct Pat { std::string name; std::vector<int> off; };
    std::vector<Pat> pats;
    auto mk = [&](std::string name, auto f) { Pat p; p.name = name; for (int l = 0; l < 64; ++l) p.off.push_back(f(l) % 32768); pats.push_back(p); };
    mk("linear lane*16", [](int l) { return l * 16; });
    mk("aligned windows [ch][64 tok]: n*16 + hsel*1024 + bsel*2048*3", [](int l) { return (l & 15) * 16 + ((l >> 4) & 1) * 1024 + (l >> 5) * 2048 * 3; });
    mk("aligned windows [ch][32 tok]: n*16 + hsel*512 + bsel*1024*3", [](int l) { return (l & 15) * 16 + ((l >> 4) & 1) * 512 + (l >> 5) * 1024 * 3; });
    mk("padded [ch][33 tok] c=1: n*16 + hsel*528 + bsel*1056", [](int l) { return (l & 15) * 16 + ((l >> 4) & 1) * 528 + (l >> 5) * 1056; });
    mk("padded [ch][33 tok] c=5: n*16 + hsel*528 + bsel*1056*5", [](int l) { return (l & 15) * 16 + ((l >> 4) & 1) * 528 + (l >> 5) * 1056 * 5; });
    mk("padded [ch][65 tok] c=3: n*16 + hsel*1040 + bsel*2080*3", [](int l) { return (l & 15) * 16 + ((l >> 4) & 1) * 1040 + (l >> 5) * 2080 * 3; });
    for (int S : {1040, 976, 528, 272, 1072, 2064})
        for (int c : {1, 5})
            mk("row-major token stride " + std::to_string(S) + ": n*S + hsel*16 + bsel*32*" + std::to_string(c), [S, c](int l) { return (l & 15) * S + ((l >> 4) & 1) * 16 + (l >> 5) * 32 * c; });
    mk("row-major token stride 1024 (conflicting): n*1024 + hsel*16 + bsel*32", [](int l) { return (l & 15) * 1024 + ((l >> 4) & 1) * 16 + (l >> 5) * 32; });
    mk("token stride 64: n*64 + hsel*16 + bsel*4096", [](int l) { return (l & 15) * 64 + ((l >> 4) & 1) * 16 + (l >> 5) * 4096; });
    mk("token stride 32: n*32 + hsel*16 + bsel*4096", [](int l) { return (l & 15) * 32 + ((l >> 4) & 1) * 16 + (l >> 5) * 4096; });
    for (int threads : {1024, 512}) {
        for (auto& p : pats) {
            hipMemcpy(d_offs, p.off.data(), 256, hipMemcpyHostToDevice);
            int iters = 4000; float ms;
            probe<<<256, threads, 65536>>>(d_offs, d_out, 100);
            hipEventRecord(e0); probe<<<256, threads, 65536>>>(d_offs, d_out, iters); hipEventRecord(e1); hipEventSynchronize(e1);
            hipEventElapsedTime(&ms, e0, e1);
            double instr_per_cu = (threads / 64.0) * iters * 8;
            double cyc = ms * 1e-3 * 2.4e9 / instr_per_cu;
            printf("threads %4d  %-75s %.2f cycles/instr  (%.0f B/clk/CU)\n", threads, p.name.c_str(), cyc, 1024.0 / cyc);
        }
    }
    return 0;
}
