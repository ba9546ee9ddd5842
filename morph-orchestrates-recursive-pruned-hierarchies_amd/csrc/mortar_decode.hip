// Decode (M <= 64) block-sparse ternary GEMV: streams the packed blocks once, bandwidth bound.
//
// Replaces the reference's mortar_gemv + combine (morph/kernels/triton/fused_decode_step.py:1341-1547).
// As there, the schedule is a work list built once per matrix (topology is frozen): every entry is a run
// of consecutive blocks of ONE row unit, one wavefront per entry, and rows that are split over several
// entries write fp32 partials that a second kernel sums in slot order (no atomics, deterministic).
//
// Per entry the wave streams block pairs (128 B of codes + 2 scales + 2 column ids), unpacks them in
// registers and contracts them with the staged activations in one 16x16x32 bf16 MFMA per 16 streams: the
// matrix pipe does the 512 multiply-adds of a block pair in one issue slot, which keeps the vector ALU free
// for the unpack -- the step that bounds this kernel when done with scalar FMAs.
#include <mutex>

#include "mortar_device.h"
#include "mortar_internal.h"

namespace {

struct GemvParams {
    const uint32_t *codes;
    const uint32_t *sdup;
    const int16_t *col;
    const int32_t *entries;
    int n_entries, nslots, kseg, mode, Cb, N;
    const uint16_t *x;
    int B;
    int64_t ldx;
    uint16_t *y;
    int64_t ldy;
    float *part;
    const float *gates;
    int n_clusters, cluster_size;
    int64_t ldg;
    const int32_t *row_act;
    int64_t ldr;
    const int32_t *col_act;
    int64_t ldc;
};

constexpr int UN = 4;   // block pairs whose loads are in flight together

template <int MSUB>
__device__ __forceinline__ void run_blocks(const GemvParams &p, int p0, int cnt, int c0, const uint4 *lx,
                                           const uint32_t *colflag, int n, int bsel, int hsel,
                                           f32x4_t (&acc)[MSUB]) {
    constexpr int LDB = 16 * MSUB + 1;
    for (int q0 = 0; q0 < cnt; q0 += 2 * UN) {
        uint32_t w[UN], sd[UN];
        int c[UN];
        bool ok[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int q = q0 + 2 * u + bsel;
            ok[u] = q < cnt;
            const int64_t j = p0 + (ok[u] ? q : 0);
            w[u] = p.codes[j * 16 + n];
            sd[u] = p.sdup[j];
            c[u] = p.col[j] - c0;
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            if (q0 + 2 * u < cnt) {
                bool on = ok[u];
                if (colflag) on = on && colflag[c[u]] != 0u;
                const u32x4_t A = mortar_unpack8(on ? (w[u] << (2 * hsel)) : 0u, sd[u]);
                const uint32_t xo = (uint32_t)((c[u] * 2 + hsel) * LDB + n);
#pragma unroll
                for (int ms = 0; ms < MSUB; ++ms) {
                    const uint4 b = lx[xo + ms * 16];
                    const u32x4_t Bv = {b.x, b.y, b.z, b.w};
                    acc[ms] = mortar_mfma(A, Bv, acc[ms]);
                }
            }
        }
    }
}

template <int MSUB>
__global__ void __launch_bounds__(256) mortar_gemv_kernel(const GemvParams p) {
    constexpr int LDB = 16 * MSUB + 1;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint4 *lx = reinterpret_cast<uint4 *>(smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, g = lane >> 4, bsel = g >> 1, hsel = g & 1;

    const int32_t *e0p = p.entries + (int64_t)blockIdx.x * 4 * 8;
    const int seg = __builtin_amdgcn_readfirstlane(e0p[7]);
    const int c0 = seg * p.kseg;
    const int ncb = (p.Cb - c0) < p.kseg ? (p.Cb - c0) : p.kseg;
    const int nch = 2 * ncb;
    uint32_t *colflag = reinterpret_cast<uint32_t *>(smem + (size_t)2 * p.kseg * LDB * 16);

    // stage the activations of this K segment: unit (ch, tok) <- x[tok, c0*16 + ch*8 .. +8]
    // (a block-column that is off for stream `tok` enters as zeros for that stream: the reference masks the block's
    // products per stream, fused_decode_step.py:1387-1393)
    for (int tok = 0; tok < p.B; ++tok)
        for (int ch = tid; ch < nch; ch += 256) {
            uint4 v = *reinterpret_cast<const uint4 *>(p.x + (int64_t)tok * p.ldx + (int64_t)c0 * 16 + ch * 8);
            if (p.col_act && p.col_act[(int64_t)tok * p.ldc + c0 + (ch >> 1)] == 0) v = uint4{0u, 0u, 0u, 0u};
            lx[ch * LDB + tok] = v;
        }
    if (p.col_act) {
        for (int c = tid; c < ncb; c += 256) {
            uint32_t f = 0;
            for (int b = 0; b < p.B; ++b) f |= (uint32_t)(p.col_act[(int64_t)b * p.ldc + c0 + c] != 0);
            colflag[c] = f;
        }
    }
    __syncthreads();

    const int32_t *ep = e0p + wave * 8;
    const int rowA = __builtin_amdgcn_readfirstlane(ep[0]);
    if (rowA < 0) return;
    const int pA = __builtin_amdgcn_readfirstlane(ep[1]), cntA = __builtin_amdgcn_readfirstlane(ep[2]);
    const int rowB = __builtin_amdgcn_readfirstlane(ep[3]);
    const int pB = __builtin_amdgcn_readfirstlane(ep[4]), cntB = __builtin_amdgcn_readfirstlane(ep[5]);
    const int slot = __builtin_amdgcn_readfirstlane(ep[6]);

    bool unit_on = true;
    if (p.row_act) {   // skip the unit when no stream has one of its rows active
        int f = 0;
        if (lane < p.B) f = p.row_act[(int64_t)lane * p.ldr + rowA] != 0 || (rowB >= 0 && p.row_act[(int64_t)lane * p.ldr + rowB] != 0);
        unit_on = __builtin_amdgcn_readfirstlane(__ballot(f) != 0ull);
    }

    f32x4_t accA[MSUB], accB[MSUB];
#pragma unroll
    for (int ms = 0; ms < MSUB; ++ms) accA[ms] = accB[ms] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    if (unit_on) {
        run_blocks<MSUB>(p, pA, cntA, c0, lx, p.col_act ? colflag : nullptr, n, bsel, hsel, accA);
        if (rowB >= 0) run_blocks<MSUB>(p, pB, cntB, c0, lx, p.col_act ? colflag : nullptr, n, bsel, hsel, accB);
    }

#pragma unroll
    for (int ms = 0; ms < MSUB; ++ms) {
        const int tok = ms * 16 + n;
        if (tok >= p.B) continue;
        if (p.row_act && unit_on) {      // the flags are per stream: a row that is off for this stream contributes zeros
            if (p.row_act[(int64_t)tok * p.ldr + rowA] == 0) accA[ms] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            if (rowB >= 0 && p.row_act[(int64_t)tok * p.ldr + rowB] == 0) accB[ms] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
        if (p.nslots > 1) {
            float *pp = p.part + ((int64_t)slot * p.B + tok) * p.N;
            *reinterpret_cast<f32x4_t *>(pp + rowA * 16 + 4 * g) = accA[ms];
            if (rowB >= 0) *reinterpret_cast<f32x4_t *>(pp + rowB * 16 + 4 * g) = accB[ms];
        } else {
            const int e0 = rowA * 16 + 4 * g;
            u32x2_t pk;
            if (p.mode == 0) {
                pk = u32x2_t{bf16_pack2(accA[ms][0], accA[ms][1]), bf16_pack2(accA[ms][2], accA[ms][3])};
            } else {
                float gv = 0.f;
                if (p.gates) gv = p.gates[(int64_t)tok * p.ldg + e0 / p.cluster_size];
                pk = swiglu_pack4(accA[ms], accB[ms], p.gates != nullptr, gv);
            }
            *reinterpret_cast<u32x2_t *>(p.y + (int64_t)tok * p.ldy + e0) = pk;
        }
    }
}

// Sums the partials of each output in slot order and applies the epilogue.  row_slots[r] = number of
// partial slots row r owns (rows of one unit own the same number).
__global__ void __launch_bounds__(256) mortar_combine_kernel(const GemvParams p, const int32_t *row_slots) {
    const int nout = p.mode == 0 ? p.N : p.N / 2;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)p.B * nout) return;
    const int tok = (int)(i / nout), o = (int)(i % nout);
    const int ns = row_slots[o >> 4];
    float a = 0.f, b = 0.f;
    for (int s = 0; s < ns; ++s) {
        const float *pp = p.part + ((int64_t)s * p.B + tok) * p.N;
        a += pp[o];
        if (p.mode == 1) b += pp[nout + o];
    }
    float r = a;
    if (p.mode == 1) {
        r = bf16r(bf16r(silu_f32(bf16r(a))) * bf16r(b));
        if (p.gates) r = bf16r(r * bf16r(p.gates[(int64_t)tok * p.ldg + o / p.cluster_size]));
    }
    p.y[(int64_t)tok * p.ldy + o] = (uint16_t)bf16_bits_rne(r);
}

template <int MSUB>
int launch_gemv(const GemvParams &p, hipStream_t st) {
    const size_t smem = (size_t)2 * p.kseg * (16 * MSUB + 1) * 16 + (size_t)p.kseg * 4;
    if (smem > 160 * 1024) return mortar_fail(MORTAR_ERR_LIMIT, "gemv: K segment of %d block-columns needs %zu bytes of LDS", p.kseg, smem);
    auto kern = mortar_gemv_kernel<MSUB>;
    static size_t attr_set = 0;
    if (smem > attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
        attr_set = smem;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)(p.n_entries / 4)), dim3(256), smem, st, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "gemv launch: %s", hipGetErrorString(e));
    return MORTAR_OK;
}

}  // namespace

namespace {

int gemv_run(const char *who, const mortar_bcsr_t *W, const int32_t *entries, int64_t n_entries, int32_t nslots,
             const int32_t *row_slots, int32_t kseg, int32_t mode, const uint16_t *x, int32_t B, int64_t ldx,
             uint16_t *y, int64_t ldy, float *part, const float *gates, int32_t n_clusters, int64_t ldg,
             const int32_t *row_act, int64_t ldr, const int32_t *col_act, int64_t ldc, void *stream) {
    GemvParams p{};
    const int64_t nout = mode == 0 ? (int64_t)W->Rb * 16 : (int64_t)W->Rb * 8;
    p.codes = W->codes; p.sdup = W->sdup; p.col = W->col; p.entries = entries; p.n_entries = (int)n_entries;
    p.nslots = nslots; p.kseg = kseg; p.mode = mode; p.Cb = W->Cb; p.N = W->Rb * 16;
    p.x = x; p.B = B; p.ldx = ldx; p.y = y; p.ldy = ldy; p.part = part;
    p.n_clusters = 1; p.cluster_size = 1 << 30;
    if (gates) {
        if (mode != 1 || n_clusters <= 0 || nout % n_clusters || (nout / n_clusters) % 4)
            return mortar_fail(MORTAR_ERR_ARG, "%s: gates need mode 1 and d_ff / n_clusters a whole multiple of 4", who);
        p.gates = gates; p.n_clusters = n_clusters; p.cluster_size = (int)(nout / n_clusters); p.ldg = ldg;
    }
    p.row_act = row_act; p.ldr = ldr; p.col_act = col_act; p.ldc = ldc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int rc = B <= 16 ? launch_gemv<1>(p, st) : (B <= 32 ? launch_gemv<2>(p, st) : launch_gemv<4>(p, st));
    if (rc) return rc;
    if (nslots > 1) {
        const int64_t total = (int64_t)B * nout;
        hipLaunchKernelGGL(mortar_combine_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, p, row_slots);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "combine launch: %s", hipGetErrorString(e));
    }
    return MORTAR_OK;
}

int gemv_check(const char *who, const mortar_bcsr_t *W, const int32_t *entries, int64_t n_entries, int32_t nslots,
               const int32_t *row_slots, int32_t kseg, int32_t mode, const uint16_t *x, int32_t B, int64_t ldx,
               const uint16_t *y, int64_t ldy) {
    if (!W || !W->codes || !W->sdup || !W->col || !entries || !x || !y)
        return mortar_fail(MORTAR_ERR_ARG, "%s: null pointer", who);
    if (B <= 0 || B > 64) return mortar_fail(MORTAR_ERR_LIMIT, "%s: B=%d outside 1..64", who, B);
    if (n_entries <= 0 || n_entries % 4 || n_entries > (int64_t)0x7fffffff) return mortar_fail(MORTAR_ERR_ARG, "%s: entry count must be a positive multiple of 4", who);
    if (mode != 0 && mode != 1) return mortar_fail(MORTAR_ERR_ARG, "%s: mode must be 0 or 1", who);
    if (mode == 1 && (W->Rb & 1)) return mortar_fail(MORTAR_ERR_ARG, "%s: gate_up needs an even number of block-rows", who);
    if (nslots < 1 || (nslots > 1 && !row_slots)) return mortar_fail(MORTAR_ERR_ARG, "%s: nslots > 1 needs row_slots", who);
    if (kseg <= 0) return mortar_fail(MORTAR_ERR_ARG, "%s: kseg must be positive", who);
    const int64_t nout = mode == 0 ? (int64_t)W->Rb * 16 : (int64_t)W->Rb * 8;
    if (ldx < (int64_t)W->Cb * 16 || ldx % 8 || ldy < nout || ldy % 4 ||
        (reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(y) & 7))
        return mortar_fail(MORTAR_ERR_ARG, "%s: bad leading dimension or alignment", who);
    return MORTAR_OK;
}

}  // namespace

extern "C" int mortar_gemv_bf16(const mortar_bcsr_t *W, const int32_t *entries, int64_t n_entries,
                                int32_t nslots, const int32_t *row_slots, int32_t kseg, int32_t mode,
                                const uint16_t *x, int32_t B, int64_t ldx, uint16_t *y, int64_t ldy, float *part,
                                const float *gates, int32_t n_clusters, int64_t ldg,
                                const int32_t *row_act, int64_t ldr, const int32_t *col_act, int64_t ldc,
                                void *stream) {
    int rc = gemv_check("gemv", W, entries, n_entries, nslots, row_slots, kseg, mode, x, B, ldx, y, ldy);
    if (rc) return rc;
    if (nslots > 1 && !part) return mortar_fail(MORTAR_ERR_ARG, "gemv: nslots > 1 needs the partial workspace");
    return gemv_run("gemv", W, entries, n_entries, nslots, row_slots, kseg, mode, x, B, ldx, y, ldy, part, gates,
                    n_clusters, ldg, row_act, ldr, col_act, ldc, stream);
}

// ---- the reference engine's arithmetic: fp32 activations, exact products, fp32 sums, scale after the block sum ------
// (morph/kernels/triton/fused_decode_step.py:1335, 1341-1459; the engine runs fp32, morph/inference/engine.py:156-160).
// An fp32 activation is split exactly into three bf16 terms x = hi + mid + lo (8 + 8 + 8 mantissa bits).  One MFMA
// contracts ONE block against two of the terms at once: both K halves of the A operand hold the block's codes as
// +-2 / 0 (exact in bf16), the B operand holds hi in the first 16 K slots and mid in the second; a second MFMA adds
// the lo term.  Every product is exact, the fp32 accumulator of the matrix pipe takes the place of the reference's
// fp32 sums, and the block's fp32 scale (times one half for the +-2) multiplies the block sum afterwards:
// y = sum_j s_j * (C_j x_j), the per-block form of the reference's scale-after-sum.
namespace {

struct GemvF32Params {
    const uint32_t *codes;
    const int16_t *col;
    const float *scale;       // fp32 [nnz], or [1] when scale_count == 1
    const int32_t *entries;
    int n_entries, nslots, kseg, mode, Cb, N, scale_count, swiglu_x;
    const float *x;           // [B, ldx]; with swiglu_x the gate_up output [B, 2 * in_features]
    int B;
    int64_t ldx;
    float *y;
    int64_t ldy;
    float *part;
    const float *gates;
    int n_clusters, cluster_size;
    int64_t ldg;
    const int32_t *row_act;
    int64_t ldr;
    const int32_t *col_act;
    int64_t ldc;
};

template <int MSUB>
__device__ __forceinline__ void run_blocks_f32(const GemvF32Params &p, int p0, int cnt, int c0, const uint4 *lx, int plane,
                                               int zero_unit, const uint32_t *colflag, int n, int bsel, int hsel,
                                               f32x4_t (&acc)[MSUB]) {
    constexpr int LDB = 16 * MSUB + 1;
    for (int q0 = 0; q0 < cnt; q0 += UN) {
        uint32_t w[UN];
        float sc[UN];
        int c[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int q = q0 + u < cnt ? q0 + u : cnt - 1;
            const int64_t j = p0 + q;
            w[u] = p.codes[j * 16 + n];
            sc[u] = 0.5f * p.scale[p.scale_count == 1 ? 0 : j];
            c[u] = p.col[j] - c0;
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            if (q0 + u < cnt) {
                if (colflag && colflag[c[u]] == 0u) continue;                 // uniform: the whole wave reads the same flag
                const u32x4_t A = mortar_nib4((w[u] << (2 * hsel)) & 0xCCCCCCCCu);
                const uint32_t xo = (uint32_t)((c[u] * 2 + hsel) * LDB + n);
#pragma unroll
                for (int ms = 0; ms < MSUB; ++ms) {
                    // K slots 0..15 (bsel 0): hi, then lo;  K slots 16..31 (bsel 1): mid, then zeros
                    const uint4 b1 = lx[(bsel ? plane : 0) + xo + ms * 16];
                    const uint4 b2 = bsel ? lx[zero_unit] : lx[2 * plane + xo + ms * 16];
                    f32x4_t P = mortar_mfma(A, u32x4_t{b1.x, b1.y, b1.z, b1.w}, f32x4_t{0.f, 0.f, 0.f, 0.f});
                    P = mortar_mfma(A, u32x4_t{b2.x, b2.y, b2.z, b2.w}, P);
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[ms][v] = __builtin_fmaf(sc[u], P[v], acc[ms][v]);
                }
            }
        }
    }
}

__device__ __forceinline__ float sigmoid_f32(float g) { return 1.0f / (1.0f + __expf(-g)); }

template <int MSUB>
__global__ void __launch_bounds__(256) mortar_gemv_f32_kernel(const GemvF32Params p) {
    constexpr int LDB = 16 * MSUB + 1;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint4 *lx = reinterpret_cast<uint4 *>(smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, g = lane >> 4, bsel = g >> 1, hsel = g & 1;
    const int32_t *e0p = p.entries + (int64_t)blockIdx.x * 4 * 8;
    const int seg = __builtin_amdgcn_readfirstlane(e0p[7]);
    const int c0 = seg * p.kseg;
    const int ncb = (p.Cb - c0) < p.kseg ? (p.Cb - c0) : p.kseg;
    const int nch = 2 * ncb;
    const int plane = 2 * p.kseg * LDB;                         // 16-byte units per term plane
    const int zero_unit = 3 * plane;                            // one all-zero unit
    uint32_t *colflag = reinterpret_cast<uint32_t *>(smem + (size_t)(3 * plane + 1) * 16);
    const int I = p.Cb * 16;

    // stage the three bf16 terms of this K segment: unit (ch, tok) <- x[tok, c0*16 + ch*8 .. +8]
    for (int it = tid; it < nch * p.B; it += 256) {
        const int tok = it / nch, ch = it % nch;
        const float *src = p.x + (int64_t)tok * p.ldx + (int64_t)c0 * 16 + ch * 8;
        // a block-column that is off for this stream enters as zeros for it (per-stream flags, as the reference's kernel)
        const bool col_on = !p.col_act || p.col_act[(int64_t)tok * p.ldc + c0 + (ch >> 1)] != 0;
        uint32_t hi[4], mid[4], lo[4];
#pragma unroll
        for (int k = 0; k < 8; k += 2) {
            float v[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                float xv = src[k + e];
                if (p.swiglu_x) xv = xv * sigmoid_f32(xv) * src[I + k + e];      // h = silu(g) * u on load, fp32
                v[e] = col_on ? xv : 0.f;
            }
            const uint32_t h2 = bf16_pack2(v[0], v[1]);
            const float r0 = v[0] - bf16_to_f32(h2 & 0xffffu), r1 = v[1] - bf16_to_f32(h2 >> 16);
            const uint32_t m2 = bf16_pack2(r0, r1);
            const float s0 = r0 - bf16_to_f32(m2 & 0xffffu), s1 = r1 - bf16_to_f32(m2 >> 16);
            hi[k / 2] = h2; mid[k / 2] = m2; lo[k / 2] = bf16_pack2(s0, s1);
        }
        lx[ch * LDB + tok] = uint4{hi[0], hi[1], hi[2], hi[3]};
        lx[plane + ch * LDB + tok] = uint4{mid[0], mid[1], mid[2], mid[3]};
        lx[2 * plane + ch * LDB + tok] = uint4{lo[0], lo[1], lo[2], lo[3]};
    }
    if (tid == 0) lx[zero_unit] = uint4{0u, 0u, 0u, 0u};
    if (p.col_act) {
        for (int c = tid; c < ncb; c += 256) {
            uint32_t f = 0;
            for (int b = 0; b < p.B; ++b) f |= (uint32_t)(p.col_act[(int64_t)b * p.ldc + c0 + c] != 0);
            colflag[c] = f;
        }
    }
    __syncthreads();

    const int32_t *ep = e0p + wave * 8;
    const int rowA = __builtin_amdgcn_readfirstlane(ep[0]);
    if (rowA < 0) return;
    const int pA = __builtin_amdgcn_readfirstlane(ep[1]), cntA = __builtin_amdgcn_readfirstlane(ep[2]);
    const int rowB = __builtin_amdgcn_readfirstlane(ep[3]);
    const int pB = __builtin_amdgcn_readfirstlane(ep[4]), cntB = __builtin_amdgcn_readfirstlane(ep[5]);
    const int slot = __builtin_amdgcn_readfirstlane(ep[6]);
    bool unit_on = true;
    if (p.row_act) {
        int f = 0;
        if (lane < p.B) f = p.row_act[(int64_t)lane * p.ldr + rowA] != 0 || (rowB >= 0 && p.row_act[(int64_t)lane * p.ldr + rowB] != 0);
        unit_on = __builtin_amdgcn_readfirstlane(__ballot(f) != 0ull);
    }
    f32x4_t accA[MSUB], accB[MSUB];
#pragma unroll
    for (int ms = 0; ms < MSUB; ++ms) accA[ms] = accB[ms] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    if (unit_on) {
        run_blocks_f32<MSUB>(p, pA, cntA, c0, lx, plane, zero_unit, p.col_act ? colflag : nullptr, n, bsel, hsel, accA);
        if (rowB >= 0) run_blocks_f32<MSUB>(p, pB, cntB, c0, lx, plane, zero_unit, p.col_act ? colflag : nullptr, n, bsel, hsel, accB);
    }
#pragma unroll
    for (int ms = 0; ms < MSUB; ++ms) {
        const int tok = ms * 16 + n;
        if (tok >= p.B) continue;
        if (p.row_act && unit_on) {      // per-stream row flags: zero partial for a stream whose row is off (fused_decode_step.py:1378-1381)
            if (p.row_act[(int64_t)tok * p.ldr + rowA] == 0) accA[ms] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            if (rowB >= 0 && p.row_act[(int64_t)tok * p.ldr + rowB] == 0) accB[ms] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
        if (p.nslots > 1) {
            float *pp = p.part + ((int64_t)slot * p.B + tok) * p.N;
            *reinterpret_cast<f32x4_t *>(pp + rowA * 16 + 4 * g) = accA[ms];
            if (rowB >= 0) *reinterpret_cast<f32x4_t *>(pp + rowB * 16 + 4 * g) = accB[ms];
        } else {
            const int e0 = rowA * 16 + 4 * g;
            f32x4_t r = accA[ms];
            if (p.mode == 1) {
                const float gv = p.gates ? p.gates[(int64_t)tok * p.ldg + e0 / p.cluster_size] : 1.0f;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    r[v] = accA[ms][v] * sigmoid_f32(accA[ms][v]) * accB[ms][v];
                    if (p.gates) r[v] *= gv;
                }
            }
            *reinterpret_cast<f32x4_t *>(p.y + (int64_t)tok * p.ldy + e0) = r;
        }
    }
}

__global__ void __launch_bounds__(256) mortar_combine_f32_kernel(const GemvF32Params p, const int32_t *row_slots) {
    const int nout = p.mode == 0 ? p.N : p.N / 2;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)p.B * nout) return;
    const int tok = (int)(i / nout), o = (int)(i % nout);
    const int ns = row_slots[o >> 4];
    float a = 0.f, b = 0.f;
    for (int s = 0; s < ns; ++s) {
        const float *pp = p.part + ((int64_t)s * p.B + tok) * p.N;
        a += pp[o];
        if (p.mode == 1) b += pp[nout + o];
    }
    float r = a;
    if (p.mode == 1) {
        r = a * sigmoid_f32(a) * b;
        if (p.gates) r *= p.gates[(int64_t)tok * p.ldg + o / p.cluster_size];
    }
    p.y[(int64_t)tok * p.ldy + o] = r;
}

template <int MSUB>
int launch_gemv_f32(const GemvF32Params &p, hipStream_t st) {
    const size_t smem = ((size_t)3 * 2 * p.kseg * (16 * MSUB + 1) + 1) * 16 + (size_t)p.kseg * 4;
    if (smem > 160 * 1024) return mortar_fail(MORTAR_ERR_LIMIT, "gemv_f32: K segment of %d block-columns needs %zu bytes of LDS", p.kseg, smem);
    auto kern = mortar_gemv_f32_kernel<MSUB>;
    static size_t attr_set = 0;
    if (smem > attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
        attr_set = smem;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)(p.n_entries / 4)), dim3(256), smem, st, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "gemv_f32 launch: %s", hipGetErrorString(e));
    return MORTAR_OK;
}

// ---- one scale for the whole matrix, no flags: the product runs on the bandwidth-bound SpMM kernels ----------------
// The three bf16 terms of every activation row become three rows of a bf16 matrix [3B, in_features] (hi rows, then
// mid, then lo); the SpMM kernels for matrices with one scale contract them with the +-2 / 0 blocks (every product
// exact, fp32 sums in the matrix pipe) and store the sums unrounded; a last kernel adds the three sums of a row, applies
// the fp32 scale once (the reference's scale-after-sum) and the SwiGLU / gate epilogue.  Same arithmetic as the
// work-list kernel above up to the order of the fp32 additions.

// thread = 8 consecutive features of one row: x (or silu(g) * u of a gate_up output) -> 16 bytes of each term row
// A chunk whose input column is off for its stream is written as zeros, which is what masking its blocks' products for
// that stream amounts to (the flags are per stream, fused_decode_step.py:1387-1393).
__global__ void __launch_bounds__(256) gemv_f32_split_kernel(const float *x, int B, int K, int64_t ldx, int swiglu_x,
                                                             uint16_t *xs, const int32_t *col_act, int64_t ldc) {
    const int nch = K / 8;
    const int64_t it = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (it >= (int64_t)B * nch) return;
    const int tok = (int)(it / nch), ch = (int)(it % nch);
    const float4 *src = reinterpret_cast<const float4 *>(x + (int64_t)tok * ldx + ch * 8);
    float4 q[2] = {src[0], src[1]};
    if (swiglu_x) {
        const float4 u0 = src[K / 4], u1 = src[K / 4 + 1];
        q[0] = float4{q[0].x * sigmoid_f32(q[0].x) * u0.x, q[0].y * sigmoid_f32(q[0].y) * u0.y,
                      q[0].z * sigmoid_f32(q[0].z) * u0.z, q[0].w * sigmoid_f32(q[0].w) * u0.w};
        q[1] = float4{q[1].x * sigmoid_f32(q[1].x) * u1.x, q[1].y * sigmoid_f32(q[1].y) * u1.y,
                      q[1].z * sigmoid_f32(q[1].z) * u1.z, q[1].w * sigmoid_f32(q[1].w) * u1.w};
    }
    const float xv[8] = {q[0].x, q[0].y, q[0].z, q[0].w, q[1].x, q[1].y, q[1].z, q[1].w};
    uint32_t hi[4], mid[4], lo[4];
#pragma unroll
    for (int k = 0; k < 8; k += 2) {
        const float v[2] = {xv[k], xv[k + 1]};
        const uint32_t h2 = bf16_pack2(v[0], v[1]);
        const float r0 = v[0] - bf16_to_f32(h2 & 0xffffu), r1 = v[1] - bf16_to_f32(h2 >> 16);
        const uint32_t m2 = bf16_pack2(r0, r1);
        const float s0 = r0 - bf16_to_f32(m2 & 0xffffu), s1 = r1 - bf16_to_f32(m2 >> 16);
        hi[k / 2] = h2; mid[k / 2] = m2; lo[k / 2] = bf16_pack2(s0, s1);
    }
    if (col_act && col_act[(int64_t)tok * ldc + (ch >> 1)] == 0) {
#pragma unroll
        for (int k = 0; k < 4; ++k) hi[k] = mid[k] = lo[k] = 0u;
    }
    uint4 *dst = reinterpret_cast<uint4 *>(xs + (int64_t)tok * K + ch * 8);
    const int64_t plane = (int64_t)B * K / 8;                    // 16-byte units per term
    dst[0] = uint4{hi[0], hi[1], hi[2], hi[3]};
    dst[plane] = uint4{mid[0], mid[1], mid[2], mid[3]};
    dst[2 * plane] = uint4{lo[0], lo[1], lo[2], lo[3]};
}

// y3 [3B, N]: the sums of the hi, mid and lo rows.  y = scale * ((hi + mid) + lo), then the epilogue of the mode.
__global__ void __launch_bounds__(256) gemv_f32_combine3_kernel(const float *y3, const float *scale, int B, int N, int mode,
                                                                const float *gates, int cluster_size, int64_t ldg,
                                                                const int32_t *row_act, int64_t ldr, float *y, int64_t ldy) {
    const int nout = mode == 0 ? N : N / 2;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)B * nout) return;
    const int tok = (int)(i / nout), o = (int)(i % nout);
    // per-stream row flags (fused_decode_step.py:1378-1381): the sum of a row that is off for this stream is zero
    const bool on_a = !row_act || row_act[(int64_t)tok * ldr + (o >> 4)] != 0;
    const float s = scale[0];
    const float *r0 = y3 + (int64_t)tok * N, *r1 = r0 + (int64_t)B * N, *r2 = r1 + (int64_t)B * N;
    const float a = on_a ? s * ((r0[o] + r1[o]) + r2[o]) : 0.f;
    float r = a;
    if (mode == 1) {
        const bool on_b = !row_act || row_act[(int64_t)tok * ldr + ((nout + o) >> 4)] != 0;
        const float b = on_b ? s * ((r0[nout + o] + r1[nout + o]) + r2[nout + o]) : 0.f;
        r = a * sigmoid_f32(a) * b;
        if (gates) r *= gates[(int64_t)tok * ldg + o / cluster_size];
    }
    y[(int64_t)tok * ldy + o] = r;
}

int64_t gemv_f32_fast_bytes(const mortar_bcsr_t *W, int B) {
    return (int64_t)3 * B * ((int64_t)W->Rb * 16 * 4 + (int64_t)W->Cb * 16 * 2);
}

// Returns MORTAR_NO_KERNEL when the SpMM kernels cannot serve the shape (the caller then runs the work-list kernel).
int gemv_f32_fast(const mortar_bcsr_t *W, const int32_t *sched, const GemvF32Params &p, void *ws, hipStream_t st) {
    const int K = W->Cb * 16, N = W->Rb * 16;
    float *y3 = reinterpret_cast<float *>(ws);
    uint16_t *xs = reinterpret_cast<uint16_t *>(y3 + (int64_t)3 * p.B * N);
    const int64_t nsplit = (int64_t)p.B * (K / 8);
    const int split_blocks = (int)((nsplit + 255) / 256);
    hipLaunchKernelGGL(gemv_f32_split_kernel, dim3((unsigned)split_blocks), dim3(256), 0, st, p.x, p.B, K, p.ldx, p.swiglu_x, xs,
                       p.col_act, p.ldc);
    const int rc = mortar_spmm_codes_f32(W, sched, xs, 3 * p.B, K, y3, N, st);
    if (rc) return rc;
    const int64_t total = (int64_t)p.B * (p.mode == 0 ? N : N / 2);
    hipLaunchKernelGGL(gemv_f32_combine3_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, y3, p.scale, p.B, N,
                       p.mode, p.gates, p.cluster_size, p.ldg, p.row_act, p.ldr, p.y, p.ldy);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "gemv_f32 launch: %s", hipGetErrorString(e));
    return MORTAR_OK;
}

}  // namespace

extern "C" int64_t mortar_gemv_f32_workspace_bytes(const mortar_bcsr_t *W, int32_t B, int32_t nslots) {
    if (!W || W->Rb <= 0 || W->Cb <= 0 || B <= 0 || B > 64 || nslots < 1)
        return mortar_fail(MORTAR_ERR_ARG, "gemv_f32_workspace_bytes: bad argument");
    const int64_t slots = nslots > 1 ? (int64_t)nslots * B * W->Rb * 16 * 4 : 0, fast = gemv_f32_fast_bytes(W, B);
    return slots > fast ? slots : fast;
}

extern "C" int mortar_gemv_f32(const mortar_bcsr_t *W, const float *scale, int64_t scale_count, const int32_t *sched,
                               const int32_t *entries,
                               int64_t n_entries, int32_t nslots, const int32_t *row_slots, int32_t kseg, int32_t mode,
                               int32_t swiglu_x, const float *x, int32_t B, int64_t ldx, float *y, int64_t ldy, float *part,
                               int64_t part_bytes, const float *gates, int32_t n_clusters, int64_t ldg,
                               const int32_t *row_act, int64_t ldr, const int32_t *col_act, int64_t ldc, void *stream) {
    if (!W || !W->codes || !W->col || !scale || !entries || !x || !y) return mortar_fail(MORTAR_ERR_ARG, "gemv_f32: null pointer");
    if (scale_count != 1 && scale_count != W->nnz) return mortar_fail(MORTAR_ERR_ARG, "gemv_f32: scale_count must be 1 or nnz");
    if (B <= 0 || B > 64) return mortar_fail(MORTAR_ERR_LIMIT, "gemv_f32: B=%d outside 1..64", B);
    if (n_entries <= 0 || n_entries % 4 || n_entries > (int64_t)0x7fffffff) return mortar_fail(MORTAR_ERR_ARG, "gemv_f32: entry count must be a positive multiple of 4");
    if (mode != 0 && mode != 1) return mortar_fail(MORTAR_ERR_ARG, "gemv_f32: mode must be 0 or 1");
    if (mode == 1 && (W->Rb & 1)) return mortar_fail(MORTAR_ERR_ARG, "gemv_f32: gate_up needs an even number of block-rows");
    if (nslots < 1 || (nslots > 1 && (!part || !row_slots))) return mortar_fail(MORTAR_ERR_ARG, "gemv_f32: nslots > 1 needs the partial workspace and row_slots");
    if (kseg <= 0) return mortar_fail(MORTAR_ERR_ARG, "gemv_f32: kseg must be positive");
    const int64_t nout = mode == 0 ? (int64_t)W->Rb * 16 : (int64_t)W->Rb * 8;
    const int64_t need_x = (int64_t)W->Cb * 16 * (swiglu_x ? 2 : 1);
    if (ldx < need_x || ldy < nout || ldy % 4 || (reinterpret_cast<uintptr_t>(x) & 3) || (reinterpret_cast<uintptr_t>(y) & 15))
        return mortar_fail(MORTAR_ERR_ARG, "gemv_f32: bad leading dimension or alignment (y 16-byte aligned, ldy %% 4 == 0)");
    GemvF32Params p{};
    p.codes = W->codes; p.col = W->col; p.scale = scale; p.scale_count = (int)scale_count; p.entries = entries;
    p.n_entries = (int)n_entries; p.nslots = nslots; p.kseg = kseg; p.mode = mode; p.Cb = W->Cb; p.N = W->Rb * 16;
    p.swiglu_x = swiglu_x != 0; p.x = x; p.B = B; p.ldx = ldx; p.y = y; p.ldy = ldy; p.part = part;
    p.n_clusters = 1; p.cluster_size = 1 << 30;
    if (gates) {
        if (mode != 1 || n_clusters <= 0 || nout % n_clusters || (nout / n_clusters) % 4)
            return mortar_fail(MORTAR_ERR_ARG, "gemv_f32: gates need mode 1 and d_ff / n_clusters a whole multiple of 4");
        p.gates = gates; p.n_clusters = n_clusters; p.cluster_size = (int)(nout / n_clusters); p.ldg = ldg;
    }
    p.row_act = row_act; p.ldr = ldr; p.col_act = col_act; p.ldc = ldc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (nslots > 1 && part_bytes < (int64_t)nslots * B * W->Rb * 16 * 4)
        return mortar_fail(MORTAR_ERR_ARG, "gemv_f32: the partial workspace holds %lld bytes, need %lld", (long long)part_bytes,
                           (long long)nslots * B * W->Rb * 16 * 4);
    if (scale_count == 1 && sched && W->codes_o && part && !(reinterpret_cast<uintptr_t>(part) & 15) &&
        part_bytes >= gemv_f32_fast_bytes(W, B) && ldx % 4 == 0 && !(reinterpret_cast<uintptr_t>(x) & 15)) {
        const int rc = gemv_f32_fast(W, sched, p, part, st);
        if (rc != MORTAR_NO_KERNEL) return rc;
    }
    int rc = B <= 16 ? launch_gemv_f32<1>(p, st) : (B <= 32 ? launch_gemv_f32<2>(p, st) : launch_gemv_f32<4>(p, st));
    if (rc) return rc;
    if (nslots > 1) {
        const int64_t total = (int64_t)B * nout;
        hipLaunchKernelGGL(mortar_combine_f32_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, p, row_slots);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "combine launch: %s", hipGetErrorString(e));
    }
    return MORTAR_OK;
}

// ---- the same GEMV for callers that cannot allocate ------------------------------------------------------------
// The partial sums of split rows go to this array inside the library instead of a caller workspace.  Every device
// the library runs on holds its own copy at its own address; host code must use that address (looked up once per
// device below), never the array's name, which in host code is only a stand-in for the symbol.
namespace {

constexpr int64_t NOALLOC_FLOATS = MORTAR_GEMV_NOALLOC_MAX_FLOATS;
static __device__ __align__(256) float scratch[NOALLOC_FLOATS];

constexpr int MAX_DEVICES = 64;
float *scratch_addr[MAX_DEVICES];                 // per device, filled on the first call there
std::mutex scratch_lock;

int scratch_for_current_device(float **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "gemv_noalloc: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= MAX_DEVICES) return mortar_fail(MORTAR_ERR_LIMIT, "gemv_noalloc: device ordinal %d not below %d", dev, MAX_DEVICES);
    std::lock_guard<std::mutex> g(scratch_lock);
    if (!scratch_addr[dev]) {
        float *ptr = nullptr;
        e = hipGetSymbolAddress(reinterpret_cast<void **>(&ptr), HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            return mortar_fail(MORTAR_ERR_HIP, "gemv_noalloc: hipGetSymbolAddress: %s", hipGetErrorString(e));
        scratch_addr[dev] = ptr;
    }
    *out = scratch_addr[dev];
    return MORTAR_OK;
}

}  // namespace

extern "C" int64_t mortar_gemv_noalloc_max_floats(void) { return NOALLOC_FLOATS; }

extern "C" int mortar_gemv_bf16_noalloc(const mortar_bcsr_t *W, const int32_t *entries, int64_t n_entries,
                                        int32_t nslots, const int32_t *row_slots, int32_t kseg, int32_t mode,
                                        const uint16_t *x, int32_t B, int64_t ldx, uint16_t *y, int64_t ldy,
                                        const float *gates, int32_t n_clusters, int64_t ldg,
                                        const int32_t *row_act, int64_t ldr, const int32_t *col_act, int64_t ldc,
                                        void *stream) {
    int rc = gemv_check("gemv_noalloc", W, entries, n_entries, nslots, row_slots, kseg, mode, x, B, ldx, y, ldy);
    if (rc) return rc;
    float *part = nullptr;
    if (nslots > 1) {
        const int64_t need = (int64_t)nslots * B * W->Rb * 16;
        if (need > NOALLOC_FLOATS)
            return mortar_fail(MORTAR_ERR_LIMIT, "gemv_noalloc: nslots * B * out_features = %lld floats of partial sums exceed the "
                               "built-in buffer of %lld (use mortar_gemv_bf16 with a workspace, fewer streams per call or a "
                               "work list with fewer slots)", (long long)need, (long long)NOALLOC_FLOATS);
        if ((rc = scratch_for_current_device(&part))) return rc;
    }
    // every slot the combine pass reads is written by the entries of this same call (skipped units write zeros), so
    // nothing in the shared buffer has to be cleared first
    return gemv_run("gemv_noalloc", W, entries, n_entries, nslots, row_slots, kseg, mode, x, B, ldx, y, ldy, part, gates,
                    n_clusters, ldg, row_act, ldr, col_act, ldc, stream);
}
