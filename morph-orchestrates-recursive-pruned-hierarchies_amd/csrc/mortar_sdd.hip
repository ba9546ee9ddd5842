// Weight gradient on the carved topology: out[j] = a[:, rows of block j]^T @ b[:, columns of block j].
//
// Reference: stk_sdd_at_b (morph/sparse/stk/backend/custom_ops.py:78-96) -> _sdd_kernel
// (morph/sparse/stk/backend/triton_kernels.py): one 16x16 output tile per kept block, contracted over the M tokens,
// bf16 operands, fp32 accumulation, output in the operand dtype.
//
// Shape of the work: the contraction runs over tokens, so both MFMA operands need 8 tokens of ONE feature per lane
// while memory holds 16 features of ONE token per 32 bytes.  The tiles are staged row-major (straight 16-byte
// copies) and read back with the transposing LDS load (ds_read_b64_tr_b16): 16 lanes hand in the addresses of 4
// token rows x 4 chunks of 4 features and each lane gets 4 tokens of one feature.  A workgroup keeps the fp32 tiles
// of up to WAVES*NB blocks of a few consecutive block-rows in registers and walks the tokens in steps of 32; per
// step it stages the 32 x (columns of its K segment) slice of b once and the slice of a for its rows.  Workgroups
// that share a token range run on the same XCD (the range index is the low part of the workgroup index), so the
// slice of b is fetched from HBM about once per XCD and served from L2 after that.  Token ranges are combined with
// fp32 atomic adds into a workspace; a last pass rounds to bf16.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <vector>

#include "mortar_internal.h"

namespace {

constexpr int SDD_WAVES = 16;
constexpr int SDD_NB = 22;                       // blocks per wavefront (4 accumulator registers each)
constexpr int SDD_G = SDD_WAVES * SDD_NB;        // blocks per workgroup
constexpr int SDD_RMAX = 16;                     // block-rows per workgroup (slice of a in LDS)
constexpr int SDD_SEG = 128;                     // block-columns per K segment (slice of b in LDS)
constexpr int SDD_XS = 1024 + 32;                // bytes per (block-column, 32 tokens) tile: 32 B per token + skew
constexpr int SDD_STEP = 32;                     // tokens per step = K of one MFMA

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct SddArgs {
    const int32_t *plan;
    const uint16_t *a, *b;
    int64_t lda, ldb, M;
    float *acc;
    uint16_t *out;
    int32_t Cb, seg_cb, tsplit, steps_per_split, nsteps;
};

__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

// 8 tokens of one feature: tokens 4g .. 4g+3 and 16+4g .. 16+4g+3 of the 32-token tile at `tile` (LDS byte address of
// a [32 tokens][16 features] bf16 tile), feature = lane & 15, g = lane >> 4.  `off` = this lane's chunk address.
__device__ __forceinline__ bf16x8 read_tr(const char *smem, int tile, int off) {
    typedef __attribute__((address_space(3))) s16x4 *lds_ptr;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(smem + tile + off));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(smem + tile + off + 16 * 32));
    union { s16x4 h[2]; bf16x8 v; } u;
    u.h[0] = lo;
    u.h[1] = hi;
    return u.v;
}

__global__ __launch_bounds__(SDD_WAVES * 64) void sdd_kernel(SddArgs p) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ts = blockIdx.x % p.tsplit, wg = blockIdx.x / p.tsplit;
    const int n_wg = p.plan[0];
    const int32_t *desc = p.plan + 4 + wg * 4;
    const int row0 = desc[0], nrows = desc[1], seg = desc[2];
    const int c0 = seg * p.seg_cb;
    const int ncb = min(p.seg_cb, p.Cb - c0);
    // this wavefront's blocks: block index (-1 = none) and (row slot << 16 | column in the segment) (-1 = none)
    const int32_t *ent_j = p.plan + 4 + n_wg * 4 + (int64_t)(wg * SDD_WAVES + wave) * SDD_NB;
    const int32_t *ent_o = ent_j + (int64_t)n_wg * SDD_G;
    f32x4 acc[SDD_NB];
#pragma unroll
    for (int b = 0; b < SDD_NB; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int a_base = SDD_SEG * SDD_XS;                                     // slice of a behind the slice of b
    const int tr_off = (4 * (lane >> 4) + ((lane & 15) >> 2)) * 32 + (lane & 3) * 8;
    const int s_begin = ts * p.steps_per_split, s_end = min(p.nsteps, s_begin + p.steps_per_split);
    for (int s = s_begin; s < s_end; ++s) {
        const int64_t t0 = (int64_t)s * SDD_STEP;
        __syncthreads();                                                      // previous step's reads are done
        // slice of b: 32 tokens x ncb block-columns; a wavefront copies whole token rows, 16 bytes per lane
        for (int tok = wave; tok < SDD_STEP; tok += SDD_WAVES) {
            const bool live = t0 + tok < p.M;
            const uint16_t *src = p.b + (t0 + tok) * p.ldb + (int64_t)c0 * 16;
            for (int ch = lane; ch < ncb * 2; ch += 64) {
                u32x4 v = {0u, 0u, 0u, 0u};
                if (live) v = *reinterpret_cast<const u32x4 *>(src + ch * 8);
                *reinterpret_cast<u32x4 *>(smem + (ch >> 1) * SDD_XS + tok * 32 + (ch & 1) * 16) = v;
            }
        }
        // slice of a: 32 tokens x nrows block-rows
        for (int idx = tid; idx < SDD_STEP * SDD_RMAX * 2; idx += SDD_WAVES * 64) {
            const int tok = idx >> 5, rs = (idx >> 1) & (SDD_RMAX - 1), half = idx & 1;
            if (rs < nrows) {
                u32x4 v = {0u, 0u, 0u, 0u};
                if (t0 + tok < p.M)
                    v = *reinterpret_cast<const u32x4 *>(p.a + (t0 + tok) * p.lda + (int64_t)(row0 + rs) * 16 + half * 8);
                *reinterpret_cast<u32x4 *>(smem + a_base + rs * SDD_XS + tok * 32 + half * 16) = v;
            }
        }
        __syncthreads();
        // the entries are read again every step (scalar loads) instead of living in registers across the loop
        const int32_t *eo = ent_o;
        asm volatile("" : "+s"(eo));
        int rs_prev = -1;
        bf16x8 A = {};
#pragma unroll
        for (int b = 0; b < SDD_NB; ++b) {
            const int e = eo[b];
            if (e >= 0) {
                const int rs = e >> 16, cr = e & 0xffff;
                if (rs != rs_prev) {
                    A = read_tr(smem, a_base + rs * SDD_XS, tr_off);
                    rs_prev = rs;
                }
                const bf16x8 B = read_tr(smem, cr * SDD_XS, tr_off);
                acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A, B, acc[b], 0, 0, 0);
            }
        }
    }
    // accumulator register r of lane (column = lane & 15, g = lane >> 4) is out[4g + r][column]
    const int oc = lane & 15, og = lane >> 4;
#pragma unroll
    for (int b = 0; b < SDD_NB; ++b) {
        const int j = ent_j[b];
        if (j >= 0) {
            const int64_t base = (int64_t)j * 256 + (4 * og) * 16 + oc;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if (p.tsplit > 1) atomicAdd(p.acc + base + r * 16, acc[b][r]);
                else p.out[base + r * 16] = f32_to_bf16(acc[b][r]);
            }
        }
    }
}

__global__ __launch_bounds__(256) void sdd_zero_kernel(float *acc, int64_t n4) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n4) reinterpret_cast<f32x4 *>(acc)[i] = f32x4{0.f, 0.f, 0.f, 0.f};
}

__global__ __launch_bounds__(256) void sdd_round_kernel(const float *acc, uint16_t *out, int64_t n4) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n4) {
        const f32x4 v = reinterpret_cast<const f32x4 *>(acc)[i];
        uint2 o;
        o.x = (uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
        o.y = (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
        reinterpret_cast<uint2 *>(out)[i] = o;
    }
}

}  // namespace

// Plan: {n_wg, seg_cb, nseg, 0}, then per workgroup {first row, rows, segment, blocks}, then per (workgroup, wavefront,
// slot) the block index or -1, then per (workgroup, wavefront, slot) (row - first row) << 16 | (column - segment start)
// or -1.
extern "C" int64_t mortar_sdd_plan_host(const int32_t *row_ptr, const int16_t *col, int32_t Rb, int32_t Cb,
                                        int32_t *plan_out, int64_t plan_words) {
    const int rc = mortar_check_bcsr_host(row_ptr, col, Rb, Cb);
    if (rc) return rc;
    const int nseg = (Cb + SDD_SEG - 1) / SDD_SEG;
    const int seg_cb = (Cb + nseg - 1) / nseg;
    struct Wg { int row0, nrows, seg; std::vector<int32_t> j, o; };
    std::vector<Wg> wgs;
    for (int sg = 0; sg < nseg; ++sg) {
        Wg cur{0, 0, sg, {}, {}};
        auto flush = [&]() {
            if (!cur.j.empty()) wgs.push_back(cur);
            cur = Wg{0, 0, sg, {}, {}};
        };
        for (int r = 0; r < Rb; ++r) {
            int lo = row_ptr[r];
            const int e = row_ptr[r + 1];
            while (lo < e && col[lo] < sg * seg_cb) ++lo;
            int hi = lo;
            while (hi < e && col[hi] < (sg + 1) * seg_cb) ++hi;
            if (hi == lo) continue;
            if (!cur.j.empty() && ((int)cur.j.size() + (hi - lo) > SDD_G || r - cur.row0 + 1 > SDD_RMAX)) flush();
            if (cur.j.empty()) cur.row0 = r;
            cur.nrows = r - cur.row0 + 1;
            for (int j = lo; j < hi; ++j) {
                cur.j.push_back(j);
                cur.o.push_back(((r - cur.row0) << 16) | (col[j] - sg * seg_cb));
            }
        }
        flush();
    }
    const int64_t n_wg = (int64_t)wgs.size();
    const int64_t words = 4 + n_wg * 4 + n_wg * SDD_G * 2;
    if (!plan_out) return words;
    if (plan_words < words) return mortar_fail(MORTAR_ERR_ARG, "sdd_plan: buffer holds %lld words, need %lld",
                                               (long long)plan_words, (long long)words);
    plan_out[0] = (int32_t)n_wg; plan_out[1] = seg_cb; plan_out[2] = nseg; plan_out[3] = 0;
    int32_t *ent_j = plan_out + 4 + n_wg * 4, *ent_o = ent_j + n_wg * SDD_G;
    for (int64_t w = 0; w < n_wg; ++w) {
        int32_t *d = plan_out + 4 + w * 4;
        d[0] = wgs[w].row0; d[1] = wgs[w].nrows; d[2] = wgs[w].seg; d[3] = (int32_t)wgs[w].j.size();
        for (int i = 0; i < SDD_G; ++i) {
            const bool ok = i < (int)wgs[w].j.size();
            ent_j[w * SDD_G + i] = ok ? wgs[w].j[i] : -1;
            ent_o[w * SDD_G + i] = ok ? wgs[w].o[i] : -1;
        }
    }
    return words;
}

extern "C" int mortar_sdd_bf16(const int32_t *plan, int32_t n_wg, int32_t Rb, int32_t Cb, int32_t nnz,
                               const uint16_t *a, int64_t lda, const uint16_t *b, int64_t ldb, int64_t M,
                               float *acc, uint16_t *out, void *stream) {
    if (!plan || !out || !acc || (M > 0 && (!a || !b))) return mortar_fail(MORTAR_ERR_ARG, "sdd: null pointer");
    if (n_wg <= 0 || Rb <= 0 || Cb <= 0 || nnz <= 0 || M < 0) return mortar_fail(MORTAR_ERR_ARG, "sdd: bad shape");
    if (reinterpret_cast<uintptr_t>(out) & 15) return mortar_fail(MORTAR_ERR_ARG, "sdd: out must be 16-byte aligned");
    if (M == 0) {                                          // no tokens: the gradient is zero
        hipLaunchKernelGGL(sdd_zero_kernel, dim3((unsigned)(((int64_t)nnz * 32 + 255) / 256)), dim3(256), 0,
                           static_cast<hipStream_t>(stream), reinterpret_cast<float *>(out), (int64_t)nnz * 32);
        return MORTAR_OK;
    }
    if (lda < (int64_t)Rb * 16 || ldb < (int64_t)Cb * 16 || (lda & 7) || (ldb & 7) ||
        (reinterpret_cast<uintptr_t>(a) & 15) || (reinterpret_cast<uintptr_t>(b) & 15) ||
        (reinterpret_cast<uintptr_t>(acc) & 15) || (reinterpret_cast<uintptr_t>(out) & 15))
        return mortar_fail(MORTAR_ERR_ARG, "sdd: operands need 16-byte aligned rows (leading dimensions multiples of 8)");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t n4 = (int64_t)nnz * 64;
    const int nseg = (Cb + SDD_SEG - 1) / SDD_SEG;
    SddArgs p;
    p.plan = plan; p.a = a; p.b = b; p.lda = lda; p.ldb = ldb; p.M = M; p.acc = acc; p.out = out;
    p.Cb = Cb; p.seg_cb = (Cb + nseg - 1) / nseg;
    p.nsteps = (int)((M + SDD_STEP - 1) / SDD_STEP);
    int tsplit = std::max(1, std::min(p.nsteps, (256 + n_wg - 1) / n_wg));
    p.steps_per_split = (p.nsteps + tsplit - 1) / tsplit;
    p.tsplit = (p.nsteps + p.steps_per_split - 1) / p.steps_per_split;
    static bool configured = false;
    const int smem = (SDD_SEG + SDD_RMAX) * SDD_XS;
    if (!configured) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(sdd_kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
        configured = true;
    }
    if (p.tsplit > 1)
        hipLaunchKernelGGL(sdd_zero_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, st, acc, n4);
    hipLaunchKernelGGL(sdd_kernel, dim3((unsigned)(n_wg * p.tsplit)), dim3(SDD_WAVES * 64), smem, st, p);
    if (p.tsplit > 1)
        hipLaunchKernelGGL(sdd_round_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, st, acc, out, n4);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "sdd: %s", hipGetErrorString(e));
    return MORTAR_OK;
}
