// Weight gradient on the carved topology: out[j] = a[:, rows of block j]^T @ b[:, columns of block j].
//
// Reference: stk_sdd_at_b (morph/sparse/stk/backend/custom_ops.py:78-96) -> _sdd_kernel
// (morph/sparse/stk/backend/triton_kernels.py): one 16x16 output tile per kept block, contracted over the M tokens,
// bf16 operands, fp32 accumulation, output in the operand dtype.
//
// Shape of the work: the contraction runs over tokens, so both MFMA operands need 8 tokens of ONE feature per lane
// while memory holds 16 features of ONE token per 32 bytes.  The slices are staged row-major with direct
// global->LDS loads (whole 128-byte lines: 4 block-columns of 8 tokens per instruction) and read back with the
// transposing LDS load (ds_read_b64_tr_b16): 16 lanes hand in the addresses of 4 token rows x 4 pieces of 4
// features and each lane gets 4 tokens of one feature.  A workgroup keeps the fp32 tiles of up to WAVES*NB blocks of
// a few consecutive block-rows in registers and walks the tokens in steps of 32; per step it stages the
// 32 x (columns of its K segment) slice of b once and the slice of a for its rows, into one of two buffers: the
// loads of the next step are in flight while the current one multiplies.  Workgroup ids are laid out per XCD (each
// has its own L2) as runs of (token range, row group) pairs with the K segments of a pair side by side, so that a
// slice of a is fetched from HBM once and a slice of b only by the XCDs that hold its token range.  Every token range
// writes its fp32 sums to its own slab of the workspace; a last pass adds the slabs in a fixed order and rounds to
// bf16, so results are reproducible.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <climits>
#include <cstdint>
#include <vector>

#include "mortar_internal.h"

namespace {

constexpr int SDD_WAVES = 16;
constexpr int SDD_NB_MAX = 22;                   // most blocks per wavefront (4 accumulator registers each)
constexpr int SDD_NB_SIZES[] = {8, 10, 12, 14, 16, 18, 20, 22};      // the kernels that are built
constexpr int SDD_RMAX = 32;                     // block-rows per workgroup (slice of a in LDS)
constexpr int SDD_SEG = 44;                      // block-columns per K segment (slice of b in LDS)
constexpr int SDD_TARGET_WGS = 256;              // workgroups wanted in flight (one per CU: two slice buffers each)
constexpr int SDD_NQ = SDD_SEG / 4;              // quads of block-columns per segment
constexpr int SDD_CS = 1024 + 32;                // LDS bytes per chunk = 8 tokens x 128 bytes (a quad's line) + skew
constexpr int SDD_QS = 4 * SDD_CS;               // LDS bytes per quad: 32 tokens
constexpr int SDD_BUF = (SDD_NQ + SDD_RMAX / 4) * SDD_QS;    // one buffer: the slice of b, then the slice of a
constexpr int SDD_STEP = 32;                     // tokens per step = K of one MFMA
constexpr int SDD_SLAB_BLOCKS = 272;             // blocks of one fp32 slab (written, read back) that cost one unit
#ifndef SDD_PF
#define SDD_PF 1
#endif

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
    int32_t Cb, tsplit, steps_per_split, nsteps, nnz, per_xcd;
};

__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

// 8 tokens of one feature (= lane & 15) of the block-column (or block-row) whose first token sits at LDS byte `tile`:
// group g = lane >> 4 gets tokens {8r + g} and {8r + 4 + g}, r = 0..3 - one token of each 8-token chunk per read, which
// spreads the 32 lanes served together over all banks.  Both operands use the same order, so the contraction is
// unchanged.  `off` = this lane's row/piece address inside the quad.
__device__ __forceinline__ bf16x8 read_tr(const char *smem, int tile, int off) {
    typedef __attribute__((address_space(3))) s16x4 *lds_ptr;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(smem + tile + off));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(smem + tile + off + 4 * 128));
    union { s16x4 h[2]; bf16x8 v; } u;
    u.h[0] = lo;
    u.h[1] = hi;
    return u.v;
}

// Asynchronous 16-byte-per-lane copy global -> LDS: lane l's 16 bytes land at lds_base + 16 * l.  Written as inline
// assembly so that the compiler does not make the LDS reads of the other buffer wait for it; the caller waits with
// s_waitcnt vmcnt(0) and a barrier before the destination is read.  (One wait state separates the write of M0 from
// its use as the LDS base.)
__device__ __forceinline__ void load_to_lds_async(const void *gsrc, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(gsrc) : "memory", "m0");
}

__device__ __forceinline__ uint32_t lds_addr(const char *p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char *)p;
}

template <int SDD_NB>
__global__ __launch_bounds__(SDD_WAVES * 64) void sdd_kernel(SddArgs p) {
    constexpr int SDD_G = SDD_WAVES * SDD_NB;        // blocks per workgroup
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Workgroup -> (token range, row group, K segment).  Ids are dealt round-robin over the 8 XCDs, each with its own
    // L2.  The (token range, workgroup) items, workgroups in the plan's order (row groups of about the same rows side by
    // side over the K segments), are cut into 8 equal runs, one per XCD: the slice of a is then fetched from HBM once
    // (its nseg readers share an L2) and a slice of b only by the few XCDs that hold its token range.
    const int n_wg = p.plan[0];
    const int32_t *order = p.plan + p.plan[3];
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int item = xcd * p.per_xcd + slot;
    if (slot >= p.per_xcd || item >= p.tsplit * n_wg) return;
    const int ts = item / n_wg;
    const int wg = order[item - ts * n_wg];
    const int32_t *desc = p.plan + 4 + wg * 4;
    const int row0 = desc[0], nrows = desc[1], seg = desc[2];
    const int seg_cb = p.plan[1];
    const int c0 = seg * seg_cb;
    const int ncb = min(seg_cb, p.Cb - c0);
    const int nq = (ncb + 3) >> 2, nrq = (nrows + 3) >> 2;          // quads of block-columns / block-rows
    // this wavefront's blocks: block index (-1 = none) and (row slot << 20 | LDS byte offset of the column's tile);
    // the second list stays in scalar registers for the whole kernel
    const int32_t *ent_j = p.plan + 4 + n_wg * 4 + (int64_t)(wg * SDD_WAVES + wave) * SDD_NB;
    const int32_t *ent_o = ent_j + (int64_t)n_wg * SDD_G;
    int eo[SDD_NB];
#pragma unroll
    for (int b = 0; b < SDD_NB; ++b) eo[b] = __builtin_amdgcn_readfirstlane(ent_o[b]);
    uint32_t new_row = 1u;                // bit b: slot b is in another block-row than slot b - 1 (reload the a operand)
#pragma unroll
    for (int b = 1; b < SDD_NB; ++b) new_row |= (uint32_t)((eo[b] >> 20) != (eo[b - 1] >> 20)) << b;
    new_row = __builtin_amdgcn_readfirstlane(new_row);
    f32x4 acc[SDD_NB];
#pragma unroll
    for (int b = 0; b < SDD_NB; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int tr_off = ((lane & 15) >> 2) * SDD_CS + (lane >> 4) * 128 + (lane & 3) * 8;
    // staging role of this lane inside one instruction: token 8c + (lane >> 3), 16-byte piece lane & 7 of the 128-byte line
    const int st_tok = lane >> 3, st_piece = lane & 7;
    const int s_begin = ts * p.steps_per_split, s_end = min(p.nsteps, s_begin + p.steps_per_split);

    // Stage the slices of step s into buffer `buf` with direct global->LDS loads (asynchronous, no registers held).
    // One wavefront instruction moves 8 tokens x one 128-byte line (4 block-columns, or 4 block-rows of a) into 1 KB
    // of contiguous LDS.  Rows past M are not loaded; in the one partial step they are cleared with plain stores
    // (disjoint addresses from the loads).
    auto stage = [&](int s, int buf) {
        const int64_t t0 = (int64_t)s * SDD_STEP;
        char *dst = smem + buf * SDD_BUF;
        const bool partial = t0 + SDD_STEP > p.M;
        for (int i = wave; i < (nq + nrq) * 4; i += SDD_WAVES) {
            const int q = i >> 2, c = i & 3;
            const int64_t t = t0 + 8 * c + st_tok;
            const int qq = q < nq ? q : SDD_NQ + q - nq;
            if (partial && t >= p.M)
                *reinterpret_cast<u32x4 *>(dst + qq * SDD_QS + c * SDD_CS + lane * 16) = u32x4{0u, 0u, 0u, 0u};
            if (q < nq) {
                if (t < p.M && 4 * q + (st_piece >> 1) < ncb)
                    load_to_lds_async(p.b + t * p.ldb + (int64_t)(c0 + 4 * q) * 16 + st_piece * 8,
                                      __builtin_amdgcn_readfirstlane(lds_addr(dst + qq * SDD_QS + c * SDD_CS)));
            } else {
                if (t < p.M && 4 * (q - nq) + (st_piece >> 1) < nrows)
                    load_to_lds_async(p.a + t * p.lda + (int64_t)(row0 + 4 * (q - nq)) * 16 + st_piece * 8,
                                      __builtin_amdgcn_readfirstlane(lds_addr(dst + qq * SDD_QS + c * SDD_CS)));
            }
        }
    };

    if (s_begin < s_end) stage(s_begin, 0);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    int buf = 0;
    for (int s = s_begin; s < s_end; ++s) {
        if (s + 1 < s_end) stage(s + 1, buf ^ 1);            // in flight while this step multiplies
        const char *cur = smem + buf * SDD_BUF;
        // re-materialise the flag word every step: otherwise the 22 loop-invariant tests are hoisted as 22 lane masks
        uint32_t nr = new_row;
        asm volatile("" : "+s"(nr));
        nr = __builtin_amdgcn_readfirstlane(nr);
        bf16x8 A = {};
        // the b operand is fetched SDD_PF blocks ahead of its MFMA
        bf16x8 Bq[SDD_PF];
#pragma unroll
        for (int k = 0; k < SDD_PF; ++k) Bq[k] = read_tr(cur, eo[k] & 0xfffff, tr_off);
#pragma unroll
        for (int b = 0; b < SDD_NB; ++b) {
            if (nr & (1u << b)) {                 // (an empty slot repeats a valid tile: its sum is never stored)
                const int rs = eo[b] >> 20;
                A = read_tr(cur, SDD_NQ * SDD_QS + (rs >> 2) * SDD_QS + (rs & 3) * 32, tr_off);
            }
            const bf16x8 B = Bq[b % SDD_PF];
            if (b + SDD_PF < SDD_NB) Bq[b % SDD_PF] = read_tr(cur, eo[b + SDD_PF] & 0xfffff, tr_off);
            acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A, B, acc[b], 0, 0, 0);
        }
        __builtin_amdgcn_s_waitcnt(0);                       // the next step's slices have landed
        __syncthreads();                                     // ... for every wavefront, and this buffer is free again
        buf ^= 1;
    }
    // accumulator register r of lane (column = lane & 15, g = lane >> 4) is out[4g + r][column]
    const int oc = lane & 15, og = lane >> 4;
    float *part = p.acc + (int64_t)ts * p.nnz * 256;
#pragma unroll
    for (int b = 0; b < SDD_NB; ++b) {
        const int j = __builtin_amdgcn_readfirstlane(ent_j[b]);
        if (j >= 0) {
            const int64_t base = (int64_t)j * 256 + (4 * og) * 16 + oc;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if (p.tsplit > 1) part[base + r * 16] = acc[b][r];
                else p.out[base + r * 16] = f32_to_bf16(acc[b][r]);
            }
        }
    }
}

__global__ __launch_bounds__(256) void sdd_zero_kernel(float *acc, int64_t n4) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n4) reinterpret_cast<f32x4 *>(acc)[i] = f32x4{0.f, 0.f, 0.f, 0.f};
}

// out = bf16(sum over the token ranges, in range order)
__global__ __launch_bounds__(256) void sdd_round_kernel(const float *acc, uint16_t *out, int64_t n4, int tsplit) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n4) {
        f32x4 v = reinterpret_cast<const f32x4 *>(acc)[i];
        for (int t = 1; t < tsplit; ++t) v += reinterpret_cast<const f32x4 *>(acc)[i + (int64_t)t * n4];
        uint2 o;
        o.x = (uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
        o.y = (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
        reinterpret_cast<uint2 *>(out)[i] = o;
    }
}

}  // namespace

// Workgroups of a plan with `nb` blocks per wavefront: per K segment, runs of consecutive block-rows holding at most
// 16 * nb blocks of the segment and at most SDD_RMAX rows.
struct SddGroup { int row0, nrows, seg; std::vector<int32_t> j, o; };

static bool sdd_nb_built(int nb) {
    for (int v : SDD_NB_SIZES) if (v == nb) return true;
    return false;
}

static void sdd_groups(const int32_t *row_ptr, const int16_t *col, int Rb, int Cb, int nb, bool fill,
                       std::vector<SddGroup> &wgs, int &nseg, int &seg_cb) {
    const int G = SDD_WAVES * nb;
    nseg = (Cb + SDD_SEG - 1) / SDD_SEG;
    seg_cb = ((Cb + nseg - 1) / nseg + 3) & ~3;                    // whole 128-byte lines
    for (int sg = 0; sg < nseg; ++sg) {
        SddGroup cur{0, 0, sg, {}, {}};
        int held = 0;
        auto flush = [&]() {
            if (held) wgs.push_back(cur);
            cur = SddGroup{0, 0, sg, {}, {}};
            held = 0;
        };
        for (int r = 0; r < Rb; ++r) {
            int lo = row_ptr[r];
            const int e = row_ptr[r + 1];
            while (lo < e && col[lo] < sg * seg_cb) ++lo;
            int hi = lo;
            while (hi < e && col[hi] < (sg + 1) * seg_cb) ++hi;
            if (hi == lo) continue;
            if (held && (held + (hi - lo) > G || r - cur.row0 + 1 > SDD_RMAX)) flush();
            if (!held) cur.row0 = r;
            cur.nrows = r - cur.row0 + 1;
            held += hi - lo;
            if (!fill) continue;
            for (int j = lo; j < hi; ++j) {
                cur.j.push_back(j);
                const int cr = col[j] - sg * seg_cb;
                cur.o.push_back(((r - cur.row0) << 20) | ((cr >> 2) * SDD_QS + (cr & 3) * 32));
            }
        }
        flush();
    }
}

// Token ranges for M tokens over the n_wg workgroups of a plan with nb blocks per wavefront.  One workgroup runs per
// CU and the (range, workgroup) items are dealt evenly over the XCDs, so the launch takes
// ceil(items per XCD / CUs per XCD) rounds of ceil(steps / ranges) + 1 steps, a step costing nb + 7 units (one per
// block and wavefront, plus staging and the barrier); every extra range adds one slab of fp32 sums to write and to
// read back, priced per block.  The constants are a fit to launch times over group sizes, range counts and 1024 to
// 16384 tokens (4.5 % rms).  Returns the cost of the cheapest count of ranges.
static int64_t sdd_split(int32_t n_wg, int32_t nnz, int nb, int64_t M, int &nsteps, int &steps_per_split, int &tsplit) {
    nsteps = (int)((M + SDD_STEP - 1) / SDD_STEP);
    int best = 1;
    int64_t best_cost = INT64_MAX;
    for (int t = 1; t <= std::min(nsteps, 16); ++t) {
        const int sps = (nsteps + t - 1) / t, tt = (nsteps + sps - 1) / sps;
        const int64_t per_xcd = ((int64_t)n_wg * tt + 7) / 8;
        const int64_t rounds = (per_xcd + SDD_TARGET_WGS / 8 - 1) / (SDD_TARGET_WGS / 8);
        const int64_t cost = rounds * (sps + 1) * (nb + 7) + (tt > 1 ? (int64_t)tt * nnz / SDD_SLAB_BLOCKS : 0);
        if (cost < best_cost) { best_cost = cost; best = t; }
    }
    steps_per_split = std::max(1, (nsteps + best - 1) / best);
    tsplit = std::max(1, (nsteps + steps_per_split - 1) / steps_per_split);
    return best_cost;
}

// Blocks per wavefront for this topology at M tokens: the built size whose plan is cheapest by sdd_split's measure.
// Fewer blocks per workgroup mean more row groups, which fill the chip with fewer token ranges (fewer slabs), at the
// price of more staged bytes per block.
extern "C" int32_t mortar_sdd_blocks_per_wave_host(const int32_t *row_ptr, const int16_t *col, int32_t Rb, int32_t Cb, int64_t M) {
    const int rc = mortar_check_bcsr_host(row_ptr, col, Rb, Cb);
    if (rc) return rc;
    if (M < 0) return mortar_fail(MORTAR_ERR_ARG, "sdd_blocks_per_wave: M < 0");
    int best = SDD_NB_MAX;
    int64_t best_cost = INT64_MAX;
    for (int nb : SDD_NB_SIZES) {
        std::vector<SddGroup> wgs;
        int nseg, seg_cb, nsteps, sps, tsplit;
        sdd_groups(row_ptr, col, Rb, Cb, nb, false, wgs, nseg, seg_cb);
        const int64_t cost = sdd_split((int32_t)wgs.size(), row_ptr[Rb], nb, M, nsteps, sps, tsplit);
        if (cost <= best_cost) { best_cost = cost; best = nb; }      // ties: the larger group (fewer staged bytes)
    }
    return best;
}

// Plan: {n_wg, seg_cb, nseg, offset of the launch order}, then per workgroup {first row, rows, segment, blocks}, then
// per (workgroup, wavefront, slot) the block index or -1, then per (workgroup, wavefront, slot)
// (row - first row) << 20 | LDS byte offset of the tile of (column - segment start); an empty slot repeats the
// workgroup's last block there; last the launch order: the workgroups (stored segment by segment) sorted by their
// position inside the segment, then by segment, so that row groups of about the same rows are neighbours.
extern "C" int64_t mortar_sdd_plan_host(const int32_t *row_ptr, const int16_t *col, int32_t Rb, int32_t Cb,
                                        int32_t blocks_per_wave, int32_t *plan_out, int64_t plan_words) {
    const int rc = mortar_check_bcsr_host(row_ptr, col, Rb, Cb);
    if (rc) return rc;
    if (!sdd_nb_built(blocks_per_wave))
        return mortar_fail(MORTAR_ERR_ARG, "sdd_plan: blocks_per_wave=%d is not a built size (8, 10, ... 22)", blocks_per_wave);
    const int SDD_G = SDD_WAVES * blocks_per_wave;
    std::vector<SddGroup> wgs;
    int nseg, seg_cb;
    sdd_groups(row_ptr, col, Rb, Cb, blocks_per_wave, true, wgs, nseg, seg_cb);
    const int64_t n_wg = (int64_t)wgs.size();
    const int64_t tab = 4 + n_wg * 4 + n_wg * SDD_G * 2;          // word offset of the per-segment table
    const int64_t words = tab + n_wg;
    if (tab > INT32_MAX) return mortar_fail(MORTAR_ERR_LIMIT, "sdd_plan: plan too large");
    if (!plan_out) return words;
    if (plan_words < words) return mortar_fail(MORTAR_ERR_ARG, "sdd_plan: buffer holds %lld words, need %lld",
                                               (long long)plan_words, (long long)words);
    plan_out[0] = (int32_t)n_wg; plan_out[1] = seg_cb; plan_out[2] = nseg; plan_out[3] = (int32_t)tab;
    {
        std::vector<int> first(nseg + 1, 0);                       // first workgroup of every segment
        for (int64_t w = 0; w < n_wg; ++w) first[wgs[w].seg + 1] = (int)w + 1;
        for (int sg = 0; sg < nseg; ++sg) first[sg + 1] = std::max(first[sg + 1], first[sg]);
        int32_t *order = plan_out + tab;
        int64_t n = 0;
        for (int k = 0; n < n_wg; ++k)
            for (int sg = 0; sg < nseg; ++sg)
                if (first[sg] + k < first[sg + 1]) order[n++] = first[sg] + k;
    }
    int32_t *ent_j = plan_out + 4 + n_wg * 4, *ent_o = ent_j + n_wg * SDD_G;
    for (int64_t w = 0; w < n_wg; ++w) {
        int32_t *d = plan_out + 4 + w * 4;
        d[0] = wgs[w].row0; d[1] = wgs[w].nrows; d[2] = wgs[w].seg; d[3] = (int32_t)wgs[w].j.size();
        for (int i = 0; i < SDD_G; ++i) {
            const bool ok = i < (int)wgs[w].j.size();
            ent_j[w * SDD_G + i] = ok ? wgs[w].j[i] : -1;
            ent_o[w * SDD_G + i] = ok ? wgs[w].o[i] : wgs[w].o.back();
        }
    }
    return words;
}

extern "C" int64_t mortar_sdd_workspace_bytes(int32_t n_wg, int32_t nnz, int32_t blocks_per_wave, int64_t M) {
    if (n_wg <= 0 || nnz <= 0 || M < 0 || !sdd_nb_built(blocks_per_wave))
        return mortar_fail(MORTAR_ERR_ARG, "sdd_workspace_bytes: bad argument");
    int nsteps, sps, tsplit;
    sdd_split(n_wg, nnz, blocks_per_wave, M, nsteps, sps, tsplit);
    return (int64_t)tsplit * nnz * 256 * (int64_t)sizeof(float);
}

template <int NB>
static hipError_t sdd_launch(const SddArgs &p, hipStream_t st) {
    static bool configured = false;
    const int smem = 2 * SDD_BUF;
    if (!configured) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(sdd_kernel<NB>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) return e;
        configured = true;
    }
    hipLaunchKernelGGL(sdd_kernel<NB>, dim3((unsigned)(8 * p.per_xcd)), dim3(SDD_WAVES * 64), smem, st, p);
    return hipSuccess;
}

extern "C" int mortar_sdd_bf16(const int32_t *plan, int32_t n_wg, int32_t blocks_per_wave,
                               int32_t Rb, int32_t Cb, int32_t nnz,
                               const uint16_t *a, int64_t lda, const uint16_t *b, int64_t ldb, int64_t M,
                               float *acc, uint16_t *out, void *stream) {
    if (!plan || !out || !acc || (M > 0 && (!a || !b))) return mortar_fail(MORTAR_ERR_ARG, "sdd: null pointer");
    if (n_wg <= 0 || Rb <= 0 || Cb <= 0 || nnz <= 0 || M < 0) return mortar_fail(MORTAR_ERR_ARG, "sdd: bad shape");
    if (!sdd_nb_built(blocks_per_wave))
        return mortar_fail(MORTAR_ERR_ARG, "sdd: blocks_per_wave=%d is not a built size (8, 10, ... 22)", blocks_per_wave);
    if (reinterpret_cast<uintptr_t>(out) & 15) return mortar_fail(MORTAR_ERR_ARG, "sdd: out must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (M == 0) {                                          // no tokens: the gradient is zero
        hipLaunchKernelGGL(sdd_zero_kernel, dim3((unsigned)(((int64_t)nnz * 32 + 255) / 256)), dim3(256), 0, st,
                           reinterpret_cast<float *>(out), (int64_t)nnz * 32);
        return MORTAR_OK;
    }
    if (lda < (int64_t)Rb * 16 || ldb < (int64_t)Cb * 16 || (lda & 7) || (ldb & 7) ||
        (reinterpret_cast<uintptr_t>(a) & 15) || (reinterpret_cast<uintptr_t>(b) & 15) ||
        (reinterpret_cast<uintptr_t>(acc) & 15))
        return mortar_fail(MORTAR_ERR_ARG, "sdd: operands need 16-byte aligned rows (leading dimensions multiples of 8)");
    const int64_t n4 = (int64_t)nnz * 64;
    SddArgs p;
    p.plan = plan; p.a = a; p.b = b; p.lda = lda; p.ldb = ldb; p.M = M; p.acc = acc; p.out = out;
    p.Cb = Cb; p.nnz = nnz;
    sdd_split(n_wg, nnz, blocks_per_wave, M, p.nsteps, p.steps_per_split, p.tsplit);
    p.per_xcd = (p.tsplit * n_wg + 7) / 8;
    hipError_t e = hipSuccess;
    switch (blocks_per_wave) {
        case 8: e = sdd_launch<8>(p, st); break;
        case 10: e = sdd_launch<10>(p, st); break;
        case 12: e = sdd_launch<12>(p, st); break;
        case 14: e = sdd_launch<14>(p, st); break;
        case 16: e = sdd_launch<16>(p, st); break;
        case 18: e = sdd_launch<18>(p, st); break;
        case 20: e = sdd_launch<20>(p, st); break;
        default: e = sdd_launch<22>(p, st); break;
    }
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    if (p.tsplit > 1)
        hipLaunchKernelGGL(sdd_round_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, st, acc, out, n4, p.tsplit);
    e = hipGetLastError();
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "sdd: %s", hipGetErrorString(e));
    return MORTAR_OK;
}
