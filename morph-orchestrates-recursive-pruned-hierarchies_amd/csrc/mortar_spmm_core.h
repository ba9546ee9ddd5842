// Octet-stream SpMM kernels shared by the prefill (large M) and decode (M <= 64) entry points.
//
// Both kernels keep a token tile of the activations in LDS and let every wavefront walk whole row units of
// the octet weight stream: unpack the ternary codes of two blocks in registers, read the activation operand
// from LDS, one 16x16x32 bf16 MFMA per 16 tokens.  They differ in how much of K the LDS tile holds:
//   mortar_resident_kernel   all of in_features (no K loop, one barrier); the K segments of the stream are
//                            walked back to back against the one resident tile
//   mortar_segmented_kernel  one K segment at a time (a barrier pair per segment); a wave owns UPW row units
//                            whose accumulators stay in registers across the segments
// A launch can carry several independent problems of one shape ("layers"): blockIdx.y then selects an entry
// of a parameter table in device memory.
#ifndef MORTAR_SPMM_CORE_H
#define MORTAR_SPMM_CORE_H

#include "mortar_device.h"
#include "mortar_internal.h"

struct SpmmParams {
    const u32x4_t *row_desc;  // octet stream: {first octet, end octet, blocks, 0} per (segment, block-row)
    const u32x4_t *codes_o;
    const u32x4_t *sd_o;
    const u32x4_t *col_o;
    const u32x4_t *sched;     // part descriptors {first octet, end octet, blocks, unit} in schedule order
                              // [(position * nseg + segment) * rows_per_unit + a], or null: position = unit
    const uint16_t *x;
    uint16_t *y;
    const float *gates;       // [M, n_clusters] fp32 or null
    const uint8_t *active;    // [M, n_clusters] input mask or null
    const int32_t *tok_cnt;   // routed: [n_mtiles, n_clusters]
    const uint8_t *tok_list;  // routed: [n_mtiles, n_clusters, MT]
    int64_t ldx, ldy;
    int n_units, Cb, M, Rb;
    int n_clusters, cluster_size;
    int n_mtiles, n_split;    // token tiles; workgroups that share one token tile
    int seg_cb, nseg;         // K segments of the octet stream
    int xcd_map;              // 1: workgroup ids are renumbered per XCD (grid padded to a multiple of 8)
    int norm;                 // 1: rows of x are RMS-normalised while they are staged (single-segment tiles only)
    float norm_eps;
    float uscale;             // CODE_UNIFORM kernels: half the matrix's (bf16-rounded) scale
    float *y32;               // plain products: unrounded fp32 output [M, ldy] in place of the bf16 store, or null
    const uint16_t *norm_w;   // bf16 [in_features] weight of that norm, or null for none
    // hyper-connection POST write in place of the plain store (small tiles, plain products): out[t, i, :] =
    // sum_j hc_res[t, i, j] * hc_h[t, j, :] + hc_post[t, i] * y[t, :] (+ hc_term[t, :]); null hc_h = plain store
    const void *hc_h;         // carrier streams [M, hc_n, out_features], bf16 or fp32 (hc_f32)
    void *hc_out;             // result, same shape and type as hc_h
    const float *hc_res;      // [M, hc_n, hc_n]
    const float *hc_post;     // [M, hc_n]
    const void *hc_term;      // [M, out_features], type of hc_h, or null
    int hc_n, hc_f32;
    // Hidden activations of the two-launch MLP in tile order instead of row-major (mortar_mlp_bf16): element (token, f)
    // at ((token / 32) * (features / 16) + f / 16) * 512 + (token % 32) * 16 + f % 16, i.e. the 32 tokens x 16 features
    // of one (token tile, block-column) are 1 KB of contiguous memory: gate_up's stores of a 16 x 16 result tile are 512
    // contiguous bytes, and `down` stages a K segment of its token tile as one contiguous run, asynchronously, straight
    // into LDS.  y_tiled: the SwiGLU epilogue stores so; x_tiled: the 32-token prefill tiles are staged from it.
    int x_tiled, y_tiled, pad0_, pad1_;
};

// Device-side view of the launch parameters: the pointers carry the global address space in their type, so
// that every access compiles to global_load / global_store (a pointer read from a parameter table in memory
// would otherwise be generic and cost flat instructions).
#define MORTAR_GLOBAL __attribute__((address_space(1)))
struct SpmmView {
    const MORTAR_GLOBAL u32x4_t *row_desc, *codes_o, *sched;
    const MORTAR_GLOBAL uint32_t *sd_dw, *cc_dw;      // scale patterns / block-columns of the octet stream as dwords
    const MORTAR_GLOBAL char *x;
    MORTAR_GLOBAL uint16_t *y;
    MORTAR_GLOBAL float *y32;
    const MORTAR_GLOBAL float *gates;
    const MORTAR_GLOBAL uint8_t *active;
    const MORTAR_GLOBAL int32_t *tok_cnt;
    const MORTAR_GLOBAL uint8_t *tok_list;
    int64_t ldx, ldy;
    int n_units, Cb, M, n_clusters, cluster_size, n_mtiles, n_split, seg_cb, nseg, Rb, xcd_map, norm;
    float norm_eps, uscale;
    const MORTAR_GLOBAL u32x4_t *norm_w;
    const MORTAR_GLOBAL char *hc_h, *hc_term;
    MORTAR_GLOBAL char *hc_out;
    const MORTAR_GLOBAL float *hc_res, *hc_post;
    int hc_n, hc_f32, x_tiled, y_tiled;
};
static_assert(sizeof(SpmmParams) % 16 == 0, "table entries are copied in 16-byte words");
// Entry i of a parameter table in device memory (uniform address: scalar loads).
__device__ __forceinline__ SpmmParams mortar_table_entry(const SpmmParams *table, unsigned i) {
    constexpr unsigned NW16 = sizeof(SpmmParams) / 16;
    union { SpmmParams p; u32x4_t w[NW16]; } u;
    const MORTAR_GLOBAL u32x4_t *src = (const MORTAR_GLOBAL u32x4_t *)table + (size_t)i * NW16;
#pragma unroll
    for (unsigned k = 0; k < NW16; ++k) u.w[k] = src[k];
    return u.p;
}
__device__ __forceinline__ SpmmView mortar_view(const SpmmParams &q) {
    SpmmView v;
    v.row_desc = (const MORTAR_GLOBAL u32x4_t *)q.row_desc; v.codes_o = (const MORTAR_GLOBAL u32x4_t *)q.codes_o;
    v.sched = (const MORTAR_GLOBAL u32x4_t *)q.sched;
    v.sd_dw = (const MORTAR_GLOBAL uint32_t *)q.sd_o; v.cc_dw = (const MORTAR_GLOBAL uint32_t *)q.col_o;
    v.x = (const MORTAR_GLOBAL char *)q.x; v.y = (MORTAR_GLOBAL uint16_t *)q.y; v.y32 = (MORTAR_GLOBAL float *)q.y32;
    v.gates = (const MORTAR_GLOBAL float *)q.gates; v.active = (const MORTAR_GLOBAL uint8_t *)q.active;
    v.tok_cnt = (const MORTAR_GLOBAL int32_t *)q.tok_cnt; v.tok_list = (const MORTAR_GLOBAL uint8_t *)q.tok_list;
    v.ldx = q.ldx; v.ldy = q.ldy; v.n_units = q.n_units; v.Cb = q.Cb; v.M = q.M; v.n_clusters = q.n_clusters;
    v.cluster_size = q.cluster_size; v.n_mtiles = q.n_mtiles; v.n_split = q.n_split; v.seg_cb = q.seg_cb; v.nseg = q.nseg; v.Rb = q.Rb; v.xcd_map = q.xcd_map;
    v.norm = q.norm; v.norm_eps = q.norm_eps; v.uscale = q.uscale; v.norm_w = (const MORTAR_GLOBAL u32x4_t *)q.norm_w;
    v.hc_h = (const MORTAR_GLOBAL char *)q.hc_h; v.hc_term = (const MORTAR_GLOBAL char *)q.hc_term;
    v.hc_out = (MORTAR_GLOBAL char *)q.hc_out; v.hc_res = (const MORTAR_GLOBAL float *)q.hc_res;
    v.hc_post = (const MORTAR_GLOBAL float *)q.hc_post; v.hc_n = q.hc_n; v.hc_f32 = q.hc_f32;
    v.x_tiled = q.x_tiled; v.y_tiled = q.y_tiled;
    return v;
}

// How a kernel reads the code stream (template parameter CODE): bit 0 = the 4-bit stream, bit 1 = one scale for the
// whole matrix (the reference's per-tensor mortar_scale): the blocks are multiplied as +-2 / 0 and the accumulators
// are scaled once in the epilogue, which saves the packed multiplies and the scale broadcast of every pair.
constexpr int CODE_2BIT = 0, CODE_4BIT = 1, CODE_UNIFORM = 2;

constexpr int MORTAR_SMALLM_MAX = 64;    // rows up to which the small-tile (decode) instantiations are used
constexpr int MORTAR_PARTSPLIT_MAX = 128; // rows up to which a plain product over several K segments runs 8-token tiles of all K
constexpr int RES_GROUPS = 4;            // octets (4 block pairs each) loaded per batch
constexpr int LDS_BUDGET = 156 * 1024;   // bytes of LDS a token tile may take
constexpr int LDS_PAD = 32;              // 16-byte units past the tile that idle lanes of a narrow tile may read

// Tile layout in LDS: [block-column][token][column half] in 16-byte units, i.e. the 32 bytes (16 values) of one token
// and block-column are adjacent and a block-column is a run of MT * 32 bytes.  The 32 lanes that fetch one block's MFMA
// operand (16 tokens x 2 column halves) then read 512 contiguous bytes, which ds_read_b128 serves at full rate
// (measured: 4.4 cycles per wave instruction, against 8.1 for any layout whose 16-lane windows are not aligned).
constexpr int tile_bytes(int mt, int ncb) { return ncb * mt * 32 + LDS_PAD * 16; }
constexpr int LDS_EXTRA = 16 + 256;      // bytes after the tile: the resident kernel's unit counter, per-row norm factors
constexpr int NORM_MAX_CB = 128;         // block-columns up to which a row fits the registers of the staging wave

// Lane k of every 16-lane row broadcast to the whole row (DPP row_newbcast); K must fold to a constant.
template <int K>
__device__ __forceinline__ uint32_t mortar_row_bcast_k(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x150 + K, 0xf, 0xf, true);
}
__device__ __forceinline__ uint32_t mortar_row_bcast(uint32_t v, int k) {
    switch (k) {
        case 0: return mortar_row_bcast_k<0>(v);   case 1: return mortar_row_bcast_k<1>(v);
        case 2: return mortar_row_bcast_k<2>(v);   case 3: return mortar_row_bcast_k<3>(v);
        case 4: return mortar_row_bcast_k<4>(v);   case 5: return mortar_row_bcast_k<5>(v);
        case 6: return mortar_row_bcast_k<6>(v);   case 7: return mortar_row_bcast_k<7>(v);
        case 8: return mortar_row_bcast_k<8>(v);   case 9: return mortar_row_bcast_k<9>(v);
        case 10: return mortar_row_bcast_k<10>(v); case 11: return mortar_row_bcast_k<11>(v);
        case 12: return mortar_row_bcast_k<12>(v); case 13: return mortar_row_bcast_k<13>(v);
        case 14: return mortar_row_bcast_k<14>(v); default: return mortar_row_bcast_k<15>(v);
    }
}

// s_setprio with a value that folds to a constant after unrolling (the instruction takes an immediate 0..3).
__device__ __forceinline__ void mortar_setprio(int p) {
    switch (p) {
        case 0: __builtin_amdgcn_s_setprio(0); break;
        case 1: __builtin_amdgcn_s_setprio(1); break;
        case 2: __builtin_amdgcn_s_setprio(2); break;
        default: __builtin_amdgcn_s_setprio(3); break;
    }
}

// One batch of the octet stream in registers: RES_GROUPS octets (8 blocks = 4 pairs each) = 16 block pairs.
// A lane holds its code dwords of the 16 pairs (one 16-byte load per octet) and, as lane k of its 16-lane row,
// the scale pattern and block-column of pair k (one dword each); pair u's metadata reaches the row by a DPP
// broadcast when it is used.
struct MortarBatch {
    u32x4_t cw[RES_GROUPS];
    uint32_t sdv, ccv;
};

// Loads the batch that starts at octet gq of a row part ending at octet g1 (octets past the end repeat the last).
// FP4: the code stream is the 4-bit one (a lane's dword holds the 8 codes of its own column half, so the four
// lane groups read four different 16-byte runs per octet instead of two).
// gq and g1 are wave-uniform, so every address is (stream base, scalar byte offset of the octet, per-lane constant):
// raw buffer loads take exactly these three and cost no address arithmetic on the vector ALU, which the kernels
// are short of (the one vector instruction left is the clamp of the metadata octet at the end of a part).
template <int CODE = 0>
__device__ __forceinline__ void mortar_load_batch(const SpmmView &p, MortarBatch &b, int gq, int g1, int n, int bsel,
                                                  int hsel = 0) {
    constexpr int OB = (CODE & CODE_4BIT) ? 1024 : 512;          // bytes of codes per octet
    const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc((void *)p.codes_o, 0, -1, 0x00020000);
    const int lane_c = (CODE & CODE_4BIT) ? ((bsel * 2 + hsel) * 16 + n) * 16 : (bsel * 16 + n) * 16;
#pragma unroll
    for (int k = 0; k < RES_GROUPS; ++k) {
        const int go = gq + k < g1 ? gq + k : g1 - 1;
        b.cw[k] = __builtin_amdgcn_raw_buffer_load_b128(rc, lane_c, go * OB, 0);
    }
    const uint32_t ko = (uint32_t)(n >> 2), last = (uint32_t)(g1 - 1 - gq);
    const int lane_m = (int)((ko < last ? ko : last) * 32u) + (bsel * 4 + (n & 3)) * 4;
    if (CODE & CODE_UNIFORM) b.sdv = 0u;
    else b.sdv = __builtin_amdgcn_raw_buffer_load_b32(__builtin_amdgcn_make_buffer_rsrc((void *)p.sd_dw, 0, -1, 0x00020000), lane_m, gq * 32, 0);
    b.ccv = __builtin_amdgcn_raw_buffer_load_b32(__builtin_amdgcn_make_buffer_rsrc((void *)p.cc_dw, 0, -1, 0x00020000), lane_m, gq * 32, 0);
}

// One row part: octets [g0, g1) (nb blocks) of the stream against the tile at `lx`.
// `xo_base` is the lane's byte offset inside a block-column (token, column half) plus the segment's origin.
// `b` holds the part's first batch, loaded by the caller (mortar_load_batch at g0) where it suits it.
// FIRST_ONLY: only the batch in `b` (the part's first RES_GROUPS octets) is multiplied and no load is issued here, so
// that a caller which keeps the next part's batch in flight gets a counted wait for `b` instead of a full one.
template <int MSUB, int MT, bool ROUTED, int CODE = 0, bool FIRST_ONLY = false>
__device__ __forceinline__ void mortar_row_part(const SpmmView &p, const uint4 *lx, MortarBatch b, int g0, int g1,
                                                int nb, uint32_t xo_base, const uint32_t (&tk)[MSUB], int nsub, int n,
                                                int bsel, int hsel, f32x4_t (&acc)[MSUB]) {
    const unsigned char *lb = reinterpret_cast<const unsigned char *>(lx);
    for (int gq = g0; gq < (FIRST_ONLY ? g0 + 1 : g1); gq += RES_GROUPS) {
        if (!FIRST_ONLY && gq != g0) mortar_load_batch<CODE>(p, b, gq, g1, n, bsel, hsel);
        const uint32_t ccs = __umul24(b.ccv, (uint32_t)(MT * 32));   // byte offset of the block-column in the tile
        const int pairs = ((nb - (gq - g0) * 8) + 1) >> 1;      // block pairs left in the row from this batch on
        // Activation operands are fetched two pairs ahead of the MFMAs that use them.  The only branches are
        // per octet (a whole octet past the end of the part is skipped) and, for prefill tiles, per half octet;
        // otherwise the pairs run straight, pairs past the end being the all-zero padding blocks of the stream.
        constexpr int NP = 4 * RES_GROUPS;
        constexpr int PD = MT == 64 ? 1 : 2;      // pairs ahead (the distance makes no difference in time; the 64-token tile has no registers to spare)
        uint4 Bq[PD + 1][MSUB];
#pragma unroll
        for (int d = 0; d < PD; ++d) {
            const uint32_t xo = mortar_row_bcast(ccs, d) + xo_base;
#pragma unroll
            for (int ms = 0; ms < MSUB; ++ms) Bq[d][ms] = *reinterpret_cast<const uint4 *>(lb + xo + (ROUTED ? tk[ms] * 32u : ms * 512u));
        }
#pragma unroll
        for (int k = 0; k < RES_GROUPS; ++k) {
            if (4 * k < pairs) {
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int u = 4 * k + t;
                    if (t == 2 && u >= pairs) break;                  // the padded half of the last octet
                    const uint32_t nib = (CODE & CODE_4BIT) ? b.cw[k][t] : ((b.cw[k][t] << (2 * hsel)) & 0xCCCCCCCCu);
                    const u32x4_t A = (CODE & CODE_UNIFORM) ? mortar_nib4(nib) : mortar_scale4(nib, mortar_row_bcast(b.sdv, u));
                    if (u + PD < NP) {
                        const uint32_t xo = mortar_row_bcast(ccs, u + PD) + xo_base;
#pragma unroll
                        for (int ms = 0; ms < MSUB; ++ms)
                            Bq[(u + PD) % (PD + 1)][ms] = *reinterpret_cast<const uint4 *>(lb + xo + (ROUTED ? tk[ms] * 32u : ms * 512u));
                    }
#pragma unroll
                    for (int ms = 0; ms < MSUB; ++ms) {
                        if (!ROUTED || ms < nsub) {
                            const uint4 bq = Bq[u % (PD + 1)][ms];
                            const u32x4_t Bv = {bq.x, bq.y, bq.z, bq.w};
                            acc[ms] = mortar_mfma(A, Bv, acc[ms]);
                        }
                    }
                }
            }
        }
    }
}

// Stages x[m0 .. m0+MT, 16*c0 .. 16*(c0+ncb)] into the tile.  One wave instruction moves 16 rows x 64 bytes: the four
// lanes of a quad read 64 contiguous bytes of one row (two block-columns), so global reads stay coalesced in 64-byte
// pieces while the 16 lanes that the LDS serves together write 16 different bank groups (4 tokens x 4 units).
// Rows past M are not staged: their LDS units keep whatever they held and only feed accumulator columns that are
// never stored.  With MASKED, units of (token, input cluster) pairs that are off are zeroed.
// NORM: the rows are scaled by their factor in `rs` (LDS, one float per tile row) and the weight, as rms_apply8 does.
template <int MT, int WAVES, bool MASKED, bool NORM>
__device__ __forceinline__ void mortar_stage_quads(const SpmmView &p, unsigned char *lb, int m0, int c0, int ncb, int tid,
                                                   const float *rs) {
    // a wave instruction covers RPI rows x LPR consecutive 16-byte units: 16 rows x 64 bytes for the MFMA-sized
    // tiles, 4 rows x 256 bytes for the narrow decode tiles (whose LDS write pattern does not matter)
    constexpr int RPI = MT >= 16 ? 16 : 4, LPR = 64 / RPI;
    constexpr int RG = (MT + RPI - 1) / RPI;             // row groups
    constexpr int KC = RG >= 4 ? 2 : (RG == 2 ? 4 : 8);  // unit blocks in flight per wave: 8 loads per lane
    const int nch = 2 * ncb;                             // 16-byte units per row
    const int nck = (nch + LPR - 1) / LPR;               // blocks of LPR units per row
    const int rlast = (p.M - m0 < MT ? p.M - m0 : MT) - 1;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int rsub = lane / LPR, li = lane % LPR;
    const MORTAR_GLOBAL char *xt = p.x + (int64_t)m0 * p.ldx * 2 + (int64_t)c0 * 32;
    const bool has_w = NORM && p.norm_w != nullptr;
    for (int ck0 = wave; ck0 < nck; ck0 += WAVES * KC) {
        u32x4_t v[KC][RG], wv[KC];
#pragma unroll
        for (int k = 0; k < KC; ++k) {
            if (ck0 + k * WAVES >= nck) break;           // uniform: nothing left for this wave
            int u = (ck0 + k * WAVES) * LPR + li;
            u = u < nch ? u : nch - 1;
            if (NORM) wv[k] = has_w ? p.norm_w[c0 * 2 + u] : u32x4_t{0u, 0u, 0u, 0u};
#pragma unroll
            for (int rg = 0; rg < RG; ++rg) {
                int row = rg * RPI + rsub;
                row = row < rlast ? row : rlast;
                v[k][rg] = *(const MORTAR_GLOBAL u32x4_t *)(xt + (int64_t)row * p.ldx * 2 + (uint32_t)u * 16u);
                if (MASKED && p.active[(int64_t)(m0 + row) * p.n_clusters + (c0 * 16 + u * 8) / p.cluster_size] == 0)
                    v[k][rg] = u32x4_t{0u, 0u, 0u, 0u};
            }
        }
#pragma unroll
        for (int k = 0; k < KC; ++k) {
            if (ck0 + k * WAVES >= nck) break;
            const int u = (ck0 + k * WAVES) * LPR + li;
#pragma unroll
            for (int rg = 0; rg < RG; ++rg) {
                const int row = rg * RPI + rsub;
                if (row <= rlast && u < nch) {
                    u32x4_t o = v[k][rg];
                    if (NORM) o = rms_apply8(o, rs[row], wv[k], has_w);
                    *reinterpret_cast<u32x4_t *>(lb + (uint32_t)(u >> 1) * (uint32_t)(MT * 32) + row * 32 + (u & 1) * 16) = o;
                }
            }
        }
    }
}

// Asynchronous 16-byte-per-lane copy global -> LDS (lane l's bytes land at lds_base + 16 * l): no registers, no
// address arithmetic beyond the source pointer.  The caller waits with s_waitcnt vmcnt(0) and a barrier before the
// destination is read.  (One wait state separates the write of M0 from its use as the LDS base.)
__device__ __forceinline__ void mortar_load_to_lds(const MORTAR_GLOBAL char *gsrc, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(gsrc) : "memory", "m0");
}

// Stages block-columns [c0, c0 + ncb) of token tile `mt` from activations stored in tile order (SpmmParams::x_tiled):
// the 1 KB of a (token tile, block-column) is already in the tile's LDS layout, so one wave instruction copies it.
// Rows past M hold whatever the buffer held: they feed accumulator columns that are never stored.
template <int WAVES>
__device__ __forceinline__ void mortar_stage_tiled32(const SpmmView &p, uint4 *lx, int mt, int c0, int ncb, int tid) {
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const MORTAR_GLOBAL char *src = p.x + ((int64_t)mt * p.Cb + c0) * 1024 + lane * 16;
    const uint32_t dst = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lx;
    for (int c = wave; c < ncb; c += WAVES) mortar_load_to_lds(src + (int64_t)c * 1024, __builtin_amdgcn_readfirstlane(dst + c * 1024));
    __builtin_amdgcn_s_waitcnt(0);
}

// XT: the activations are stored in tile order (SpmmParams::x_tiled, set by the host for exactly these instantiations).
// A compile-time choice: the register-staged path holds up to eight 16-byte loads per lane, which the kernels that
// copy straight into LDS should not pay for in their register budget.
template <int MT, int WAVES, bool MASKED, bool XT = false>
__device__ __forceinline__ void mortar_stage_tile(const SpmmView &p, uint4 *lx, int m0, int c0, int ncb, int tid) {
    if constexpr (XT) {
        static_assert(MT == 32 && !MASKED, "tile-ordered activations are staged by the 32-token plain kernels");
        mortar_stage_tiled32<WAVES>(p, lx, m0 / 32, c0, ncb, tid);
    } else {
        mortar_stage_quads<MT, WAVES, MASKED, false>(p, reinterpret_cast<unsigned char *>(lx), m0, c0, ncb, tid, nullptr);
    }
}

// The same staging with the rows RMS-normalised on the way (gate_up with the block's norm folded in).  First every
// wave adds the squares of whole rows (lanes = consecutive 16-byte units, ascending, then the xor butterfly: the order
// of the stand-alone RMSNorm kernel, so both give the same bits) and leaves the row factors in LDS at `rs`; after a
// barrier the tile is staged as above with bf16(bf16(x * r) * w) applied (the second read of x hits the cache).
// The host admits the fused norm for ncb <= NORM_MAX_CB only (a row is at most 256 units = 4 per lane).
template <int MT, int WAVES>
__device__ __forceinline__ void mortar_stage_tile_norm(const SpmmView &p, uint4 *lx, int m0, int ncb, int tid, float *rs) {
    constexpr int CU = 4;
    const int nch = 2 * ncb;
    const int rlast = (p.M - m0 < MT ? p.M - m0 : MT) - 1;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const MORTAR_GLOBAL char *xt = p.x + (int64_t)m0 * p.ldx * 2;
    for (int row = wave; row <= rlast; row += WAVES) {
        const MORTAR_GLOBAL char *xr = xt + (int64_t)row * p.ldx * 2;
        u32x4_t v[CU];
#pragma unroll
        for (int b = 0; b < CU; ++b) {
            int ch = b * 64 + lane;
            ch = ch < nch ? ch : nch - 1;
            v[b] = *(const MORTAR_GLOBAL u32x4_t *)(xr + (uint32_t)ch * 16u);
        }
        float ss = 0.f;
#pragma unroll
        for (int b = 0; b < CU; ++b)
            if (b * 64 + lane < nch) ss = rms_sumsq8(v[b], ss);
        const float r = rms_scale(rms_wave_sum(ss), 8 * nch, p.norm_eps);
        if (lane == 0) rs[row] = r;
    }
    __syncthreads();
    mortar_stage_quads<MT, WAVES, false, true>(p, reinterpret_cast<unsigned char *>(lx), m0, 0, ncb, tid, rs);
}

// Four consecutive values of a carrier stream (bf16 or fp32 storage) as floats, and back.
__device__ __forceinline__ f32x4_t mortar_load4(const MORTAR_GLOBAL char *base, int64_t elem, bool f32) {
    if (f32) return *(const MORTAR_GLOBAL f32x4_t *)(base + elem * 4);
    const u32x2_t u = *(const MORTAR_GLOBAL u32x2_t *)(base + elem * 2);
    return f32x4_t{bf16_to_f32(u[0] & 0xffffu), bf16_to_f32(u[0] >> 16), bf16_to_f32(u[1] & 0xffffu), bf16_to_f32(u[1] >> 16)};
}
__device__ __forceinline__ void mortar_store4(MORTAR_GLOBAL char *base, int64_t elem, bool f32, f32x4_t v) {
    if (f32) *(MORTAR_GLOBAL f32x4_t *)(base + elem * 4) = v;
    else *(MORTAR_GLOBAL u32x2_t *)(base + elem * 2) = u32x2_t{bf16_pack2(v[0], v[1]), bf16_pack2(v[2], v[3])};
}

// Hyper-connection POST write for the four features a lane holds (reference: _hc_post_fwd_kernel,
// morph/kernels/triton/fused_hyper_connection.py:927-970, called from engine._hc, morph/inference/engine.py:1052-1060;
// wide form hc_post_wide, fused_decode_step.py:1725-1739): the MLP output y (rounded to bf16, the dtype the unfused
// path hands over) never goes to memory; fp32 arithmetic in the reference's order (j ascending, then y, then term).
template <int N>
__device__ __forceinline__ void mortar_hc_post(const SpmmView &p, int tok, int f0, f32x4_t y) {
    const int64_t C = (int64_t)p.Rb * 16;
    const bool f32 = p.hc_f32 != 0;
    f32x4_t h[N];
#pragma unroll
    for (int j = 0; j < N; ++j) h[j] = mortar_load4(p.hc_h, ((int64_t)tok * N + j) * C + f0, f32);
    f32x4_t term = f32x4_t{0.f, 0.f, 0.f, 0.f};
    if (p.hc_term) term = mortar_load4(p.hc_term, (int64_t)tok * C + f0, f32);
#pragma unroll
    for (int i = 0; i < N; ++i) {
        f32x4_t a = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const float hij = p.hc_res[((int64_t)tok * N + i) * N + j];
#pragma unroll
            for (int v = 0; v < 4; ++v) a[v] = __builtin_fmaf(hij, h[j][v], a[v]);
        }
        const float pi = p.hc_post[(int64_t)tok * N + i];
#pragma unroll
        for (int v = 0; v < 4; ++v) a[v] = __builtin_fmaf(pi, y[v], a[v]);
        if (p.hc_term) a += term;
        mortar_store4(p.hc_out, ((int64_t)tok * N + i) * C + f0, f32, a);
    }
}

// Epilogue of one row unit for the 16 tokens of sub-tile `ms`: the lane holds D[4g+v][token].
// `gv` is the router gate of the lane's four features for this token (read when has_gates).
template <int NACC, int CODE = 0, bool HC = false, bool YT = false>
__device__ __forceinline__ void mortar_store_unit(const SpmmView &p, int unit, int tok, int g, bool has_gates, float gv,
                                                  f32x4_t a0, f32x4_t a1) {
    if (CODE & CODE_UNIFORM) {      // the blocks were multiplied as +-2: p.uscale is half the matrix's scale
        a0 *= p.uscale;
        if (NACC == 2) a1 *= p.uscale;
    }
    u32x2_t pk;
    if (NACC == 1) {
        if (p.y32 != nullptr) {      // the fp32 sums as they are (the three-term fp32 decode product adds them up later)
            *(MORTAR_GLOBAL f32x4_t *)(p.y32 + (int64_t)tok * p.ldy + unit * 16 + 4 * g) = a0;
            return;
        }
        pk = u32x2_t{bf16_pack2(a0[0], a0[1]), bf16_pack2(a0[2], a0[3])};
        if (HC && p.hc_h != nullptr) {
            const f32x4_t y = {bf16_to_f32(pk[0] & 0xffffu), bf16_to_f32(pk[0] >> 16), bf16_to_f32(pk[1] & 0xffffu), bf16_to_f32(pk[1] >> 16)};
            switch (p.hc_n) {
                case 1: mortar_hc_post<1>(p, tok, unit * 16 + 4 * g, y); break;
                case 2: mortar_hc_post<2>(p, tok, unit * 16 + 4 * g, y); break;
                case 3: mortar_hc_post<3>(p, tok, unit * 16 + 4 * g, y); break;
                default: mortar_hc_post<4>(p, tok, unit * 16 + 4 * g, y); break;
            }
            return;
        }
    } else {
        pk = swiglu_pack4(a0, a1, has_gates, gv);
        if constexpr (YT) {    // tile-ordered hidden activations (SpmmParams::y_tiled; host: M * features < 2^31)
            const uint32_t e = ((uint32_t)(tok >> 5) * (uint32_t)p.n_units + (uint32_t)unit) * 512u + (uint32_t)(tok & 31) * 16u + 4u * g;
            *(MORTAR_GLOBAL u32x2_t *)(p.y + e) = pk;
            return;
        }
    }
    *(MORTAR_GLOBAL u32x2_t *)(p.y + (int64_t)tok * p.ldy + unit * 16 + 4 * g) = pk;
}

// Epilogue of one row unit for all sub-tiles of the token tile.  tl[ms] is the tile row of the lane's token in
// sub-tile ms, `cnt` the number of live rows per 16-row sub-tile set (MT, or the routed list length).  The cluster of
// the lane's features is found once per unit and the gates of all sub-tiles are requested before the first SwiGLU.
template <int MSUB, int NACC, int CODE, bool HC, bool YT = false>
__device__ __forceinline__ void mortar_store_tile(const SpmmView &p, int unit, int m0, const uint32_t (&tl)[MSUB], int cnt,
                                                  int n, int g, bool has_gates, const f32x4_t (&a0)[MSUB],
                                                  const f32x4_t (&a1)[MSUB]) {
    float gv[MSUB];
    bool ok[MSUB];
#pragma unroll
    for (int ms = 0; ms < MSUB; ++ms) {
        ok[ms] = ms * 16 + n < cnt && m0 + (int)tl[ms] < p.M;
        gv[ms] = 0.f;
    }
    if (NACC == 2 && has_gates) {
        const int gcol = (unit * 16 + 4 * g) / p.cluster_size;
#pragma unroll
        for (int ms = 0; ms < MSUB; ++ms)
            if (ok[ms]) gv[ms] = p.gates[(int64_t)(m0 + (int)tl[ms]) * p.n_clusters + gcol];
    }
#pragma unroll
    for (int ms = 0; ms < MSUB; ++ms)
        if (ok[ms]) mortar_store_unit<NACC, CODE, HC, YT>(p, unit, m0 + (int)tl[ms], g, has_gates, gv[ms], a0[ms], a1[ms]);
}

// Part descriptor of schedule position `pos`, segment `sg`, row `a` of the unit: {g0, g1, nb, unit}.
// One load site for both sources (schedule table, or row descriptors in natural order) so that the compiler can
// keep the load in flight instead of waiting at a control-flow join.
template <int NACC>
__device__ __forceinline__ u32x4_t mortar_part_desc(const SpmmView &p, int pos, int sg, int a) {
    pos = pos < p.n_units ? pos : p.n_units - 1;
    const bool sc = p.sched != nullptr;
    const MORTAR_GLOBAL u32x4_t *base = sc ? p.sched : p.row_desc;
    const uint32_t idx = sc ? ((uint32_t)pos * (uint32_t)p.nseg + (uint32_t)sg) * NACC + a
                            : (uint32_t)(sg * p.Rb + pos + a * p.n_units);
    u32x4_t d = base[idx];
    d[3] = sc ? d[3] : (uint32_t)pos;
    return d;
}

// ---------------------------------------------------------------------------------------------------------
// Resident kernel.  The workgroup stages x[MT, K] once; then every wave walks whole row units on its own,
// streaming the unit's block pairs straight from global memory in batches (a row's blocks are contiguous).
// No barrier after the first one.  A wave's work is a chain of row parts (unit, segment, row of the unit) whose
// descriptors come from the schedule table one part ahead; latency is hidden by the waves that share a SIMD.
// ---------------------------------------------------------------------------------------------------------
// TL: the hidden activations of the two-launch MLP are in tile order: a plain product (NACC = 1) stages its input from
// them (SpmmParams::x_tiled), a gate_up (NACC = 2) stores its result so (SpmmParams::y_tiled).
template <int MT, int NACC, bool ROUTED, int WAVES, bool TABLE, int CODE, bool TL = false>
__global__ void __launch_bounds__(WAVES * 64) mortar_resident_kernel(const SpmmParams p0, const SpmmParams *table) {
    constexpr int MSUB = (MT + 15) / 16;
    constexpr bool XT = TL && NACC == 1, YT = TL && NACC == 2;
    const SpmmView p = mortar_view(TABLE ? mortar_table_entry(table, blockIdx.y) : p0);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint4 *lx = reinterpret_cast<uint4 *>(smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, g = lane >> 4, bsel = g >> 1, hsel = g & 1;
    // Workgroups are dealt round-robin over the 8 XCDs (each with its own L2): renumber them so that the
    // n_split workgroups that stage the same token tile run on one XCD and share its copy of the tile.
    const int wg = p.xcd_map ? (int)(blockIdx.x & 7) * (int)(gridDim.x >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
    if (wg >= p.n_mtiles * p.n_split) return;
    const int mt = wg / p.n_split, sp = wg % p.n_split;
    const int m0 = mt * MT;
    const uint32_t lane_xo = (uint32_t)(hsel * 16 + (ROUTED ? 0 : n * 32));
    const bool has_gates = p.gates != nullptr;

    const int per = (p.n_units + p.n_split - 1) / p.n_split;
    const int u_end = (sp + 1) * per < p.n_units ? (sp + 1) * per : p.n_units;
    // Units are handed out dynamically: a wave starts with position `wave` of the workgroup's window and draws
    // its next position from a counter in LDS when it begins a unit (one unit ahead, so that the descriptor of the
    // next unit's first part can still be fetched early).  The SIMD arbiter favours the oldest wave, so with a
    // fixed assignment the waves of a SIMD would finish one after another and leave it with one or two waves;
    // drawing positions keeps all waves busy until the window is empty.
    uint32_t *next_unit = reinterpret_cast<uint32_t *>(smem + tile_bytes(MT, p.Cb));
    if (tid == 0) *next_unit = WAVES;
    const int base = sp * per;
    int pos = base + wave;
    u32x4_t d0 = mortar_part_desc<NACC>(p, pos, 0, 0);

    if (NACC == 2 && p.norm) mortar_stage_tile_norm<MT, WAVES>(p, lx, m0, p.Cb, tid, reinterpret_cast<float *>(next_unit + 4));      // gate_up may carry the norm
    else mortar_stage_tile<MT, WAVES, false, XT>(p, lx, m0, 0, p.Cb, tid);
    __syncthreads();

    while (pos < u_end) {
        uint32_t drawn = 0;
        if (lane == 0) drawn = atomicAdd(next_unit, 1u);
        // coordinates of the part after the current one; its descriptor is fetched while the current part runs
        int p1 = pos, s1 = 0, a1 = 0;
        int npos = -1;       // position of this wave's next unit, known from the second part on
        auto advance = [&](int &ps, int &s, int &a_) {
            if (++a_ == NACC) { a_ = 0; if (++s == p.nseg) { s = 0; ps = npos; } }
        };
        const int unit = __builtin_amdgcn_readfirstlane((int)d0[3]);
        int cnt = MT;
        uint32_t tk[MSUB];
#pragma unroll
        for (int ms = 0; ms < MSUB; ++ms) tk[ms] = ms * 16 + n;
        bool skip = false;
        if (ROUTED) {
            const int cl = (unit * 16) / p.cluster_size;
            const int64_t e = (int64_t)mt * p.n_clusters + cl;
            cnt = __builtin_amdgcn_readfirstlane(p.tok_cnt[e]);
            skip = cnt == 0;
#pragma unroll
            for (int ms = 0; ms < MSUB; ++ms) {
                const int i = ms * 16 + n;
                tk[ms] = i < cnt ? p.tok_list[e * MT + i] : 0;
            }
        }
        const int nsub = ROUTED ? (cnt + 15) >> 4 : MSUB;
        f32x4_t acc[NACC][MSUB];
#pragma unroll
        for (int a = 0; a < NACC; ++a)
#pragma unroll
            for (int ms = 0; ms < MSUB; ++ms) acc[a][ms] = f32x4_t{0.f, 0.f, 0.f, 0.f};

        for (int sg = 0; sg < p.nseg; ++sg) {
            const uint32_t xo_base = lane_xo + (uint32_t)(sg * p.seg_cb) * (uint32_t)(MT * 32);
#pragma unroll
            for (int a = 0; a < NACC; ++a) {
                const bool last_part = sg + 1 == p.nseg && a + 1 == NACC;
                if (last_part) npos = base + (int)__builtin_amdgcn_readfirstlane(drawn);
                advance(p1, s1, a1);
                const u32x4_t d1 = mortar_part_desc<NACC>(p, p1, s1, a1);
                const int g0 = __builtin_amdgcn_readfirstlane((int)d0[0]), g1 = __builtin_amdgcn_readfirstlane((int)d0[1]);
                const int nb = __builtin_amdgcn_readfirstlane((int)d0[2]);
                if (!skip && g0 < g1) {
                    MortarBatch b;
                    mortar_load_batch<CODE>(p, b, g0, g1, n, bsel, hsel);
                    mortar_row_part<MSUB, MT, ROUTED, CODE>(p, lx, b, g0, g1, nb, xo_base, tk, nsub, n, bsel, hsel, acc[a]);
                }
                d0 = d1;
            }
        }
        pos = npos;
        if (skip) continue;

        mortar_store_tile<MSUB, NACC, CODE, (MT <= 16 && NACC == 1 && !TABLE), YT>(p, unit, m0, tk, ROUTED ? cnt : MT, n, g, has_gates,
                                                                                   acc[0], acc[NACC - 1]);
    }
}

// ---------------------------------------------------------------------------------------------------------
// Segmented kernel for matrices whose K does not fit in LDS at once (e.g. `down`, K = d_ff).  The workgroup
// walks the K segments of the octet stream: per segment it stages x[MT, 16*seg_cb] (one barrier pair), and
// every wave multiplies the segment's blocks of its own UPW row units, whose accumulators stay in registers.
// The descriptors of the next segment are fetched before the barrier pair, so their latency hides behind the
// staging.
// ---------------------------------------------------------------------------------------------------------
template <int MT, int NACC, bool MASKED, int WAVES, int UPW, bool TABLE, int CODE, bool TL = false>
__global__ void __launch_bounds__(WAVES * 64) mortar_segmented_kernel(const SpmmParams p0, const SpmmParams *table) {
    constexpr int MSUB = (MT + 15) / 16, NP = UPW * NACC;
    constexpr bool XT = TL && NACC == 1, YT = TL && NACC == 2;
    const SpmmView p = mortar_view(TABLE ? mortar_table_entry(table, blockIdx.y) : p0);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint4 *lx = reinterpret_cast<uint4 *>(smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, g = lane >> 4, bsel = g >> 1, hsel = g & 1;
    // Workgroups are dealt round-robin over the 8 XCDs (each with its own L2): renumber them so that the
    // n_split workgroups that stage the same token tile run on one XCD and share its copy of the tile.
    const int wg = p.xcd_map ? (int)(blockIdx.x & 7) * (int)(gridDim.x >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
    if (wg >= p.n_mtiles * p.n_split) return;
    const int mt = wg / p.n_split, sp = wg % p.n_split;
    const int m0 = mt * MT;
    const uint32_t lane_xo = (uint32_t)(hsel * 16 + n * 32);
    const bool has_gates = p.gates != nullptr;

    // this wave's units: schedule positions sp*per + wave + WAVES*k
    constexpr int per = WAVES * UPW;
    const int pos0 = sp * per + wave;
    f32x4_t acc[UPW][NACC][MSUB];
    uint32_t tk[MSUB];
#pragma unroll
    for (int ms = 0; ms < MSUB; ++ms) tk[ms] = ms * 16;
#pragma unroll
    for (int k = 0; k < UPW; ++k)
#pragma unroll
        for (int a = 0; a < NACC; ++a)
#pragma unroll
            for (int ms = 0; ms < MSUB; ++ms) acc[k][a][ms] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    u32x4_t dn[NP];     // descriptors of the coming segment, part q = k * NACC + a
#pragma unroll
    for (int q = 0; q < NP; ++q) dn[q] = mortar_part_desc<NACC>(p, pos0 + WAVES * (q / NACC), 0, q % NACC);
    int units[UPW];

    for (int sg = 0; sg < p.nseg; ++sg) {
        const int c0 = sg * p.seg_cb;
        const int ncb = p.Cb - c0 < p.seg_cb ? p.Cb - c0 : p.seg_cb;
        int g0[NP], g1[NP], nb[NP];
#pragma unroll
        for (int q = 0; q < NP; ++q) {
            const bool on = pos0 + WAVES * (q / NACC) < p.n_units;
            g0[q] = on ? __builtin_amdgcn_readfirstlane((int)dn[q][0]) : 0;
            g1[q] = on ? __builtin_amdgcn_readfirstlane((int)dn[q][1]) : 0;
            nb[q] = __builtin_amdgcn_readfirstlane((int)dn[q][2]);
            if (q % NACC == 0) units[q / NACC] = on ? __builtin_amdgcn_readfirstlane((int)dn[q][3]) : -1;
        }
        if (sg + 1 < p.nseg) {
#pragma unroll
            for (int q = 0; q < NP; ++q) dn[q] = mortar_part_desc<NACC>(p, pos0 + WAVES * (q / NACC), sg + 1, q % NACC);
        }
        // The first batch of every part is requested one part ahead (the first part's before the tile is staged), always
        // and in a fixed order (an empty part reads octet 0), and a part's first batch is multiplied without a load in
        // between: the wait for it then counts the loads issued since and never includes the newest ones.
        // (Prefill tiles only: the decode tiles of this kernel run many waves per SIMD on few registers.)
        constexpr int FIRST = 8 * RES_GROUPS;                      // blocks of a part's first batch
        constexpr bool BATCH_AHEAD = MT >= 32;
        auto first_batch = [&](MortarBatch &bb, int q) {
            const bool any = g0[q] < g1[q];
            mortar_load_batch<CODE>(p, bb, any ? g0[q] : 0, any ? g1[q] : 1, n, bsel, hsel);
        };
        MortarBatch bq;
        if (BATCH_AHEAD) first_batch(bq, 0);
        if (sg > 0) __syncthreads();
        mortar_stage_tile<MT, WAVES, MASKED, XT>(p, lx, m0, c0, ncb, tid);
        __syncthreads();
        if (!BATCH_AHEAD) {
#pragma unroll
            for (int q = 0; q < NP; ++q) {
                if (g0[q] < g1[q]) {
                    MortarBatch b;
                    mortar_load_batch<CODE>(p, b, g0[q], g1[q], n, bsel, hsel);
                    mortar_row_part<MSUB, MT, false, CODE>(p, lx, b, g0[q], g1[q], nb[q], lane_xo, tk, MSUB, n, bsel, hsel,
                                                           acc[q / NACC][q % NACC]);
                }
            }
            continue;
        }
#pragma unroll
        for (int q = 0; q < NP; ++q) {
            // A wave lowers its priority with every part of the segment it has finished: the arbiter serves the oldest wave of
            // a SIMD first, so without this the four waves finish a segment one after another (4.8 / 6.3 / 8.0 / 9.4 us measured)
            // and the SIMD runs the end of it on one or two waves.  Tile-ordered form only: with the register-staged forms the
            // same priorities cost time (the staging of the next segment then starts from uneven waves).
            if constexpr (XT) mortar_setprio(NP - 1 - q);
            MortarBatch bn;
            if (q + 1 < NP) first_batch(bn, q + 1);
            const int nbq = g0[q] < g1[q] ? nb[q] : 0;
            mortar_row_part<MSUB, MT, false, CODE, true>(p, lx, bq, g0[q], g1[q], nbq < FIRST ? nbq : FIRST, lane_xo, tk, MSUB,
                                                         n, bsel, hsel, acc[q / NACC][q % NACC]);
            if (nbq > FIRST) {                                      // the rest of a long part
                MortarBatch bt;
                mortar_load_batch<CODE>(p, bt, g0[q] + RES_GROUPS, g1[q], n, bsel, hsel);
                mortar_row_part<MSUB, MT, false, CODE>(p, lx, bt, g0[q] + RES_GROUPS, g1[q], nbq - FIRST, lane_xo, tk, MSUB,
                                                       n, bsel, hsel, acc[q / NACC][q % NACC]);
            }
            if (q + 1 < NP) bq = bn;
        }
        if constexpr (XT) mortar_setprio(0);
    }

    uint32_t tl[MSUB];
#pragma unroll
    for (int ms = 0; ms < MSUB; ++ms) tl[ms] = ms * 16 + n;
#pragma unroll
    for (int k = 0; k < UPW; ++k) {
        if (units[k] < 0) continue;
        mortar_store_tile<MSUB, NACC, CODE, (MT <= 16 && NACC == 1 && !TABLE), YT>(p, units[k], m0, tl, MT, n, g, has_gates, acc[k][0],
                                                                                   acc[k][NACC - 1]);
    }
}

// ---------------------------------------------------------------------------------------------------------
// Part-split kernel: the latency form for ONE small-M product that has to be spread over the whole chip.
// The row parts of a unit (its K segments x its gate/up rows) are dealt to PW waves that run side by side;
// their partial accumulators meet in LDS and the unit's first wave applies the epilogue.  A workgroup holds UW
// units (PW * UW waves) and one resident token tile.  Every wave fetches its first descriptor and weight batch
// before the tile is staged, so the only serial global round trips are descriptor -> batch.
// ---------------------------------------------------------------------------------------------------------
template <int MT, int NACC, bool ROUTED, bool MASKED, int PW, int UW, int CODE>
__global__ void __launch_bounds__(PW * UW * 64) mortar_partsplit_kernel(const SpmmParams p0) {
    constexpr int MSUB = (MT + 15) / 16, WAVES = PW * UW;
    const SpmmView p = mortar_view(p0);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint4 *lx = reinterpret_cast<uint4 *>(smem);
    f32x4_t *red = reinterpret_cast<f32x4_t *>(smem + tile_bytes(MT, p.Cb));   // [WAVES][NACC][MSUB][64]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, g = lane >> 4, bsel = g >> 1, hsel = g & 1;
    const int mt = blockIdx.x / p.n_split, sp = blockIdx.x % p.n_split;
    const int m0 = mt * MT;
    const uint32_t lane_xo = (uint32_t)(hsel * 16 + (ROUTED ? 0 : n * 32));
    const bool has_gates = p.gates != nullptr;
    const int ug = wave / PW, wq = wave % PW;            // unit slot in the workgroup, this wave's share of its parts
    const int pos = sp * UW + ug;
    const bool valid = pos < p.n_units;
    const int nparts = p.nseg * NACC;

    // first part of this wave: q = wq  (q = segment * NACC + a)
    MortarBatch first;
    u32x4_t d = u32x4_t{0u, 0u, 0u, 0u};
    if (valid && wq < nparts) {
        d = mortar_part_desc<NACC>(p, pos, wq / NACC, wq % NACC);
        const int g0 = __builtin_amdgcn_readfirstlane((int)d[0]), g1 = __builtin_amdgcn_readfirstlane((int)d[1]);
        if (g0 < g1) mortar_load_batch<CODE>(p, first, g0, g1, n, bsel, hsel);
    }
    const int unit = valid ? __builtin_amdgcn_readfirstlane((int)mortar_part_desc<NACC>(p, pos, 0, 0)[3]) : 0;

    int cnt = MT;
    uint32_t tk[MSUB];
#pragma unroll
    for (int ms = 0; ms < MSUB; ++ms) tk[ms] = ms * 16 + n;
    bool skip = !valid;
    if (ROUTED && valid) {
        const int cl = (unit * 16) / p.cluster_size;
        const int64_t e = (int64_t)mt * p.n_clusters + cl;
        cnt = __builtin_amdgcn_readfirstlane(p.tok_cnt[e]);
        skip = cnt == 0;
#pragma unroll
        for (int ms = 0; ms < MSUB; ++ms) {
            const int i = ms * 16 + n;
            tk[ms] = i < cnt ? p.tok_list[e * MT + i] : 0;
        }
    }
    const int nsub = ROUTED ? (cnt + 15) >> 4 : MSUB;
    // Gated gate_up without token lists: a unit whose cluster is off for every token of the tile multiplies nothing
    // (its accumulators stay zero and the epilogue stores the zeros the gates would have produced).  The gates are
    // requested here and looked at after the tile is staged.
    constexpr bool GATE_SKIP = NACC == 2 && !ROUTED && MT <= 16;
    float gsk = 0.f;
    if (GATE_SKIP && valid && has_gates && p.cluster_size % 16 == 0 && n < MT && m0 + n < p.M)
        gsk = p.gates[(int64_t)(m0 + n) * p.n_clusters + (unit * 16) / p.cluster_size];

    if (NACC == 2 && !MASKED && p.norm) mortar_stage_tile_norm<MT, WAVES>(p, lx, m0, p.Cb, tid, reinterpret_cast<float *>(red));
    else mortar_stage_tile<MT, WAVES, MASKED>(p, lx, m0, 0, p.Cb, tid);
    __syncthreads();
    bool idle = skip;
    if (GATE_SKIP && valid && has_gates && p.cluster_size % 16 == 0) idle = __ballot(gsk != 0.f) == 0ull;      // NaN and negative gates multiply like any other

    f32x4_t acc[NACC][MSUB];
#pragma unroll
    for (int a = 0; a < NACC; ++a)
#pragma unroll
        for (int ms = 0; ms < MSUB; ++ms) acc[a][ms] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    if (!idle) {
        for (int sg = 0; sg < p.nseg; ++sg) {
            const uint32_t xo_base = lane_xo + (uint32_t)(sg * p.seg_cb) * (uint32_t)(MT * 32);
#pragma unroll
            for (int a = 0; a < NACC; ++a) {
                const int q = sg * NACC + a;
                if (q % PW != wq) continue;
                const bool is_first = q == wq;
                const u32x4_t dq = is_first ? d : mortar_part_desc<NACC>(p, pos, sg, a);
                const int g0 = __builtin_amdgcn_readfirstlane((int)dq[0]), g1 = __builtin_amdgcn_readfirstlane((int)dq[1]);
                const int nb = __builtin_amdgcn_readfirstlane((int)dq[2]);
                if (g0 >= g1) continue;
                if (!is_first) mortar_load_batch<CODE>(p, first, g0, g1, n, bsel, hsel);
                mortar_row_part<MSUB, MT, ROUTED, CODE>(p, lx, first, g0, g1, nb, xo_base, tk, nsub, n, bsel, hsel, acc[a]);
            }
        }
    }
    // partial sums of the unit's waves meet in LDS; its first wave finishes the unit
    if (PW > 1) {
#pragma unroll
        for (int a = 0; a < NACC; ++a)
#pragma unroll
            for (int ms = 0; ms < MSUB; ++ms) red[((wave * NACC + a) * MSUB + ms) * 64 + lane] = acc[a][ms];
        __syncthreads();
        if (wq != 0) return;
#pragma unroll
        for (int w = 1; w < PW; ++w)
#pragma unroll
            for (int a = 0; a < NACC; ++a)
#pragma unroll
                for (int ms = 0; ms < MSUB; ++ms) acc[a][ms] += red[(((wave + w) * NACC + a) * MSUB + ms) * 64 + lane];
    }
    if (skip) return;
    mortar_store_tile<MSUB, NACC, CODE, (MT <= 16 && NACC == 1)>(p, unit, m0, tk, ROUTED ? cnt : MT, n, g, has_gates, acc[0],
                                                                 acc[NACC - 1]);
}

// ---- launchers -------------------------------------------------------------------------------------------
// `layers` > 1 launches the table variant: `table` points at `layers` SpmmParams in device memory whose
// n_mtiles / n_split fields were filled from the same shape as `p`.

template <typename K>
inline int mortar_allow_big_lds(K kern, bool &done) {
    if (!done) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
        done = true;
    }
    return MORTAR_OK;
}

inline int mortar_launch_check(int64_t grid, int layers) {
    if (grid <= 0 || grid > 0x7fffffff || layers <= 0 || layers > 65535)
        return mortar_fail(MORTAR_ERR_LIMIT, "spmm grid %lld x %d out of range", (long long)grid, layers);
    return MORTAR_OK;
}

// Grid width for n_mtiles * n_split workgroups.  When several workgroups share a token tile of a large single
// launch, the ids are renumbered per XCD in the kernel and the grid is padded to a multiple of 8.
inline int64_t mortar_grid_width(SpmmParams &p, int layers) {
    const int64_t n = (int64_t)p.n_mtiles * p.n_split;
    p.xcd_map = layers == 1 && p.n_split > 1 && n >= 64;
    return p.xcd_map ? (n + 7) / 8 * 8 : n;
}

// Fills the launch-shape fields of `p` for the resident kernel and returns the grid width.
template <int MT, int WAVES>
inline int64_t mortar_resident_shape(SpmmParams &p, int layers) {
    p.n_mtiles = (p.M + MT - 1) / MT;
    // Prefill tiles: one workgroup per CU (every workgroup stages a whole tile and the last units of its window
    // leave waves idle, so few large ones: one round measured faster than two).  Decode tiles stage little: many
    // small workgroups (about 12 per CU) so that the hardware dispatcher evens out the load, with a few units
    // per wave when many layers share the launch and one unit per wave when a single matrix has to be spread
    // over the whole chip.
    const bool wide = (int64_t)layers * p.n_units >= 8 * 512;
    int upw = 1;
    if (MT <= 16 && wide) {
        // up to 4 units per wave, 8 for the 16-token tile whose staging costs more (fewer workgroups, each staging
        // its tile once), but never so few workgroups that the launch cannot fill the chip's resident slots about
        // once: a second, mostly empty round is what a count just above the slot count costs, and half-empty CUs
        // what a count far below it costs
        const int by_lds = (160 * 1024) / (tile_bytes(MT, p.Cb) + LDS_EXTRA), by_waves = 32 / WAVES;
        const int64_t slots = 256 * (int64_t)(by_lds < by_waves ? by_lds : by_waves);
        for (upw = MT == 16 ? 8 : 4; upw > 1; --upw)
            if ((int64_t)layers * p.n_mtiles * ((p.n_units + WAVES * upw - 1) / (WAVES * upw)) * 10 >= slots * 9) break;
    }
    // prefill tiles: never more workgroups than CUs (one workgroup fills a CU's LDS, so 264 of them take two rounds
    // where 252 take one)
    const int target = MT <= 16 ? 256 * 12 : 256;
    int split = MT <= 16 ? (target + layers * p.n_mtiles - 1) / (layers * p.n_mtiles) : target / (layers * p.n_mtiles);
    const int max_split = (p.n_units + WAVES * upw - 1) / (WAVES * upw);
    split = split < 1 ? 1 : (split > max_split ? max_split : split);
    p.n_split = split;
    return mortar_grid_width(p, layers);
}

template <int MT, int NACC, bool ROUTED, int WAVES, bool TABLE = false, int CODE = 0, bool TL = false>
int mortar_launch_resident(SpmmParams &p, const SpmmParams *table, int layers, hipStream_t st) {
    if (TABLE != (table != nullptr)) return mortar_fail(MORTAR_ERR_ARG, "spmm launch: parameter table mismatch");
    const int smem = tile_bytes(MT, p.Cb) + LDS_EXTRA;
    if (smem > LDS_BUDGET + LDS_PAD * 16 + LDS_EXTRA) return mortar_fail(MORTAR_ERR_LIMIT, "resident tile of %d bytes does not fit LDS", smem);
    static bool attr_done = false;
    if (TL != ((NACC == 1 ? p.x_tiled : p.y_tiled) != 0)) return mortar_fail(MORTAR_ERR_ARG, "spmm launch: activation layout mismatch");
    auto kern = mortar_resident_kernel<MT, NACC, ROUTED, WAVES, TABLE, CODE, TL>;
    int rc = mortar_allow_big_lds(kern, attr_done);
    if (rc) return rc;
    const int64_t grid = mortar_resident_shape<MT, WAVES>(p, layers);
    if ((rc = mortar_launch_check(grid, layers))) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid, (unsigned)layers), dim3(WAVES * 64), smem, st, p, table);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "spmm launch: %s", hipGetErrorString(e));
    return MORTAR_OK;
}

template <int MT, int WAVES, int UPW>
inline int64_t mortar_segmented_shape(SpmmParams &p, int layers) {
    p.n_mtiles = (p.M + MT - 1) / MT;
    p.n_split = (p.n_units + WAVES * UPW - 1) / (WAVES * UPW);
    return mortar_grid_width(p, layers);
}

template <int MT, int NACC, bool MASKED, int WAVES, int UPW, bool TABLE = false, int CODE = 0, bool TL = false>
int mortar_launch_segmented(SpmmParams &p, const SpmmParams *table, int layers, hipStream_t st) {
    if (TABLE != (table != nullptr)) return mortar_fail(MORTAR_ERR_ARG, "spmm launch: parameter table mismatch");
    const int smem = tile_bytes(MT, p.seg_cb);
    if (smem > LDS_BUDGET + LDS_PAD * 16) return mortar_fail(MORTAR_ERR_LIMIT, "segment tile of %d bytes does not fit LDS", smem);
    static bool attr_done = false;
    if (TL != ((NACC == 1 ? p.x_tiled : p.y_tiled) != 0)) return mortar_fail(MORTAR_ERR_ARG, "spmm launch: activation layout mismatch");
    auto kern = mortar_segmented_kernel<MT, NACC, MASKED, WAVES, UPW, TABLE, CODE, TL>;
    int rc = mortar_allow_big_lds(kern, attr_done);
    if (rc) return rc;
    const int64_t grid = mortar_segmented_shape<MT, WAVES, UPW>(p, layers);
    if ((rc = mortar_launch_check(grid, layers))) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid, (unsigned)layers), dim3(WAVES * 64), smem, st, p, table);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "spmm launch: %s", hipGetErrorString(e));
    return MORTAR_OK;
}

template <int MT, int NACC, bool ROUTED, bool MASKED, int PW, int UW, int CODE = 0>
int mortar_launch_partsplit(SpmmParams &p, hipStream_t st) {
    constexpr int WAVES = PW * UW;
    const int smem = tile_bytes(MT, p.Cb) + WAVES * NACC * ((MT + 15) / 16) * 64 * 16;
    if (smem > 160 * 1024) return mortar_fail(MORTAR_ERR_LIMIT, "part-split tile of %d bytes does not fit LDS", smem);
    static bool attr_done = false;
    auto kern = mortar_partsplit_kernel<MT, NACC, ROUTED, MASKED, PW, UW, CODE>;
    int rc = mortar_allow_big_lds(kern, attr_done);
    if (rc) return rc;
    p.n_mtiles = (p.M + MT - 1) / MT;
    p.n_split = (p.n_units + UW - 1) / UW;
    p.xcd_map = 0;
    const int64_t grid = (int64_t)p.n_mtiles * p.n_split;
    if ((rc = mortar_launch_check(grid, 1))) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(WAVES * 64), smem, st, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "spmm launch: %s", hipGetErrorString(e));
    return MORTAR_OK;
}

// Small-M (decode) dispatch, compiled in its own translation unit.  kind: 0 spmm, 1 gate_up + SwiGLU,
// 2 gate_up + SwiGLU routed, 3 spmm with an input mask.  Returns -1 when the shape has no small-M variant.
__attribute__((visibility("hidden"))) int mortar_smallm_launch(int kind, SpmmParams &p, const SpmmParams *table,
                                                               int layers, hipStream_t st);
__attribute__((visibility("hidden"))) int mortar_smallm_tile(int Cb, int seg_cb, int64_t M, int kind);
// Fills the launch-shape fields (n_mtiles, n_split) of a table entry exactly as mortar_smallm_launch would.
__attribute__((visibility("hidden"))) int mortar_smallm_shape(int kind, SpmmParams &p, int layers);

#endif
