// Prefill (large M) block-sparse ternary SpMM on bf16 MFMA, fp32 accumulate.
//
// Replaces the reference's stk dds forward (morph/sparse/stk/backend/triton_kernels.py:170-230 behind
// custom_ops.py:35-56) and, in gate_up mode, fuses the SwiGLU of _SwiGLUMortar.forward
// (morph/model/transformer.py:402-431) into the epilogue.
//
// Three kernels share the inner step (unpack the ternary codes of two blocks in registers, read the
// activation operand from LDS, one 16x16x32 MFMA per 16 tokens):
//   mortar_resident_kernel   in_features fits LDS for a 32..96-token tile: stage x once, every wave then walks
//                            whole row units on its own from the octet weight stream (no K loop, no barriers)
//   mortar_segmented_kernel  wide K (e.g. `down`): the same, with K cut into LDS-sized segments and the
//                            accumulators of a wave's few row units kept in registers across segments
//   mortar_spmm_kernel       K-chunked kernel with 128-token tiles and one wave per SIMD; serves the routed
//                            gate_up of matrices that are too wide for the resident kernel
#include "mortar_spmm_core.h"

#include <vector>

namespace {

constexpr int KCB = MORTAR_PREFILL_KCB;
constexpr int NW = 4;   // wavefronts per workgroup (one per SIMD, 512 registers each)

template <int MSUB, int RW, int NACC, bool ROUTED, bool MASKED>
__global__ void __launch_bounds__(NW * 64, 1) mortar_spmm_kernel(const SpmmParams p) {
    constexpr int MT = 16 * MSUB, LDM = MT + 1, NA = RW * NACC, NT = NW * 64;
    constexpr int XUNITS = 2 * KCB * LDM;                 // one activation buffer, in 16-byte units
    constexpr int WBLK = NA * KCB + 4;                    // block slots in a wave's staging list (+ pads)
    constexpr int WDW = WBLK * 18;                        // codes [WBLK*16] + scale [WBLK] + x offset [WBLK]
    constexpr int NIT = (2 * KCB * MT + NT - 1) / NT;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint4 *lxbuf = reinterpret_cast<uint4 *>(smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, g = lane >> 4, bsel = g >> 1, hsel = g & 1;
    uint32_t *lwc = reinterpret_cast<uint32_t *>(smem + 2 * XUNITS * 16) + wave * WDW;
    uint32_t *lws = lwc + WBLK * 16;
    uint32_t *lwl = lws + WBLK;

    // Workgroup -> (token tile, unit group).  Consecutive workgroup ids land on consecutive XCDs; with the
    // XCD map every workgroup that reads one token tile runs on the same XCD and shares its L2.
    int mt, ug;
    {
        const int L = blockIdx.x;
        if (p.xcd_map) {
            const int xcd = L & 7, s = L >> 3;
            mt = xcd + 8 * (s / p.n_groups);
            ug = s % p.n_groups;
        } else {
            mt = L / p.n_groups;
            ug = L % p.n_groups;
        }
    }
    if (mt >= p.n_mtiles) return;
    const int m0 = mt * MT;

    int rows[NA];
    int outb[RW];
#pragma unroll
    for (int rw = 0; rw < RW; ++rw) {
        const int pos = (ug * NW + wave) * RW + rw;
        int unit = -1;
        if (pos < p.n_units) unit = p.unit_order ? p.unit_order[pos] : pos;
        unit = __builtin_amdgcn_readfirstlane(unit);
        outb[rw] = unit;
        rows[rw * NACC] = unit;
        if (NACC == 2) rows[rw * NACC + 1] = unit < 0 ? -1 : unit + p.n_units;
    }

    // Routed mode: tokens of this tile that have the unit's cluster active, compacted (ascending).
    int cnt[RW];
    uint32_t tk[RW][MSUB];
#pragma unroll
    for (int rw = 0; rw < RW; ++rw) {
        cnt[rw] = MT;
#pragma unroll
        for (int ms = 0; ms < MSUB; ++ms) tk[rw][ms] = ms * 16 + n;
        if (ROUTED && outb[rw] >= 0) {
            const int cl = (outb[rw] * 16) / p.cluster_size;
            const int64_t e = (int64_t)mt * p.n_clusters + cl;
            cnt[rw] = __builtin_amdgcn_readfirstlane(p.tok_cnt[e]);
#pragma unroll
            for (int ms = 0; ms < MSUB; ++ms) {
                const int i = ms * 16 + n;
                tk[rw][ms] = i < cnt[rw] ? p.tok_list[e * MT + i] : 0;
            }
        }
    }

    f32x4_t acc[NA][MSUB];
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int ms = 0; ms < MSUB; ++ms) acc[a][ms] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // Per-wave copy of the chunk pointer rows of its NA block-rows (read once; the table is then consulted
    // from LDS so that no global round trip sits between the loads of a chunk).
    int32_t *lcp = reinterpret_cast<int32_t *>(smem + 2 * XUNITS * 16 + NW * WDW * 4) + wave * NA * (p.nkc + 1);
#pragma unroll
    for (int a = 0; a < NA; ++a)
        for (int c = lane; c <= p.nkc; c += 64)
            lcp[a * (p.nkc + 1) + c] = rows[a] >= 0 ? p.chunk_ptr[(int64_t)rows[a] * (p.nkc + 1) + c] : 0;

    // Registers that carry chunk kc+1 from global memory to LDS while chunk kc is being multiplied.
    // Staging map: thread t < 2*KCB*8 owns column-half ch = t % (2*KCB) of rows r0 + 8*it, r0 = t / (2*KCB).
    constexpr int RG = 8, NITX = MT / RG;
    const bool stager = tid < 2 * KCB * RG;
    const int ch = tid % (2 * KCB), r0 = tid / (2 * KCB);
    const int rlast = (p.M - m0 < MT ? p.M - m0 : MT) - 1;          // last valid token row of the tile
    const bool full_tile = rlast == MT - 1;
    const uint32_t ldxB = (uint32_t)p.ldx * 2u;
    const char *xtile = reinterpret_cast<const char *>(p.x) + (int64_t)m0 * ldxB;
    uint4 xv[NITX];
    uint32_t xm[MASKED ? NITX : 1];
    uint32_t wv[NA][4], wsd[NA];
    int wcl[NA], nbn[NA], np[NA], nxt[NA], c0n = 0;

    // All global loads of one chunk.  Addresses are clamped into the tensor instead of predicated: rows past
    // M and columns past in_features receive copies of valid data that no block or output ever refers to.
    auto load_chunk = [&](int kc) {
        const int c0 = kc * KCB;
        c0n = c0;
        if (stager) {
            int cu = c0 * 2 + ch;
            cu = cu < 2 * p.Cb ? cu : 2 * p.Cb - 1;
            int clus = 0;
            if (MASKED) clus = (cu * 8) / p.cluster_size;
            if (full_tile) {
                const uint32_t voff = (uint32_t)r0 * ldxB + (uint32_t)cu * 16u;
#pragma unroll
                for (int it = 0; it < NITX; ++it) {
                    xv[it] = *reinterpret_cast<const uint4 *>(xtile + (int64_t)(RG * it) * ldxB + voff);
                    if (MASKED) xm[it] = p.active[(int64_t)(m0 + r0 + RG * it) * p.n_clusters + clus];
                }
            } else {
#pragma unroll
                for (int it = 0; it < NITX; ++it) {
                    int r = r0 + RG * it;
                    r = r < rlast ? r : rlast;
                    xv[it] = *reinterpret_cast<const uint4 *>(xtile + (uint32_t)r * ldxB + (uint32_t)cu * 16u);
                    if (MASKED) xm[it] = p.active[(int64_t)(m0 + r) * p.n_clusters + clus];
                }
            }
        }
        int P0v = 0, P1v = 0;
        if (lane < NA) {
            P0v = lcp[lane * (p.nkc + 1) + kc];
            P1v = lcp[lane * (p.nkc + 1) + kc + 1];
        }
#pragma unroll
        for (int a = 0; a < NA; ++a) {
            const int P0 = __builtin_amdgcn_readlane(P0v, a);
            int nb = __builtin_amdgcn_readlane(P1v, a) - P0;
            if (ROUTED && cnt[a / NACC] == 0) nb = 0;
            nbn[a] = nb;
            if (nb > 0) {
                const int last = nb * 16 - 1;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int i = lane + 64 * k;
                    if (k == 0 || nb * 16 > 64 * k) wv[a][k] = p.codes[(int64_t)P0 * 16 + (i < last ? i : last)];
                }
                const int j = lane < nb ? lane : 0;
                wsd[a] = p.sdup[P0 + j];
                wcl[a] = p.col[P0 + j];        // chunk base is subtracted at store time: no ALU use here,
                                               // so no wait for this load sits between the loads of a chunk
            }
        }
    };
    // Registers -> LDS: activation buffer `buf` (shared) and this wave's own block list.  The rows' blocks are
    // laid back to back, each row padded to a whole pair with an all-zero block, and the list ends with two
    // zero blocks so that the software pipeline below may read one pair past the end.
    auto store_chunk = [&](int buf) {
        uint4 *lx = lxbuf + buf * XUNITS;
        if (stager) {
#pragma unroll
            for (int it = 0; it < NITX; ++it) {
                uint4 v = xv[it];
                if (MASKED && xm[it] == 0u) v = make_uint4(0u, 0u, 0u, 0u);
                lx[ch * LDM + r0 + RG * it] = v;
            }
        }
        int o = 0;
#pragma unroll
        for (int a = 0; a < NA; ++a) {
            const int nb = nbn[a];
            np[a] = (nb + 1) >> 1;
            if (nb > 0) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int i = lane + 64 * k;
                    if (i < nb * 16) lwc[o * 16 + i] = wv[a][k];
                }
                if (lane < nb) {
                    lws[o + lane] = wsd[a];
                    lwl[o + lane] = (uint32_t)((wcl[a] - c0n) * 2 * LDM);
                }
                if (nb & 1) {
                    if (lane < 16) lwc[(o + nb) * 16 + lane] = 0u;
                    if (lane == 0) {
                        lws[o + nb] = 0u;
                        lwl[o + nb] = 0u;
                    }
                }
            }
            o += 2 * np[a];
        }
        if (lane < 32) lwc[o * 16 + lane] = 0u;
        if (lane < 2) {
            lws[o + lane] = 0u;
            lwl[o + lane] = 0u;
        }
        // row unit of the next non-empty row after a (routed mode: whose token list the look-ahead uses)
        int nx = RW - 1;
#pragma unroll
        for (int a = NA - 1; a >= 0; --a) {
            nxt[a] = nx;
            if (np[a] > 0) nx = a / NACC;
        }
    };

    load_chunk(0);
    store_chunk(0);
    __syncthreads();
    for (int kc = 0; kc < p.nkc; ++kc) {
        const bool more = kc + 1 < p.nkc;
        if (more) load_chunk(kc + 1);
        const uint4 *lx = lxbuf + (kc & 1) * XUNITS;
        // ---- MFMA over the chunk: one software pipeline across all rows of the wave --------------------
        // stage 1 reads a pair's codes/scale/offset, stage 2 unpacks it and issues its activation reads,
        // stage 3 multiplies; three consecutive pairs are in flight.
        int first_rw = 0;
        if (ROUTED) {
            first_rw = RW - 1;
#pragma unroll
            for (int a = NA - 1; a >= 0; --a)
                if (np[a] > 0) first_rw = a / NACC;
        }
        int cur = bsel;                                   // block index (this lane's half of the pair)
        uint32_t w1 = lwc[cur * 16 + n], sd1 = lws[cur], xo1 = lwl[cur] + hsel * LDM;
        u32x4_t A = mortar_unpack8(w1 << (8 * hsel), sd1);
        uint4 B[MSUB];
#pragma unroll
        for (int ms = 0; ms < MSUB; ++ms) B[ms] = lx[xo1 + tk[ROUTED ? first_rw : 0][ms]];
        cur += 2;
        w1 = lwc[cur * 16 + n]; sd1 = lws[cur]; xo1 = lwl[cur] + hsel * LDM;
#pragma unroll
        for (int a = 0; a < NA; ++a) {
            const int rw = a / NACC;
            const int nsub = ROUTED ? (cnt[rw] + 15) >> 4 : MSUB;
            for (int q = 0; q < np[a]; ++q) {
                // stage 1 for the pair after the next one
                cur += 2;
                const uint32_t w0 = lwc[cur * 16 + n], sd0 = lws[cur], xo0 = lwl[cur] + hsel * LDM;
                // stage 2 (unpack) of the next pair
                const u32x4_t An = mortar_unpack8(w1 << (8 * hsel), sd1);
                // the next pair belongs to this row, except after the row's last pair
                const int rn = (ROUTED && q + 1 == np[a]) ? nxt[a] : rw;
                // stage 3: multiply, and refill each activation register for the next pair as soon as its
                // MFMA has been issued
#pragma unroll
                for (int ms = 0; ms < MSUB; ++ms) {
                    if (!ROUTED || ms < nsub) {
                        const u32x4_t Bv = {B[ms].x, B[ms].y, B[ms].z, B[ms].w};
                        acc[a][ms] = mortar_mfma(A, Bv, acc[a][ms]);
                    }
                    B[ms] = lx[xo1 + (ROUTED ? tk[rn][ms] : tk[0][ms])];
                }
                A = An;
                w1 = w0; sd1 = sd0; xo1 = xo0;
            }
        }
        if (more) store_chunk((kc + 1) & 1);
        __syncthreads();
    }

    // ---- epilogue: lane holds D[4g+v][token n] ------------------------------------------------------
    const bool has_gates = p.gates != nullptr;
#pragma unroll
    for (int rw = 0; rw < RW; ++rw) {
        if (outb[rw] < 0) continue;
#pragma unroll
        for (int ms = 0; ms < MSUB; ++ms) {
            const int li = ms * 16 + n;
            if (ROUTED && li >= cnt[rw]) continue;
            const int tok = m0 + (int)tk[rw][ms];
            if (tok >= p.M) continue;
            u32x2_t pk;
            if (NACC == 1) {
                pk = u32x2_t{bf16_pack2(acc[rw][ms][0], acc[rw][ms][1]), bf16_pack2(acc[rw][ms][2], acc[rw][ms][3])};
            } else {
                float gv = 0.f;
                if (has_gates) gv = p.gates[(int64_t)tok * p.n_clusters + (outb[rw] * 16 + 4 * g) / p.cluster_size];
                pk = swiglu_pack4(acc[rw * NACC][ms], acc[rw * NACC + NACC - 1][ms], has_gates, gv);
            }
            *reinterpret_cast<u32x2_t *>(p.y + (int64_t)tok * p.ldy + outb[rw] * 16 + 4 * g) = pk;
        }
    }
}

template <int MSUB, int RW, int NACC>
constexpr int smem_fixed_bytes() {
    return 2 * 2 * KCB * (16 * MSUB + 1) * 16 + NW * (RW * NACC * KCB + 4) * 18 * 4;
}

template <int MSUB, int RW, int NACC, bool ROUTED, bool MASKED>
int launch(SpmmParams &p, hipStream_t st) {
    constexpr int MT = 16 * MSUB;
    const int smem = smem_fixed_bytes<MSUB, RW, NACC>() + NW * RW * NACC * (p.nkc + 1) * 4;
    if (smem > 160 * 1024) return mortar_fail(MORTAR_ERR_LIMIT, "prefill: in_features too large for the LDS chunk table (%d bytes)", smem);
    static bool attr_done = false;
    auto kern = mortar_spmm_kernel<MSUB, RW, NACC, ROUTED, MASKED>;
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
        attr_done = true;
    }
    p.n_mtiles = (p.M + MT - 1) / MT;
    p.n_groups = (p.n_units + NW * RW - 1) / (NW * RW);
    p.xcd_map = p.n_mtiles >= 8;
    const int mt_slots = p.xcd_map ? (p.n_mtiles + 7) / 8 * 8 : p.n_mtiles;
    const int64_t grid = (int64_t)mt_slots * p.n_groups;
    if (grid <= 0 || grid > 0x7fffffff) return mortar_fail(MORTAR_ERR_LIMIT, "prefill grid %lld out of range", (long long)grid);
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NW * 64), smem, st, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "prefill launch: %s", hipGetErrorString(e));
    return MORTAR_OK;
}


int check_common(const mortar_bcsr_t *W, const int32_t *chunk_ptr, const uint16_t *x, int64_t M, int64_t ldx,
                 const uint16_t *y, int64_t ldy, int64_t out_cols) {
    if (!W || !W->codes || !W->sdup || !W->col || !W->row_ptr || !W->row_desc || !W->codes_o || !W->sd_o || !W->col_o || !chunk_ptr || !x || !y)
        return mortar_fail(MORTAR_ERR_ARG, "prefill: null pointer");
    if (W->Rb <= 0 || W->Cb <= 0 || W->nnz <= 0) return mortar_fail(MORTAR_ERR_ARG, "prefill: empty matrix");
    if (W->seg_cb <= 0 || (int64_t)2 * (W->seg_cb < W->Cb ? W->seg_cb : W->Cb) * 33 * 16 > 156 * 1024)
        return mortar_fail(MORTAR_ERR_ARG, "prefill: seg_cb=%d does not fit LDS (max %d)", W->seg_cb, 156 * 1024 / (2 * 33 * 16));
    if (M <= 0 || M > (1 << 30)) return mortar_fail(MORTAR_ERR_ARG, "prefill: M=%lld out of range", (long long)M);
    if (ldx < (int64_t)W->Cb * 16 || ldx % 8) return mortar_fail(MORTAR_ERR_ARG, "prefill: ldx=%lld must be >= in_features and a multiple of 8", (long long)ldx);
    if (ldy < out_cols || ldy % 4) return mortar_fail(MORTAR_ERR_ARG, "prefill: ldy=%lld must be >= out_features and a multiple of 4", (long long)ldy);
    if ((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(y) & 7))
        return mortar_fail(MORTAR_ERR_ARG, "prefill: x must be 16-byte and y 8-byte aligned");
    return MORTAR_OK;
}

void fill(SpmmParams &p, const mortar_bcsr_t *W, const int32_t *chunk_ptr, const int32_t *unit_order,
          const uint16_t *x, int64_t M, int64_t ldx, uint16_t *y, int64_t ldy) {
    p = SpmmParams{};
    p.codes = W->codes; p.sdup = W->sdup; p.col = W->col; p.chunk_ptr = chunk_ptr; p.row_ptr = W->row_ptr;
    p.row_desc = reinterpret_cast<const u32x4_t *>(W->row_desc);
    p.codes_o = reinterpret_cast<const u32x4_t *>(W->codes_o);
    p.sd_o = reinterpret_cast<const u32x4_t *>(W->sd_o);
    p.col_o = reinterpret_cast<const u32x4_t *>(W->col_o);
    p.seg_cb = W->seg_cb < W->Cb ? W->seg_cb : W->Cb; p.nseg = (W->Cb + p.seg_cb - 1) / p.seg_cb; p.Rb = W->Rb;
    p.unit_order = unit_order;
    p.nkc = (W->Cb + KCB - 1) / KCB; p.Cb = W->Cb;
    p.x = x; p.ldx = ldx; p.M = (int)M; p.y = y; p.ldy = ldy;
    p.n_clusters = 1; p.cluster_size = 1 << 30;
}

// Token tile of the resident prefill kernel for a matrix with Cb block-columns (0 = does not fit).
int resident_mt(int Cb) {
    for (int mt : {96, 64, 32})
        if (tile_bytes(mt, Cb) <= LDS_BUDGET) return mt;
    return 0;
}

// prefill tiles: 16 wavefronts (4 per SIMD, 128 registers) for the 32-token tile, 8 for larger tiles
template <int NACC, bool ROUTED>
int launch_resident_any(SpmmParams &p, hipStream_t st) {
    switch (resident_mt(p.Cb)) {
        case 96: return mortar_launch_resident<96, NACC, ROUTED, 8>(p, nullptr, 1, st);
        case 64: return mortar_launch_resident<64, NACC, ROUTED, 8>(p, nullptr, 1, st);
        default: return mortar_launch_resident<32, NACC, ROUTED, 16>(p, nullptr, 1, st);
    }
}

constexpr int SEG_WAVES = 16, SEG_UPW = 4;

// kind: 0 spmm, 1 gate_up + SwiGLU, 2 routed gate_up + SwiGLU, 3 spmm with an input mask
int dispatch(int kind, SpmmParams &p, hipStream_t st) {
    if (p.M <= 16) {
        const int rc = mortar_smallm_launch(kind, p, nullptr, 1, st);
        if (rc >= 0) return rc;
    }
    switch (kind) {
        case 0:
            if (p.nseg == 1) return launch_resident_any<1, false>(p, st);
            return mortar_launch_segmented<32, 1, false, SEG_WAVES, SEG_UPW>(p, nullptr, 1, st);
        case 1:
            if (p.nseg == 1) return launch_resident_any<2, false>(p, st);
            return mortar_launch_segmented<32, 2, false, SEG_WAVES, SEG_UPW>(p, nullptr, 1, st);
        case 2:
            if (p.nseg == 1) return launch_resident_any<2, true>(p, st);
            return launch<8, 4, 2, true, false>(p, st);
        default:
            return mortar_launch_segmented<32, 1, true, SEG_WAVES, SEG_UPW>(p, nullptr, 1, st);
    }
}

}  // namespace

extern "C" int mortar_prefill_max_seg_cb(void) { return (LDS_BUDGET / 16 - LDS_PAD) / (2 * 33); }

extern "C" int mortar_prefill_tile(int32_t Cb, int64_t M) {
    if (M > 0 && M <= 16) {
        const int t = mortar_smallm_tile(Cb, Cb, M, 2);
        if (t > 0) return t;
    }
    const int mt = resident_mt(Cb);
    return mt ? mt : MORTAR_PREFILL_MT;
}

extern "C" int mortar_prefill_group(int swiglu) { return swiglu ? NW * 4 : NW * 8; }

extern "C" int mortar_spmm_bf16(const mortar_bcsr_t *W, const int32_t *chunk_ptr, const int32_t *unit_order,
                                const uint16_t *x, int64_t M, int64_t ldx, uint16_t *y, int64_t ldy,
                                void *stream) {
    int rc = check_common(W, chunk_ptr, x, M, ldx, y, ldy, W ? (int64_t)W->Rb * 16 : 0);
    if (rc) return rc;
    SpmmParams p;
    fill(p, W, chunk_ptr, unit_order, x, M, ldx, y, ldy);
    p.n_units = W->Rb;
    return dispatch(0, p, static_cast<hipStream_t>(stream));
}

extern "C" int mortar_spmm_bf16_masked(const mortar_bcsr_t *W, const int32_t *chunk_ptr,
                                       const int32_t *unit_order, const uint16_t *x, int64_t M, int64_t ldx,
                                       uint16_t *y, int64_t ldy, const uint8_t *active, int32_t n_clusters,
                                       void *stream) {
    int rc = check_common(W, chunk_ptr, x, M, ldx, y, ldy, W ? (int64_t)W->Rb * 16 : 0);
    if (rc) return rc;
    if (!active || n_clusters <= 0 || (W->Cb * 16) % n_clusters || ((W->Cb * 16) / n_clusters) % 8)
        return mortar_fail(MORTAR_ERR_ARG, "spmm_masked: in_features/n_clusters must be a multiple of 8");
    SpmmParams p;
    fill(p, W, chunk_ptr, unit_order, x, M, ldx, y, ldy);
    p.n_units = W->Rb;
    p.active = active; p.n_clusters = n_clusters; p.cluster_size = (W->Cb * 16) / n_clusters;
    return dispatch(3, p, static_cast<hipStream_t>(stream));
}

extern "C" int mortar_gateup_swiglu_bf16(const mortar_bcsr_t *W, const int32_t *chunk_ptr,
                                         const int32_t *unit_order, const uint16_t *x, int64_t M, int64_t ldx,
                                         uint16_t *h, int64_t ldh, const float *gates, int32_t n_clusters,
                                         const int32_t *tok_cnt, const uint8_t *tok_list, void *stream) {
    if (W && (W->Rb & 1)) return mortar_fail(MORTAR_ERR_ARG, "gateup: odd number of block-rows");
    const int64_t d_ff = W ? (int64_t)W->Rb * 8 : 0;
    int rc = check_common(W, chunk_ptr, x, M, ldx, h, ldh, d_ff);
    if (rc) return rc;
    SpmmParams p;
    fill(p, W, chunk_ptr, unit_order, x, M, ldx, h, ldh);
    p.n_units = W->Rb / 2;
    if (gates) {
        if (n_clusters <= 0 || d_ff % n_clusters || (d_ff / n_clusters) % 4)
            return mortar_fail(MORTAR_ERR_ARG, "gateup: d_ff / n_clusters must be a whole multiple of 4");
        p.gates = gates; p.n_clusters = n_clusters; p.cluster_size = (int)(d_ff / n_clusters);
    }
    if (tok_cnt || tok_list) {
        if (!tok_cnt || !tok_list || !gates) return mortar_fail(MORTAR_ERR_ARG, "gateup: routed mode needs gates, tok_cnt and tok_list");
        if (p.cluster_size % 16) return mortar_fail(MORTAR_ERR_ARG, "gateup: routed mode needs cluster_size %% 16 == 0");
        p.tok_cnt = tok_cnt; p.tok_list = tok_list;
        return dispatch(2, p, static_cast<hipStream_t>(stream));
    }
    return dispatch(1, p, static_cast<hipStream_t>(stream));
}

// ---- layer-batched small-M launches ---------------------------------------------------------------------

extern "C" int64_t mortar_stack_table_bytes(int32_t n_layers) {
    return n_layers > 0 ? (int64_t)n_layers * (int64_t)sizeof(SpmmParams) : 0;
}

extern "C" int mortar_stack_prepare(int32_t swiglu, int32_t n_layers, const mortar_bcsr_t *W,
                                    const uint16_t *const *x, uint16_t *const *y, int64_t M, int64_t ldx,
                                    int64_t ldy, void *table_dev, void *stream) {
    if (n_layers <= 0 || n_layers > 65535 || !W || !x || !y || !table_dev)
        return mortar_fail(MORTAR_ERR_ARG, "stack_prepare: bad arguments");
    if (M > 16) return mortar_fail(MORTAR_ERR_LIMIT, "stack_prepare: layer-batched launches serve M <= 16 (got %lld)", (long long)M);
    static const int32_t dummy_chunk = 0;
    std::vector<SpmmParams> tab((size_t)n_layers);
    for (int l = 0; l < n_layers; ++l) {
        if (W[l].Rb != W[0].Rb || W[l].Cb != W[0].Cb || W[l].seg_cb != W[0].seg_cb)
            return mortar_fail(MORTAR_ERR_ARG, "stack_prepare: layer %d differs in shape from layer 0", l);
        if (swiglu && (W[l].Rb & 1)) return mortar_fail(MORTAR_ERR_ARG, "stack_prepare: odd number of block-rows");
        const int64_t out_cols = swiglu ? (int64_t)W[l].Rb * 8 : (int64_t)W[l].Rb * 16;
        int rc = check_common(&W[l], &dummy_chunk, x[l], M, ldx, y[l], ldy, out_cols);
        if (rc) return rc;
        SpmmParams &p = tab[(size_t)l];
        fill(p, &W[l], nullptr, nullptr, x[l], M, ldx, y[l], ldy);
        p.n_units = swiglu ? W[l].Rb / 2 : W[l].Rb;
        rc = mortar_smallm_shape(swiglu ? 1 : 0, p, n_layers);
        if (rc) return rc;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipError_t e = hipMemcpyAsync(table_dev, tab.data(), tab.size() * sizeof(SpmmParams), hipMemcpyHostToDevice, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "stack_prepare: %s", hipGetErrorString(e));
    return MORTAR_OK;
}

extern "C" int mortar_stack_run(int32_t swiglu, int32_t n_layers, const mortar_bcsr_t *W0, int64_t M,
                                const void *table_dev, void *stream) {
    if (n_layers <= 0 || n_layers > 65535 || !W0 || !table_dev || M <= 0 || M > 16)
        return mortar_fail(MORTAR_ERR_ARG, "stack_run: bad arguments");
    SpmmParams p;
    fill(p, W0, nullptr, nullptr, nullptr, M, 0, nullptr, 0);
    p.n_units = swiglu ? W0->Rb / 2 : W0->Rb;
    const int rc = mortar_smallm_launch(swiglu ? 1 : 0, p, static_cast<const SpmmParams *>(table_dev), n_layers,
                                        static_cast<hipStream_t>(stream));
    if (rc < 0) return mortar_fail(MORTAR_ERR_LIMIT, "stack_run: shape has no small-M kernel");
    return rc;
}
