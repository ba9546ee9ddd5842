// Prefill (large M) block-sparse ternary SpMM on bf16 MFMA, fp32 accumulate.
//
// Replaces the reference's stk dds forward (morph/sparse/stk/backend/triton_kernels.py:170-230 behind
// custom_ops.py:35-56) and, in gate_up mode, fuses the SwiGLU of _SwiGLUMortar.forward
// (morph/model/transformer.py:402-431) into the epilogue.
//
// Work decomposition.  A workgroup (4 wavefronts) owns a tile of MT = 16*MSUB tokens and NW*RW row units
// (a unit is one 16-row block-row, or a gate/up pair of block-rows).  It walks K in chunks of KCB
// block-columns.  Per chunk the token tile x[MT, 16*KCB] is staged in LDS as 16-byte units
// [column-half][token] (token stride padded by one unit so both the staging writes and the MFMA operand
// reads are bank-conflict free), and every wave stages the packed blocks of its own rows that fall into the
// chunk (found through the chunk pointer table).  Accumulators stay in registers across all chunks, so each
// output element is written exactly once.  Per MFMA the weights of two blocks are unpacked in registers once
// and reused for the MSUB token sub-tiles; the activation operand is one 16-byte LDS read per lane.
#include "mortar_device.h"
#include "mortar_internal.h"

namespace {

constexpr int KCB = MORTAR_PREFILL_KCB;
constexpr int NW = 4;

struct SpmmParams {
    const uint32_t *codes;
    const uint32_t *sdup;
    const int16_t *col;
    const int32_t *chunk_ptr;
    const int32_t *unit_order;
    int n_units, nkc, Cb;
    const uint16_t *x;
    int64_t ldx;
    int M;
    uint16_t *y;
    int64_t ldy;
    const float *gates;       // [M, n_clusters] fp32 or null
    const uint8_t *active;    // [M, n_clusters] input mask or null
    const int32_t *tok_cnt;   // routed: [n_mtiles, n_clusters]
    const uint8_t *tok_list;  // routed: [n_mtiles, n_clusters, MT]
    int n_clusters, cluster_size;
    int xcd_map, n_mtiles, n_groups;
};

template <int MSUB, int RW, int NACC, bool ROUTED, bool MASKED>
__global__ void __launch_bounds__(256, 2) mortar_spmm_kernel(const SpmmParams p) {
    constexpr int MT = 16 * MSUB, LDM = MT + 1, NA = RW * NACC;
    constexpr int XUNITS = 2 * KCB * LDM;
    constexpr int WDW = NA * KCB * 18;   // per wave: codes [NA*KCB*16] + scale [NA*KCB] + x offset [NA*KCB]
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint4 *lx = reinterpret_cast<uint4 *>(smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, g = lane >> 4, bsel = g >> 1, hsel = g & 1;
    uint32_t *lwc = reinterpret_cast<uint32_t *>(smem + XUNITS * 16) + wave * WDW;
    uint32_t *lws = lwc + NA * KCB * 16;
    uint32_t *lwl = lws + NA * KCB;

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

    for (int kc = 0; kc < p.nkc; ++kc) {
        const int c0 = kc * KCB;
        __syncthreads();
        // ---- issue every global load of this chunk first (token tile + this wave's blocks), with clamped
        //      addresses so that no load sits behind a branch, then write LDS -----------------------------
        int nb[NA];
        uint32_t wv[NA][4], wsd[NA];
        int wcl[NA];
#pragma unroll
        for (int a = 0; a < NA; ++a) {
            nb[a] = 0;
            const int r = rows[a];
            if (r >= 0 && (!ROUTED || cnt[a / NACC] > 0)) {
                const int32_t *cp = p.chunk_ptr + (int64_t)r * (p.nkc + 1) + kc;
                const int P0 = __builtin_amdgcn_readfirstlane(cp[0]);
                const int P1 = __builtin_amdgcn_readfirstlane(cp[1]);
                nb[a] = P1 - P0;
                const int last = nb[a] > 0 ? nb[a] * 16 - 1 : 0;
                const int64_t base = nb[a] > 0 ? (int64_t)P0 : 0;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int i = lane + 64 * k;
                    wv[a][k] = p.codes[base * 16 + (i < last ? i : last)];
                }
                const int j = lane < nb[a] ? lane : 0;
                wsd[a] = p.sdup[base + j];
                wcl[a] = p.col[base + j];
            }
        }
        // token tile in two batches of loads (bounds the registers held across the loads)
        constexpr int NIT = (2 * KCB * MT + 255) / 256, NH = (NIT + 1) / 2;
#pragma unroll
        for (int hb = 0; hb < NIT; hb += NH) {
            uint4 xv[NH];
            bool xok[NH];
#pragma unroll
            for (int it = 0; it < NH; ++it) {
                const int i = (hb + it) * 256 + tid;
                const int ch = i % (2 * KCB), row = i / (2 * KCB);
                const int cb = c0 + (ch >> 1), tok = m0 + row;
                xok[it] = (hb + it < NIT) && (i < 2 * KCB * MT) && tok < p.M && cb < p.Cb;
                const int tokc = tok < p.M ? tok : p.M - 1;
                const int e0 = (cb < p.Cb ? cb : p.Cb - 1) * 16 + (ch & 1) * 8;
                xv[it] = *reinterpret_cast<const uint4 *>(p.x + (int64_t)tokc * p.ldx + e0);
                if (MASKED) xok[it] = xok[it] && p.active[(int64_t)tokc * p.n_clusters + e0 / p.cluster_size] != 0;
            }
#pragma unroll
            for (int it = 0; it < NH; ++it) {
                const int i = (hb + it) * 256 + tid;
                if ((hb + it < NIT) && i < 2 * KCB * MT) {
                    const int ch = i % (2 * KCB), row = i / (2 * KCB);
                    lx[ch * LDM + row] = xok[it] ? xv[it] : make_uint4(0u, 0u, 0u, 0u);
                }
            }
        }
#pragma unroll
        for (int a = 0; a < NA; ++a) {
            if (nb[a] > 0) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int i = lane + 64 * k;
                    if (i < nb[a] * 16) lwc[a * KCB * 16 + i] = wv[a][k];
                }
                if (lane < nb[a]) {
                    lws[a * KCB + lane] = wsd[a];
                    lwl[a * KCB + lane] = (uint32_t)((wcl[a] - c0) * 2 * LDM);
                }
                if (nb[a] & 1) {   // pad to a whole pair with an all-zero block
                    if (lane < 16) lwc[(a * KCB + nb[a]) * 16 + lane] = 0u;
                    if (lane == 0) {
                        lws[a * KCB + nb[a]] = 0u;
                        lwl[a * KCB + nb[a]] = 0u;
                    }
                }
            }
        }
        __syncthreads();
        // ---- MFMA over the chunk -----------------------------------------------------------------
#pragma unroll
        for (int a = 0; a < NA; ++a) {
            const int rw = a / NACC;
            const int np = (nb[a] + 1) >> 1;
            const int nsub = ROUTED ? (cnt[rw] + 15) >> 4 : MSUB;
            for (int q = 0; q < np; ++q) {
                const int blk = a * KCB + 2 * q + bsel;
                const uint32_t w = lwc[blk * 16 + n];
                const uint32_t sd = lws[blk];
                const uint32_t xo = lwl[blk] + hsel * LDM;
                const u32x4_t A = mortar_unpack8(w << (8 * hsel), sd);
#pragma unroll
                for (int ms = 0; ms < MSUB; ++ms) {
                    if (!ROUTED || ms < nsub) {
                        const uint4 b = lx[xo + tk[rw][ms]];
                        const u32x4_t B = {b.x, b.y, b.z, b.w};
                        acc[a][ms] = mortar_mfma(A, B, acc[a][ms]);
                    }
                }
            }
        }
    }

    // ---- epilogue: lane holds D[4g+v][token n] ------------------------------------------------------
#pragma unroll
    for (int rw = 0; rw < RW; ++rw) {
        if (outb[rw] < 0) continue;
#pragma unroll
        for (int ms = 0; ms < MSUB; ++ms) {
            const int li = ms * 16 + n;
            if (ROUTED && li >= cnt[rw]) continue;
            const int tok = m0 + (int)tk[rw][ms];
            if (tok >= p.M) continue;
            uint32_t o[4];
            if (NACC == 1) {
#pragma unroll
                for (int v = 0; v < 4; ++v) o[v] = bf16_bits_rne(acc[rw][ms][v]);
            } else {
                const int e0 = outb[rw] * 16 + 4 * g;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float gt = bf16r(acc[rw * 2][ms][v]);
                    const float up = bf16r(acc[rw * 2 + 1][ms][v]);
                    float h = bf16r(bf16r(silu_f32(gt)) * up);
                    if (p.gates) {
                        const float gv = p.gates[(int64_t)tok * p.n_clusters + (e0 + v) / p.cluster_size];
                        h = bf16r(h * bf16r(gv));
                    }
                    o[v] = bf16_bits_rne(h);
                }
            }
            u32x2_t pk = {o[0] | (o[1] << 16), o[2] | (o[3] << 16)};
            *reinterpret_cast<u32x2_t *>(p.y + (int64_t)tok * p.ldy + outb[rw] * 16 + 4 * g) = pk;
        }
    }
}

template <int MSUB, int RW, int NACC>
constexpr int smem_bytes() {
    return 2 * KCB * (16 * MSUB + 1) * 16 + NW * RW * NACC * KCB * 18 * 4;
}

template <int MSUB, int RW, int NACC, bool ROUTED, bool MASKED>
int launch(SpmmParams &p, hipStream_t st) {
    constexpr int MT = 16 * MSUB;
    constexpr int smem = smem_bytes<MSUB, RW, NACC>();
    static bool attr_done = false;
    auto kern = mortar_spmm_kernel<MSUB, RW, NACC, ROUTED, MASKED>;
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
        attr_done = true;
    }
    p.n_mtiles = (p.M + MT - 1) / MT;
    p.n_groups = (p.n_units + NW * RW - 1) / (NW * RW);
    p.xcd_map = p.n_mtiles >= 8;
    const int mt_slots = p.xcd_map ? (p.n_mtiles + 7) / 8 * 8 : p.n_mtiles;
    const int64_t grid = (int64_t)mt_slots * p.n_groups;
    if (grid <= 0 || grid > 0x7fffffff) return mortar_fail(MORTAR_ERR_LIMIT, "prefill grid %lld out of range", (long long)grid);
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), smem, st, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "prefill launch: %s", hipGetErrorString(e));
    return MORTAR_OK;
}

int check_common(const mortar_bcsr_t *W, const int32_t *chunk_ptr, const uint16_t *x, int64_t M, int64_t ldx,
                 const uint16_t *y, int64_t ldy, int64_t out_cols) {
    if (!W || !W->codes || !W->sdup || !W->col || !W->row_ptr || !chunk_ptr || !x || !y)
        return mortar_fail(MORTAR_ERR_ARG, "prefill: null pointer");
    if (W->Rb <= 0 || W->Cb <= 0 || W->nnz <= 0) return mortar_fail(MORTAR_ERR_ARG, "prefill: empty matrix");
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
    p.codes = W->codes; p.sdup = W->sdup; p.col = W->col; p.chunk_ptr = chunk_ptr; p.unit_order = unit_order;
    p.nkc = (W->Cb + KCB - 1) / KCB; p.Cb = W->Cb;
    p.x = x; p.ldx = ldx; p.M = (int)M; p.y = y; p.ldy = ldy;
    p.n_clusters = 1; p.cluster_size = 1 << 30;
}

}  // namespace

extern "C" int mortar_prefill_group(int swiglu) { return swiglu ? NW * 2 : NW * 4; }

extern "C" int mortar_spmm_bf16(const mortar_bcsr_t *W, const int32_t *chunk_ptr, const int32_t *unit_order,
                                const uint16_t *x, int64_t M, int64_t ldx, uint16_t *y, int64_t ldy,
                                void *stream) {
    int rc = check_common(W, chunk_ptr, x, M, ldx, y, ldy, W ? (int64_t)W->Rb * 16 : 0);
    if (rc) return rc;
    SpmmParams p;
    fill(p, W, chunk_ptr, unit_order, x, M, ldx, y, ldy);
    p.n_units = W->Rb;
    return launch<8, 4, 1, false, false>(p, static_cast<hipStream_t>(stream));
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
    return launch<8, 4, 1, false, true>(p, static_cast<hipStream_t>(stream));
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
        if (n_clusters <= 0 || d_ff % n_clusters) return mortar_fail(MORTAR_ERR_ARG, "gateup: d_ff %% n_clusters != 0");
        p.gates = gates; p.n_clusters = n_clusters; p.cluster_size = (int)(d_ff / n_clusters);
    }
    if (tok_cnt || tok_list) {
        if (!tok_cnt || !tok_list || !gates) return mortar_fail(MORTAR_ERR_ARG, "gateup: routed mode needs gates, tok_cnt and tok_list");
        if (p.cluster_size % 16) return mortar_fail(MORTAR_ERR_ARG, "gateup: routed mode needs cluster_size %% 16 == 0");
        p.tok_cnt = tok_cnt; p.tok_list = tok_list;
        return launch<8, 2, 2, true, false>(p, static_cast<hipStream_t>(stream));
    }
    return launch<8, 2, 2, false, false>(p, static_cast<hipStream_t>(stream));
}
