// Entry points of the block-sparse ternary SpMM on bf16 MFMA (fp32 accumulate), prefill-sized instantiations.
//
// Replaces the reference's stk dds forward (morph/sparse/stk/backend/triton_kernels.py:170-230 behind
// custom_ops.py:35-56) and, in gate_up mode, fuses the SwiGLU of _SwiGLUMortar.forward
// (morph/model/transformer.py:402-431) into the epilogue.  The kernels live in mortar_spmm_core.h:
//   mortar_resident_kernel   in_features fits LDS for a 32- or 64-token tile
//   mortar_segmented_kernel  wide K (e.g. `down`): K cut into LDS-sized segments, 32-token tile
// Batches of up to 16 rows go to the small-tile instantiations in mortar_smallm.hip.
#include "mortar_spmm_core.h"

#include <vector>

namespace {

int check_common(const mortar_bcsr_t *W, const uint16_t *x, int64_t M, int64_t ldx, const uint16_t *y, int64_t ldy,
                 int64_t out_cols) {
    if (!W || !W->row_desc || !W->codes_o || !W->sd_o || !W->col_o || !x || !y)
        return mortar_fail(MORTAR_ERR_ARG, "spmm: null pointer");
    if (W->Rb <= 0 || W->Cb <= 0 || W->nnz <= 0) return mortar_fail(MORTAR_ERR_ARG, "spmm: empty matrix");
    {   // K segments as wide as a 32-token tile allows serve every row count; a decode stream laid out with wider segments
        // (as wide as a 4- or 16-token tile allows, mortar_decode_max_seg_cb) serves calls of up to 4 or 16 rows
        const int seg = W->seg_cb < W->Cb ? W->seg_cb : W->Cb;
        if (W->seg_cb <= 0 || tile_bytes(M <= 4 ? 4 : M <= 16 ? 16 : 32, seg) > LDS_BUDGET)
            return mortar_fail(MORTAR_ERR_ARG, "spmm: K segments of %d block-columns do not fit LDS for %lld rows (max %d; %d up to 16 rows, %d up to 4)",
                               W->seg_cb, (long long)M, mortar_prefill_max_seg_cb(), mortar_decode_max_seg_cb(16), mortar_decode_max_seg_cb(4));
    }
    {   // the kernels address the octet stream with 32-bit byte offsets (1 KiB of 4-bit codes per octet)
        const int64_t nseg = (W->Cb + W->seg_cb - 1) / W->seg_cb;
        if ((int64_t)W->nnz / 8 + (int64_t)W->Rb * nseg >= ((int64_t)1 << 22))
            return mortar_fail(MORTAR_ERR_LIMIT, "spmm: octet stream of %d blocks in %d x %lld row parts exceeds 4 GiB",
                               W->nnz, W->Rb, (long long)nseg);
    }
    if (M <= 0 || M > (1 << 30)) return mortar_fail(MORTAR_ERR_ARG, "spmm: M=%lld out of range", (long long)M);
    if (ldx < (int64_t)W->Cb * 16 || ldx % 8) return mortar_fail(MORTAR_ERR_ARG, "spmm: ldx=%lld must be >= in_features and a multiple of 8", (long long)ldx);
    if (ldy < out_cols || ldy % 4) return mortar_fail(MORTAR_ERR_ARG, "spmm: ldy=%lld must be >= out_features and a multiple of 4", (long long)ldy);
    if ((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(y) & 7))
        return mortar_fail(MORTAR_ERR_ARG, "spmm: x must be 16-byte and y 8-byte aligned");
    return MORTAR_OK;
}

void fill(SpmmParams &p, const mortar_bcsr_t *W, const int32_t *sched, const uint16_t *x, int64_t M, int64_t ldx,
          uint16_t *y, int64_t ldy) {
    p = SpmmParams{};
    p.row_desc = reinterpret_cast<const u32x4_t *>(W->row_desc);
    p.codes_o = reinterpret_cast<const u32x4_t *>(W->codes_o);
    p.sd_o = reinterpret_cast<const u32x4_t *>(W->sd_o);
    p.col_o = reinterpret_cast<const u32x4_t *>(W->col_o);
    p.sched = reinterpret_cast<const u32x4_t *>(sched);
    p.seg_cb = W->seg_cb < W->Cb ? W->seg_cb : W->Cb; p.nseg = (W->Cb + p.seg_cb - 1) / p.seg_cb; p.Rb = W->Rb;
    p.Cb = W->Cb;
    p.x = x; p.ldx = ldx; p.M = (int)M; p.y = y; p.ldy = ldy;
    p.n_clusters = 1; p.cluster_size = 1 << 30;
    p.uscale = 0.5f * W->uniform_scale;
}

// Token tile of the resident prefill kernel for a matrix with Cb block-columns (0 = does not fit).
int resident_mt(int Cb) {
    for (int mt : {64, 32})
        if (tile_bytes(mt, Cb) <= LDS_BUDGET) return mt;
    return 0;
}

// prefill tiles: 16 wavefronts (4 per SIMD) for both tiles (the 64-token tile with 8 wavefronts was measured 18 % slower
// on the base-width gate_up; the 16-wave form fits its 128 registers with the LDS operands fetched one pair ahead
// instead of two; a 96-token tile of a narrow matrix leaves only two waves per SIMD and is slower still)
template <int NACC, bool ROUTED, int CODE, bool TL = false>
int launch_resident_any(SpmmParams &p, hipStream_t st) {
    switch (resident_mt(p.Cb)) {
        case 64: return mortar_launch_resident<64, NACC, ROUTED, 16, false, CODE, TL>(p, nullptr, 1, st);
        default: return mortar_launch_resident<32, NACC, ROUTED, 16, false, CODE, TL>(p, nullptr, 1, st);
    }
}

constexpr int SEG_WAVES = 16, SEG_UPW = 4;

// Row units per wave of the K-segmented plain product: 4, 2 or 1.  Fewer units per wave mean more workgroups per token
// tile (64 units per workgroup left 8 workgroups for 128 tokens) but every workgroup stages the tile's segments again,
// and workgroups beyond the 256 CUs wait for a second round: take the choice with the least rounds x (staging + units),
// staging weighing about three units.
int segmented_upw(const SpmmParams &p) {
    const int64_t tiles = (p.M + 31) / 32;
    int best = SEG_UPW;
    int64_t best_cost = 0;
    for (int upw = SEG_UPW; upw >= 1; upw >>= 1) {
        const int64_t wgs = tiles * ((p.n_units + SEG_WAVES * upw - 1) / (SEG_WAVES * upw));
        const int64_t cost = ((wgs + 255) / 256) * (3 + upw);
        if (upw == SEG_UPW || cost < best_cost) { best = upw; best_cost = cost; }
    }
    return best;
}

// Plain product of a `down` whose input is stored in tile order (mortar_mlp_bf16): the instantiations that copy their
// token tiles straight into LDS.  The caller has checked that the matrix runs 32-token tiles.
template <int CODE>
int dispatch_gateup_tiled(SpmmParams &p, hipStream_t st) {     // gate_up + SwiGLU storing tile-ordered hidden activations
    if (p.nseg == 1) return launch_resident_any<2, false, CODE, true>(p, st);
    return mortar_launch_segmented<32, 2, false, SEG_WAVES, 2, false, CODE, true>(p, nullptr, 1, st);
}

template <int CODE>
int dispatch_prefill_tiled(SpmmParams &p, hipStream_t st) {
    if (p.nseg == 1) return mortar_launch_resident<32, 1, false, 16, false, CODE, true>(p, nullptr, 1, st);
    switch (segmented_upw(p)) {
        case 1: return mortar_launch_segmented<32, 1, false, SEG_WAVES, 1, false, CODE, true>(p, nullptr, 1, st);
        case 2: return mortar_launch_segmented<32, 1, false, SEG_WAVES, 2, false, CODE, true>(p, nullptr, 1, st);
    }
    return mortar_launch_segmented<32, 1, false, SEG_WAVES, SEG_UPW, false, CODE, true>(p, nullptr, 1, st);
}

template <int CODE>
int dispatch_prefill(int kind, SpmmParams &p, hipStream_t st) {
    switch (kind) {
        case 0:
            if (p.nseg == 1) return launch_resident_any<1, false, CODE>(p, st);
            switch (segmented_upw(p)) {
                case 1: return mortar_launch_segmented<32, 1, false, SEG_WAVES, 1, false, CODE>(p, nullptr, 1, st);
                case 2: return mortar_launch_segmented<32, 1, false, SEG_WAVES, 2, false, CODE>(p, nullptr, 1, st);
            }
            return mortar_launch_segmented<32, 1, false, SEG_WAVES, SEG_UPW, false, CODE>(p, nullptr, 1, st);
        case 1:
            if (p.nseg == 1) return launch_resident_any<2, false, CODE>(p, st);
            return mortar_launch_segmented<32, 2, false, SEG_WAVES, 2, false, CODE>(p, nullptr, 1, st);
        case 2:
            return launch_resident_any<2, true, CODE>(p, st);
        default:
            switch (segmented_upw(p)) {
                case 1: return mortar_launch_segmented<32, 1, true, SEG_WAVES, 1, false, CODE>(p, nullptr, 1, st);
                case 2: return mortar_launch_segmented<32, 1, true, SEG_WAVES, 2, false, CODE>(p, nullptr, 1, st);
            }
            return mortar_launch_segmented<32, 1, true, SEG_WAVES, SEG_UPW, false, CODE>(p, nullptr, 1, st);
    }
}

// kind: 0 spmm, 1 gate_up + SwiGLU, 2 routed gate_up + SwiGLU, 3 spmm with an input mask.
// Prefill-sized launches read the 4-bit code stream when the matrix carries one (cheaper unpack: one conversion
// per register instead of shift + mask); decode-sized launches always stream the 2-bit codes (half the bytes).
// A matrix with one scale (uniform_scale != 0) runs the kernels that multiply +-2 / 0 blocks and scale the
// accumulators once (decode-sized launches always, prefill-sized ones through the 4-bit stream).
int dispatch(int kind, SpmmParams &p, const mortar_bcsr_t *W, hipStream_t st) {
    // products over several K segments have small-tile forms beyond the decode sizes as well (the launcher returns -1
    // once they would need more than one round of workgroups)
    if (p.M <= MORTAR_SMALLM_MAX || ((kind == 0 || kind == 1 || kind == 3) && p.nseg > 1)) {
        const int rc = mortar_smallm_launch(kind, p, nullptr, 1, st);
        if (rc >= 0) return rc;
    }
    if (W->codes4_o) {
        p.codes_o = reinterpret_cast<const u32x4_t *>(W->codes4_o);
        if (p.uscale != 0.f) return dispatch_prefill<CODE_4BIT | CODE_UNIFORM>(kind, p, st);
        return dispatch_prefill<CODE_4BIT>(kind, p, st);
    }
    p.uscale = 0.f;      // per-block path: the 2-bit prefill kernels multiply every block by its own pattern
    return dispatch_prefill<CODE_2BIT>(kind, p, st);
}

}  // namespace

extern "C" int mortar_prefill_max_seg_cb(void) { return (LDS_BUDGET - LDS_PAD * 16) / (32 * 32); }
extern "C" int mortar_decode_max_seg_cb(int32_t rows) {
    return (LDS_BUDGET - LDS_PAD * 16) / ((rows <= 4 ? 4 : rows <= 16 ? 16 : 32) * 32);
}

extern "C" int mortar_route_tile(int32_t Cb, int64_t M) {
    if (M > 0 && M <= MORTAR_SMALLM_MAX) {
        const int t = mortar_smallm_tile(Cb, Cb, M, 2);
        if (t > 0) return t;
    }
    return resident_mt(Cb);
}

extern "C" int mortar_spmm_bf16(const mortar_bcsr_t *W, const int32_t *sched, const uint16_t *x, int64_t M,
                                int64_t ldx, uint16_t *y, int64_t ldy, void *stream) {
    int rc = check_common(W, x, M, ldx, y, ldy, W ? (int64_t)W->Rb * 16 : 0);
    if (rc) return rc;
    SpmmParams p;
    fill(p, W, sched, x, M, ldx, y, ldy);
    p.n_units = W->Rb;
    return dispatch(0, p, W, static_cast<hipStream_t>(stream));
}

int mortar_spmm_codes_f32(const mortar_bcsr_t *W, const int32_t *sched, const uint16_t *x, int64_t M, int64_t ldx,
                          float *y32, int64_t ldy, void *stream) {
    int rc = check_common(W, x, M, ldx, reinterpret_cast<const uint16_t *>(y32), ldy, W ? (int64_t)W->Rb * 16 : 0);
    if (rc) return rc;
    if (reinterpret_cast<uintptr_t>(y32) & 15) return mortar_fail(MORTAR_ERR_ARG, "spmm: the fp32 output must be 16-byte aligned");
    SpmmParams p;
    fill(p, W, sched, x, M, ldx, nullptr, ldy);
    p.n_units = W->Rb;
    p.y32 = y32;
    p.uscale = 0.5f;                       // the kernels multiply the blocks as +-2 / 0
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (M <= MORTAR_SMALLM_MAX) {
        rc = mortar_smallm_launch(0, p, nullptr, 1, st);
        if (rc >= 0) return rc;
    }
    if (!W->codes4_o) return MORTAR_NO_KERNEL;      // prefill-sized tiles multiply +-2 / 0 blocks only from the 4-bit stream
    p.codes_o = reinterpret_cast<const u32x4_t *>(W->codes4_o);
    return dispatch_prefill<CODE_4BIT | CODE_UNIFORM>(0, p, st);
}

extern "C" int mortar_spmm_bf16_masked(const mortar_bcsr_t *W, const int32_t *sched, const uint16_t *x, int64_t M,
                                       int64_t ldx, uint16_t *y, int64_t ldy, const uint8_t *active,
                                       int32_t n_clusters, void *stream) {
    int rc = check_common(W, x, M, ldx, y, ldy, W ? (int64_t)W->Rb * 16 : 0);
    if (rc) return rc;
    if (!active || n_clusters <= 0 || (W->Cb * 16) % n_clusters || ((W->Cb * 16) / n_clusters) % 8)
        return mortar_fail(MORTAR_ERR_ARG, "spmm_masked: in_features/n_clusters must be a multiple of 8");
    SpmmParams p;
    fill(p, W, sched, x, M, ldx, y, ldy);
    p.n_units = W->Rb;
    p.active = active; p.n_clusters = n_clusters; p.cluster_size = (W->Cb * 16) / n_clusters;
    return dispatch(3, p, W, static_cast<hipStream_t>(stream));
}

extern "C" int mortar_spmm_hc_post(const mortar_bcsr_t *W, const int32_t *sched, const uint16_t *x, int64_t M, int64_t ldx,
                                   const void *carrier, int32_t carrier_f32, int32_t n_streams, const float *hres,
                                   const float *hpost, const void *term, void *out, const uint8_t *active,
                                   int32_t n_clusters, void *stream) {
    // the plain store is replaced, so y / ldy only have to pass the common checks
    int rc = check_common(W, x, M, ldx, reinterpret_cast<const uint16_t *>(out), W ? (int64_t)W->Rb * 16 : 0, W ? (int64_t)W->Rb * 16 : 0);
    if (rc) return rc;
    if (M > MORTAR_SMALLM_MAX)
        return mortar_fail(MORTAR_ERR_LIMIT, "spmm_hc_post: the fused POST write serves decode batches (M <= %d, got %lld); "
                           "call mortar_spmm_bf16 and combine separately", MORTAR_SMALLM_MAX, (long long)M);
    if (!carrier || !hres || !hpost || !out) return mortar_fail(MORTAR_ERR_ARG, "spmm_hc_post: null pointer");
    if (n_streams < 1 || n_streams > 4) return mortar_fail(MORTAR_ERR_LIMIT, "spmm_hc_post: %d carrier streams outside 1..4", n_streams);
    const uintptr_t al = carrier_f32 ? 15 : 7;
    if ((reinterpret_cast<uintptr_t>(carrier) & al) || (reinterpret_cast<uintptr_t>(out) & al) || (reinterpret_cast<uintptr_t>(term) & al))
        return mortar_fail(MORTAR_ERR_ARG, "spmm_hc_post: carrier, term and out must be %d-byte aligned", (int)al + 1);
    SpmmParams p;
    fill(p, W, sched, x, M, ldx, reinterpret_cast<uint16_t *>(out), (int64_t)W->Rb * 16);
    p.n_units = W->Rb;
    p.hc_h = carrier; p.hc_out = out; p.hc_res = hres; p.hc_post = hpost; p.hc_term = term; p.hc_n = n_streams; p.hc_f32 = carrier_f32 != 0;
    int kind = 0;
    if (active) {
        if (n_clusters <= 0 || (W->Cb * 16) % n_clusters || ((W->Cb * 16) / n_clusters) % 8)
            return mortar_fail(MORTAR_ERR_ARG, "spmm_hc_post: in_features/n_clusters must be a multiple of 8");
        p.active = active; p.n_clusters = n_clusters; p.cluster_size = (W->Cb * 16) / n_clusters;
        kind = 3;
    }
    rc = mortar_smallm_launch(kind, p, nullptr, 1, static_cast<hipStream_t>(stream));
    if (rc < 0 && rc != MORTAR_ERR_HIP) return mortar_fail(MORTAR_ERR_LIMIT, "spmm_hc_post: shape has no small-tile kernel");
    return rc;
}

namespace {
int gateup_common(const mortar_bcsr_t *W, const int32_t *sched, const uint16_t *x, int64_t M, int64_t ldx, bool norm,
                  const uint16_t *norm_w, float norm_eps, uint16_t *h, int64_t ldh, const float *gates,
                  int32_t n_clusters, const int32_t *tok_cnt, const uint8_t *tok_list, void *stream);
}

extern "C" int mortar_gateup_swiglu_bf16(const mortar_bcsr_t *W, const int32_t *sched, const uint16_t *x, int64_t M,
                                         int64_t ldx, uint16_t *h, int64_t ldh, const float *gates,
                                         int32_t n_clusters, const int32_t *tok_cnt, const uint8_t *tok_list,
                                         void *stream) {
    return gateup_common(W, sched, x, M, ldx, false, nullptr, 0.f, h, ldh, gates, n_clusters, tok_cnt, tok_list, stream);
}

extern "C" int mortar_norm_gateup_swiglu_bf16(const mortar_bcsr_t *W, const int32_t *sched, const uint16_t *x,
                                              int64_t M, int64_t ldx, const uint16_t *norm_w, float norm_eps,
                                              uint16_t *h, int64_t ldh, const float *gates, int32_t n_clusters,
                                              const int32_t *tok_cnt, const uint8_t *tok_list, void *stream) {
    return gateup_common(W, sched, x, M, ldx, true, norm_w, norm_eps, h, ldh, gates, n_clusters, tok_cnt, tok_list, stream);
}

extern "C" int mortar_norm_fusable(int32_t Cb) { return Cb > 0 && Cb <= NORM_MAX_CB && resident_mt(Cb) != 0; }

namespace {
int gateup_common(const mortar_bcsr_t *W, const int32_t *sched, const uint16_t *x, int64_t M, int64_t ldx, bool norm,
                  const uint16_t *norm_w, float norm_eps, uint16_t *h, int64_t ldh, const float *gates,
                  int32_t n_clusters, const int32_t *tok_cnt, const uint8_t *tok_list, void *stream) {
    if (W && (W->Rb & 1)) return mortar_fail(MORTAR_ERR_ARG, "gateup: odd number of block-rows");
    const int64_t d_ff = W ? (int64_t)W->Rb * 8 : 0;
    int rc = check_common(W, x, M, ldx, h, ldh, d_ff);
    if (rc) return rc;
    SpmmParams p;
    fill(p, W, sched, x, M, ldx, h, ldh);
    p.n_units = W->Rb / 2;
    if (norm) {
        if (!mortar_norm_fusable(W->Cb) || p.nseg != 1)
            return mortar_fail(MORTAR_ERR_LIMIT, "gateup: the fused RMSNorm needs in_features <= %d in one K segment "
                               "(mortar_norm_fusable() == 0: call mortar_rmsnorm_bf16 first)", NORM_MAX_CB * 16);
        if (!(norm_eps >= 0.f)) return mortar_fail(MORTAR_ERR_ARG, "gateup: norm_eps must be >= 0");
        if (reinterpret_cast<uintptr_t>(norm_w) & 15) return mortar_fail(MORTAR_ERR_ARG, "gateup: norm_w must be 16-byte aligned");
        p.norm = 1; p.norm_eps = norm_eps; p.norm_w = norm_w;
    }
    if (gates) {
        if (n_clusters <= 0 || d_ff % n_clusters || (d_ff / n_clusters) % 4)
            return mortar_fail(MORTAR_ERR_ARG, "gateup: d_ff / n_clusters must be a whole multiple of 4");
        p.gates = gates; p.n_clusters = n_clusters; p.cluster_size = (int)(d_ff / n_clusters);
    }
    if (tok_cnt || tok_list) {
        if (!tok_cnt || !tok_list || !gates) return mortar_fail(MORTAR_ERR_ARG, "gateup: routed mode needs gates, tok_cnt and tok_list");
        if (p.cluster_size % 16) return mortar_fail(MORTAR_ERR_ARG, "gateup: routed mode needs cluster_size %% 16 == 0");
        if (mortar_route_tile(W->Cb, M) == 0)
            return mortar_fail(MORTAR_ERR_LIMIT, "gateup: routed mode needs in_features to fit one LDS tile "
                               "(mortar_route_tile() == 0: call without tok_cnt / tok_list)");
        p.tok_cnt = tok_cnt; p.tok_list = tok_list;
        return dispatch(2, p, W, static_cast<hipStream_t>(stream));
    }
    return dispatch(1, p, W, static_cast<hipStream_t>(stream));
}
}  // namespace

// ---- the MLP as one call ------------------------------------------------------------------------------------

namespace {
// Rows from which both launches of the MLP certainly run the 32-token prefill tiles (below, products over several K
// segments have small-tile forms): the hidden activations then travel in tile order.
constexpr int64_t MLP_TILED_MIN_ROWS = 513;

bool mlp_tiled(const mortar_bcsr_t *Wgu, const mortar_bcsr_t *Wdn, int64_t M) {
    if (M < MLP_TILED_MIN_ROWS || !Wgu->codes4_o || !Wdn->codes4_o) return false;
    const int seg = Wdn->seg_cb < Wdn->Cb ? Wdn->seg_cb : Wdn->Cb;
    if (tile_bytes(32, seg) > LDS_BUDGET) return false;
    if (seg == Wdn->Cb && resident_mt(Wdn->Cb) != 32) return false;      // a narrow `down` runs 64-token tiles
    return ((M + 31) / 32 * 32) * ((int64_t)Wdn->Cb * 16) < ((int64_t)1 << 31);
}
}  // namespace

extern "C" int64_t mortar_mlp_hidden_bytes(int64_t M, int32_t d_ff) {
    if (M <= 0 || d_ff <= 0 || d_ff % 16) return 0;
    return (M + 31) / 32 * 32 * (int64_t)d_ff * 2;
}

extern "C" int mortar_mlp_bf16(const mortar_bcsr_t *Wgu, const int32_t *sched_gu, const mortar_bcsr_t *Wdn,
                               const int32_t *sched_dn, const uint16_t *x, int64_t M, int64_t ldx, int32_t norm,
                               const uint16_t *norm_w, float norm_eps, const float *gates, int32_t n_clusters,
                               void *hidden, uint16_t *y, int64_t ldy, int32_t phase, void *stream) {
    if (!Wgu || !Wdn || !hidden) return mortar_fail(MORTAR_ERR_ARG, "mlp: null pointer");
    if (Wgu->Rb & 1) return mortar_fail(MORTAR_ERR_ARG, "mlp: gate_up has an odd number of block-rows");
    if (Wdn->Cb * 2 != Wgu->Rb) return mortar_fail(MORTAR_ERR_ARG, "mlp: down has %d input block-columns, gate_up %d gate/up units", Wdn->Cb, Wgu->Rb / 2);
    if (phase < 0 || phase > 2) return mortar_fail(MORTAR_ERR_ARG, "mlp: phase %d not in 0..2", phase);
    if (reinterpret_cast<uintptr_t>(hidden) & 15) return mortar_fail(MORTAR_ERR_ARG, "mlp: hidden must be 16-byte aligned");
    const int64_t d_ff = (int64_t)Wdn->Cb * 16;
    uint16_t *h = static_cast<uint16_t *>(hidden);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool tiled = M > 0 && mlp_tiled(Wgu, Wdn, M);
    if (!tiled) {        // row-major hidden activations through the separate entry points
        int rc = MORTAR_OK;
        if (phase != 2)
            rc = gateup_common(Wgu, sched_gu, x, M, ldx, norm != 0, norm_w, norm_eps, h, d_ff, gates, n_clusters, nullptr, nullptr, stream);
        if (rc == MORTAR_OK && phase != 1) rc = mortar_spmm_bf16(Wdn, sched_dn, h, M, d_ff, y, ldy, stream);
        return rc;
    }
    if (phase != 2) {
        int rc = check_common(Wgu, x, M, ldx, h, d_ff, d_ff);
        if (rc) return rc;
        SpmmParams p;
        fill(p, Wgu, sched_gu, x, M, ldx, h, d_ff);
        p.n_units = Wgu->Rb / 2;
        if (norm) {
            if (!mortar_norm_fusable(Wgu->Cb) || p.nseg != 1)
                return mortar_fail(MORTAR_ERR_LIMIT, "mlp: the fused RMSNorm needs in_features <= %d in one K segment "
                                   "(mortar_norm_fusable() == 0: call mortar_rmsnorm_bf16 first)", NORM_MAX_CB * 16);
            if (!(norm_eps >= 0.f)) return mortar_fail(MORTAR_ERR_ARG, "mlp: norm_eps must be >= 0");
            if (reinterpret_cast<uintptr_t>(norm_w) & 15) return mortar_fail(MORTAR_ERR_ARG, "mlp: norm_w must be 16-byte aligned");
            p.norm = 1; p.norm_eps = norm_eps; p.norm_w = norm_w;
        }
        if (gates) {
            if (n_clusters <= 0 || d_ff % n_clusters || (d_ff / n_clusters) % 4)
                return mortar_fail(MORTAR_ERR_ARG, "mlp: d_ff / n_clusters must be a whole multiple of 4");
            p.gates = gates; p.n_clusters = n_clusters; p.cluster_size = (int)(d_ff / n_clusters);
        }
        p.y_tiled = 1;
        p.codes_o = reinterpret_cast<const u32x4_t *>(Wgu->codes4_o);
        rc = p.uscale != 0.f ? dispatch_gateup_tiled<CODE_4BIT | CODE_UNIFORM>(p, st) : dispatch_gateup_tiled<CODE_4BIT>(p, st);
        if (rc) return rc;
    }
    if (phase != 1) {
        int rc = check_common(Wdn, h, M, d_ff, y, ldy, (int64_t)Wdn->Rb * 16);
        if (rc) return rc;
        SpmmParams p;
        fill(p, Wdn, sched_dn, h, M, d_ff, y, ldy);
        p.n_units = Wdn->Rb;
        p.x_tiled = 1;
        p.codes_o = reinterpret_cast<const u32x4_t *>(Wdn->codes4_o);
        rc = p.uscale != 0.f ? dispatch_prefill_tiled<CODE_4BIT | CODE_UNIFORM>(p, st) : dispatch_prefill_tiled<CODE_4BIT>(p, st);
        if (rc) return rc;
    }
    return MORTAR_OK;
}

// ---- layer-batched small-M launches ---------------------------------------------------------------------

extern "C" int64_t mortar_stack_table_bytes(int32_t n_layers) {
    return n_layers > 0 ? (int64_t)n_layers * (int64_t)sizeof(SpmmParams) : 0;
}

extern "C" int mortar_stack_prepare(int32_t swiglu, int32_t n_layers, const mortar_bcsr_t *W,
                                    const int32_t *const *sched, const uint16_t *const *x, uint16_t *const *y,
                                    int64_t M, int64_t ldx, int64_t ldy, void *table_dev, void *stream) {
    if (n_layers <= 0 || n_layers > 65535 || !W || !x || !y || !table_dev)
        return mortar_fail(MORTAR_ERR_ARG, "stack_prepare: bad arguments");
    if (M > 64) return mortar_fail(MORTAR_ERR_LIMIT, "stack_prepare: layer-batched launches serve M <= 64 (got %lld)", (long long)M);
    std::vector<SpmmParams> tab((size_t)n_layers);
    for (int l = 0; l < n_layers; ++l) {
        if (W[l].Rb != W[0].Rb || W[l].Cb != W[0].Cb || W[l].seg_cb != W[0].seg_cb)
            return mortar_fail(MORTAR_ERR_ARG, "stack_prepare: layer %d differs in shape from layer 0", l);
        if (swiglu && (W[l].Rb & 1)) return mortar_fail(MORTAR_ERR_ARG, "stack_prepare: odd number of block-rows");
        if ((W[l].uniform_scale != 0.f) != (W[0].uniform_scale != 0.f))
            return mortar_fail(MORTAR_ERR_ARG, "stack_prepare: layer %d and layer 0 differ in having a uniform scale "
                               "(set uniform_scale = 0 on all layers to run them together)", l);
        const int64_t out_cols = swiglu ? (int64_t)W[l].Rb * 8 : (int64_t)W[l].Rb * 16;
        int rc = check_common(&W[l], x[l], M, ldx, y[l], ldy, out_cols);
        if (rc) return rc;
        SpmmParams &p = tab[(size_t)l];
        fill(p, &W[l], sched ? sched[l] : nullptr, x[l], M, ldx, y[l], ldy);
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
    if (n_layers <= 0 || n_layers > 65535 || !W0 || !table_dev || M <= 0 || M > 64)
        return mortar_fail(MORTAR_ERR_ARG, "stack_run: bad arguments");
    SpmmParams p;
    fill(p, W0, nullptr, nullptr, M, 0, nullptr, 0);
    p.n_units = swiglu ? W0->Rb / 2 : W0->Rb;
    const int rc = mortar_smallm_launch(swiglu ? 1 : 0, p, static_cast<const SpmmParams *>(table_dev), n_layers,
                                        static_cast<hipStream_t>(stream));
    if (rc < 0) return mortar_fail(MORTAR_ERR_LIMIT, "stack_run: shape has no small-M kernel");
    return rc;
}
