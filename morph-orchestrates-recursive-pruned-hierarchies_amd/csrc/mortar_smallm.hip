// Small-M (decode, M <= 16) instantiations of the octet-stream SpMM kernels.
//
// Replaces the reference's decode GEMV over packed ternary strips (morph/kernels/triton/fused_decode_step.py:
// 1701-1842, mortar_gemv) for batches of up to 16 rows: the batch is one token tile of 4 or 16 tokens, so a
// weight block is read once per launch and the kernel is bound by the weight stream.  Workgroups are small
// (2 wavefronts) when one matrix has to cover the chip and 8 wavefronts when many layers share a launch.
#include "mortar_spmm_core.h"

namespace {

template <int MT, int WAVES>
int launch_kind(int kind, bool resident, SpmmParams &p, const SpmmParams *table, int layers, hipStream_t st) {
    if (table) {      // layer-batched: plain products and unrouted gate_up only
        if (resident && kind == 0) return mortar_launch_resident<MT, 1, false, WAVES, true>(p, table, layers, st);
        if (resident && kind == 1) return mortar_launch_resident<MT, 2, false, WAVES, true>(p, table, layers, st);
        if (!resident && kind == 0 && MT == 16) return mortar_launch_segmented<16, 1, false, WAVES, 1, true>(p, table, layers, st);
    } else if (resident) {
        switch (kind) {
            case 0: return mortar_launch_resident<MT, 1, false, WAVES>(p, nullptr, 1, st);
            case 1: return mortar_launch_resident<MT, 2, false, WAVES>(p, nullptr, 1, st);
            case 2: return mortar_launch_resident<MT, 2, true, WAVES>(p, nullptr, 1, st);
        }
    } else if (MT == 16) {
        switch (kind) {
            case 0: return mortar_launch_segmented<16, 1, false, WAVES, 1>(p, nullptr, 1, st);
            case 3: return mortar_launch_segmented<16, 1, true, WAVES, 1>(p, nullptr, 1, st);
        }
    }
    return mortar_fail(MORTAR_ERR_ARG, "small-M dispatch: no kernel for kind %d", kind);
}

bool fits(int mt, int ncb) { return tile_bytes(mt, ncb) <= LDS_BUDGET; }

}  // namespace

// Token tile of the small-M path: 4 or 16, negative when the tile is served by the segmented kernel,
// 0 when (M, kind) has no small-M variant.
int mortar_smallm_tile(int Cb, int seg_cb, int64_t M, int kind) {
    (void)seg_cb;
    if (M <= 4 && kind != 3 && fits(4, Cb)) return 4;
    if (M <= 16) {
        if (kind != 3 && fits(16, Cb)) return 16;
        if (kind == 0 || kind == 3) return -16;
    }
    return 0;
}

int mortar_smallm_launch(int kind, SpmmParams &p, const SpmmParams *table, int layers, hipStream_t st) {
    const int t = mortar_smallm_tile(p.Cb, p.seg_cb, p.M, kind);
    if (t == 0) return -1;
    const bool resident = t > 0;
    const bool wide = (int64_t)layers * p.n_units >= 8 * 512;   // enough units to fill the chip with 8-wave groups
    if (t == 4) return wide ? launch_kind<4, 8>(kind, true, p, table, layers, st) : launch_kind<4, 2>(kind, true, p, table, layers, st);
    return wide ? launch_kind<16, 8>(kind, resident, p, table, layers, st) : launch_kind<16, 2>(kind, resident, p, table, layers, st);
}

int mortar_smallm_shape(int kind, SpmmParams &p, int layers) {
    const int t = mortar_smallm_tile(p.Cb, p.seg_cb, p.M, kind);
    if (t == 0) return mortar_fail(MORTAR_ERR_LIMIT, "shape has no small-M kernel");
    const bool wide = (int64_t)layers * p.n_units >= 8 * 512;
    if (t == 4) {
        if (wide) mortar_resident_shape<4, 8>(p, layers); else mortar_resident_shape<4, 2>(p, layers);
    } else if (t == 16) {
        if (wide) mortar_resident_shape<16, 8>(p, layers); else mortar_resident_shape<16, 2>(p, layers);
    } else {
        if (wide) mortar_segmented_shape<16, 8, 1>(p); else mortar_segmented_shape<16, 2, 1>(p);
    }
    return MORTAR_OK;
}
