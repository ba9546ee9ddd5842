// Small-M (decode, M <= 64) instantiations of the octet-stream SpMM kernels.
//
// Replaces the reference's decode GEMV over packed ternary strips (morph/kernels/triton/fused_decode_step.py:
// 1502-1547 mortar_gemv, kernels 1341-1459) for batches of up to 64 rows: the batch is one token tile of 4 or 16 tokens (up to four
// 16-token tiles above 16 rows), so a weight block is read from HBM once per launch and the kernel is bound by
// the weight stream.  Workgroups are small
// (2 wavefronts) when one matrix has to cover the chip and 8 or 16 wavefronts when many layers share a launch.
#include "mortar_spmm_core.h"

namespace {

// Row units per wave of the layer-batched K-segmented kernel: two (half the workgroups, so half the tile staging and
// barriers; measured 61 against 69 us for 160 `down` layers at b = 16, three units 64 us, four 75 us) as long as the
// workgroups still fill the chip's resident slots about once.
int segmented_stack_upw(const SpmmParams &p, int layers, int waves) {
    const int by_lds = (160 * 1024) / tile_bytes(16, p.seg_cb), by_waves = 32 / waves;
    const int64_t slots = 256 * (int64_t)(by_lds < by_waves ? by_lds : by_waves);
    const int64_t n_mtiles = (p.M + 15) / 16;
    return (int64_t)layers * n_mtiles * ((p.n_units + waves * 2 - 1) / (waves * 2)) * 10 >= slots * 9 ? 2 : 1;
}

template <int MT, int WAVES, int CODE>
int launch_kind(int kind, bool resident, SpmmParams &p, const SpmmParams *table, int layers, hipStream_t st) {
    if (table) {      // layer-batched: plain products and unrouted gate_up only
        if (resident && kind == 0) return mortar_launch_resident<MT, 1, false, WAVES, true, CODE>(p, table, layers, st);
        if (resident && kind == 1) return mortar_launch_resident<MT, 2, false, WAVES, true, CODE>(p, table, layers, st);
        if (!resident && kind == 0 && MT == 16) {
            if (segmented_stack_upw(p, layers, WAVES) == 2)
                return mortar_launch_segmented<16, 1, false, WAVES, 2, true, CODE>(p, table, layers, st);
            return mortar_launch_segmented<16, 1, false, WAVES, 1, true, CODE>(p, table, layers, st);
        }
    } else if (resident) {
        switch (kind) {
            case 0: return mortar_launch_resident<MT, 1, false, WAVES, false, CODE>(p, nullptr, 1, st);
            case 1: return mortar_launch_resident<MT, 2, false, WAVES, false, CODE>(p, nullptr, 1, st);
            case 2: return mortar_launch_resident<MT, 2, true, WAVES, false, CODE>(p, nullptr, 1, st);
        }
    } else if (MT == 16) {
        switch (kind) {
            case 0: return mortar_launch_segmented<16, 1, false, WAVES, 1, false, CODE>(p, nullptr, 1, st);
            case 1: if (WAVES == 8) return mortar_launch_segmented<16, 2, false, 8, 1, false, CODE>(p, nullptr, 1, st); break;
            case 3: return mortar_launch_segmented<16, 1, true, WAVES, 1, false, CODE>(p, nullptr, 1, st);
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
    if (M <= MORTAR_SMALLM_MAX) {      // up to four 16-token tiles
        if (kind != 3 && fits(16, Cb)) return 16;
        if (kind == 0 || kind == 3) return -16;
    }
    return 0;
}

// Wavefronts per workgroup: 2 when one matrix has to cover the chip; otherwise 8, or 16 when the tile is so
// large that only two workgroups fit in a CU's LDS (keeps 32 wavefronts per CU resident either way).
static int pick_waves(int t, const SpmmParams &p, int layers) {
    if ((int64_t)layers * p.n_units < 8 * 512) return 2;
    const int bytes = t > 0 ? tile_bytes(t, p.Cb) : tile_bytes(16, p.seg_cb);
    return bytes > 40 * 1024 ? 16 : 8;
}

// Part-split launch for one matrix: PW waves per unit, PW = 4, 3 or 2, dividing the unit's part count where one does.
template <int MT, int CODE>
static int launch_partsplit(int kind, SpmmParams &p, hipStream_t st) {
    const int nacc = (kind == 0 || kind == 3) ? 1 : 2, nparts = p.nseg * nacc;
    // a part count no wave count divides (5, 7, 11 ... K segments): the waves of a unit take parts q, q + PW, ... and
    // some take one more than others - still far better than one wave per unit ([4096, 11008] at one row: 9.0 -> 5.6 us)
    int pw = nparts % 4 == 0 ? 4 : (nparts % 3 == 0 ? 3 : (nparts % 2 == 0 ? 2 : 0));
    if (pw == 0 && nparts >= 5) pw = (nparts + 3) / 4 < (nparts + 2) / 3 ? 4 : 3;
    // LDS: the tile, then the partial sums of the workgroup's PW * 4 waves (1 KB per wave, accumulator and sub-tile)
    if (pw == 0 || tile_bytes(MT, p.Cb) + pw * 4 * nacc * ((MT + 15) / 16) * 1024 > 160 * 1024) return -1;
    // more tiles x 4-unit workgroups than one round holds (one workgroup fills a CU): 8 units per workgroup, two waves
    // each (gate_up of d_model 2048 at 33..64 rows: 8.3 -> 6.1 us)
    if (kind != 2 && nparts >= 2 && (p.M + MT - 1) / MT * (int64_t)((p.n_units + 3) / 4) > 256 &&
        tile_bytes(MT, p.Cb) + 16 * nacc * ((MT + 15) / 16) * 1024 <= 160 * 1024) {
        switch (kind) {
            case 0: return mortar_launch_partsplit<MT, 1, false, false, 2, 8, CODE>(p, st);
            case 1: return mortar_launch_partsplit<MT, 2, false, false, 2, 8, CODE>(p, st);
            case 3: return mortar_launch_partsplit<MT, 1, false, true, 2, 8, CODE>(p, st);
        }
    }
    switch (kind * 10 + pw) {
        case 2: return mortar_launch_partsplit<MT, 1, false, false, 2, 4, CODE>(p, st);
        case 3: return mortar_launch_partsplit<MT, 1, false, false, 3, 4, CODE>(p, st);
        case 4: return mortar_launch_partsplit<MT, 1, false, false, 4, 4, CODE>(p, st);
        case 12: return mortar_launch_partsplit<MT, 2, false, false, 2, 4, CODE>(p, st);
        case 13: return mortar_launch_partsplit<MT, 2, false, false, 3, 4, CODE>(p, st);
        case 14: return mortar_launch_partsplit<MT, 2, false, false, 4, 4, CODE>(p, st);
        case 22: return mortar_launch_partsplit<MT, 2, true, false, 2, 4, CODE>(p, st);
        case 23: return mortar_launch_partsplit<MT, 2, true, false, 3, 4, CODE>(p, st);
        case 24: return mortar_launch_partsplit<MT, 2, true, false, 4, 4, CODE>(p, st);
        case 32: return mortar_launch_partsplit<MT, 1, false, true, 2, 4, CODE>(p, st);
        case 33: return mortar_launch_partsplit<MT, 1, false, true, 3, 4, CODE>(p, st);
        case 34: return mortar_launch_partsplit<MT, 1, false, true, 4, 4, CODE>(p, st);
    }
    return -1;
}

// Layer-batched launches of 17..64 rows run the 32-token prefill tiles (one unpack feeds two MFMAs) when the shape has
// one: 1 = resident tile, 2 = K-segmented (plain products only), 0 = none (16-token tiles serve the rows).  They keep
// reading the 2-bit stream: the 4-bit one (two instructions less per block pair, twice the bytes) was measured no
// faster for 160 layers at 32 and 64 rows.
static int stack_tile32(int kind, const SpmmParams &p) {
    // 17..32 and 49..64 rows: one or two 32-token tiles instead of two or four 16-token ones (33..48 rows would leave
    // the second 32-token tile half empty: three 16-token tiles cost the same there)
    if (p.M <= 16 || (p.M > 32 && p.M <= 48) || kind > 1) return 0;
    if (p.nseg == 1 && fits(32, p.Cb)) return 1;
    if (kind == 0 && p.nseg > 1 && fits(32, p.seg_cb)) return 2;
    return 0;
}

static bool wide_gate_up_table(int kind, const SpmmParams &p) {
    return kind == 1 && p.M <= MORTAR_SMALLM_MAX && p.nseg > 1 && !fits(16, p.Cb) && fits(16, p.seg_cb) && !(p.M <= 4 && fits(4, p.Cb));
}

template <int CODE>
static int smallm_launch_code(int kind, SpmmParams &p, const SpmmParams *table, int layers, hipStream_t st) {
    if (table) {
        switch (stack_tile32(kind, p)) {
            case 1:
                if (kind == 0) return mortar_launch_resident<32, 1, false, 16, true, CODE>(p, table, layers, st);
                return mortar_launch_resident<32, 2, false, 16, true, CODE>(p, table, layers, st);
            case 2: return mortar_launch_segmented<32, 1, false, 16, 4, true, CODE>(p, table, layers, st);
        }
    }
    if (!table && p.M > MORTAR_SMALLM_MAX) {
        // 65 rows and more: a plain product over several K segments, whose 32-token prefill tiles walk the segments
        // one after another in few workgroups, has faster small-tile forms, as long as these fit one round of
        // workgroups: 8-token tiles of all K with a row's parts on different waves up to 128 rows (`down`: 10.7 against
        // 13.3 us), else 16-token K-segmented tiles with 8 waves (256 rows: 11.1 against 13.7 us) or 16 waves (384 rows:
        // 12.8 against 14.0 us).
        // gate_up over several K segments: the 16-token tiles with 8 waves of one gate/up unit each, while they fit the
        // chip's slots once (d_model 3072 at 65..128 rows: 12.2..13.2 against 20..21 us for the 32-token tiles)
        if (kind == 1 && p.nseg > 1 && fits(16, p.seg_cb)) {
            if ((p.M + 15) / 16 * (int64_t)((p.n_units + 7) / 8) <= 512) return launch_kind<16, 8, CODE>(1, false, p, nullptr, 1, st);
            return -1;
        }
        if ((kind != 0 && kind != 3) || p.nseg <= 1) return -1;
        if (p.M <= MORTAR_PARTSPLIT_MAX && fits(8, p.Cb)) {
            const int rc = launch_partsplit<8, CODE>(kind, p, st);
            if (rc >= 0) return rc;
        }
        const int64_t tiles = (p.M + 15) / 16;
        if (tiles * ((p.n_units + 7) / 8) <= 256) return launch_kind<16, 8, CODE>(kind, false, p, nullptr, 1, st);
        if (tiles * ((p.n_units + 15) / 16) <= 256) return launch_kind<16, 16, CODE>(kind, false, p, nullptr, 1, st);
        return -1;
    }
    const int t = mortar_smallm_tile(p.Cb, p.seg_cb, p.M, kind);
    // One matrix whose 16-token tile of all K leaves no room for the partial sums of the part-split form, or (gate_up)
    // does not fit at all: several 8-token tiles, else 4-token tiles, while they make few enough workgroups - the weights
    // are then read from L2 once per tile, which beats one 2-wave workgroup per CU staging 130 KB or the 32-token
    // prefill tiles (gate_up [22016, 4096] at 12.5 %: 5.6 us at 5..8 rows against 17..19 us; [43648, 8192] with 4-token
    // tiles: 16 against 22.5 us at 5..8 rows, but 34 against 23 us at 16).
    auto narrow_tiles = [&]() {
        // limits in 4-unit workgroups, one of which fills a CU's LDS (the launcher packs 8 units into one beyond 256):
        // 768 for 8-token tiles, 512 for 4-token ones, which re-read the weights more often (704 when there are only
        // two tiles); twice these limits measured slower than the K-segmented tiles that follow
        const int64_t per_tile = (p.n_units + 3) / 4;
        int rc = -1;
        if ((p.M + 7) / 8 * per_tile <= 768) rc = launch_partsplit<8, CODE>(kind, p, st);
        const int64_t t4 = (p.M + 3) / 4;
        if (rc < 0 && (t4 * per_tile <= 512 || (t4 <= 2 && t4 * per_tile <= 704)) && fits(4, p.Cb)) rc = launch_partsplit<4, CODE>(kind, p, st);
        // rows of more than 19904 values: one or two 2-token tiles (down [8192, 21824] at 25 %, 12 MB of weights:
        // 11.5 us at 1..4 rows against 18.7 us for the work-list kernel; the same time as that kernel at 8 rows)
        if (rc < 0 && !fits(4, p.Cb) && p.M <= 4 && fits(2, p.Cb)) rc = launch_partsplit<2, CODE>(kind, p, st);
        return rc;
    };
    // gate_up over several K segments with more rows than the narrow tiles take: K-segmented 16-token tiles, 8 waves of
    // one gate/up unit each, while they fit the chip's slots once (two workgroups per CU) - the 32-token prefill tiles
    // leave most CUs idle at these row counts
    auto segmented_gate_up = [&]() {
        if (kind != 1 || p.nseg <= 1 || !fits(16, p.seg_cb)) return -1;
        if ((p.M + 15) / 16 * (int64_t)((p.n_units + 7) / 8) > 512) return -1;
        return launch_kind<16, 8, CODE>(1, false, p, nullptr, 1, st);
    };
    // gate_up: one narrow tile where the rows fit one (5.6..7 us), else the K-segmented tiles (10..12 us at 16..32 rows,
    // where two to four 8-token tiles take 10..15 us and two 4-token tiles of d_model 8192 17 us), else narrow tiles
    auto wide_gate_up = [&]() {
        int rc = -1;
        if (p.M <= 8) rc = launch_partsplit<8, CODE>(kind, p, st);
        if (rc < 0 && p.M <= 4 && fits(4, p.Cb)) rc = launch_partsplit<4, CODE>(kind, p, st);
        if (rc < 0) rc = segmented_gate_up();
        if (rc < 0) rc = narrow_tiles();
        return rc;
    };
    if (t == 0) {
        if (!table && layers == 1 && kind == 1 && p.M <= MORTAR_SMALLM_MAX) {
            const int rc = wide_gate_up();
            if (rc >= 0) return rc;
        }
        // layer-batched gate_up whose rows fit no 16-token tile of all K: K-segmented 16-token tiles, one gate/up unit
        // per wave
        if (table && wide_gate_up_table(kind, p)) {
            if (pick_waves(-16, p, layers) == 16) return mortar_launch_segmented<16, 2, false, 16, 1, true, CODE>(p, table, layers, st);
            return mortar_launch_segmented<16, 2, false, 8, 1, true, CODE>(p, table, layers, st);
        }
        return -1;
    }
    const bool resident = t > 0;
    const int w = pick_waves(t, p, layers);
    if (!table && layers == 1 && w == 2) {      // one matrix over the whole chip: latency form
        int rc = -1;
        if (resident) {
            rc = t == 4 ? launch_partsplit<4, CODE>(kind, p, st) : launch_partsplit<16, CODE>(kind, p, st);
            if (rc < 0 && t == 16 && kind == 1) rc = wide_gate_up();
            if (rc < 0 && t == 16 && kind != 2) rc = narrow_tiles();      // (fails as well where a row is one part)
        } else {
            if (fits(8, p.Cb)) rc = launch_partsplit<8, CODE>(kind, p, st);      // 8-token tiles of all K instead of K segments
            if (rc < 0) rc = narrow_tiles();
        }
        if (rc >= 0) return rc;
        // no part-split form (a plain product whose rows are one part each): above one 16-token tile the 32-token
        // prefill tiles of the caller are faster than 2-wave workgroups per 16-token tile (48 rows: 7.5 against 15.5 us)
        if (resident && t == 16 && p.M > 16 && !p.hc_h) return -1;      // (the POST write exists in the small tiles only)
    }
    if (t == 4) {
        if (w == 16) return launch_kind<4, 16, CODE>(kind, true, p, table, layers, st);
        return w == 8 ? launch_kind<4, 8, CODE>(kind, true, p, table, layers, st) : launch_kind<4, 2, CODE>(kind, true, p, table, layers, st);
    }
    // one matrix whose rows are too wide for an 8-token tile of all K: K-segmented 16-token tiles with 8 waves, which
    // stage a segment four times faster than 2-wave workgroups (4096 x 11008 at 5..64 rows: 13 against 20 us; 16 waves 15 us)
    if (!table && !resident) return launch_kind<16, 8, CODE>(kind, resident, p, table, layers, st);
    if (w == 16) return launch_kind<16, 16, CODE>(kind, resident, p, table, layers, st);
    return w == 8 ? launch_kind<16, 8, CODE>(kind, resident, p, table, layers, st) : launch_kind<16, 2, CODE>(kind, resident, p, table, layers, st);
}

// p.uscale != 0 (set by the caller for a matrix with one scale) selects the kernels that scale after the sums.
int mortar_smallm_launch(int kind, SpmmParams &p, const SpmmParams *table, int layers, hipStream_t st) {
    return p.uscale != 0.f ? smallm_launch_code<CODE_UNIFORM>(kind, p, table, layers, st)
                           : smallm_launch_code<CODE_2BIT>(kind, p, table, layers, st);
}


int mortar_smallm_shape(int kind, SpmmParams &p, int layers) {
    switch (stack_tile32(kind, p)) {       // table launches only: the choice of smallm_launch_code
        case 1: mortar_resident_shape<32, 16>(p, layers); return MORTAR_OK;
        case 2: mortar_segmented_shape<32, 16, 4>(p, layers); return MORTAR_OK;
    }
    if (wide_gate_up_table(kind, p)) {
        if (pick_waves(-16, p, layers) == 16) mortar_segmented_shape<16, 16, 1>(p, layers);
        else mortar_segmented_shape<16, 8, 1>(p, layers);
        return MORTAR_OK;
    }
    const int t = mortar_smallm_tile(p.Cb, p.seg_cb, p.M, kind);
    if (t == 0) return mortar_fail(MORTAR_ERR_LIMIT, "shape has no small-M kernel");
    const int w = pick_waves(t, p, layers);
    if (t == 4) {
        if (w == 16) mortar_resident_shape<4, 16>(p, layers);
        else if (w == 8) mortar_resident_shape<4, 8>(p, layers);
        else mortar_resident_shape<4, 2>(p, layers);
    } else if (t == 16) {
        if (w == 16) mortar_resident_shape<16, 16>(p, layers);
        else if (w == 8) mortar_resident_shape<16, 8>(p, layers);
        else mortar_resident_shape<16, 2>(p, layers);
    } else if (segmented_stack_upw(p, layers, w) == 2) {
        if (w == 16) mortar_segmented_shape<16, 16, 2>(p, layers);
        else if (w == 8) mortar_segmented_shape<16, 8, 2>(p, layers);
        else mortar_segmented_shape<16, 2, 2>(p, layers);
    } else {
        if (w == 16) mortar_segmented_shape<16, 16, 1>(p, layers);
        else if (w == 8) mortar_segmented_shape<16, 8, 1>(p, layers);
        else mortar_segmented_shape<16, 2, 1>(p, layers);
    }
    return MORTAR_OK;
}
