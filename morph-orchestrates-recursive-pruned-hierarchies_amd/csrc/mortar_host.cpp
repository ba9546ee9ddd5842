// Host-side packing and scheduling for the MORTAR device format (no GPU calls in this file).
//
// The reference keeps carved weights as mortar_packed (flat 2-bit codes, u = code + 1) plus a scale
// (morph/inference/deploy_quant.py:344-374) and re-packs them once for its decode engine
// (mortar_pack_strips, morph/kernels/triton/fused_decode_step.py:1465-1499).  This file is the
// equivalent one-time re-pack for the gfx950 kernels.
#include "mortar_internal.h"

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <numeric>
#include <utility>
#include <vector>

static thread_local char g_err[512] = "";

int mortar_fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

extern "C" const char *mortar_last_error(void) { return g_err; }
extern "C" int mortar_abi_version(void) { return 7; }

static inline uint16_t f32_to_bf16_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// Bit position (in 2-bit slots) of column c inside a row dword: columns 0..7 in the odd slots, columns 8..15 in
// the even slots, so that (dword << 2*(c/8)) & 0xCCCCCCCC leaves the 8 codes of a column half as the top two
// bits of the 8 nibbles, in column order.
static inline int slot_of_col(int c) { return c < 8 ? 2 * c + 1 : 2 * (c - 8); }

extern "C" int mortar_encode_blocks_host(const uint8_t *packed, int64_t nnz, const float *scale,
                                         int64_t scale_count, uint32_t *codes_out, uint32_t *sdup_out) {
    if (!packed || !scale || !codes_out || !sdup_out || nnz < 0)
        return mortar_fail(MORTAR_ERR_ARG, "encode_blocks: null pointer or negative nnz");
    if (scale_count != 1 && scale_count != nnz)
        return mortar_fail(MORTAR_ERR_ARG, "encode_blocks: scale_count must be 1 or nnz (got %lld, nnz %lld)",
                           (long long)scale_count, (long long)nnz);
    for (int64_t j = 0; j < nnz; ++j) {
        const uint16_t s = f32_to_bf16_bits(scale[scale_count == 1 ? 0 : j]);
        const int e8 = (s >> 7) & 0xff;
        uint32_t sd = 0;
        if ((s & 0x7fff) != 0) {
            if (e8 < 27 || e8 > 227)
                return mortar_fail(MORTAR_ERR_SCALE,
                                   "encode_blocks: scale of block %lld (%g) outside [2^-100, 2^100]",
                                   (long long)j, (double)scale[scale_count == 1 ? 0 : j]);
            const uint32_t adj = (uint32_t)s - 0x0400u;   // half the value when read as a 16-bit float
            sd = adj | (adj << 16);
        }
        sdup_out[j] = sd;
        for (int n = 0; n < 16; ++n) {
            uint32_t flat;
            memcpy(&flat, packed + j * 64 + n * 4, 4);    // 16 codes of row n, 2 bits each, col c at bits 2c
            uint32_t w = 0;
            for (int c = 0; c < 16; ++c) {
                const uint32_t u = (flat >> (2 * c)) & 3u;      // 0:-1  1:0  2:+1  (3 never produced)
                if (u == 3u)
                    return mortar_fail(MORTAR_ERR_ARG, "encode_blocks: invalid 2-bit code 3 in block %lld",
                                       (long long)j);
                const uint32_t enc = sd == 0 ? 0u : (u == 0u ? 3u : (u == 2u ? 1u : 0u));  // bit1 sign, bit0 nonzero
                w |= enc << (2 * slot_of_col(c));
            }
            codes_out[j * 16 + n] = w;
        }
    }
    return MORTAR_OK;
}

extern "C" int mortar_uniform_scale_host(const uint32_t *sdup, int64_t nnz, float *scale_out) {
    if (!sdup || !scale_out || nnz <= 0) return mortar_fail(MORTAR_ERR_ARG, "uniform_scale: bad argument");
    *scale_out = 0.f;
    for (int64_t j = 1; j < nnz; ++j)
        if (sdup[j] != sdup[0]) return MORTAR_OK;
    if (sdup[0] == 0u) return MORTAR_OK;
    const uint32_t bits = ((sdup[0] & 0xffffu) + 0x0400u) << 16;     // undo the exponent step: bf16 bits of the scale
    memcpy(scale_out, &bits, 4);
    return MORTAR_OK;
}

extern "C" int mortar_decode_blocks_host(const uint32_t *codes, int64_t nnz, int8_t *codes_out) {
    if (!codes || !codes_out) return mortar_fail(MORTAR_ERR_ARG, "decode_blocks: null pointer");
    for (int64_t j = 0; j < nnz; ++j)
        for (int n = 0; n < 16; ++n) {
            const uint32_t w = codes[j * 16 + n];
            for (int c = 0; c < 16; ++c) {
                const uint32_t enc = (w >> (2 * slot_of_col(c))) & 3u;
                codes_out[j * 256 + n * 16 + c] = enc == 1u ? 1 : (enc == 3u ? -1 : 0);
            }
        }
    return MORTAR_OK;
}

int mortar_check_bcsr_host(const int32_t *row_ptr, const int16_t *col, int32_t Rb, int32_t Cb) {
    if (!row_ptr || !col || Rb <= 0 || Cb <= 0) return mortar_fail(MORTAR_ERR_ARG, "bcsr: null pointer or empty shape");
    if (row_ptr[0] != 0) return mortar_fail(MORTAR_ERR_ARG, "bcsr: offsets[0] != 0");
    for (int r = 0; r < Rb; ++r) {
        if (row_ptr[r + 1] < row_ptr[r]) return mortar_fail(MORTAR_ERR_ARG, "bcsr: offsets decrease at row %d", r);
        for (int p = row_ptr[r]; p < row_ptr[r + 1]; ++p) {
            if (col[p] < 0 || col[p] >= Cb)
                return mortar_fail(MORTAR_ERR_ARG, "bcsr: column index %d out of range at block %d", (int)col[p], p);
            if (p > row_ptr[r] && col[p] <= col[p - 1])
                return mortar_fail(MORTAR_ERR_ARG, "bcsr: columns of row %d not strictly ascending", r);
        }
    }
    return MORTAR_OK;
}

extern "C" int mortar_validate_bcsr_host(const int32_t *row_ptr, const int16_t *col, int32_t Rb, int32_t Cb) {
    return mortar_check_bcsr_host(row_ptr, col, Rb, Cb);
}

extern "C" int64_t mortar_octet_layout_host(const int32_t *row_ptr, int32_t Rb, int32_t Cb, int32_t seg_cb,
                                            const uint32_t *codes, const uint32_t *sdup, const int16_t *col,
                                            int32_t *row_desc_out, uint32_t *codes_o_out, uint32_t *sd_o_out,
                                            int32_t *col_o_out) {
    if (!row_ptr || !col || !row_desc_out || Rb <= 0 || Cb <= 0 || seg_cb <= 0)
        return mortar_fail(MORTAR_ERR_ARG, "octet_layout: bad argument");
    const int nseg = (Cb + seg_cb - 1) / seg_cb;
    // block range of (segment, row): columns are ascending inside a row
    std::vector<int32_t> lo((size_t)nseg * Rb), hi((size_t)nseg * Rb);
    for (int r = 0; r < Rb; ++r) {
        int p = row_ptr[r];
        for (int sg = 0; sg < nseg; ++sg) {
            lo[(size_t)sg * Rb + r] = p;
            while (p < row_ptr[r + 1] && col[p] < (sg + 1) * seg_cb) ++p;
            hi[(size_t)sg * Rb + r] = p;
        }
    }
    int64_t ng = 0;
    for (int64_t v = 0; v < (int64_t)nseg * Rb; ++v) {
        const int nb = hi[v] - lo[v];
        row_desc_out[4 * v] = (int32_t)ng;
        ng += (nb + 7) / 8;
        row_desc_out[4 * v + 1] = (int32_t)ng;
        row_desc_out[4 * v + 2] = nb;
        row_desc_out[4 * v + 3] = 0;
        if (ng > 0x7fffffff / 128) return mortar_fail(MORTAR_ERR_LIMIT, "octet_layout: too many blocks");
    }
    if (!codes_o_out) return ng;
    if (!codes || !sdup || !sd_o_out || !col_o_out) return mortar_fail(MORTAR_ERR_ARG, "octet_layout: null pointer");
    for (int64_t v = 0; v < (int64_t)nseg * Rb; ++v) {
        const int nb = hi[v] - lo[v];
        const int c0 = (int)(v / Rb) * seg_cb;
        for (int gl = 0; gl * 8 < nb; ++gl) {
            const int64_t gidx = row_desc_out[4 * v] + gl;
            for (int s2 = 0; s2 < 2; ++s2)
                for (int t = 0; t < 4; ++t) {
                    const int b = 8 * gl + 2 * t + s2;
                    const bool ok = b < nb;
                    const int64_t j = (int64_t)lo[v] + b;
                    sd_o_out[(gidx * 2 + s2) * 4 + t] = ok ? sdup[j] : 0u;
                    col_o_out[(gidx * 2 + s2) * 4 + t] = ok ? (int32_t)col[j] - c0 : 0;
                    for (int n = 0; n < 16; ++n)
                        codes_o_out[((gidx * 2 + s2) * 16 + n) * 4 + t] = ok ? codes[j * 16 + n] : 0u;
                }
        }
    }
    return ng;
}

extern "C" int mortar_octet_positions_host(const int32_t *row_ptr, int32_t Rb, int32_t Cb, int32_t seg_cb,
                                           const int16_t *col, int32_t *pos_out) {
    if (!row_ptr || !col || !pos_out || Rb <= 0 || Cb <= 0 || seg_cb <= 0)
        return mortar_fail(MORTAR_ERR_ARG, "octet_positions: bad argument");
    const int nseg = (Cb + seg_cb - 1) / seg_cb;
    // same walk as mortar_octet_layout_host: segments outermost, rows inside, 8 blocks per octet
    std::vector<int32_t> lo((size_t)nseg * Rb), hi((size_t)nseg * Rb);
    for (int r = 0; r < Rb; ++r) {
        int p = row_ptr[r];
        for (int sg = 0; sg < nseg; ++sg) {
            lo[(size_t)sg * Rb + r] = p;
            while (p < row_ptr[r + 1] && col[p] < (sg + 1) * seg_cb) ++p;
            hi[(size_t)sg * Rb + r] = p;
        }
    }
    int64_t ng = 0;
    for (int64_t v = 0; v < (int64_t)nseg * Rb; ++v) {
        const int nb = hi[v] - lo[v];
        for (int b = 0; b < nb; ++b) {
            const int64_t g = ng + b / 8;
            pos_out[lo[v] + b] = (int32_t)((g * 2 + (b & 1)) * 4 + ((b & 7) >> 1));
        }
        ng += (nb + 7) / 8;
    }
    return MORTAR_OK;
}

extern "C" int mortar_transpose_topology_host(const int32_t *row_ptr, const int16_t *col, int32_t Rb, int32_t Cb,
                                              int32_t *offsets_t_out, int16_t *col_t_out, int32_t *src_block_out) {
    if (!offsets_t_out || !col_t_out || !src_block_out)
        return mortar_fail(MORTAR_ERR_ARG, "transpose_topology: null pointer");
    const int rc = mortar_check_bcsr_host(row_ptr, col, Rb, Cb);
    if (rc) return rc;
    const int32_t nnz = row_ptr[Rb];
    std::fill(offsets_t_out, offsets_t_out + Cb + 1, 0);
    for (int32_t j = 0; j < nnz; ++j) ++offsets_t_out[col[j] + 1];
    for (int c = 0; c < Cb; ++c) offsets_t_out[c + 1] += offsets_t_out[c];
    std::vector<int32_t> fill(offsets_t_out, offsets_t_out + Cb);
    for (int r = 0; r < Rb; ++r)                        // ascending rows: blocks of one column stay in row order
        for (int32_t j = row_ptr[r]; j < row_ptr[r + 1]; ++j) {
            const int32_t o = fill[col[j]]++;
            col_t_out[o] = (int16_t)r;
            src_block_out[o] = j;
        }
    return MORTAR_OK;
}

extern "C" int mortar_fp4_stream_host(const uint32_t *codes_o, int64_t ngroups, uint32_t *codes4_o_out) {
    if (!codes_o || !codes4_o_out || ngroups < 0) return mortar_fail(MORTAR_ERR_ARG, "fp4_stream: bad argument");
    for (int64_t gs = 0; gs < ngroups * 2; ++gs)          // (octet, s)
        for (int n = 0; n < 16; ++n)
            for (int t = 0; t < 4; ++t) {
                const uint32_t w = codes_o[(gs * 16 + n) * 4 + t];
                for (int h = 0; h < 2; ++h) {
                    uint32_t o = 0;
                    for (int q = 0; q < 8; ++q) {
                        const int c = 8 * h + q;
                        const uint32_t enc = (w >> (2 * slot_of_col(c))) & 3u;
                        o |= (enc << 2) << (4 * q);
                    }
                    const int64_t g = gs >> 1, s2 = gs & 1;
                    codes4_o_out[(((g * 4 + 2 * s2 + h) * 16) + n) * 4 + t] = o;
                }
            }
    return MORTAR_OK;
}

extern "C" int mortar_unit_order_host(const int32_t *row_ptr, int32_t Rb, int32_t rows_per_unit,
                                      int32_t group, int32_t snake, int32_t *order_out) {
    if (!row_ptr || !order_out || Rb <= 0 || group <= 0 || (rows_per_unit != 1 && rows_per_unit != 2) ||
        Rb % rows_per_unit)
        return mortar_fail(MORTAR_ERR_ARG, "unit_order: bad argument");
    const int nu = Rb / rows_per_unit;
    std::vector<int64_t> cost(nu);
    bool uniform = true;
    for (int u = 0; u < nu; ++u) {
        cost[u] = row_ptr[u + 1] - row_ptr[u];
        if (rows_per_unit == 2) cost[u] += row_ptr[u + nu + 1] - row_ptr[u + nu];
        if (cost[u] != cost[0]) uniform = false;
    }
    if (uniform) {   // natural order keeps neighbouring output columns in one wave
        std::iota(order_out, order_out + nu, 0);
        return MORTAR_OK;
    }
    std::vector<int> idx(nu);
    std::iota(idx.begin(), idx.end(), 0);
    std::stable_sort(idx.begin(), idx.end(), [&](int a, int b) { return cost[a] > cost[b]; });
    const int ng = (nu + group - 1) / group;
    std::vector<int64_t> load(ng, 0);
    std::vector<std::vector<int>> members(ng);
    std::vector<int> cap(ng, group);
    cap[ng - 1] = nu - (ng - 1) * group;
    for (int u : idx) {
        int best = -1;
        for (int g = 0; g < ng; ++g)
            if ((int)members[g].size() < cap[g] && (best < 0 || load[g] < load[best])) best = g;
        members[best].push_back(u);
        load[best] += cost[u];
    }
    // Members are in descending cost.  Where wave w of a workgroup takes the positions w, w + group, ... of its
    // window (every group hands one unit to each wave) the odd groups are reversed so that no wave collects the
    // heaviest unit of every group; where the waves draw positions one after another every group stays heaviest
    // first, so that a window ends with light units (ragged gate_up, 160 layers at one row: 91 -> 84 us).
    int o = 0;
    for (int g = 0; g < ng; ++g) {
        const int n = (int)members[g].size();
        for (int i = 0; i < n; ++i) order_out[o++] = members[g][(snake && (g & 1)) ? n - 1 - i : i];
    }
    return MORTAR_OK;
}

extern "C" int mortar_unit_order_segments_host(const int32_t *row_desc, int32_t Rb, int32_t nseg,
                                               int32_t rows_per_unit, int32_t waves, int32_t units_per_wave,
                                               int32_t *order) {
    if (!row_desc || !order || Rb <= 0 || nseg <= 0 || waves <= 0 || units_per_wave <= 0 ||
        (rows_per_unit != 1 && rows_per_unit != 2) || Rb % rows_per_unit)
        return mortar_fail(MORTAR_ERR_ARG, "unit_order_segments: bad argument");
    const int nu = Rb / rows_per_unit;
    if (nseg == 1 || units_per_wave == 1) return MORTAR_OK;   // no barrier between parts / nothing to deal
    // cost[u][s]: block pairs the kernel multiplies for unit u in segment s (parts run in half octets)
    std::vector<int32_t> cost((size_t)nu * nseg);
    for (int u = 0; u < nu; ++u) {
        if (order[u] < 0 || order[u] >= nu) return mortar_fail(MORTAR_ERR_ARG, "unit_order_segments: order out of range");
        for (int s = 0; s < nseg; ++s) {
            int32_t c = 0;
            for (int a = 0; a < rows_per_unit; ++a)
                c += (row_desc[4 * ((int64_t)s * Rb + u + (int64_t)a * nu) + 2] + 3) / 4 * 2;
            cost[(size_t)u * nseg + s] = c;
        }
    }
    const int per = waves * units_per_wave;
    std::vector<int64_t> load((size_t)waves * nseg);
    std::vector<std::vector<int>> mem(waves);
    // sum over the segments of the heaviest wave: what the barriers make the workgroup wait for
    auto objective = [&]() {
        int64_t t = 0;
        for (int s = 0; s < nseg; ++s) {
            int64_t m = 0;
            for (int w = 0; w < waves; ++w) m = std::max(m, load[(size_t)w * nseg + s]);
            t += m;
        }
        return t;
    };
    auto move = [&](int w, int u, int sign) {
        for (int s = 0; s < nseg; ++s) load[(size_t)w * nseg + s] += sign * cost[(size_t)u * nseg + s];
    };
    for (int p0 = 0; p0 < nu; p0 += per) {
        const int n = std::min(per, nu - p0);
        std::vector<int> units(order + p0, order + p0 + n);
        auto peak = [&](int u) { return *std::max_element(&cost[(size_t)u * nseg], &cost[(size_t)u * nseg] + nseg); };
        std::stable_sort(units.begin(), units.end(), [&](int a, int b) { return peak(a) > peak(b); });
        std::fill(load.begin(), load.end(), 0);
        std::vector<int> cap(waves);
        for (int w = 0; w < waves; ++w) {       // wave w owns the window's positions w, w + waves, ...
            mem[w].clear();
            cap[w] = w < n ? (n - w + waves - 1) / waves : 0;
        }
        for (int u : units) {                   // greedy: the wave whose heaviest segment stays lightest
            int best = -1;
            int64_t best_peak = 0, best_sum = 0;
            for (int w = 0; w < waves; ++w) {
                if ((int)mem[w].size() >= cap[w]) continue;
                int64_t pk = 0, sm = 0;
                for (int s = 0; s < nseg; ++s) {
                    const int64_t v = load[(size_t)w * nseg + s] + cost[(size_t)u * nseg + s];
                    pk = std::max(pk, v);
                    sm += v;
                }
                if (best < 0 || pk < best_peak || (pk == best_peak && sm < best_sum)) best = w, best_peak = pk, best_sum = sm;
            }
            mem[best].push_back(u);
            move(best, u, +1);
        }
        int64_t cur = objective();              // then exchanges of two units while one lowers the objective
        for (int pass = 0; pass < 16; ++pass) {
            bool improved = false;
            for (int a = 0; a < waves; ++a)
                for (int b = a + 1; b < waves; ++b)
                    for (size_t i = 0; i < mem[a].size(); ++i)
                        for (size_t j = 0; j < mem[b].size(); ++j) {
                            const int ua = mem[a][i], ub = mem[b][j];
                            move(a, ua, -1); move(a, ub, +1); move(b, ub, -1); move(b, ua, +1);
                            const int64_t t = objective();
                            if (t < cur) {
                                cur = t;
                                std::swap(mem[a][i], mem[b][j]);
                                improved = true;
                            } else {
                                move(a, ub, -1); move(a, ua, +1); move(b, ua, -1); move(b, ub, +1);
                            }
                        }
            if (!improved) break;
        }
        // A kernel that gives a wave half as many units (the layer-batched decode form) cuts the window into two
        // windows of the same waves, each a workgroup of its own.  The greedy above hands every wave its heaviest unit
        // first, which would make the first half several times the second: order every wave's units (the sums above
        // stay as they are) so that the halves cost the same - heaviest with lightest to start with, then exchanges
        // inside a wave while the costlier half gets cheaper.  A half is priced by its blocks first and by the measure
        // above second: the decode launches stream their weights once and wait little at the barriers, and equal
        // blocks per workgroup measured faster there than equal barrier waits (160 `down` layers with Zipf rows at
        // 16 rows: 63.7 against 71.4 us; 83 us with the halves left as the greedy makes them).
        if (units_per_wave % 2 == 0) {
            const int hk = units_per_wave / 2;
            auto total = [&](int u) { return std::accumulate(&cost[(size_t)u * nseg], &cost[(size_t)u * nseg] + nseg, (int64_t)0); };
            for (int w = 0; w < waves; ++w) {
                std::vector<int> &m = mem[w];
                std::stable_sort(m.begin(), m.end(), [&](int a, int b) { return total(a) > total(b); });
                std::vector<int> first, second;                   // 0, 3, 4, 7, ... | 1, 2, 5, 6, ...
                for (size_t i = 0; i < m.size(); ++i) ((i % 4 == 0 || i % 4 == 3) ? first : second).push_back(m[i]);
                while ((int)first.size() > hk) { second.push_back(first.back()); first.pop_back(); }
                while ((int)first.size() < hk && !second.empty()) { first.push_back(second.back()); second.pop_back(); }
                m = first;
                m.insert(m.end(), second.begin(), second.end());
            }
            std::vector<int64_t> hl((size_t)2 * waves * nseg, 0);
            auto hmove = [&](int h, int w, int u, int sign) {
                for (int s = 0; s < nseg; ++s) hl[((size_t)h * waves + w) * nseg + s] += sign * cost[(size_t)u * nseg + s];
            };
            auto hobjective = [&]() {                              // (costlier half, both halves)
                int64_t t[2] = {0, 0};
                for (int h = 0; h < 2; ++h)
                    for (int s = 0; s < nseg; ++s) {
                        int64_t mx = 0;
                        for (int w = 0; w < waves; ++w) mx = std::max(mx, hl[((size_t)h * waves + w) * nseg + s]);
                        t[h] += mx;
                    }
                int64_t tot[2] = {0, 0};
                for (int h = 0; h < 2; ++h)
                    for (int w = 0; w < waves; ++w)
                        for (int s = 0; s < nseg; ++s) tot[h] += hl[((size_t)h * waves + w) * nseg + s];
                const int64_t k0 = tot[0] * 64 + t[0], k1 = tot[1] * 64 + t[1];
                return std::make_pair(std::max(k0, k1), k0 + k1);
            };
            for (int w = 0; w < waves; ++w)
                for (size_t k = 0; k < mem[w].size(); ++k) hmove((int)k < hk ? 0 : 1, w, mem[w][k], +1);
            auto hcur = hobjective();
            for (int pass = 0; pass < 16; ++pass) {
                bool improved = false;
                for (int w = 0; w < waves; ++w)
                    for (size_t i = 0; i < mem[w].size() && (int)i < hk; ++i)
                        for (size_t j = hk; j < mem[w].size(); ++j) {
                            const int ui = mem[w][i], uj = mem[w][j];
                            hmove(0, w, ui, -1); hmove(0, w, uj, +1); hmove(1, w, uj, -1); hmove(1, w, ui, +1);
                            const auto t = hobjective();
                            if (t < hcur) {
                                hcur = t;
                                std::swap(mem[w][i], mem[w][j]);
                                improved = true;
                            } else {
                                hmove(0, w, uj, -1); hmove(0, w, ui, +1); hmove(1, w, ui, -1); hmove(1, w, uj, +1);
                            }
                        }
                if (!improved) break;
            }
        }
        for (int w = 0; w < waves; ++w)
            for (size_t k = 0; k < mem[w].size(); ++k) order[p0 + w + waves * (int)k] = mem[w][k];
    }
    return MORTAR_OK;
}

extern "C" int mortar_schedule_host(const int32_t *row_desc, int32_t Rb, int32_t nseg, int32_t rows_per_unit,
                                    const int32_t *order, int32_t *sched_out) {
    if (!row_desc || !sched_out || Rb <= 0 || nseg <= 0 || (rows_per_unit != 1 && rows_per_unit != 2) ||
        Rb % rows_per_unit)
        return mortar_fail(MORTAR_ERR_ARG, "schedule: bad argument");
    const int nu = Rb / rows_per_unit;
    std::vector<char> seen((size_t)nu, 0);
    for (int pos = 0; pos < nu; ++pos) {
        const int u = order ? order[pos] : pos;
        if (u < 0 || u >= nu || seen[(size_t)u]) return mortar_fail(MORTAR_ERR_ARG, "schedule: order is not a permutation");
        seen[(size_t)u] = 1;
        for (int sg = 0; sg < nseg; ++sg)
            for (int a = 0; a < rows_per_unit; ++a) {
                const int32_t *d = row_desc + 4 * ((int64_t)sg * Rb + u + (int64_t)a * nu);
                int32_t *o = sched_out + 4 * (((int64_t)pos * nseg + sg) * rows_per_unit + a);
                o[0] = d[0]; o[1] = d[1]; o[2] = d[2]; o[3] = u;
            }
    }
    return MORTAR_OK;
}

extern "C" int64_t mortar_decode_worklist_host(const int32_t *row_ptr, const int16_t *col, int32_t Rb,
                                               int32_t Cb, int32_t rows_per_unit, int32_t kseg,
                                               int32_t max_blocks, int32_t *entries_out, int32_t *nslots_out,
                                               int32_t *row_slots_out) {
    if (kseg <= 0 || max_blocks <= 0 || (rows_per_unit != 1 && rows_per_unit != 2) || Rb % rows_per_unit)
        return mortar_fail(MORTAR_ERR_ARG, "decode_worklist: bad argument");
    int rc = mortar_check_bcsr_host(row_ptr, col, Rb, Cb);
    if (rc) return rc;
    const int nu = Rb / rows_per_unit;
    const int nseg = (Cb + kseg - 1) / kseg;
    struct Ent { int32_t v[8]; };
    std::vector<std::vector<Ent>> per_seg(nseg);
    std::vector<int> slot_of_unit(nu, 0);
    int nslots = 1;
    // range of row r inside segment s
    auto seg_range = [&](int r, int s, int &a, int &b) {
        a = row_ptr[r];
        const int e = row_ptr[r + 1];
        while (a < e && col[a] < s * kseg) ++a;
        b = a;
        while (b < e && col[b] < (s + 1) * kseg) ++b;
    };
    for (int s = 0; s < nseg; ++s)
        for (int u = 0; u < nu; ++u) {
            int a0, b0, a1 = 0, b1 = 0;
            seg_range(u, s, a0, b0);
            if (rows_per_unit == 2) seg_range(u + nu, s, a1, b1);
            const int n0 = b0 - a0, n1 = b1 - a1;
            const int nch = std::max((n0 + max_blocks - 1) / max_blocks, (n1 + max_blocks - 1) / max_blocks);
            for (int i = 0; i < nch; ++i) {
                Ent e;
                const int c0 = std::max(0, std::min(max_blocks, n0 - i * max_blocks));
                const int c1 = std::max(0, std::min(max_blocks, n1 - i * max_blocks));
                e.v[0] = u; e.v[1] = c0 > 0 ? a0 + i * max_blocks : a0; e.v[2] = c0;
                e.v[3] = rows_per_unit == 2 ? u + nu : -1; e.v[4] = c1 > 0 ? a1 + i * max_blocks : a1; e.v[5] = c1;
                e.v[6] = slot_of_unit[u]++; e.v[7] = s;
                per_seg[s].push_back(e);
            }
        }
    for (int u = 0; u < nu; ++u) nslots = std::max(nslots, slot_of_unit[u]);
    // a unit with no block at all (cannot happen after carve, which keeps >= 1 block per row) still needs
    // one entry so its output is written
    for (int u = 0; u < nu; ++u)
        if (slot_of_unit[u] == 0) {
            Ent e = {{u, row_ptr[u], 0, rows_per_unit == 2 ? u + nu : -1,
                      rows_per_unit == 2 ? row_ptr[u + nu] : 0, 0, 0, 0}};
            per_seg[0].push_back(e);
        }
    int64_t total = 0;
    for (int s = 0; s < nseg; ++s) total += ((int64_t)per_seg[s].size() + 3) / 4 * 4;   // workgroup = 4 entries
    if (nslots_out) *nslots_out = nslots;
    if (row_slots_out)
        for (int u = 0; u < nu; ++u) {
            row_slots_out[u] = std::max(1, slot_of_unit[u]);
            if (rows_per_unit == 2) row_slots_out[u + nu] = row_slots_out[u];
        }
    if (!entries_out) return total;
    int64_t o = 0;
    for (int s = 0; s < nseg; ++s) {
        for (const Ent &e : per_seg[s]) { memcpy(entries_out + o * 8, e.v, 32); ++o; }
        while (o % 4) {
            const int32_t nul[8] = {-1, 0, 0, -1, 0, 0, 0, s};
            memcpy(entries_out + o * 8, nul, 32);
            ++o;
        }
    }
    return total;
}
