// Block-sparse product over stored bf16 block VALUES: y = x W^T with W given as the reference's BCSR arrays
// (mortar_data [nnz,16,16], mortar_offsets, mortar_column_indices), whatever values the blocks hold.
//
// This is the arithmetic of the reference's stk_dds operator itself (morph/sparse/stk/backend/custom_ops.py:35-56,
// kernel triton_kernels.py:170-230 with trans_B: bf16 operands, fp32 accumulation, bf16 store), which multiplies any
// bf16 data.  The ternary kernels of this library stream 2- and 4-bit codes and therefore serve ternary blocks only; this
// kernel is the general form behind the operator-level drop-in.  It needs no unpacking at all: a block row of 16 values
// is 32 contiguous bytes, so the lane that holds row n, column half h of a block pair in the MFMA's A operand fetches
// exactly its 16 bytes with one global load; the activation operand comes from the same 32-token LDS tile layout as the
// ternary kernels ([block-column][token][32 B]).
#include "mortar_spmm_core.h"

namespace {

constexpr int VAL_MT = 32, VAL_WAVES = 16, VAL_UPW = 4, VAL_PB = 4;

struct ValArgs {
    const int32_t *row_ptr;     // [Rb + 1]
    const int32_t *seg_ptr;     // [Rb, nseg + 1]: first block of row r in K segment s (mortar_segment_ptr_host); null for nseg == 1
    const int16_t *col;         // [nnz]
    const uint16_t *data;       // [nnz, 16, 16] bf16
    int per;                    // block-rows per workgroup
    int upw;                    // K-segmented form: block-rows per wave (<= VAL_UPW)
};

// Blocks [j0, j1) of one block-row (columns inside the staged tile, which starts at block-column c0) against the tile.
// The values of the next VAL_PB pairs are requested before the current ones are multiplied.
__device__ __forceinline__ void val_run(const ValArgs &a, const unsigned char *lb, int j0, int j1, int c0, int n, int bsel,
                                        int hsel, f32x4_t (&acc)[2]) {
    const uint32_t lane_xo = (uint32_t)(n * 32 + hsel * 16);
    u32x4_t A[VAL_PB], An[VAL_PB];
    int cc[VAL_PB], cn[VAL_PB];
    auto fetch = [&](int j, u32x4_t (&Av)[VAL_PB], int (&cv)[VAL_PB]) {
#pragma unroll
        for (int u = 0; u < VAL_PB; ++u) {
            const int jj = j + 2 * u + bsel;
            const bool ok = jj < j1;
            const int64_t js = ok ? jj : j0;
            Av[u] = *reinterpret_cast<const u32x4_t *>(reinterpret_cast<const char *>(a.data) + js * 512 + n * 32 + hsel * 16);
            if (!ok) Av[u] = u32x4_t{0u, 0u, 0u, 0u};
            cv[u] = (int)a.col[js] - c0;
        }
    };
    if (j0 < j1) fetch(j0, A, cc);
    for (int j = j0; j < j1; j += 2 * VAL_PB) {
        if (j + 2 * VAL_PB < j1) fetch(j + 2 * VAL_PB, An, cn);
#pragma unroll
        for (int u = 0; u < VAL_PB; ++u) {
            if (j + 2 * u < j1) {
                const uint32_t xo = (uint32_t)cc[u] * (uint32_t)(VAL_MT * 32) + lane_xo;
#pragma unroll
                for (int ms = 0; ms < 2; ++ms) {
                    const uint4 b = *reinterpret_cast<const uint4 *>(lb + xo + ms * 512);
                    acc[ms] = mortar_mfma(A[u], u32x4_t{b.x, b.y, b.z, b.w}, acc[ms]);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < VAL_PB; ++u) { A[u] = An[u]; cc[u] = cn[u]; }
    }
}

__device__ __forceinline__ void val_store(const SpmmView &p, int row, int m0, int n, int g, const f32x4_t (&acc)[2]) {
#pragma unroll
    for (int ms = 0; ms < 2; ++ms) {
        const int tok = m0 + ms * 16 + n;
        if (tok < p.M)
            *(MORTAR_GLOBAL u32x2_t *)(p.y + (int64_t)tok * p.ldy + row * 16 + 4 * g) =
                u32x2_t{bf16_pack2(acc[ms][0], acc[ms][1]), bf16_pack2(acc[ms][2], acc[ms][3])};
    }
}

// SEG = false: the tile holds all of K; a wave walks the block-rows w, w + 16, ... of its workgroup's share.
// SEG = true: K is walked in segments (one barrier pair each); a wave owns VAL_UPW block-rows whose accumulators stay
// in registers across the segments.
template <bool SEG>
__global__ void __launch_bounds__(VAL_WAVES * 64) values_kernel(const SpmmParams p0, const ValArgs a) {
    const SpmmView p = mortar_view(p0);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint4 *lx = reinterpret_cast<uint4 *>(smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, g = lane >> 4, bsel = g >> 1, hsel = g & 1;
    const int mt = blockIdx.x / p.n_split, sp = blockIdx.x % p.n_split;
    const int m0 = mt * VAL_MT;
    const int r0 = sp * a.per, r1 = r0 + a.per < p.Rb ? r0 + a.per : p.Rb;
    if (!SEG) {
        mortar_stage_tile<VAL_MT, VAL_WAVES, false>(p, lx, m0, 0, p.Cb, tid);
        __syncthreads();
        for (int r = r0 + wave; r < r1; r += VAL_WAVES) {
            f32x4_t acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
            val_run(a, smem, a.row_ptr[r], a.row_ptr[r + 1], 0, n, bsel, hsel, acc);
            val_store(p, r, m0, n, g, acc);
        }
        return;
    }
    f32x4_t acc[VAL_UPW][2];
#pragma unroll
    for (int k = 0; k < VAL_UPW; ++k) acc[k][0] = acc[k][1] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    for (int sg = 0; sg < p.nseg; ++sg) {
        const int c0 = sg * p.seg_cb;
        const int ncb = p.Cb - c0 < p.seg_cb ? p.Cb - c0 : p.seg_cb;
        if (sg > 0) __syncthreads();
        mortar_stage_tile<VAL_MT, VAL_WAVES, false>(p, lx, m0, c0, ncb, tid);
        __syncthreads();
#pragma unroll
        for (int k = 0; k < VAL_UPW; ++k) {
            const int r = r0 + wave + VAL_WAVES * k;
            if (k < a.upw && r < r1) {
                const int32_t *sp_ = a.seg_ptr + (int64_t)r * (p.nseg + 1) + sg;
                val_run(a, smem, __builtin_amdgcn_readfirstlane(sp_[0]), __builtin_amdgcn_readfirstlane(sp_[1]), c0, n, bsel, hsel, acc[k]);
            }
        }
    }
#pragma unroll
    for (int k = 0; k < VAL_UPW; ++k) {
        const int r = r0 + wave + VAL_WAVES * k;
        if (k < a.upw && r < r1) val_store(p, r, m0, n, g, acc[k]);
    }
}

}  // namespace

extern "C" int32_t mortar_values_seg_cb(int32_t Cb) {
    if (Cb <= 0) return 0;
    const int max_seg = mortar_prefill_max_seg_cb();
    const int nseg = (Cb + max_seg - 1) / max_seg;
    return (Cb + nseg - 1) / nseg;
}

extern "C" int mortar_segment_ptr_host(const int32_t *row_ptr, const int16_t *col, int32_t Rb, int32_t Cb, int32_t seg_cb,
                                       int32_t *seg_ptr_out) {
    if (!row_ptr || !col || !seg_ptr_out || seg_cb <= 0) return mortar_fail(MORTAR_ERR_ARG, "segment_ptr: bad argument");
    const int rc = mortar_check_bcsr_host(row_ptr, col, Rb, Cb);
    if (rc) return rc;
    const int nseg = (Cb + seg_cb - 1) / seg_cb;
    for (int r = 0; r < Rb; ++r) {
        int j = row_ptr[r];
        for (int s = 0; s <= nseg; ++s) {
            while (j < row_ptr[r + 1] && col[j] < s * seg_cb) ++j;
            seg_ptr_out[(int64_t)r * (nseg + 1) + s] = s == nseg ? row_ptr[r + 1] : j;
        }
    }
    return MORTAR_OK;
}

extern "C" int mortar_dds_values_bf16(const int32_t *row_ptr, const int16_t *col, const int32_t *seg_ptr, const uint16_t *data,
                                      int32_t Rb, int32_t Cb, int64_t nnz, const uint16_t *x, int64_t M, int64_t ldx, uint16_t *y,
                                      int64_t ldy, void *stream) {
    if (!row_ptr || !col || !data || !x || !y) return mortar_fail(MORTAR_ERR_ARG, "dds_values: null pointer");
    if (Rb <= 0 || Cb <= 0 || nnz < 0 || nnz > 0x7fffffff) return mortar_fail(MORTAR_ERR_ARG, "dds_values: bad shape");
    if (M <= 0 || M > (1 << 30)) return mortar_fail(MORTAR_ERR_ARG, "dds_values: M=%lld out of range", (long long)M);
    if (ldx < (int64_t)Cb * 16 || ldx % 8 || ldy < (int64_t)Rb * 16 || ldy % 4)
        return mortar_fail(MORTAR_ERR_ARG, "dds_values: bad leading dimension (ldx %% 8 == 0, ldy %% 4 == 0)");
    if ((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(y) & 7) || (reinterpret_cast<uintptr_t>(data) & 15))
        return mortar_fail(MORTAR_ERR_ARG, "dds_values: x and data must be 16-byte and y 8-byte aligned");
    const int seg_cb = mortar_values_seg_cb(Cb);
    const int nseg = (Cb + seg_cb - 1) / seg_cb;
    if (nseg > 1 && !seg_ptr) return mortar_fail(MORTAR_ERR_ARG, "dds_values: %d K segments need seg_ptr (mortar_segment_ptr_host)", nseg);
    SpmmParams p{};
    p.x = x; p.ldx = ldx; p.M = (int)M; p.y = y; p.ldy = ldy; p.Rb = Rb; p.Cb = Cb; p.seg_cb = seg_cb; p.nseg = nseg;
    p.n_clusters = 1; p.cluster_size = 1 << 30; p.n_units = Rb;
    p.n_mtiles = (int)((M + VAL_MT - 1) / VAL_MT);
    ValArgs a{row_ptr, seg_ptr, col, data, 0, VAL_UPW};
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int smem = tile_bytes(VAL_MT, seg_cb);
    static bool attr_done[2] = {false, false};
    int rc;
    if (nseg == 1) {
        // about one workgroup per CU and round; every workgroup stages the whole token tile, so few splits
        int split = (int)(256 / p.n_mtiles);
        const int max_split = (Rb + VAL_WAVES - 1) / VAL_WAVES;
        split = split < 1 ? 1 : (split > max_split ? max_split : split);
        p.n_split = split;
        a.per = (Rb + split - 1) / split;
        if ((rc = mortar_allow_big_lds(values_kernel<false>, attr_done[0]))) return rc;
        if ((rc = mortar_launch_check((int64_t)p.n_mtiles * split, 1))) return rc;
        hipLaunchKernelGGL(values_kernel<false>, dim3((unsigned)(p.n_mtiles * split)), dim3(VAL_WAVES * 64), smem, st, p, a);
    } else {
        // fewer block-rows per wave while the launch would leave CUs idle (every workgroup stages the tile's segments again)
        int upw = VAL_UPW;
        while (upw > 1 && (int64_t)p.n_mtiles * ((Rb + VAL_WAVES * upw - 1) / (VAL_WAVES * upw)) < 256) upw >>= 1;
        a.upw = upw;
        a.per = VAL_WAVES * upw;
        p.n_split = (Rb + a.per - 1) / a.per;
        if ((rc = mortar_allow_big_lds(values_kernel<true>, attr_done[1]))) return rc;
        if ((rc = mortar_launch_check((int64_t)p.n_mtiles * p.n_split, 1))) return rc;
        hipLaunchKernelGGL(values_kernel<true>, dim3((unsigned)(p.n_mtiles * p.n_split)), dim3(VAL_WAVES * 64), smem, st, p, a);
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mortar_fail(MORTAR_ERR_HIP, "dds_values launch: %s", hipGetErrorString(e));
    return MORTAR_OK;
}
