// Device helpers shared by the gfx950 kernels: ternary block unpack, MFMA wrappers, bf16 rounding.
#ifndef MORTAR_DEVICE_H
#define MORTAR_DEVICE_H

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

// Lane decomposition used by every MFMA kernel here (v_mfma_f32_16x16x32_bf16):
//   n = lane & 15   row of the A operand (output feature inside the block-row) / column of B (token)
//   g = lane >> 4   K group: the lane holds K slots 8g .. 8g+7
// One MFMA contracts two 16x16 blocks: bsel = g >> 1 picks the block, hsel = g & 1 its column half.
// The accumulator lane holds D[4g + v][n], v = 0..3: four consecutive output features of token n.

// 8 ternary codes -> 8 bf16 weights (+-bf16(scale) or 0) in four dwords.
// A row dword holds its 16 two-bit codes (bit 1 = negative, bit 0 = non-zero) interleaved: column c < 8 in slot
// 2c + 1, column c >= 8 in slot 2(c - 8).  `t` is the dword shifted left by 2*hsel, so that the lane's 8 columns
// sit in the odd slots: masked with 0xCCCCCCCC every nibble is {sign, non-zero, 0, 0}, which read as FP4 (E2M1) is
// -2, 0 or +2, and one hardware conversion per register (v_cvt_scalef32_pk_bf16_fp4, scale 1) gives the two bf16
// patterns 0xC000 / 0 / 0x4000 of a column pair.  Read as 16-bit floats those are -2, 0, +2 as well; `sd` holds
// the block scale's bf16 pattern minus one 16-bit-float exponent step in both halves, so one packed half multiply
// returns exactly +-scale or 0 in bf16 bits (a power-of-two product is exact; the host rejects scales whose
// pattern would leave the normal range).
// The 4-bit stream stores the nibbles themselves (byte i = {column 2i, column 2i + 1}): no shift, no mask.
__device__ __forceinline__ u32x4_t mortar_scale4(uint32_t nib, uint32_t sd) {
    const f16x2_t s = __builtin_bit_cast(f16x2_t, sd);
    u32x4_t r;
    r[0] = __builtin_bit_cast(uint32_t, s * __builtin_bit_cast(f16x2_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(nib, 1.0f, 0)));
    r[1] = __builtin_bit_cast(uint32_t, s * __builtin_bit_cast(f16x2_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(nib, 1.0f, 1)));
    r[2] = __builtin_bit_cast(uint32_t, s * __builtin_bit_cast(f16x2_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(nib, 1.0f, 2)));
    r[3] = __builtin_bit_cast(uint32_t, s * __builtin_bit_cast(f16x2_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(nib, 1.0f, 3)));
    return r;
}
__device__ __forceinline__ u32x4_t mortar_unpack8(uint32_t t, uint32_t sd) {
    return mortar_scale4(t & 0xCCCCCCCCu, sd);
}
// The conversions alone: bf16 +-2 / 0 for the eight nibbles (matrices with one scale, applied after the sums).
__device__ __forceinline__ u32x4_t mortar_nib4(uint32_t nib) {
    u32x4_t r;
    r[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(nib, 1.0f, 0));
    r[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(nib, 1.0f, 1));
    r[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(nib, 1.0f, 2));
    r[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(nib, 1.0f, 3));
    return r;
}

__device__ __forceinline__ f32x4_t mortar_mfma(u32x4_t a, u32x4_t b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// fp32 -> bf16 (round to nearest even) through the hardware conversion (v_cvt_pk_bf16_f32).
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t bf16_pack2(float lo, float hi) {
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ uint32_t bf16_bits_rne(float f) { return bf16_pack2(f, 0.f) & 0xffffu; }
__device__ __forceinline__ float bf16_to_f32(uint32_t b) { return __builtin_bit_cast(float, b << 16); }
// f rounded to bf16, as a float: the conversion of (0, f) leaves the bf16 of f in the high half and zeros below it.
__device__ __forceinline__ float bf16r(float f) { return __builtin_bit_cast(float, bf16_pack2(0.f, f)); }

// ---- RMSNorm pieces shared by the stand-alone kernel and the fused staging of gate_up, so that both round alike.
// A row is handled by one wavefront in 16-byte units (8 bf16): a lane adds the squares of its units in ascending
// unit order (fused multiply-adds, low half-word first), the lanes meet in a xor butterfly.
__device__ __forceinline__ float rms_sumsq8(u32x4_t u, float s) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float lo = __builtin_bit_cast(float, u[j] << 16), hi = __builtin_bit_cast(float, u[j] & 0xffff0000u);
        s = __builtin_fmaf(lo, lo, s);
        s = __builtin_fmaf(hi, hi, s);
    }
    return s;
}
__device__ __forceinline__ float rms_wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float rms_scale(float sumsq, int d, float eps) { return 1.0f / sqrtf(sumsq / (float)d + eps); }
// bf16(bf16(x * r) * w) on 8 values; has_w = false leaves out the weight.
__device__ __forceinline__ u32x4_t rms_apply8(u32x4_t u, float r, u32x4_t w, bool has_w) {
    u32x4_t o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float lo = __builtin_bit_cast(float, u[j] << 16), hi = __builtin_bit_cast(float, u[j] & 0xffff0000u);
        uint32_t pk = bf16_pack2(lo * r, hi * r);
        if (has_w) {
            const float wl = __builtin_bit_cast(float, w[j] << 16), wh = __builtin_bit_cast(float, w[j] & 0xffff0000u);
            pk = bf16_pack2(__builtin_bit_cast(float, pk << 16) * wl, __builtin_bit_cast(float, pk & 0xffff0000u) * wh);
        }
        o[j] = pk;
    }
    return o;
}

// silu in fp32 from a bf16-rounded input; the result is rounded to bf16 by the caller, which absorbs the
// 1-ulp error of the hardware exp and reciprocal.
__device__ __forceinline__ float silu_f32(float g) { return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)); }

// SwiGLU epilogue for the four consecutive hidden features a lane holds: every intermediate is rounded to
// bf16 where the reference materialises a bf16 tensor (gate_up output, silu, product, gated product).
// `gate` is the router gate of these features (they lie in one cluster); pass has_gate = false for none.
__device__ __forceinline__ u32x2_t swiglu_pack4(f32x4_t g, f32x4_t u, bool has_gate, float gate) {
    // each value is rounded on its own (one conversion, no unpacking of a packed pair)
    float h[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) h[v] = bf16r(silu_f32(bf16r(g[v]))) * bf16r(u[v]);
    if (has_gate) {
        const float gb = bf16r(gate);
#pragma unroll
        for (int v = 0; v < 4; ++v) h[v] = bf16r(h[v]) * gb;
    }
    return u32x2_t{bf16_pack2(h[0], h[1]), bf16_pack2(h[2], h[3])};
}

#endif
