// Shared device/host helpers for the gfx950 MoE kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/moe_abi.h"

namespace moe {

constexpr int kWave = 64;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define MOE_DEVICE __device__ __forceinline__

// Launch-error plumbing: entries return hipError_t values as positive ints.
#define MOE_RETURN_IF_HIP(expr)                  \
    do {                                         \
        hipError_t moe_e_ = (expr);              \
        if (moe_e_ != hipSuccess) return (int)moe_e_; \
    } while (0)

static inline int launch_status() { return (int)hipGetLastError(); }

template <typename T>
__host__ __device__ static inline T ceil_div(T a, T b) {
    return (a + b - 1) / b;
}

// ---- bf16 <-> fp32 ------------------------------------------------------------------------
MOE_DEVICE float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// Round-to-nearest-even fp32 -> bf16 pair packed in a dword (low half = a).
MOE_DEVICE uint32_t pack_bf16x2(float a, float b) {
    f32x2 v = {a, b};
    bf16x2 r = __builtin_convertvector(v, bf16x2);
    return __builtin_bit_cast(uint32_t, r);
}

MOE_DEVICE uint16_t f32_to_bf16_bits(float a) {
    __bf16 r = (__bf16)a;
    return __builtin_bit_cast(uint16_t, r);
}

// ---- MXFP4 -> bf16 --------------------------------------------------------------------------
// General routine, every scale byte: integer assembly of the bf16 bit pattern of
// LUT[code] * 2^(scale-127), LUT = {0,.5,1,1.5,2,3,4,6} with bit 3 of the code as sign
// (tools/model_export/gpt-oss-20b/export_model_bin.py:75-92, 129).
MOE_DEVICE uint32_t mxfp4_code_to_bf16_bits(uint32_t code, uint32_t scale) {
    const uint32_t sign = (code & 8u) << 12;
    const uint32_t mag = code & 7u;
    // p = exponent step of the magnitude, f = 1 when the magnitude has the half bit
    // magnitude = (1 + f/2) * 2^(pp-1): pp = 0,0,1,1,2,2,3,3 and f = 0,0,0,1,0,1,0,1 for mag 0..7
    const uint32_t pp = mag >> 1;
    const uint32_t f = (mag >= 3u) ? (mag & 1u) : 0u;
    if (scale == 255u) return mag == 0u ? 0x7FC0u : (sign | 0x7F80u);
    if (mag == 0u) return sign;
    const int biased = (int)pp + (int)scale - 1;
    if (biased >= 255) return sign | 0x7F80u;
    if (biased >= 1) return sign | ((uint32_t)biased << 7) | (f << 6);
    return sign | ((2u + f) << (biased + 5));
}

// Fast routine for the fused GEMM path: one dword = 8 codes sharing one scale byte, expanded to
// four bf16x2 dwords in element order (low nibble of byte 0 first) by the gfx950 scaled
// conversion.  The scale operand is the fp32 value 2^(scale-127).
MOE_DEVICE float mxfp4_scale_to_f32(uint32_t scale_byte) { return __uint_as_float(scale_byte << 23); }

MOE_DEVICE void mxfp4_dword_to_bf16x8(uint32_t codes, float scale, uint32_t out[4]) {
    out[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 0));
    out[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 1));
    out[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 2));
    out[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 3));
}

// ---- MFMA -----------------------------------------------------------------------------------
// D(16x16) += A(16x32) * B(32x16); lane l holds A[row l%16][8*(l/16) .. +8), B[.. same k ..][col l%16],
// D[rows 4*(l/16) .. +4][col l%16].
MOE_DEVICE f32x4 mfma_16x16x32(const u32x4& a, const u32x4& b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// D(32x32) += A(32x16) * B(16x32); lane l holds A[row l%32][8*(l/32) .. +8), B[..][col l%32],
// D[rows 8*(i/4) + 4*(l/32) + i%4 for i in 0..15][col l%32].
MOE_DEVICE f32x16 mfma_32x32x16(const u32x4& a, const u32x4& b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// ---- wave-wide reductions on the DPP path -----------------------------------------------------
// Six data-parallel-primitive steps (shift right by 1, 2, 4, 8 inside each row of 16 lanes, then
// the two row broadcasts) leave the combination of all 64 lanes in lane 63; a lane whose source
// falls outside its row keeps `identity`.  No LDS traffic and no waiting on the LDS queue, unlike
// the ds_bpermute behind __shfl_xor.  The result is read from lane 63 into a scalar register, so
// every lane gets it.
template <int CTRL, int ROW_MASK>
MOE_DEVICE uint32_t dpp_move(uint32_t identity, uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp((int)identity, (int)v, CTRL, ROW_MASK, 0xf, false);
}

#define MOE_DPP_STEPS(STEP) \
    STEP(0x111, 0xf)        \
    STEP(0x112, 0xf)        \
    STEP(0x114, 0xf)        \
    STEP(0x118, 0xf)        \
    STEP(0x142, 0xa)        \
    STEP(0x143, 0xc)

MOE_DEVICE float wave_sum(float v) {
#define MOE_STEP(C, M) v += __uint_as_float(dpp_move<C, M>(0u, __float_as_uint(v)));
    MOE_DPP_STEPS(MOE_STEP)
#undef MOE_STEP
    return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), 63));
}

MOE_DEVICE int wave_sum(int v) {
#define MOE_STEP(C, M) v += (int)dpp_move<C, M>(0u, (uint32_t)v);
    MOE_DPP_STEPS(MOE_STEP)
#undef MOE_STEP
    return __builtin_amdgcn_readlane(v, 63);
}

// for v >= 0
MOE_DEVICE float wave_max_nonneg(float v) {
#define MOE_STEP(C, M) v = fmaxf(v, __uint_as_float(dpp_move<C, M>(0u, __float_as_uint(v))));
    MOE_DPP_STEPS(MOE_STEP)
#undef MOE_STEP
    return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), 63));
}

// Fixed combination order (a pure function of the lane values), so results are reproducible.
MOE_DEVICE double wave_sum(double v) {
#define MOE_STEP(C, M)                                                          \
    {                                                                           \
        const uint64_t b = __builtin_bit_cast(uint64_t, v);                     \
        const uint32_t lo = dpp_move<C, M>(0u, (uint32_t)b);                    \
        const uint32_t hi = dpp_move<C, M>(0u, (uint32_t)(b >> 32));            \
        v += __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);             \
    }
    MOE_DPP_STEPS(MOE_STEP)
#undef MOE_STEP
    const uint64_t b = __builtin_bit_cast(uint64_t, v);
    const uint32_t lo = __builtin_amdgcn_readlane((uint32_t)b, 63);
    const uint32_t hi = __builtin_amdgcn_readlane((uint32_t)(b >> 32), 63);
    return __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
}

// ---- clamped SwiGLU (src/run.cpp:673-689) ---------------------------------------------------
MOE_DEVICE float swiglu(float gate, float up, float alpha, float limit) {
    gate = gate > limit ? limit : gate;
    up = up > limit ? limit : up;
    up = up < -limit ? -limit : up;
    // sigmoid through the hardware's exp2 and reciprocal (each good to one unit in the last place:
    // relative error ~1e-7, far inside the 1e-2 output tolerance; the reference's own GPU kernel uses
    // __expf as well, src/hip/moe.hip:189).  The IEEE division the plain expression compiles to costs
    // ten more instructions per output, and the epilogue runs with the matrix pipe idle.
    const float sig = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(gate * (alpha * -1.44269504088896f)));
    return (gate * sig) * (up + 1.0f);
}

// Storage order of weight rows inside a group of 64 rows: MFMA tile r (0..3), tile row q (0..15)
// holds weight row (q/4)*16 + r*4 + q%4 of the group.  With this order lane group g = lane/16 of
// the 16x16 accumulator layout owns rows g*16 + r*4 + j (j = 0..3) across the four tiles, i.e. 16
// consecutive weight rows, so epilogue stores are contiguous and gate/up pairs stay in one lane.
MOE_DEVICE int tile_row_in_group(int r, int q) { return (q >> 2) * 16 + r * 4 + (q & 3); }

}  // namespace moe
