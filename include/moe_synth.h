/*
 * moe_synth.h — counter-based synthetic tensor generator shared by host and device code.
 *
 * Every element of every synthetic tensor is a pure function of (seed, tensor_id, flat_index):
 * a 64-bit integer mix followed by a table lookup or an integer range reduction.  No libm call
 * is made per element, so a host loop and a HIP kernel produce bit-identical tensors, and a
 * multi-gigabyte weight set can be generated directly in device memory.
 *
 * Distributions used by the MoE workloads (shapes follow the reference checkpoint layout,
 * tools/model_export/gpt-oss-20b/export_model_bin.py:51-71, and its config.json):
 *   - activations      fp32  N(0,1)         -> normal table lookup
 *   - bf16 weights     bf16  N(0,0.02)      -> bf16_rne(0.02f * normal table lookup)
 *   - MXFP4 codes      u8    two uniform e2m1 codes per byte (low nibble = even element)
 *   - MXFP4 scales     u8    uniform in [lo, lo+span)   (e8m0, value 2^(s-127))
 *
 * The normal table holds MOE_SYNTH_TABLE_SIZE quantiles of N(0,1); it is computed once on the
 * host (moe_synth_build_normal_table) and handed to whichever side consumes it.
 */
#ifndef MOE_SYNTH_H
#define MOE_SYNTH_H

#include <stdint.h>
#include <stddef.h>

#if defined(__HIPCC__)
#define MOE_SYNTH_HD __host__ __device__ static inline
#else
#define MOE_SYNTH_HD static inline
#endif

#define MOE_SYNTH_TABLE_BITS 16
#define MOE_SYNTH_TABLE_SIZE (1u << MOE_SYNTH_TABLE_BITS)

/* tensor ids: one stream per logical tensor; layers add MOE_SYNTH_LAYER_STRIDE * layer */
enum {
    MOE_SYNTH_X = 1,
    MOE_SYNTH_W_ROUTER = 2,
    MOE_SYNTH_B_ROUTER = 3,
    MOE_SYNTH_W_MLP1 = 4,
    MOE_SYNTH_B_MLP1 = 5,
    MOE_SYNTH_W_MLP2 = 6,
    MOE_SYNTH_B_MLP2 = 7,
    MOE_SYNTH_W_MLP1_SCALES = 8,
    MOE_SYNTH_W_MLP2_SCALES = 9,
    MOE_SYNTH_LAYER_STRIDE = 16
};

/* splitmix64-style finaliser over (seed, tensor_id, idx); returns the high 32 bits */
MOE_SYNTH_HD uint32_t moe_synth_hash(uint32_t seed, uint32_t tensor_id, uint64_t idx) {
    uint64_t z = idx + 0x9E3779B97F4A7C15ull * (((uint64_t)seed << 20) + (uint64_t)tensor_id + 1ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z = z ^ (z >> 31);
    return (uint32_t)(z >> 32);
}

/* fp32 -> bf16 bits, round to nearest even (finite inputs; NaN kept quiet) */
MOE_SYNTH_HD uint16_t moe_synth_f32_to_bf16_bits(float f) {
    union { float f; uint32_t u; } v;
    v.f = f;
    if ((v.u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((v.u >> 16) | 0x0040u);
    uint32_t lsb = (v.u >> 16) & 1u;
    return (uint16_t)((v.u + 0x7FFFu + lsb) >> 16);
}

MOE_SYNTH_HD float moe_synth_bf16_bits_to_f32(uint16_t b) {
    union { float f; uint32_t u; } v;
    v.u = (uint32_t)b << 16;
    return v.f;
}

MOE_SYNTH_HD float moe_synth_normal_f32(const float* table, float scale, uint32_t seed,
                                        uint32_t tensor_id, uint64_t idx) {
    return scale * table[moe_synth_hash(seed, tensor_id, idx) >> (32 - MOE_SYNTH_TABLE_BITS)];
}

MOE_SYNTH_HD uint16_t moe_synth_normal_bf16(const float* table, float scale, uint32_t seed,
                                            uint32_t tensor_id, uint64_t idx) {
    return moe_synth_f32_to_bf16_bits(moe_synth_normal_f32(table, scale, seed, tensor_id, idx));
}

MOE_SYNTH_HD uint8_t moe_synth_byte(uint32_t seed, uint32_t tensor_id, uint64_t idx) {
    return (uint8_t)(moe_synth_hash(seed, tensor_id, idx) >> 24);
}

/* uniform integer in [lo, lo+span), span <= 256 */
MOE_SYNTH_HD uint8_t moe_synth_range_byte(uint32_t seed, uint32_t tensor_id, uint64_t idx,
                                          uint32_t lo, uint32_t span) {
    uint32_t h = moe_synth_hash(seed, tensor_id, idx);
    return (uint8_t)(lo + (uint32_t)(((uint64_t)h * span) >> 32));
}

#if !defined(__HIP_DEVICE_COMPILE__)
#include <math.h>
/* Quantile table of N(0,1): table[i] = Phi^-1((i + 0.5) / size), by Acklam's rational
 * approximation refined with one Halley step on erfc (relative error < 1e-15 before the final
 * rounding to fp32).  Host only. */
static inline double moe_synth_ndtri(double p) {
    static const double a[6] = {-3.969683028665376e+01, 2.209460984245205e+02, -2.759285104469687e+02,
                                1.383577518672690e+02,  -3.066479806614716e+01, 2.506628277459239e+00};
    static const double b[5] = {-5.447609879822406e+01, 1.615858368580409e+02, -1.556989798598866e+02,
                                6.680131188771972e+01,  -1.328068155288572e+01};
    static const double c[6] = {-7.784894002430293e-03, -3.223964580411365e-01, -2.400758277161838e+00,
                                -2.549732539343734e+00, 4.374664141464968e+00,  2.938163982698783e+00};
    static const double d[4] = {7.784695709041462e-03, 3.224671290700398e-01, 2.445134137142996e+00,
                                3.754408661907416e+00};
    double q, r, x;
    if (p < 0.02425) {
        q = sqrt(-2.0 * log(p));
        x = (((((c[0] * q + c[1]) * q + c[2]) * q + c[3]) * q + c[4]) * q + c[5]) /
            ((((d[0] * q + d[1]) * q + d[2]) * q + d[3]) * q + 1.0);
    } else if (p > 1.0 - 0.02425) {
        q = sqrt(-2.0 * log(1.0 - p));
        x = -(((((c[0] * q + c[1]) * q + c[2]) * q + c[3]) * q + c[4]) * q + c[5]) /
            ((((d[0] * q + d[1]) * q + d[2]) * q + d[3]) * q + 1.0);
    } else {
        q = p - 0.5;
        r = q * q;
        x = (((((a[0] * r + a[1]) * r + a[2]) * r + a[3]) * r + a[4]) * r + a[5]) * q /
            (((((b[0] * r + b[1]) * r + b[2]) * r + b[3]) * r + b[4]) * r + 1.0);
    }
    {
        double e = 0.5 * erfc(-x / sqrt(2.0)) - p;
        double u = e * sqrt(2.0 * 3.14159265358979323846) * exp(x * x / 2.0);
        x = x - u / (1.0 + x * u / 2.0);
    }
    return x;
}

static inline void moe_synth_build_normal_table(float* table) {
    for (uint32_t i = 0; i < MOE_SYNTH_TABLE_SIZE; ++i)
        table[i] = (float)moe_synth_ndtri(((double)i + 0.5) / (double)MOE_SYNTH_TABLE_SIZE);
}
#endif

#endif /* MOE_SYNTH_H */
