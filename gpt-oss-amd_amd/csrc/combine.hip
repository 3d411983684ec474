// Weighted top-k combine, residual add and the FFN RMSNorm around the block.
#include "common.h"
#include "kernels.h"

namespace moe {

// The token's K (slot, weight) pairs in ascending expert id (block-uniform: scalar loads and a
// fully unrolled insertion sort on eight register entries).  slot_of == NULL: rows are stored by
// assignment, the row of (t, k) is t * K + k.
MOE_DEVICE void sorted_slots(const int* __restrict__ slot_of, const int* __restrict__ topk_i,
                             const float* __restrict__ topk_v, int t, int K, int (&sl)[8], float (&wt)[8]) {
    int ex[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        if (k < K) {
            ex[k] = topk_i[(size_t)t * K + k];
            sl[k] = slot_of ? slot_of[(size_t)t * K + k] : t * K + k;
            wt[k] = topk_v[(size_t)t * K + k];
        } else {
            ex[k] = 0x7FFFFFFF;
            sl[k] = 0;
            wt[k] = 0.f;
        }
    }
#pragma unroll
    for (int i = 1; i < 8; ++i) {
#pragma unroll
        for (int j = i; j > 0; --j) {
            if (ex[j] < ex[j - 1]) {
                const int te = ex[j]; ex[j] = ex[j - 1]; ex[j - 1] = te;
                const int ts = sl[j]; sl[j] = sl[j - 1]; sl[j - 1] = ts;
                const float tw = wt[j]; wt[j] = wt[j - 1]; wt[j - 1] = tw;
            }
        }
    }
}

// One float4 column of the token's combined row: K fused multiply-adds in ascending expert id.
MOE_DEVICE float4 combine_column(const float4* __restrict__ y, const int (&sl)[8], const float (&wt)[8], int K, int H4,
                                 int c) {
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        if (k < K) {
            const float4 v = y[(size_t)sl[k] * H4 + c];
            acc.x = fmaf(v.x, wt[k], acc.x);
            acc.y = fmaf(v.y, wt[k], acc.y);
            acc.z = fmaf(v.z, wt[k], acc.z);
            acc.w = fmaf(v.w, wt[k], acc.w);
        }
    }
    return acc;
}

// Rows stored by assignment (the row of (t, k) is t * K + k): the K rows are known without looking
// at the routing, so their loads go out together with the loads of the routing itself (one memory
// round trip instead of two).  The order of the additions is fixed afterwards: the rank of each k by
// expert id is block-uniform, and rank r is added in step r.
MOE_DEVICE float4 combine_column_by_assignment(const float4* __restrict__ y, const int* __restrict__ topk_i,
                                               const float* __restrict__ topk_v, int t, int K, int H4, int c) {
    float4 v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k)
        if (k < K) v[k] = y[((size_t)t * K + k) * H4 + c];
    int ex[8];
    float wt[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        ex[k] = k < K ? topk_i[(size_t)t * K + k] : 0x7FFFFFFF;
        wt[k] = k < K ? topk_v[(size_t)t * K + k] : 0.f;
    }
    int rank[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        rank[k] = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) rank[k] += (ex[j] < ex[k] || (ex[j] == ex[k] && j < k)) ? 1 : 0;
    }
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        if (r < K) {
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                if (k < K && rank[k] == r) {  // block-uniform
                    acc.x = fmaf(v[k].x, wt[k], acc.x);
                    acc.y = fmaf(v[k].y, wt[k], acc.y);
                    acc.z = fmaf(v[k].z, wt[k], acc.z);
                    acc.w = fmaf(v[k].w, wt[k], acc.w);
                }
            }
        }
    }
    return acc;
}

// e_agg[t,:] = sum over the token's K experts, visited in ASCENDING EXPERT ID, of
// y_by_slot[slot,:] * weight, each step one fused multiply-add — the order and rounding of the
// reference CPU loop (src/run.cpp:645-706).  Replaces the atomicAdd scatter of
// moe_mlp2_scatter_mfma_kernel (src/hip/moe.hip:464-492), whose order is not fixed.
// Optionally also residual_x += e_agg (src/forward.cpp:514).
// grid = (ceil(H/4/256), T), block = 256.
__global__ __launch_bounds__(256) void combine_kernel(const float4* __restrict__ y, const int* __restrict__ slot_of,
                                                      const int* __restrict__ topk_i,
                                                      const float* __restrict__ topk_v, float4* __restrict__ e_agg,
                                                      float4* __restrict__ residual_x, int T, int K, int H4) {
    const int t = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= H4) return;
    float4 acc;
    if (slot_of) {
        int sl[8];
        float wt[8];
        sorted_slots(slot_of, topk_i, topk_v, t, K, sl, wt);
        acc = combine_column(y, sl, wt, K, H4, c);
    } else {
        acc = combine_column_by_assignment(y, topk_i, topk_v, t, K, H4, c);
    }
    e_agg[(size_t)t * H4 + c] = acc;
    if (residual_x) {
        float4 r = residual_x[(size_t)t * H4 + c];
        r.x += acc.x;
        r.y += acc.y;
        r.z += acc.z;
        r.w += acc.w;
        residual_x[(size_t)t * H4 + c] = r;
    }
}

int launch_combine(const float* y_by_slot, const int* slot_of, const int* topk_i, const float* topk_v,
                   float* e_agg, float* residual_x, int T, int K, int H, hipStream_t stream) {
    const int H4 = H / 4;
    hipLaunchKernelGGL(combine_kernel, dim3(ceil_div(H4, 256), T), dim3(256), 0, stream,
                       reinterpret_cast<const float4*>(y_by_slot), slot_of, topk_i, topk_v,
                       reinterpret_cast<float4*>(e_agg), reinterpret_cast<float4*>(residual_x), T, K, H4);
    return launch_status();
}

// a += b * weight; b = 0   (src/hip/vecadd.hip:19-39)
__global__ void vecadd_and_zero_kernel(float* __restrict__ a, float* __restrict__ b, float weight, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    a[i] += b[i] * weight;
    b[i] = 0.0f;
}

int launch_vecadd_and_zero(float* a, float* b, float weight, int batch, int size, hipStream_t stream) {
    const size_t n = (size_t)batch * size;
    hipLaunchKernelGGL(vecadd_and_zero_kernel, dim3((unsigned)ceil_div(n, (size_t)256)), dim3(256), 0, stream, a, b,
                       weight, n);
    return launch_status();
}

// RMSNorm of src/run.cpp:306-319 with the reference CPU's mixed precision: fp32 squares summed in
// fp64, sqrtf and the reciprocal in fp32, the scaling in fp64, one rounding to fp32 at the end.
// A row is owned by one block of 256 threads; thread i holds float4 columns i, i + 256, ... and adds
// their squares in ascending order, the block-wide fp64 sum is a fixed tree: results are run-to-run
// identical, and identical between the plain kernel and the one fused into the combine.
MOE_DEVICE double sumsq(double ss, const float4& v) {
    ss += (double)__fmul_rn(v.x, v.x);
    ss += (double)__fmul_rn(v.y, v.y);
    ss += (double)__fmul_rn(v.z, v.z);
    ss += (double)__fmul_rn(v.w, v.w);
    return ss;
}

MOE_DEVICE double block_inv_rms(double ss, double* red, int size) {
    red[threadIdx.x] = ss;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    double m = red[0] / size;
    m += (double)1e-5f;
    return (double)(1.0f / sqrtf((float)m));
}

MOE_DEVICE float4 norm_scale(const float4& v, const uint16_t* __restrict__ weight, int c, double inv) {
    const uint2 wb = *reinterpret_cast<const uint2*>(weight + 4 * c);
    float4 o;
    o.x = (float)((double)bf16_bits_to_f32(wb.x & 0xFFFFu) * (inv * (double)v.x));
    o.y = (float)((double)bf16_bits_to_f32(wb.x >> 16) * (inv * (double)v.y));
    o.z = (float)((double)bf16_bits_to_f32(wb.y & 0xFFFFu) * (inv * (double)v.z));
    o.w = (float)((double)bf16_bits_to_f32(wb.y >> 16) * (inv * (double)v.w));
    return o;
}

// grid = rows, block = 256; size % 4 == 0.
__global__ __launch_bounds__(256) void rmsnorm_kernel(float* __restrict__ o, const float* __restrict__ x,
                                                      const uint16_t* __restrict__ weight, int size) {
    __shared__ double red[256];
    const int H4 = size >> 2;
    const float4* xr = reinterpret_cast<const float4*>(x + (size_t)blockIdx.x * size);
    float4* orow = reinterpret_cast<float4*>(o + (size_t)blockIdx.x * size);
    double ss = 0.0;
    for (int c = threadIdx.x; c < H4; c += 256) ss = sumsq(ss, xr[c]);
    const double inv = block_inv_rms(ss, red, size);
    for (int c = threadIdx.x; c < H4; c += 256) orow[c] = norm_scale(xr[c], weight, c, inv);
}

// Combine, residual add and the RMSNorm that follows it in the layer loop (the attention norm of the
// next layer, src/forward.cpp:262, or the final norm, :997), in one pass over the token's row:
//   e_agg = combine;  residual_x += e_agg;  norm_out = rmsnorm(residual_x, norm_weight).
// Same arithmetic as combine_kernel followed by rmsnorm_kernel.  A thread keeps its NI float4 columns
// of the updated residual in registers.  grid = T, block = 256, H/4 <= 256 * NI.
template <int NI>
__global__ __launch_bounds__(256) void combine_norm_kernel(const float4* __restrict__ y, const int* __restrict__ slot_of,
                                                           const int* __restrict__ topk_i,
                                                           const float* __restrict__ topk_v, float4* __restrict__ e_agg,
                                                           float4* __restrict__ residual_x,
                                                           const uint16_t* __restrict__ norm_weight,
                                                           float4* __restrict__ norm_out, int K, int H4) {
    __shared__ double red[256];
    const int t = blockIdx.x;
    int sl[8];
    float wt[8];
    sorted_slots(slot_of, topk_i, topk_v, t, K, sl, wt);
    float4 r[NI];
    double ss = 0.0;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int c = threadIdx.x + 256 * i;
        if (c < H4) {
            const float4 acc = combine_column(y, sl, wt, K, H4, c);
            e_agg[(size_t)t * H4 + c] = acc;
            float4 v = residual_x[(size_t)t * H4 + c];
            v.x += acc.x;
            v.y += acc.y;
            v.z += acc.z;
            v.w += acc.w;
            residual_x[(size_t)t * H4 + c] = v;
            r[i] = v;
            ss = sumsq(ss, v);
        }
    }
    const double inv = block_inv_rms(ss, red, 4 * H4);
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int c = threadIdx.x + 256 * i;
        if (c < H4) norm_out[(size_t)t * H4 + c] = norm_scale(r[i], norm_weight, c, inv);
    }
}

// Returns MOE_ERR_LIMIT when the row is too long for the fused kernel (the caller then runs the two
// kernels one after the other).
int launch_combine_norm(const float* y_by_slot, const int* slot_of, const int* topk_i, const float* topk_v,
                        float* e_agg, float* residual_x, const uint16_t* norm_weight, float* norm_out, int T, int K,
                        int H, hipStream_t stream) {
    const int H4 = H / 4;
    const int ni = ceil_div(H4, 256);
    auto y = reinterpret_cast<const float4*>(y_by_slot);
    auto e = reinterpret_cast<float4*>(e_agg);
    auto r = reinterpret_cast<float4*>(residual_x);
    auto o = reinterpret_cast<float4*>(norm_out);
    if (ni <= 1) {
        hipLaunchKernelGGL((combine_norm_kernel<1>), dim3(T), dim3(256), 0, stream, y, slot_of, topk_i, topk_v, e, r,
                           norm_weight, o, K, H4);
    } else if (ni <= 2) {
        hipLaunchKernelGGL((combine_norm_kernel<2>), dim3(T), dim3(256), 0, stream, y, slot_of, topk_i, topk_v, e, r,
                           norm_weight, o, K, H4);
    } else if (ni <= 3) {
        hipLaunchKernelGGL((combine_norm_kernel<3>), dim3(T), dim3(256), 0, stream, y, slot_of, topk_i, topk_v, e, r,
                           norm_weight, o, K, H4);
    } else if (ni <= 4) {
        hipLaunchKernelGGL((combine_norm_kernel<4>), dim3(T), dim3(256), 0, stream, y, slot_of, topk_i, topk_v, e, r,
                           norm_weight, o, K, H4);
    } else {
        return MOE_ERR_LIMIT;
    }
    return launch_status();
}

int launch_rmsnorm(float* o, const float* x, const uint16_t* weight, int batch, int size, hipStream_t stream) {
    hipLaunchKernelGGL(rmsnorm_kernel, dim3(batch), dim3(256), 0, stream, o, x, weight, size);
    return launch_status();
}

}  // namespace moe
