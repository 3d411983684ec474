// Weighted top-k combine, residual add and the FFN RMSNorm around the block.
#include "common.h"
#include "kernels.h"

namespace moe {

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
    int ex[8], sl[8];
    float wt[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        if (k < K) {
            ex[k] = topk_i[(size_t)t * K + k];
            sl[k] = slot_of[(size_t)t * K + k];
            wt[k] = topk_v[(size_t)t * K + k];
        } else {
            ex[k] = 0x7FFFFFFF;
            sl[k] = 0;
            wt[k] = 0.f;
        }
    }
    // sorting network-free insertion sort on 8 register entries (fully unrolled), key = expert id
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

// o = weight * (x / sqrt(mean(x^2) + 1e-5)) per row, with the reference CPU's mixed precision
// (src/run.cpp:306-319): fp32 squares summed in fp64 in ascending index order per lane partial,
// sqrtf and the reciprocal in fp32, the scaling in fp64, one rounding to fp32 at the end.
// One block per row; the block-wide fp64 sum is a fixed tree, so results are run-to-run identical.
__global__ __launch_bounds__(256) void rmsnorm_kernel(float* __restrict__ o, const float* __restrict__ x,
                                                      const uint16_t* __restrict__ weight, int size) {
    __shared__ double red[256];
    const float* xr = x + (size_t)blockIdx.x * size;
    float* orow = o + (size_t)blockIdx.x * size;
    double ss = 0.0;
    for (int j = threadIdx.x; j < size; j += 256) ss += (double)__fmul_rn(xr[j], xr[j]);
    red[threadIdx.x] = ss;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    double m = red[0] / size;
    m += (double)1e-5f;
    const double inv = (double)(1.0f / sqrtf((float)m));
    for (int j = threadIdx.x; j < size; j += 256) {
        const double w = (double)bf16_bits_to_f32(weight[j]);
        orow[j] = (float)(w * (inv * (double)xr[j]));
    }
}

int launch_rmsnorm(float* o, const float* x, const uint16_t* weight, int batch, int size, hipStream_t stream) {
    hipLaunchKernelGGL(rmsnorm_kernel, dim3(batch), dim3(256), 0, stream, o, x, weight, size);
    return launch_status();
}

}  // namespace moe
