// Layer normalisation of the reference's transformer layer for gfx950 (MI355X).
//
// Replaces norm() (inference-engine/src/host/transformer_layer.cpp:50-90) and the residual add that
// follows it in the layer (:476-486 and :601-611).  Numerics follow the reference statement by
// statement: the mean and the variance are accumulated in double and rounded to float, the centred
// value, its square and the three output operations (scale, weight, bias) are separately rounded fp32
// operations (this translation unit is built with -ffp-contract=off), eps = 1e-6.  The only freedom
// taken is the order of the two double-precision sums: a row is summed by 64 lanes and a butterfly
// instead of sequentially, which can move the float mean or variance by one ulp in rare rows.
#include "pimdl_internal.h"

namespace pimdl {

namespace {

__device__ __forceinline__ double wave_sum(double v)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

// one wave per row
__global__ __launch_bounds__(256) void layer_norm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                        const float* __restrict__ b,
                                                        const float* __restrict__ residual,
                                                        float* __restrict__ out, uint32_t n, uint32_t d, float eps)
{
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n) return;
    const float* xr = x + (size_t)row * d;
    double s = 0.0;
    for (uint32_t i = lane; i < d; i += 64) s += (double)xr[i];
    const float mean = (float)(wave_sum(s) / (double)d);
    double s2 = 0.0;
    for (uint32_t i = lane; i < d; i += 64) {
        const float v = __fsub_rn(xr[i], mean);
        s2 += (double)__fmul_rn(v, v);
    }
    const float variance = (float)(wave_sum(s2) / (double)d);
    const float scale = 1.0f / sqrtf(__fadd_rn(variance, eps));
    float* o = out + (size_t)row * d;
    const float* r = residual ? residual + (size_t)row * d : nullptr;
    for (uint32_t i = lane; i < d; i += 64) {
        float y = __fsub_rn(xr[i], mean);
        y = __fmul_rn(y, scale);
        y = __fmul_rn(y, w[i]);
        y = __fadd_rn(y, b[i]);
        o[i] = r ? __fadd_rn(r[i], y) : y;
    }
}

}  // namespace

int launch_layer_norm(Ctx* ctx, const float* d_x, const float* d_w, const float* d_b, const float* d_residual,
                      float* d_out, uint32_t n, uint32_t d, float eps)
{
    if (n == 0) return PIMDL_OK;
    hipLaunchKernelGGL(layer_norm_kernel, dim3((n + 3) / 4), dim3(256), 0, ctx->stream, d_x, d_w, d_b, d_residual,
                       d_out, n, d, eps);
    return hip_check(ctx, hipGetLastError(), "layer_norm_kernel launch");
}

}  // namespace pimdl
