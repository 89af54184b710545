// Layer normalisation of the reference's transformer layer for gfx950 (MI355X).
//
// Replaces norm() (inference-engine/src/host/transformer_layer.cpp:50-90) and the residual add that
// follows it in the layer (:476-486 and :601-611).  Numerics follow the reference statement by
// statement: the mean and the variance are accumulated in double and rounded to float, the centred
// value, its square and the three output operations (scale, weight, bias) are separately rounded fp32
// operations (this translation unit is built with -ffp-contract=off), eps = 1e-6.  The only freedom
// taken is the order of the two double-precision sums: a row is summed by 64 lanes and a butterfly
// instead of sequentially, which can move the float mean or variance by one ulp in rare rows.
// The centred value x - mean is computed once and reused (the reference computes the identical
// expression twice).
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

// The same for rows of up to 64 * 4 * KV floats with d % 4 == 0 and 16-byte aligned buffers: the row
// is read once with float4 loads and stays in registers for the three passes.
template <int KV>
__global__ __launch_bounds__(256) void layer_norm_vec_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                            const float* __restrict__ b,
                                                            const float* __restrict__ residual,
                                                            float* __restrict__ out, uint32_t n, uint32_t d, float eps)
{
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n) return;
    const uint32_t d4 = d / 4;
    const float4* xr = reinterpret_cast<const float4*>(x + (size_t)row * d);
    float4 xv[KV];
    double s = 0.0;
#pragma unroll
    for (int k = 0; k < KV; ++k) {
        const uint32_t i = lane + 64 * k;
        if (i < d4) {
            xv[k] = xr[i];
            s += (double)xv[k].x;
            s += (double)xv[k].y;
            s += (double)xv[k].z;
            s += (double)xv[k].w;
        }
    }
    const float mean = (float)(wave_sum(s) / (double)d);
    double s2 = 0.0;
#pragma unroll
    for (int k = 0; k < KV; ++k) {
        if (lane + 64 * k < d4) {
            xv[k].x = __fsub_rn(xv[k].x, mean);
            xv[k].y = __fsub_rn(xv[k].y, mean);
            xv[k].z = __fsub_rn(xv[k].z, mean);
            xv[k].w = __fsub_rn(xv[k].w, mean);
            s2 += (double)__fmul_rn(xv[k].x, xv[k].x);
            s2 += (double)__fmul_rn(xv[k].y, xv[k].y);
            s2 += (double)__fmul_rn(xv[k].z, xv[k].z);
            s2 += (double)__fmul_rn(xv[k].w, xv[k].w);
        }
    }
    const float variance = (float)(wave_sum(s2) / (double)d);
    const float scale = 1.0f / sqrtf(__fadd_rn(variance, eps));
    float4* o = reinterpret_cast<float4*>(out + (size_t)row * d);
    const float4* r = residual ? reinterpret_cast<const float4*>(residual + (size_t)row * d) : nullptr;
    const float4* w4 = reinterpret_cast<const float4*>(w);
    const float4* b4 = reinterpret_cast<const float4*>(b);
#pragma unroll
    for (int k = 0; k < KV; ++k) {
        const uint32_t i = lane + 64 * k;
        if (i < d4) {
            const float4 wv = w4[i], bv = b4[i];
            float4 y;
            y.x = __fadd_rn(__fmul_rn(__fmul_rn(xv[k].x, scale), wv.x), bv.x);
            y.y = __fadd_rn(__fmul_rn(__fmul_rn(xv[k].y, scale), wv.y), bv.y);
            y.z = __fadd_rn(__fmul_rn(__fmul_rn(xv[k].z, scale), wv.z), bv.z);
            y.w = __fadd_rn(__fmul_rn(__fmul_rn(xv[k].w, scale), wv.w), bv.w);
            if (r) {
                const float4 rv = r[i];
                y.x = __fadd_rn(rv.x, y.x);
                y.y = __fadd_rn(rv.y, y.y);
                y.z = __fadd_rn(rv.z, y.z);
                y.w = __fadd_rn(rv.w, y.w);
            }
            o[i] = y;
        }
    }
}

}  // namespace

int launch_layer_norm(Ctx* ctx, const float* d_x, const float* d_w, const float* d_b, const float* d_residual,
                      float* d_out, uint32_t n, uint32_t d, float eps)
{
    if (n == 0) return PIMDL_OK;
    const uintptr_t all = reinterpret_cast<uintptr_t>(d_x) | reinterpret_cast<uintptr_t>(d_w) |
                          reinterpret_cast<uintptr_t>(d_b) | reinterpret_cast<uintptr_t>(d_residual) |
                          reinterpret_cast<uintptr_t>(d_out);
    if (d % 4 == 0 && (all & 15) == 0 && d <= 64 * 4 * 8) {
        if (d <= 64 * 4 * 4)
            hipLaunchKernelGGL(layer_norm_vec_kernel<4>, dim3((n + 3) / 4), dim3(256), 0, ctx->stream, d_x, d_w, d_b,
                               d_residual, d_out, n, d, eps);
        else
            hipLaunchKernelGGL(layer_norm_vec_kernel<8>, dim3((n + 3) / 4), dim3(256), 0, ctx->stream, d_x, d_w, d_b,
                               d_residual, d_out, n, d, eps);
        return hip_check(ctx, hipGetLastError(), "layer_norm_vec_kernel launch");
    }
    hipLaunchKernelGGL(layer_norm_kernel, dim3((n + 3) / 4), dim3(256), 0, ctx->stream, d_x, d_w, d_b, d_residual,
                       d_out, n, d, eps);
    return hip_check(ctx, hipGetLastError(), "layer_norm_kernel launch");
}

}  // namespace pimdl
