// LUT construction for gfx950 (MI355X): the one dense contraction of the path, on the matrix cores.
//
// Replaces model-calibration/pim_weight_converter.py:82-91 of the reference
//     lut = bmm(centroids.view(CB, C, v), weight.view(CB, v, M))
// and lut_quant (:21-35)
//     scale = max|lut| / 127;  q = int8(round_half_even(clamp(lut / scale, -128, 127))).
//
// One wave computes a 16-centroid x 64-column tile of one codebook with v_mfma_f32_16x16x4_f32
// (K = 4 matches sub_vec_len 4 in one step; other v loop/zero-pad).  The work is tiny
// (2*C*K*M flop) and the kernel is bound by reading W and writing the LUT once.
#include "pimdl_internal.h"

namespace pimdl {

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int LG_WAVES = 4;
constexpr int LG_FT = 4;  // 16-column tiles per wave

__global__ __launch_bounds__(LG_WAVES * 64) void lutgen_f32_kernel(const float* __restrict__ cent,
                                                                  const float* __restrict__ W,
                                                                  float* __restrict__ lut, uint32_t CB,
                                                                  uint32_t C, uint32_t v, uint32_t M)
{
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t j = lane & 15, k = lane >> 4;
    const uint32_t cb = blockIdx.z;
    const uint32_t c0 = blockIdx.y * 16;
    const uint32_t f0 = (blockIdx.x * LG_WAVES + wave) * (16 * LG_FT);
    if (f0 >= M) return;  // whole wave

    v4f acc[LG_FT];
#pragma unroll
    for (int t = 0; t < LG_FT; ++t) acc[t] = (v4f){0.f, 0.f, 0.f, 0.f};

    for (uint32_t t0 = 0; t0 < v; t0 += 4) {
        const uint32_t t = t0 + k;
        // A[i = centroid c0 + j][k = t]
        float a = 0.0f;
        if (c0 + j < C && t < v) a = cent[((size_t)cb * C + c0 + j) * v + t];
#pragma unroll
        for (int ft = 0; ft < LG_FT; ++ft) {
            const uint32_t f = f0 + ft * 16 + j;
            float b = 0.0f;
            if (t < v && f < M) b = W[((size_t)cb * v + t) * M + f];
            acc[ft] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[ft], 0, 0, 0);
        }
    }
    // D[i = 4*k + r][j]: centroid c0 + 4k + r, column f0 + ft*16 + j
#pragma unroll
    for (int ft = 0; ft < LG_FT; ++ft) {
        const uint32_t f = f0 + ft * 16 + j;
        if (f >= M) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t c = c0 + 4 * k + r;
            if (c < C) lut[((size_t)cb * C + c) * M + f] = acc[ft][r];
        }
    }
}

// The same product with the v terms of every entry added in ascending order, each multiplication and each
// addition rounded on its own, starting from 0.0f: the order in which a plain loop over the sub-vector runs
// on a CPU.  torch.bmm fixes no order (pim_weight_converter.py:86-90 leaves it to the library), so neither
// form is "the" reference result; this one makes a converter's output reproducible bit for bit by scalar code.
// One thread = one output column of one codebook, all C centroids: W is read once, the LUT written once.
__global__ __launch_bounds__(256) void lutgen_ordered_kernel(const float* __restrict__ cent, const float* __restrict__ W,
                                                           float* __restrict__ lut, uint32_t C, uint32_t v, uint32_t M)
{
    const uint32_t f = blockIdx.x * blockDim.x + threadIdx.x, cb = blockIdx.y;
    if (f >= M) return;
    const float* w = W + (size_t)cb * v * M + f;
    for (uint32_t c = 0; c < C; ++c) {
        const float* a = cent + ((size_t)cb * C + c) * v;
        float acc = 0.0f;
        for (uint32_t t = 0; t < v; ++t) acc = __fadd_rn(acc, __fmul_rn(a[t], w[(size_t)t * M]));
        lut[((size_t)cb * C + c) * M + f] = acc;
    }
}

// max |x| per scale group; non-negative floats order like their bit patterns
__global__ void absmax_kernel(const float* __restrict__ lut, uint32_t* __restrict__ absmax_bits,
                              uint64_t group_elems, uint64_t total)
{
    const uint64_t grp = blockIdx.y;
    const uint64_t beg = grp * group_elems;
    const uint64_t end = beg + group_elems < total ? beg + group_elems : total;
    float m = 0.0f;
    for (uint64_t i = beg + (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < end;
         i += (uint64_t)gridDim.x * blockDim.x)
        m = fmaxf(m, fabsf(lut[i]));
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
    if ((threadIdx.x & 63) == 0) atomicMax(&absmax_bits[grp], __float_as_uint(m));
}

__global__ void quant_kernel(const float* __restrict__ lut, int8_t* __restrict__ q,
                             const uint32_t* __restrict__ absmax_bits, float* __restrict__ scales,
                             uint64_t group_elems, uint64_t total)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const uint64_t grp = i / group_elems;
    float scale = __fdiv_rn(__uint_as_float(absmax_bits[grp]), 127.0f);
    if (!(scale > 0.0f)) scale = 1.0f;  // all-zero group: any scale represents it
    if (i % group_elems == 0) scales[grp] = scale;
    float t = __fdiv_rn(lut[i], scale);
    t = fminf(fmaxf(t, -128.0f), 127.0f);
    q[i] = (int8_t)rintf(t);  // round half to even
}

// ---- diagnostics: a plain copy (HBM) and a ds_read_b128 loop (LDS) ------------------------------
__global__ void copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, uint64_t n16)
{
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (uint64_t)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

typedef int v4i __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(1024) void lds_read_kernel(int* __restrict__ sink, int iters)
{
    __shared__ __attribute__((aligned(16))) int buf[16384];
    for (int i = threadIdx.x; i < 16384; i += blockDim.x) buf[i] = i;
    __syncthreads();
    const uint32_t addr = (threadIdx.x & 63) * 16;  // 64 lanes x 16 B: contiguous, conflict-free
    v4i s = {0, 0, 0, 0};
    for (int it = 0; it < iters; ++it) {
        v4i r0, r1, r2, r3, r4, r5, r6, r7;
        asm volatile(
            "ds_read_b128 %0, %8\n ds_read_b128 %1, %8 offset:4096\n ds_read_b128 %2, %8 offset:8192\n"
            "ds_read_b128 %3, %8 offset:12288\n ds_read_b128 %4, %8 offset:16384\n"
            "ds_read_b128 %5, %8 offset:20480\n ds_read_b128 %6, %8 offset:24576\n"
            "ds_read_b128 %7, %8 offset:28672\n s_waitcnt lgkmcnt(0)"
            : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3), "=&v"(r4), "=&v"(r5), "=&v"(r6), "=&v"(r7)
            : "v"(addr));
        s += r0 + r1 + r2 + r3 + r4 + r5 + r6 + r7;
    }
    sink[blockIdx.x * blockDim.x + threadIdx.x] = s.x + s.y + s.z + s.w;
}

}  // namespace

int launch_lutgen_f32(Ctx* ctx, const float* d_cent, const float* d_w, float* d_lut, uint32_t CB, uint32_t C,
                      uint32_t v, uint32_t M, bool ordered)
{
    if (ordered) {
        hipLaunchKernelGGL(lutgen_ordered_kernel, dim3((M + 255) / 256, CB), dim3(256), 0, ctx->stream, d_cent, d_w, d_lut, C, v, M);
        return hip_check(ctx, hipGetLastError(), "lutgen_ordered_kernel launch");
    }
    dim3 grid((M + LG_WAVES * 16 * LG_FT - 1) / (LG_WAVES * 16 * LG_FT), (C + 15) / 16, CB);
    hipLaunchKernelGGL(lutgen_f32_kernel, grid, dim3(LG_WAVES * 64), 0, ctx->stream, d_cent, d_w, d_lut, CB, C, v, M);
    return hip_check(ctx, hipGetLastError(), "lutgen_f32_kernel launch");
}

int launch_lut_quant(Ctx* ctx, const float* d_lut, int8_t* d_q, float* d_scales, uint32_t CB, uint32_t C,
                     uint32_t M, uint32_t scale_group)
{
    const uint64_t total = (uint64_t)CB * C * M;
    const uint32_t ngroups = scale_group ? (CB + scale_group - 1) / scale_group : 1;
    const uint64_t group_elems = scale_group ? (uint64_t)scale_group * C * M : total;
    uint32_t* d_bits = nullptr;
    int rc = hip_check(ctx, hipMalloc(&d_bits, sizeof(uint32_t) * ngroups), "hipMalloc(absmax)");
    if (rc) return rc;
    rc = hip_check(ctx, hipMemsetAsync(d_bits, 0, sizeof(uint32_t) * ngroups, ctx->stream), "hipMemsetAsync(absmax)");
    if (!rc) {
        uint64_t bx = (group_elems + 256 * 16 - 1) / (256 * 16);
        if (bx > 1024) bx = 1024;
        if (bx < 1) bx = 1;
        hipLaunchKernelGGL(absmax_kernel, dim3((uint32_t)bx, ngroups), dim3(256), 0, ctx->stream, d_lut, d_bits,
                           group_elems, total);
        rc = hip_check(ctx, hipGetLastError(), "absmax_kernel launch");
    }
    if (!rc) {
        hipLaunchKernelGGL(quant_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, ctx->stream, d_lut, d_q,
                           d_bits, d_scales, group_elems, total);
        rc = hip_check(ctx, hipGetLastError(), "quant_kernel launch");
    }
    if (!rc) rc = hip_check(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize(quant)");
    (void)hipFree(d_bits);
    return rc;
}

int launch_diag(Ctx* ctx, uint64_t bytes, float* copy_gbps, float* lds_gbps)
{
    int rc = PIMDL_OK;
    if (copy_gbps) {
        const uint64_t n16 = bytes / 16;
        if (n16 == 0) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_diag_bandwidth: bytes < 16");
        uint4 *src = nullptr, *dst = nullptr;
        if ((rc = hip_check(ctx, hipMalloc(&src, n16 * 16), "hipMalloc(diag src)"))) return rc;
        if ((rc = hip_check(ctx, hipMalloc(&dst, n16 * 16), "hipMalloc(diag dst)"))) { (void)hipFree(src); return rc; }
        (void)hipMemsetAsync(src, 1, n16 * 16, ctx->stream);
        const uint32_t blocks = ctx->prop.multiProcessorCount * 8;
        for (int w = 0; w < 2; ++w) hipLaunchKernelGGL(copy_kernel, dim3(blocks), dim3(256), 0, ctx->stream, src, dst, n16);
        (void)hipEventRecord(ctx->ev[0], ctx->stream);
        const int reps = 10;
        for (int w = 0; w < reps; ++w) hipLaunchKernelGGL(copy_kernel, dim3(blocks), dim3(256), 0, ctx->stream, src, dst, n16);
        (void)hipEventRecord(ctx->ev[1], ctx->stream);
        rc = hip_check(ctx, hipEventSynchronize(ctx->ev[1]), "diag copy");
        float ms = 0;
        (void)hipEventElapsedTime(&ms, ctx->ev[0], ctx->ev[1]);
        *copy_gbps = ms > 0 ? (float)(2.0 * n16 * 16 * reps / (ms * 1e6)) : 0.f;  // read + write
        (void)hipFree(src);
        (void)hipFree(dst);
        if (rc) return rc;
    }
    if (lds_gbps) {
        const uint32_t blocks = ctx->prop.multiProcessorCount * 2, threads = 1024;
        int* sink = nullptr;
        if ((rc = hip_check(ctx, hipMalloc(&sink, (size_t)blocks * threads * 4), "hipMalloc(diag sink)"))) return rc;
        const int iters = 4000;
        hipLaunchKernelGGL(lds_read_kernel, dim3(blocks), dim3(threads), 0, ctx->stream, sink, iters);
        (void)hipEventRecord(ctx->ev[0], ctx->stream);
        hipLaunchKernelGGL(lds_read_kernel, dim3(blocks), dim3(threads), 0, ctx->stream, sink, iters);
        (void)hipEventRecord(ctx->ev[1], ctx->stream);
        rc = hip_check(ctx, hipEventSynchronize(ctx->ev[1]), "diag lds");
        float ms = 0;
        (void)hipEventElapsedTime(&ms, ctx->ev[0], ctx->ev[1]);
        *lds_gbps = ms > 0 ? (float)((double)blocks * threads * iters * 8 * 16 / (ms * 1e6)) : 0.f;
        (void)hipFree(sink);
    }
    return rc;
}

}  // namespace pimdl
