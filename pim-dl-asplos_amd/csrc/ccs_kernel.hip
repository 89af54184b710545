// Closest-centroid search for gfx950 (MI355X).
//
// Replaces index_calculation of the reference (inference-engine/src/host/index_calc_host.cpp:8-53).
// The result must be bit-identical to that CPU code, which fixes three things:
//   * distances are accumulated per dimension in ascending order from 0.0f with separately
//     rounded fp32 subtract, multiply and add (the reference's x86-64 build has no FMA);
//   * the "argmin" is the reference's sequential scan with a 1e-6 hysteresis
//     (index_calc_host.cpp:30-39), which is order dependent and is NOT a true argmin, so it is
//     replayed in centroid order by the lane that owns the (token, codebook) pair rather than
//     reduced across lanes;
//   * the compare `(double)(best - d) > 1e-6` equals the fp32 compare `(best - d) > 1e-6f`,
//     because (float)1e-6 < 1e-6 < nextafter((float)1e-6).
//
// Mapping.  One lane owns one token; a workgroup of 256 lanes owns 256 tokens x CBT codebooks.
// The activation tile is loaded from HBM with fully coalesced 16-byte loads, transposed through
// LDS (row pitch padded by 16 B so the per-lane 16-byte reads hit distinct banks), and each lane
// keeps its row slice in registers.  Centroids are wave-uniform, so the compiler fetches them with
// scalar loads and feeds them to the VALU as SGPR operands: no VGPRs, no LDS traffic for them.
// Indices leave packed (4 bits when C <= 16, else 8) so the gather reads them once.
#include "pimdl_internal.h"

namespace pimdl {

namespace {

template <int V>
struct CcsShape {
    static constexpr int ROW_FLOATS = (2 * V > 32) ? 2 * V : 32;  // floats of one token per tile
    static constexpr int CBT = ROW_FLOATS / V;                    // codebooks per workgroup
    static constexpr int PITCH = ROW_FLOATS + 4;                  // floats; +16 B: conflict-free b128
};

constexpr int CCS_THREADS = 256;

template <int V, int IDX_BITS>
__global__ __launch_bounds__(CCS_THREADS) void ccs_kernel(const float* __restrict__ x,
                                                         const float* __restrict__ cent,
                                                         uint8_t* __restrict__ idx, uint32_t N,
                                                         uint32_t K, uint32_t CB, uint32_t C,
                                                         uint32_t idx_row_bytes, int vec_ok)
{
    using S = CcsShape<V>;
    constexpr int RF = S::ROW_FLOATS, CBT = S::CBT, PITCH = S::PITCH;
    __shared__ __attribute__((aligned(16))) float tile[CCS_THREADS * PITCH];

    const uint32_t tok0 = blockIdx.x * CCS_THREADS;
    const uint32_t cb0 = blockIdx.y * CBT;
    const uint32_t col0 = cb0 * V;

    // ---- stage the [256 tokens][RF floats] tile, coalesced along the row --------------------
    constexpr int F4_PER_ROW = RF / 4;
    constexpr int ROWS_PER_PASS = CCS_THREADS / F4_PER_ROW;
    {
        const uint32_t q = threadIdx.x % F4_PER_ROW;
        const uint32_t r0 = threadIdx.x / F4_PER_ROW;
#pragma unroll 4
        for (uint32_t r = r0; r < CCS_THREADS; r += ROWS_PER_PASS) {
            uint32_t tok = tok0 + r;
            if (tok >= N) tok = N - 1;  // rows past N repeat the last token; never stored
            const uint32_t col = col0 + 4 * q;
            float4 val;
            const float* src = x + (size_t)tok * K + col;
            if (vec_ok && col + 4 <= K) {
                val = *reinterpret_cast<const float4*>(src);
            } else {
                val.x = (col + 0 < K) ? src[0] : 0.0f;
                val.y = (col + 1 < K) ? src[1] : 0.0f;
                val.z = (col + 2 < K) ? src[2] : 0.0f;
                val.w = (col + 3 < K) ? src[3] : 0.0f;
            }
            *reinterpret_cast<float4*>(&tile[r * PITCH + 4 * q]) = val;
        }
    }
    __syncthreads();

    // ---- each lane takes its own row into registers --------------------------------------------
    float xv[RF];
#pragma unroll
    for (int i = 0; i < RF / 4; ++i) {
        float4 t4 = *reinterpret_cast<const float4*>(&tile[threadIdx.x * PITCH + 4 * i]);
        xv[4 * i + 0] = t4.x;
        xv[4 * i + 1] = t4.y;
        xv[4 * i + 2] = t4.z;
        xv[4 * i + 3] = t4.w;
    }

    // ---- distance + hysteresis scan, centroid order, one codebook after the other ----------
    constexpr int OUT_BITS = CBT * IDX_BITS;
    constexpr int OUT_WORDS = (OUT_BITS + 31) / 32;
    uint32_t packed[OUT_WORDS];
#pragma unroll
    for (int i = 0; i < OUT_WORDS; ++i) packed[i] = 0;

#pragma unroll
    for (int cbl = 0; cbl < CBT; ++cbl) {
        const uint32_t cb = cb0 + cbl;
        uint32_t bi = 0;
        if (cb < CB) {  // wave-uniform
            const float* __restrict__ cp = cent + (size_t)cb * C * V;
            float best = 0.0f;
#pragma unroll 4
            for (uint32_t c = 0; c < C; ++c) {
                // d = ((0 + d0*d0) + d1*d1) + ... ; 0.0f + p == p exactly for every p >= 0
                float diff = __fsub_rn(xv[cbl * V + 0], cp[c * V + 0]);
                float d = __fmul_rn(diff, diff);
#pragma unroll
                for (int t = 1; t < V; ++t) {
                    diff = __fsub_rn(xv[cbl * V + t], cp[c * V + t]);
                    d = __fadd_rn(d, __fmul_rn(diff, diff));
                }
                const bool take = (c == 0) || (__fsub_rn(best, d) > 1e-6f);
                best = take ? d : best;
                bi = take ? c : bi;
            }
        }
        constexpr int per_word = 32 / IDX_BITS;
        packed[cbl / per_word] |= bi << (IDX_BITS * (cbl % per_word));
    }

    // ---- packed store -----------------------------------------------------------------------
    const uint32_t tok = tok0 + threadIdx.x;
    if (tok < N) {
        uint8_t* dst = idx + (size_t)tok * idx_row_bytes + (size_t)cb0 * IDX_BITS / 8;
        if constexpr (OUT_BITS >= 128) {
            *reinterpret_cast<uint4*>(dst) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
        } else if constexpr (OUT_BITS == 64) {
            *reinterpret_cast<uint2*>(dst) = make_uint2(packed[0], packed[1]);
        } else if constexpr (OUT_BITS == 32) {
            *reinterpret_cast<uint32_t*>(dst) = packed[0];
        } else if constexpr (OUT_BITS == 16) {
            *reinterpret_cast<uint16_t*>(dst) = (uint16_t)packed[0];
        } else {
            static_assert(OUT_BITS == 8, "unexpected packing");
            *dst = (uint8_t)packed[0];
        }
    }
}

// Generic sub-vector length (any v): one lane per (token, codebook), operands straight from
// global memory.  Correct for every shape; only used where no specialisation exists.
template <int IDX_BITS>
__global__ __launch_bounds__(256) void ccs_generic_kernel(const float* __restrict__ x,
                                                         const float* __restrict__ cent,
                                                         uint8_t* __restrict__ idx, uint32_t N,
                                                         uint32_t K, uint32_t v, uint32_t CB,
                                                         uint32_t CB_pad, uint32_t C,
                                                         uint32_t idx_row_bytes)
{
    // a lane produces one whole output byte (two codebooks when IDX_BITS == 4)
    constexpr int CB_PER_BYTE = 8 / IDX_BITS;
    const uint32_t bytes_per_row = CB_pad / CB_PER_BYTE;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)N * bytes_per_row) return;
    const uint32_t tok = gid / bytes_per_row;
    const uint32_t byte = gid % bytes_per_row;
    uint32_t outv = 0;
    for (int h = 0; h < CB_PER_BYTE; ++h) {
        const uint32_t cb = byte * CB_PER_BYTE + h;
        uint32_t bi = 0;
        if (cb < CB) {
            const float* xs = x + (size_t)tok * K + (size_t)cb * v;
            const float* cp = cent + (size_t)cb * C * v;
            float best = 0.0f;
            for (uint32_t c = 0; c < C; ++c) {
                float d = 0.0f;
                for (uint32_t t = 0; t < v; ++t) {
                    const float diff = __fsub_rn(xs[t], cp[c * v + t]);
                    d = __fadd_rn(d, __fmul_rn(diff, diff));
                }
                const bool take = (c == 0) || (__fsub_rn(best, d) > 1e-6f);
                best = take ? d : best;
                bi = take ? c : bi;
            }
        }
        outv |= bi << (IDX_BITS * h);
    }
    idx[(size_t)tok * idx_row_bytes + byte] = (uint8_t)outv;
}

// packed indices -> uint16 at the reference's tiled offset (index_calc_host.cpp:41-49)
template <int IDX_BITS>
__global__ void unpack_idx_kernel(const uint8_t* __restrict__ idx, uint16_t* __restrict__ out,
                                  uint32_t N, uint32_t CB, uint32_t idx_row_bytes, uint32_t n_stile,
                                  uint32_t cb_mtile)
{
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)N * CB) return;
    const uint32_t n = gid / CB, cb = gid % CB;
    const uint8_t b = idx[(size_t)n * idx_row_bytes + (size_t)cb * IDX_BITS / 8];
    const uint16_t val = (IDX_BITS == 4) ? ((b >> (4 * (cb & 1))) & 0xF) : b;
    const uint64_t off = (uint64_t)(n / n_stile) * n_stile * CB + (uint64_t)(cb / cb_mtile) * n_stile * cb_mtile +
                         (uint64_t)(n % n_stile) * cb_mtile + (cb % cb_mtile);
    out[off] = val;
}

// uint16 centroid ids at the reference's tiled offset -> packed rows (padded codebooks get index 0)
template <int IDX_BITS>
__global__ void pack_idx_kernel(const uint16_t* __restrict__ in, uint8_t* __restrict__ idx, uint32_t N,
                                uint32_t CB, uint32_t idx_row_bytes, uint32_t n_stile, uint32_t cb_mtile)
{
    constexpr int CB_PER_BYTE = 8 / IDX_BITS;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)N * idx_row_bytes) return;
    const uint32_t n = gid / idx_row_bytes, byte = gid % idx_row_bytes;
    uint32_t outv = 0;
    for (int h = 0; h < CB_PER_BYTE; ++h) {
        const uint32_t cb = byte * CB_PER_BYTE + h;
        if (cb < CB) {
            const uint64_t off = (uint64_t)(n / n_stile) * n_stile * CB + (uint64_t)(cb / cb_mtile) * n_stile * cb_mtile +
                                 (uint64_t)(n % n_stile) * cb_mtile + (cb % cb_mtile);
            outv |= (uint32_t)(in[off] & ((1u << IDX_BITS) - 1)) << (IDX_BITS * h);
        }
    }
    idx[gid] = (uint8_t)outv;
}

template <int V, int IDX_BITS>
int launch_ccs_t(Ctx* ctx, const AmmGeom& g, const float* d_x, const float* d_cent, uint8_t* d_idx, uint32_t n)
{
    using S = CcsShape<V>;
    dim3 grid((n + CCS_THREADS - 1) / CCS_THREADS, g.CB_pad / S::CBT);
    const int vec_ok = (g.K % 4 == 0) && ((reinterpret_cast<uintptr_t>(d_x) & 15) == 0);
    hipLaunchKernelGGL((ccs_kernel<V, IDX_BITS>), grid, dim3(CCS_THREADS), 0, ctx->stream, d_x, d_cent, d_idx, n,
                       g.K, g.CB, g.C, g.idx_row_bytes, vec_ok);
    return hip_check(ctx, hipGetLastError(), "ccs_kernel launch");
}

template <int IDX_BITS>
int launch_ccs_bits(Ctx* ctx, const AmmGeom& g, const float* d_x, const float* d_cent, uint8_t* d_idx, uint32_t n)
{
    switch (g.v) {
        case 2: return launch_ccs_t<2, IDX_BITS>(ctx, g, d_x, d_cent, d_idx, n);
        case 4: return launch_ccs_t<4, IDX_BITS>(ctx, g, d_x, d_cent, d_idx, n);
        case 8: return launch_ccs_t<8, IDX_BITS>(ctx, g, d_x, d_cent, d_idx, n);
        case 16: return launch_ccs_t<16, IDX_BITS>(ctx, g, d_x, d_cent, d_idx, n);
        case 32: return launch_ccs_t<32, IDX_BITS>(ctx, g, d_x, d_cent, d_idx, n);
        default: {
            const uint64_t total = (uint64_t)n * (g.CB_pad / (8 / IDX_BITS));
            dim3 grid((uint32_t)((total + 255) / 256));
            hipLaunchKernelGGL((ccs_generic_kernel<IDX_BITS>), grid, dim3(256), 0, ctx->stream, d_x, d_cent, d_idx,
                               n, g.K, g.v, g.CB, g.CB_pad, g.C, g.idx_row_bytes);
            return hip_check(ctx, hipGetLastError(), "ccs_generic_kernel launch");
        }
    }
}

}  // namespace

uint32_t ccs_cb_per_wg(uint32_t v)
{
    switch (v) {
        case 2: return CcsShape<2>::CBT;
        case 4: return CcsShape<4>::CBT;
        case 8: return CcsShape<8>::CBT;
        case 16: return CcsShape<16>::CBT;
        case 32: return CcsShape<32>::CBT;
        default: return 0;
    }
}

int launch_ccs(Ctx* ctx, const AmmGeom& g, const float* d_x, const float* d_cent, uint8_t* d_idx, uint32_t n)
{
    if (n == 0) return PIMDL_OK;
    return g.idx_bits == 4 ? launch_ccs_bits<4>(ctx, g, d_x, d_cent, d_idx, n)
                           : launch_ccs_bits<8>(ctx, g, d_x, d_cent, d_idx, n);
}

int launch_unpack_idx(Ctx* ctx, const AmmGeom& g, const uint8_t* d_idx, uint16_t* d_idx16, uint32_t n,
                      uint32_t n_stile, uint32_t cb_mtile)
{
    if (n == 0) return PIMDL_OK;
    const uint64_t total = (uint64_t)n * g.CB;
    dim3 grid((uint32_t)((total + 255) / 256));
    if (g.idx_bits == 4)
        hipLaunchKernelGGL((unpack_idx_kernel<4>), grid, dim3(256), 0, ctx->stream, d_idx, d_idx16, n, g.CB,
                           g.idx_row_bytes, n_stile, cb_mtile);
    else
        hipLaunchKernelGGL((unpack_idx_kernel<8>), grid, dim3(256), 0, ctx->stream, d_idx, d_idx16, n, g.CB,
                           g.idx_row_bytes, n_stile, cb_mtile);
    return hip_check(ctx, hipGetLastError(), "unpack_idx_kernel launch");
}

int launch_pack_idx(Ctx* ctx, const AmmGeom& g, const uint16_t* d_idx16, uint8_t* d_idx, uint32_t n,
                    uint32_t n_stile, uint32_t cb_mtile)
{
    if (n == 0) return PIMDL_OK;
    const uint64_t total = (uint64_t)n * g.idx_row_bytes;
    dim3 grid((uint32_t)((total + 255) / 256));
    if (g.idx_bits == 4)
        hipLaunchKernelGGL((pack_idx_kernel<4>), grid, dim3(256), 0, ctx->stream, d_idx16, d_idx, n, g.CB,
                           g.idx_row_bytes, n_stile, cb_mtile);
    else
        hipLaunchKernelGGL((pack_idx_kernel<8>), grid, dim3(256), 0, ctx->stream, d_idx16, d_idx, n, g.CB,
                           g.idx_row_bytes, n_stile, cb_mtile);
    return hip_check(ctx, hipGetLastError(), "pack_idx_kernel launch");
}

namespace {
// row-major [N][M] -> the order the reference's DPUs hand the output back in (test_amm.cpp:193-202)
__global__ void retile_output_kernel(const float* __restrict__ in, float* __restrict__ out, uint32_t N, uint32_t M,
                                     uint32_t n_stile, uint32_t f_stile, uint32_t f_mtile)
{
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)N * M) return;
    const uint32_t n = gid / M, f = gid % M;
    const uint64_t dpu = (uint64_t)(n / n_stile) * (M / f_stile) + f / f_stile;
    const uint32_t row = n % n_stile, dim = f % f_stile;
    const uint64_t off = dpu * n_stile * f_stile + (uint64_t)(dim / f_mtile) * n_stile * f_mtile +
                         (uint64_t)row * f_mtile + dim % f_mtile;
    out[off] = in[gid];
}
}  // namespace

int launch_retile_output(Ctx* ctx, const float* d_rowmajor, float* d_tiled, uint32_t n, uint32_t M, uint32_t n_stile,
                         uint32_t f_stile, uint32_t f_mtile)
{
    if (n == 0) return PIMDL_OK;
    const uint64_t total = (uint64_t)n * M;
    hipLaunchKernelGGL(retile_output_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, ctx->stream,
                       d_rowmajor, d_tiled, n, M, n_stile, f_stile, f_mtile);
    return hip_check(ctx, hipGetLastError(), "retile_output_kernel launch");
}

}  // namespace pimdl
