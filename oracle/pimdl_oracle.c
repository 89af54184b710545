/*
 * pimdl_oracle.c -- CPU restatement of PIM-DL's LUT-based approximate matrix multiply.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP path is compared against
 * (tests, the smoke check, and the cpu_baseline leg of the benchmark).  Nothing that ships
 * links, imports or calls it; the product path has no CPU fallback.
 *
 * Each function cites the reference file:line it follows (paths under the reference tree).
 * Build: see oracle/Makefile -- flags mirror the reference's host library
 * (inference-engine/src/host/CMakeLists.txt:1: -O3, no -march, no fast-math) plus
 * -ffp-contract=off so that no fused multiply-add is ever formed, on any host.
 *
 * How each function is pinned (what its tests check it against):
 *   oracle_index_calculation  -- the reference's own index_calc_host.cpp compiled from source
 *                                (oracle/_ref), golden fixtures made from it, closed forms
 *                                (scan-vs-true-argmin chains), brute force.
 *   oracle_gather_i8          -- integer one-hot matmul in numpy; LUT==1 => acc==CB;
 *                                codebook-permutation invariance.
 *   oracle_dequant            -- closed form (one line of numpy).
 *   oracle_gather_f32         -- fp64 numpy gather within 1e-6; order fixed ascending-cb.
 *   oracle_lutgen_f32         -- numpy einsum (library routine) within fp32 rounding.
 *   oracle_lut_quant          -- numpy restatement of the published formula
 *                                (torch.clamp -> round-half-even -> int8), invariants.
 *   oracle_gather_i8_grouped  -- extension absent from the reference (per-codebook-group
 *                                scale): "parity unpinned by the reference"; pinned only by
 *                                numpy restatement and by group==CB reducing to per-tensor.
 *   layout helpers            -- bijection checks + identity tiling == row-major.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

static int clamp_threads(int t) { return t < 1 ? 1 : t; }

/* ------------------------------------------------------------------------------------------
 * A1. Closest-centroid search.
 * Follows inference-engine/src/host/index_calc_host.cpp:8-53 (same arithmetic as
 * inference-engine/test/test_amm.cpp:134-159):
 *   dist[c] = sum over t (ascending, from 0.0f) of (x - cent) * (x - cent), fp32, no FMA;
 *   scan: best = dist[0]; for c = 1..C-1: if ((best - dist[c]) > 1e-6) take c.
 * The compare promotes the fp32 difference to double against the double literal 1e-6
 * (index_calc_host.cpp:34); it is kept in that form here.
 * Output position follows index_calc_host.cpp:41-49 (DPU tile order); n_stile == N and
 * cb_mtile == CB give row-major [N][CB].
 * ---------------------------------------------------------------------------------------- */
ORACLE_API void oracle_index_calculation(const float *x, const float *cent, uint16_t *idx_out,
                                         uint32_t N, uint32_t K, uint32_t v, uint32_t CB,
                                         uint32_t C, uint32_t n_stile, uint32_t cb_mtile,
                                         int threads)
{
    threads = clamp_threads(threads);
#pragma omp parallel for num_threads(threads) schedule(static)
    for (uint32_t n = 0; n < N; ++n) {
        float *dist = (float *)malloc(sizeof(float) * C);
        for (uint32_t cb = 0; cb < CB; ++cb) {
            const float *xs = x + (size_t)n * K + (size_t)v * cb;
            const float *cs = cent + (size_t)cb * C * v;
            for (uint32_t c = 0; c < C; ++c) {
                float d = 0;
                for (uint32_t t = 0; t < v; ++t) {
                    float diff = xs[t] - cs[c * v + t];
                    d += diff * diff;
                }
                dist[c] = d;
            }
            float best = dist[0];
            uint16_t bi = 0;
            for (uint32_t c = 1; c < C; ++c) {
                if ((best - dist[c]) > 1e-6) {
                    best = dist[c];
                    bi = (uint16_t)c;
                }
            }
            uint32_t nt = n / n_stile, ni = n % n_stile;
            uint32_t ct = cb / cb_mtile, ci = cb % cb_mtile;
            size_t off = (size_t)nt * n_stile * CB + (size_t)ct * n_stile * cb_mtile +
                         (size_t)ni * cb_mtile + ci;
            idx_out[off] = bi;
        }
        free(dist);
    }
}

/* Distances only (for tests that build adversarial near-tie cases). Same arithmetic as above. */
ORACLE_API void oracle_distances(const float *x, const float *cent, float *dist_out, uint32_t N,
                                 uint32_t K, uint32_t v, uint32_t CB, uint32_t C)
{
    for (uint32_t n = 0; n < N; ++n)
        for (uint32_t cb = 0; cb < CB; ++cb)
            for (uint32_t c = 0; c < C; ++c) {
                float d = 0;
                for (uint32_t t = 0; t < v; ++t) {
                    float diff = x[(size_t)n * K + v * cb + t] - cent[((size_t)cb * C + c) * v + t];
                    d += diff * diff;
                }
                dist_out[((size_t)n * CB + cb) * C + c] = d;
            }
}

/* ------------------------------------------------------------------------------------------
 * A3. Gather-accumulate, int8 table, int32 accumulator.
 * Follows inference-engine/test/test_amm.cpp:164-175 (the canonical row-major statement of
 * what the DPU kernel inference-engine/src/dpu/pim_lut_kernel.c:97-2296 computes).
 * idx row-major [N][CB]; lut [CB][C][M]; acc [N][M].
 * ---------------------------------------------------------------------------------------- */
ORACLE_API void oracle_gather_i8(const uint16_t *idx, const int8_t *lut, int32_t *acc, uint32_t N,
                                 uint32_t CB, uint32_t C, uint32_t M, int threads)
{
    threads = clamp_threads(threads);
#pragma omp parallel for num_threads(threads) schedule(static)
    for (uint32_t n = 0; n < N; ++n) {
        int32_t *row = acc + (size_t)n * M;
        memset(row, 0, sizeof(int32_t) * M);
        for (uint32_t cb = 0; cb < CB; ++cb) {
            const int8_t *src = lut + ((size_t)cb * C + idx[(size_t)n * CB + cb]) * M;
            for (uint32_t f = 0; f < M; ++f)
                row[f] += src[f];
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * A4. De-quantisation epilogue.
 * bias_mode 0 follows inference-engine/test/test_amm.cpp:178-181:
 *     out = acc*scale + lut_bias + bias_tensor[f]
 * bias_mode 1 follows inference-engine/src/host/pim_lut_host.cpp:201:
 *     out = acc*scale + lut_bias*num_codebook + bias_tensor[f]
 * Both evaluate left to right in fp32.  They agree when lut_bias == 0, which is all the
 * reference's converter ever writes (model-calibration/pim_weight_converter.py:27,34).
 * ---------------------------------------------------------------------------------------- */
ORACLE_API void oracle_dequant(const int32_t *acc, const float *bias_tensor, float *out, uint32_t N,
                               uint32_t M, uint32_t CB, float scale, float lut_bias, int bias_mode,
                               int threads)
{
    threads = clamp_threads(threads);
#pragma omp parallel for num_threads(threads) schedule(static)
    for (uint32_t n = 0; n < N; ++n)
        for (uint32_t f = 0; f < M; ++f) {
            size_t o = (size_t)n * M + f;
            if (bias_mode == 0)
                out[o] = acc[o] * scale + lut_bias + bias_tensor[f];
            else
                out[o] = acc[o] * scale + lut_bias * CB + bias_tensor[f];
        }
}

/* ------------------------------------------------------------------------------------------
 * Whole AMM, row-major: inference-engine/test/test_amm.cpp:126-183 (amm_cpu).
 * idx_scratch [N][CB] u16 and acc_scratch [N][M] i32 are caller-provided so the timed
 * baseline does not measure malloc.
 * ---------------------------------------------------------------------------------------- */
ORACLE_API void oracle_amm_cpu(const float *x, const float *cent, const int8_t *lut,
                               const float *bias_tensor, float *out, uint16_t *idx_scratch,
                               int32_t *acc_scratch, uint32_t N, uint32_t K, uint32_t v, uint32_t C,
                               uint32_t M, float scale, float lut_bias, int threads)
{
    uint32_t CB = K / v;
    oracle_index_calculation(x, cent, idx_scratch, N, K, v, CB, C, N, CB, threads);
    oracle_gather_i8(idx_scratch, lut, acc_scratch, N, CB, C, M, threads);
    oracle_dequant(acc_scratch, bias_tensor, out, N, M, CB, scale, lut_bias, 0, threads);
}

/* ------------------------------------------------------------------------------------------
 * fp32-LUT gather: out[n][f] = (sum over cb ascending, fp32, from 0.0f) lut[cb][idx][f]
 *                              + bias_tensor[f]
 * Semantics from model-calibration/LUTNeuro/LUTLinear_t.py:77-78,85-86
 * (bmm(one_hot, lut).sum(0) + bias).  The reference does not fix a summation order; this
 * oracle fixes ascending cb, and parity is stated to 1e-5 relative.
 * ---------------------------------------------------------------------------------------- */
ORACLE_API void oracle_gather_f32(const uint16_t *idx, const float *lut, const float *bias_tensor,
                                  float *out, uint32_t N, uint32_t CB, uint32_t C, uint32_t M,
                                  int threads)
{
    threads = clamp_threads(threads);
#pragma omp parallel for num_threads(threads) schedule(static)
    for (uint32_t n = 0; n < N; ++n) {
        float *row = out + (size_t)n * M;
        for (uint32_t f = 0; f < M; ++f)
            row[f] = 0.0f;
        for (uint32_t cb = 0; cb < CB; ++cb) {
            const float *src = lut + ((size_t)cb * C + idx[(size_t)n * CB + cb]) * M;
            for (uint32_t f = 0; f < M; ++f)
                row[f] += src[f];
        }
        for (uint32_t f = 0; f < M; ++f)
            row[f] += bias_tensor[f];
    }
}

/* ------------------------------------------------------------------------------------------
 * Extension (NOT in the reference): int8 LUT with one fp32 scale per group of `group`
 * consecutive codebooks.  int32 accumulate inside a group, then
 *   out = (sum over groups ascending, fp32, from 0.0f) (float)acc_g * scale[g]  + bias_tensor[f]
 * group == CB with a single scale reproduces A3+A4 with lut_bias 0 up to the order of the
 * final additions.  Parity unpinned by the reference.
 * ---------------------------------------------------------------------------------------- */
ORACLE_API void oracle_gather_i8_grouped(const uint16_t *idx, const int8_t *lut, const float *scales,
                                         const float *bias_tensor, float *out, uint32_t N,
                                         uint32_t CB, uint32_t C, uint32_t M, uint32_t group,
                                         int threads)
{
    threads = clamp_threads(threads);
    uint32_t ngroups = (CB + group - 1) / group;
#pragma omp parallel for num_threads(threads) schedule(static)
    for (uint32_t n = 0; n < N; ++n) {
        int32_t *tmp = (int32_t *)malloc(sizeof(int32_t) * M);
        float *row = out + (size_t)n * M;
        for (uint32_t f = 0; f < M; ++f)
            row[f] = 0.0f;
        for (uint32_t g = 0; g < ngroups; ++g) {
            memset(tmp, 0, sizeof(int32_t) * M);
            uint32_t cb_end = (g + 1) * group < CB ? (g + 1) * group : CB;
            for (uint32_t cb = g * group; cb < cb_end; ++cb) {
                const int8_t *src = lut + ((size_t)cb * C + idx[(size_t)n * CB + cb]) * M;
                for (uint32_t f = 0; f < M; ++f)
                    tmp[f] += src[f];
            }
            for (uint32_t f = 0; f < M; ++f)
                row[f] += (float)tmp[f] * scales[g];
        }
        for (uint32_t f = 0; f < M; ++f)
            row[f] += bias_tensor[f];
        free(tmp);
    }
}

/* ------------------------------------------------------------------------------------------
 * A5a. LUT construction: lut[cb][c][f] = sum over t ascending of cent[cb][c][t] * W[cb*v+t][f]
 * Follows model-calibration/pim_weight_converter.py:86-90 (torch.bmm of centroids.view(CB,C,v)
 * with weight.view(CB,v,M)).  W is [K][M] (the transposed nn.Linear weight,
 * model-calibration/LUTNeuro/LUTLinear_t.py:36).  torch.bmm's internal summation order is a
 * library detail; this oracle uses ascending t with separate multiply and add, and parity of
 * the fp32 LUT is stated to 1e-5 relative.
 * ---------------------------------------------------------------------------------------- */
ORACLE_API void oracle_lutgen_f32(const float *cent, const float *W, float *lut, uint32_t CB,
                                  uint32_t C, uint32_t v, uint32_t M, int threads)
{
    threads = clamp_threads(threads);
#pragma omp parallel for num_threads(threads) schedule(static)
    for (uint32_t cb = 0; cb < CB; ++cb)
        for (uint32_t c = 0; c < C; ++c) {
            float *dst = lut + ((size_t)cb * C + c) * M;
            for (uint32_t f = 0; f < M; ++f)
                dst[f] = 0.0f;
            for (uint32_t t = 0; t < v; ++t) {
                float a = cent[((size_t)cb * C + c) * v + t];
                const float *w = W + ((size_t)cb * v + t) * M;
                for (uint32_t f = 0; f < M; ++f)
                    dst[f] += a * w[f];
            }
        }
}

/* ------------------------------------------------------------------------------------------
 * A5b. LUT quantisation.  Follows model-calibration/pim_weight_converter.py:21-35:
 *   max_abs = max(|min|, |max|) over the whole tensor; scale = max_abs / 127 (zero point 0);
 *   q = int8(round_half_even(clamp(lut / scale, -128, 127)));  bias = -scale*0 = 0.
 * group_rows == 0: one scale for the whole tensor (the reference).  group_rows > 0
 * (extension, not in the reference): one scale per block of group_rows consecutive LUT rows,
 * i.e. per group of group_rows/C codebooks.  An all-zero block gets scale 1 (the reference
 * would divide by zero; its converter never meets that case).
 * rows = CB*C, cols = M.  scales_out has 1 or ceil(rows/group_rows) entries.
 * ---------------------------------------------------------------------------------------- */
ORACLE_API void oracle_lut_quant(const float *lut, int8_t *q, float *scales_out, uint64_t rows,
                                 uint64_t cols, uint64_t group_rows)
{
    if (group_rows == 0 || group_rows > rows)
        group_rows = rows;
    uint64_t g = 0;
    for (uint64_t r0 = 0; r0 < rows; r0 += group_rows, ++g) {
        uint64_t r1 = r0 + group_rows < rows ? r0 + group_rows : rows;
        float mn = lut[r0 * cols], mx = lut[r0 * cols];
        for (uint64_t i = r0 * cols; i < r1 * cols; ++i) {
            if (lut[i] < mn) mn = lut[i];
            if (lut[i] > mx) mx = lut[i];
        }
        float max_abs = fmaxf(fabsf(mn), fabsf(mx));
        float scale = max_abs / 127.0f;
        if (!(scale > 0.0f))
            scale = 1.0f;
        scales_out[g] = scale;
        for (uint64_t i = r0 * cols; i < r1 * cols; ++i) {
            float t = lut[i] / scale;
            t = t < -128.0f ? -128.0f : (t > 127.0f ? 127.0f : t);
            q[i] = (int8_t)nearbyintf(t); /* default rounding mode: to nearest, ties to even */
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * DPU layouts (only the source-compatible amm_host shim needs them).
 * ---------------------------------------------------------------------------------------- */

/* LUT [CB][C][M] -> [f_tile][CB][C][f_in_tile], tile = feature_load_tile_size (non-STATIC) or
 * feature_stile_size (STATIC): inference-engine/test/test_amm.cpp:71-121. */
ORACLE_API void oracle_reorder_pim_lut(const int8_t *cpu_lut, int8_t *dpu_lut, uint32_t CB,
                                       uint32_t C, uint32_t M, uint32_t ftile)
{
    for (uint32_t cb = 0; cb < CB; ++cb)
        for (uint32_t c = 0; c < C; ++c)
            for (uint32_t f = 0; f < M; ++f) {
                size_t src = ((size_t)cb * C + c) * M + f;
                size_t dst = (size_t)(f / ftile) * CB * C * ftile + (size_t)cb * C * ftile +
                             (size_t)c * ftile + (f % ftile);
                dpu_lut[dst] = cpu_lut[src];
            }
}

/* Offset of element (n, f) in the output buffer amm_host fills:
 * inference-engine/test/test_amm.cpp:193-202. */
ORACLE_API uint64_t oracle_output_offset(uint32_t n, uint32_t f, uint32_t n_stile, uint32_t f_stile,
                                         uint32_t f_mtile, uint32_t lut_parallelism)
{
    uint64_t dpu = (uint64_t)(n / n_stile) * lut_parallelism + f / f_stile;
    uint64_t row = n % n_stile, dim = f % f_stile;
    uint64_t mt = dim / f_mtile, in_mt = dim % f_mtile;
    return dpu * n_stile * f_stile + mt * n_stile * f_mtile + row * f_mtile + in_mt;
}

/* The in-place index rewrite pim_lut performs on the caller's index buffer before it sends it
 * to the DPUs: inference-engine/src/host/pim_lut_host.cpp:40-104.
 * load_type 0 STATIC (:59), 1 FINE_GRAIN (:80), 2 COARSE_GRAIN (:96-104).
 * idx is in the tiled order index_calculation wrote (index_calc_host.cpp:41-49). */
ORACLE_API void oracle_prepare_input_index(uint16_t *idx, uint32_t N, uint32_t CB, uint32_t C,
                                           uint32_t n_stile, uint32_t cb_mtile, int load_type,
                                           uint32_t f_stile, uint32_t f_load_tile,
                                           uint32_t cb_load_tile)
{
    for (uint32_t n = 0; n < N; ++n)
        for (uint32_t cb = 0; cb < CB; ++cb) {
            uint32_t ci = cb % cb_mtile;
            size_t off = (size_t)(n / n_stile) * n_stile * CB + (size_t)(cb / cb_mtile) * n_stile * cb_mtile +
                         (size_t)(n % n_stile) * cb_mtile + ci;
            if (load_type == 0)
                idx[off] = (uint16_t)(idx[off] * f_stile);
            else if (load_type == 1)
                idx[off] = (uint16_t)(idx[off] * f_load_tile);
            else
                idx[off] = (uint16_t)((ci % cb_load_tile) * C * f_load_tile + idx[off] * f_load_tile);
        }
}

/* ------------------------------------------------------------------------------------------
 * Layer norm as the reference's encoder layer applies it:
 * inference-engine/src/host/transformer_layer.cpp:50-90 -- per row: mean and variance with
 * double accumulators, eps 1e-6, y = (x-mean)/sqrt(var+eps) * gamma + beta.
 * (Used by the layer-level tests; not on the AMM path.)
 * ---------------------------------------------------------------------------------------- */
ORACLE_API void oracle_layer_norm(const float *x, const float *gamma, const float *beta, float *y,
                                  uint32_t N, uint32_t D)
{
    const float eps = 1e-6f;
    for (uint32_t n = 0; n < N; ++n) {
        const float *r = x + (size_t)n * D;
        double sum = 0.0;
        for (uint32_t i = 0; i < D; ++i)
            sum += (double)r[i];
        float mean = (float)(sum / D);
        double sum2 = 0.0;
        for (uint32_t i = 0; i < D; ++i) {
            float vv = r[i] - mean;
            y[(size_t)n * D + i] = vv;
            sum2 += (double)(vv * vv);
        }
        float var = (float)(sum2 / D);
        const float sc = 1.0f / sqrtf(var + eps);
        for (uint32_t i = 0; i < D; ++i)
            y[(size_t)n * D + i] = y[(size_t)n * D + i] * sc * gamma[i] + beta[i];
    }
}

ORACLE_API int oracle_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
