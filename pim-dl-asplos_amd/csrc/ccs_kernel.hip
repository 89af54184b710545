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
// Mapping.  One lane owns one token.  A workgroup of four waves owns a tile of 64 tokens x
// 4*CBT codebooks: wave w searches the w-th group of CBT codebooks for all 64 tokens.  A tile row
// is 512 contiguous bytes in HBM (v <= 16), loaded with coalesced 16-byte loads, transposed through
// LDS (row pitch padded by 16 B so the per-lane 16-byte reads hit distinct banks), and each lane
// keeps its 32-float row slice in registers.  Workgroups are persistent and fetch the next tile
// into registers before searching the current one.  In the exact scan centroids are wave-uniform
// and arrive as SGPR operands through scalar loads.
// Indices leave packed (4 bits when C <= 16, else 8) so the gather reads them once.
//
// Two-speed search.  The scan above costs 3v+3 VALU operations per centroid.  Almost every
// (token, codebook) pair has a nearest centroid that wins by far more than rounding error plus the
// 1e-6 hysteresis, and for those the scan returns the true nearest centroid whatever the order.  So
// each lane first evaluates the expanded form  |x|^2 + |c|^2 - 2 x.c  with FMAs (v+1 operations per
// centroid; -2c and |c|^2 are precomputed per operator and arrive as SGPR operands), keeps the two
// smallest values with the centroid id packed into the low mantissa bits (v_and_or, v_med3,
// v_min: 3 operations), and accepts the winner only when
//     second - best  >  2 * (error bound of both formulas + packing error) + 1e-6 .
// If any lane of the wave fails that test (near ties, non-finite data) the whole wave replays the
// reference's exact scan for that codebook, so the output is bit-identical in every case.
//
// Error bound.  u = 2^-24.  With XX = sum x_t^2, CN = sum c_t^2 and D the real-valued distance
// (D <= 2(XX+CN)): the reference chain has relative error <= (v+2)u, i.e. <= 2(v+2)u(XX+CN);
// the FMA form accumulates <= (3v+1)u(XX+CN) (v roundings in each of XX and CN, one for their sum,
// v for the FMAs whose partial sums stay below 2(XX+CN)).  Sum: (5v+5)u(XX+CN); the kernel uses
// three times that.  Packing the id into the low IDX_BITS bits moves a value by less than
// 2^IDX_BITS ulp, i.e. 2^(IDX_BITS-22) |value|, charged against the second-smallest value.
#include <math.h>
#include <string.h>

#include <vector>

#include "pimdl_internal.h"

#include <stdlib.h>

#include <type_traits>

namespace pimdl {

namespace {

template <int V>
struct CcsShape {
    // floats of one token per wave: 32, or 2 v above that, or 40 where v does not divide 32 (v = 10, 20)
    static constexpr int ROW_FLOATS = (32 % V != 0) ? 40 : (2 * V > 32) ? 2 * V : 32;
    static_assert(ROW_FLOATS % V == 0 && ROW_FLOATS % 4 == 0, "whole codebooks and whole 16-byte pieces per wave");
    static constexpr int CBT = ROW_FLOATS / V;                    // codebooks per workgroup
    static constexpr int WAVES = 4;                               // each wave: its own codebook group
    static constexpr int TILE_TOKENS = 64;                        // one token per lane
    static constexpr int PITCH = WAVES * ROW_FLOATS + 4;          // floats; +16 B: conflict-free b128
    static constexpr int LDS_BYTES = TILE_TOKENS * PITCH * 4;
};

constexpr int CCS_THREADS = 256;

inline size_t ccs_aux_floats(const AmmGeom& g)
{
    return (size_t)g.CB * (g.v + 1) * ((g.C + 15) / 16 * 16);
}

inline size_t ccs_aux_a_floats(const AmmGeom& g)
{
    return (size_t)(g.CB_pad / 2) * (g.v + 1) * 64 + g.CB_pad;  // A-operand images, padded cnmax
}

// bf16-split search (v = 4, C <= 16): offset in floats of its operands behind everything else, and
// their size.  The offset is rounded up to 16 bytes (uint4 operand images).
inline bool ccs_has_bf16(const AmmGeom& g) { return (g.v == 2 || g.v == 4 || g.v == 8) && g.C <= 32; }
// 17..32 centroids: a codebook fills all 32 rows of the matrix instruction by itself ("wide"); the operand
// images are then per codebook instead of per pair of codebooks
inline bool ccs_bf16_wide(const AmmGeom& g) { return g.C > 16; }
inline size_t ccs_bf16_units(const AmmGeom& g) { return ccs_bf16_wide(g) ? g.CB_pad : g.CB_pad / 2; }
// MFMAs (16 K-slots each) per codebook pair: 2 codebooks x v dims x 6 cross products
constexpr uint32_t ccs_bf16_nm(uint32_t v) { return (12 * v + 15) / 16; }
inline size_t ccs_bf16_offset(const AmmGeom& g)
{
    const size_t o = (size_t)g.CB * g.C * g.v + ccs_aux_floats(g) + g.CB + ccs_aux_a_floats(g);
    return (o + 3) / 4 * 4;
}
inline size_t ccs_bf16_floats(const AmmGeom& g)
{
    return ccs_has_bf16(g) ? ccs_bf16_units(g) * ccs_bf16_nm(g.v) * 64 * 4 + ccs_bf16_units(g) * 2 * 16 : 0;
}

template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

// Derived centroid data behind the raw [CB][C][v] block of a centroid buffer (C16 = C rounded up
// to a multiple of 16):
//   aux   [CB][v+1][C16] = rows t < v: -2 c_t, row v: |c|^2; centroids past C hold (0, 3e38) so
//                          they can be evaluated like real ones and never win
//   cnmax [CB]           = max_c |c|^2, NaN when any centroid of the codebook is not finite or so
//                          large that the fast form could overflow (forces the exact scan)
__global__ void ccs_prep_kernel(const float* __restrict__ cent, float* __restrict__ aux,
                                float* __restrict__ cnmax, uint32_t C, uint32_t v)
{
    __shared__ float cn_s[256];
    const uint32_t cb = blockIdx.x;
    const uint32_t C16 = (C + 15) / 16 * 16;
    float* ap = aux + (size_t)cb * (v + 1) * C16;
    for (uint32_t c = threadIdx.x; c < C16; c += blockDim.x) {
        float cn = 3e38f;
        if (c < C) {
            const float* cp = cent + ((size_t)cb * C + c) * v;
            cn = 0.0f;
            for (uint32_t t = 0; t < v; ++t) {
                cn = fmaf(cp[t], cp[t], cn);
                ap[(size_t)t * C16 + c] = -2.0f * cp[t];
            }
            cn_s[c] = cn;
        } else {
            for (uint32_t t = 0; t < v; ++t) ap[(size_t)t * C16 + c] = 0.0f;
        }
        ap[(size_t)v * C16 + c] = cn;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float m = 0.0f;
        bool bad = false;
        for (uint32_t c = 0; c < C; ++c) {
            const float cn = cn_s[c];
            if (!(cn < 1e36f)) bad = true;
            m = fmaxf(m, cn);
        }
        cnmax[cb] = bad ? __builtin_nanf("") : m;
    }
}

template <int V, int IDX_BITS, bool FAST>
__global__ __launch_bounds__(CCS_THREADS) void ccs_kernel(const float* __restrict__ x,
                                                         const float* __restrict__ cent,
                                                         const float* __restrict__ aux,
                                                         const float* __restrict__ cnmax,
                                                         uint8_t* __restrict__ idx, uint32_t N,
                                                         uint32_t K, uint32_t CB, uint32_t C,
                                                         uint32_t idx_row_bytes, int idx_tiled, int vec_ok,
                                                         uint32_t CB_pad, uint32_t tiles_cb,
                                                         uint32_t total_tiles)
{
    using S = CcsShape<V>;
    constexpr int RF = S::ROW_FLOATS, CBT = S::CBT, PITCH = S::PITCH, TT = S::TILE_TOKENS;
    static_assert(S::WAVES * 64 == CCS_THREADS, "one wave per codebook group");
    __shared__ __attribute__((aligned(16))) float tile[TT * PITCH];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

    // ---- persistent loop over (token tile, codebook group) tiles; the next tile's activations
    //      are fetched into registers before the current tile is searched, so HBM latency and
    //      bandwidth hide under the VALU work -----------------------------------------------------
    // A tile is 64 tokens x 4*RF floats: rows of 4*RF*4 bytes (512 B for v <= 16) are contiguous in
    // HBM, and wave w searches the w-th quarter of the columns for all 64 tokens.
    constexpr int F4_PER_ROW = S::WAVES * RF / 4;
    constexpr int PASSES = TT * F4_PER_ROW / CCS_THREADS;     // float4 per lane per tile (= RF / 4)
    static_assert(TT * F4_PER_ROW % CCS_THREADS == 0, "the tile's 16-byte pieces divide among the threads");
    // Piece e = threadIdx.x + CCS_THREADS * i of the tile is column piece e % F4_PER_ROW of row e / F4_PER_ROW.
    // Where the threads cover whole rows per pass (256 % F4_PER_ROW == 0) that is the same column piece and
    // a fixed row step in every pass; otherwise (40 pieces per row) both are worked out per pass.
    constexpr bool WHOLE_ROWS = CCS_THREADS % F4_PER_ROW == 0;
    constexpr int ROWS_PER_PASS = CCS_THREADS / F4_PER_ROW;
    auto piece_row = [&](int i) -> uint32_t {
        return WHOLE_ROWS ? threadIdx.x / F4_PER_ROW + i * ROWS_PER_PASS : (threadIdx.x + CCS_THREADS * i) / F4_PER_ROW;
    };
    auto piece_col = [&](int i) -> uint32_t {
        return WHOLE_ROWS ? threadIdx.x % F4_PER_ROW : (threadIdx.x + CCS_THREADS * i) % F4_PER_ROW;
    };
    auto fetch = [&](float4 (&pf)[PASSES], uint32_t tile_id) {
        const uint32_t t_tok0 = (tile_id / tiles_cb) * TT;
#pragma unroll
        for (int i = 0; i < PASSES; ++i) {
            const uint32_t col = (tile_id % tiles_cb) * (S::WAVES * RF) + 4 * piece_col(i);
            uint32_t tok = t_tok0 + piece_row(i);
            if (tok >= N) tok = N - 1;  // rows past N repeat the last token; never stored
            const float* src = x + (size_t)tok * K + col;
            if (vec_ok && col + 4 <= K) {
                pf[i] = *reinterpret_cast<const float4*>(src);
            } else {
                pf[i].x = (col + 0 < K) ? src[0] : 0.0f;
                pf[i].y = (col + 1 < K) ? src[1] : 0.0f;
                pf[i].z = (col + 2 < K) ? src[2] : 0.0f;
                pf[i].w = (col + 3 < K) ? src[3] : 0.0f;
            }
        }
    };
    float4 pf[PASSES];
    if (blockIdx.x < total_tiles) fetch(pf, blockIdx.x);

    for (uint32_t tile_id = blockIdx.x; tile_id < total_tiles; tile_id += gridDim.x) {
    const uint32_t tok0 = (tile_id / tiles_cb) * TT;
    const uint32_t cb0 = ((tile_id % tiles_cb) * S::WAVES + wave) * CBT;

    // transpose through LDS: coalesced rows in, one row slice per lane out
#pragma unroll
    for (int i = 0; i < PASSES; ++i)
        *reinterpret_cast<float4*>(&tile[piece_row(i) * PITCH + 4 * piece_col(i)]) = pf[i];
    __syncthreads();
    float xv[RF];
#pragma unroll
    for (int i = 0; i < RF / 4; ++i) {
        float4 t4 = *reinterpret_cast<const float4*>(&tile[lane * PITCH + wave * RF + 4 * i]);
        xv[4 * i + 0] = t4.x;
        xv[4 * i + 1] = t4.y;
        xv[4 * i + 2] = t4.z;
        xv[4 * i + 3] = t4.w;
    }
    __syncthreads();  // every lane has its row slice: the tile may be overwritten
    if (tile_id + gridDim.x < total_tiles) fetch(pf, tile_id + gridDim.x);

    // ---- distance + hysteresis scan, centroid order, one codebook after the other ----------
    constexpr int OUT_BITS = CBT * IDX_BITS;
    constexpr int OUT_WORDS = (OUT_BITS + 31) / 32;
    uint32_t packed[OUT_WORDS];
#pragma unroll
    for (int i = 0; i < OUT_WORDS; ++i) packed[i] = 0;

    // Fast-form operands of one codebook: lane 16r+j holds (-2 c_0 .. -2 c_{v-1}, |c|^2) of centroid
    // 16*grp+j, and a row_newbcast:j DPP operand hands that to all 16 lanes of the row.
    const uint32_t groups = (C + 15) / 16;
    auto load_aux = [&](float (&am)[V + 1], uint32_t cb, uint32_t grp) {
        const uint32_t cbc = cb < CB ? cb : CB - 1;  // padded codebooks: any valid address
        const float* __restrict__ ap = aux + ((size_t)cbc * (V + 1) * groups + grp) * 16 + (lane & 15);
#pragma unroll
        for (int t = 0; t <= V; ++t) am[t] = ap[(size_t)t * (16 * groups)];
    };
    constexpr bool PREFETCH = FAST && IDX_BITS == 4;  // C <= 16: one group per codebook
    float am_ring[2][V + 1];
    if constexpr (PREFETCH) load_aux(am_ring[0], cb0, 0);
    // more than 16 centroids: the operands of the next group of 16 (of this codebook or the next) are requested
    // before the current group is scanned, so a group's scan covers the next one's loads
    float am_cur[V + 1], am_nxt[V + 1];
    if constexpr (FAST && !PREFETCH) load_aux(am_cur, cb0, 0);

    static_for<CBT>([&](auto cbl_c) {
        constexpr int cbl = decltype(cbl_c)::value;
        const uint32_t cb = cb0 + cbl;
        uint32_t bi = 0;
        bool exact = (cb < CB);  // wave-uniform
        if constexpr (PREFETCH && cbl + 1 < CBT) load_aux(am_ring[(cbl + 1) & 1], cb + 1, 0);
        if (FAST && cb < CB) {
            constexpr uint32_t ID_MASK = (1u << IDX_BITS) - 1u;
            float xx = xv[cbl * V] * xv[cbl * V];
#pragma unroll
            for (int t = 1; t < V; ++t) xx = fmaf(xv[cbl * V + t], xv[cbl * V + t], xx);
            float m1 = __builtin_inff(), m2 = __builtin_inff();
            auto scan16 = [&](const float (&am)[V + 1], uint32_t c0) {
                static_for<16>([&](auto jc) {
                    constexpr int J = decltype(jc)::value;
                    float sc;
                    asm("v_add_f32_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf"
                        : "=v"(sc) : "v"(am[V]), "v"(xx), "n"(J));
#pragma unroll
                    for (int t = 0; t < V; ++t)
                        asm("v_fmac_f32_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf"
                            : "+v"(sc) : "v"(am[t]), "v"(xv[cbl * V + t]), "n"(J));
                    const uint32_t id = (IDX_BITS == 4) ? (uint32_t)J : (c0 | (uint32_t)J);
                    const float key = __uint_as_float((__float_as_uint(sc) & ~ID_MASK) | id);
                    m2 = __builtin_amdgcn_fmed3f(m1, m2, key);
                    // plain v_min_f32: fminf() would first canonicalise the bit-cast key (one more op)
                    asm("v_min_f32_e32 %0, %1, %2" : "=v"(m1) : "v"(m1), "v"(key));
                });
            };
            if constexpr (PREFETCH) {
                scan16(am_ring[cbl & 1], 0);
            } else {
                for (uint32_t grp = 0; grp < groups; ++grp) {
                    const bool last = grp + 1 == groups;
                    load_aux(am_nxt, last ? cb + 1 : cb, last ? 0 : grp + 1);
                    scan16(am_cur, 16 * grp);
#pragma unroll
                    for (int t = 0; t <= V; ++t) am_cur[t] = am_nxt[t];
                }
            }
            bi = __float_as_uint(m1) & ID_MASK;
            const float mag = xx + cnmax[cb];
            constexpr float A = 3.0f * (5 * V + 5) * 5.9604645e-8f;          // 3 (5v+5) u
            constexpr float B = (float)(1u << IDX_BITS) * 2.3841858e-7f * 2;  // 2 * 2^(IDX_BITS-22)
            const float thr = fmaf(A * 2.0f, mag, fmaf(B, fabsf(m2), 1.001e-6f));
            // NaN anywhere makes a compare false, which counts as "not safe"
            const bool safe = ((m2 - m1) > thr) && (mag < 1e36f);
            exact = __builtin_amdgcn_ballot_w64(!safe) != 0;
        }
        if (exact) {
            const float* __restrict__ cp = cent + (size_t)cb * C * V;
            float best = 0.0f;
            bi = 0;
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
    });

    // ---- packed store -----------------------------------------------------------------------
    const uint32_t tok = tok0 + lane;
    if (tok < N && cb0 < CB_pad) {
        const uint32_t byte0 = cb0 * IDX_BITS / 8;
        uint8_t* dst = idx + idx_offset(tok, byte0, idx_row_bytes, idx_tiled);
        if (idx_tiled && OUT_BITS >= 64) {  // one 32-bit word at a time: consecutive words are 256 bytes apart
#pragma unroll
            for (int w = 0; w < (OUT_BITS >= 128 ? 4 : 2); ++w)
                *reinterpret_cast<uint32_t*>(idx + idx_offset(tok, byte0 + 4 * w, idx_row_bytes, 1)) = packed[w];
        } else if constexpr (OUT_BITS >= 128) {
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
    }  // tiles
}

// =============================================================================================
// Matrix-core search for C <= 16 (4-bit indices), v in {2, 4, 8}.
//
// The score  |c|^2 - 2 x.c  of 16 centroids x 2 codebooks x 32 tokens is one chain of v+1
// v_mfma_f32_32x32x2_f32: the A operand holds, per codebook pair, a 32 x (2v+2) matrix whose row
// for (codebook half h, centroid r) carries -2c in the v columns of its own codebook, zeros in the
// other codebook's columns and |c|^2 in column 2v; the B operand holds the 2v activation values of
// the pair and a 1.0 in row 2v.  Rows are ordered so that the result registers of lane (j, h)
// are exactly the 16 scores of token j against codebook h of the pair:
//     result register r of lane l = D[8*(r/4) + 4*(l/32) + r%4][l%32]   (hardware layout)
//     => row i belongs to half h = (i/4)%2 and centroid r = i%4 + 4*(i/8).
// The search is then lane-local: pack the centroid id into the low 4 mantissa bits, keep the two
// smallest (v_and_or, v_med3, v_med3 per centroid) and apply the margin test described at the top
// of this file.  (token, codebook) pairs that fail the test are replayed with the exact scan by
// their own lane after the fast pass, from LDS copies of the activations and the raw centroids.
//
// A tile is 128 tokens x 16 codebooks.  Wave w owns codebook pairs 2w and 2w+1, whose A operands
// stay in registers for the four 32-token groups of the tile; the next item's MFMA chain is issued
// before the current item's scores are searched so the matrix pipe and the VALU overlap.
// Workgroups are persistent and fetch the next tile's activations into registers meanwhile.
//
// Error bound of this form: |c|^2 carries <= v u CN, the MFMA chain rounds at most v+2 partial sums
// each below 2(XX+CN): together with the reference chain's 2(v+2)u(XX+CN) that is below
// (5v+8)u(XX+CN); the kernel uses twice that.
// =============================================================================================
template <int V, bool WIDE = false, int TTOK = 128>
struct CcsMfmaShape {
    static constexpr int TILE_TOKENS = TTOK;               // 128, or 64 for batches with few tiles
    static constexpr int CBW = 16;                         // codebooks per tile: 2 pairs per wave
    static constexpr int RCB = WIDE ? CBW / 2 : CBW;       // wide: a "pair" is the two 16-centroid halves of one codebook
    static constexpr int TF = RCB * V;                     // floats per tile row
    static constexpr int PITCH = TF + 4;                   // +16 B: odd number of 16-byte units
    static constexpr int NQ = V + 1;                       // MFMAs (K = 2 each) per item
    static constexpr int TG = TILE_TOKENS / 32;            // 32-token groups
    static constexpr int ITEMS = 2 * TG;                   // (pair, token group) items per wave
    static constexpr int X_FLOATS = TILE_TOKENS * PITCH;
    static constexpr int CENT_FLOATS = CBW * 16 * V;       // raw centroids of the tile's codebooks
    static constexpr int LDS_BYTES = (X_FLOATS + CENT_FLOATS) * 4 + TILE_TOKENS * (CBW / 2);
};

typedef float floatx16 __attribute__((ext_vector_type(16)));

// Plain hardware min/max on bit patterns that are already valid floats.  fminf()/fmaxf() would
// first canonicalise operands that come from integer operations (one more VALU op each).
__device__ __forceinline__ float vmin(float a, float b)
{
    float r;
    asm("v_min_f32_e32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ float vmax(float a, float b)
{
    float r;
    asm("v_max_f32_e32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ float vmin3(float a, float b, float c)
{
    float r;
    asm("v_min3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// Operands of the MFMA search behind the other derived data of a centroid buffer:
//   aux_a     [CB_pad/2 pairs][v+1][64 lanes]  A-operand images
//   cnmax_pad [CB_pad]                         cnmax, 0 for padded codebooks
// A padded codebook scores r against centroid r, so it yields index 0 with a margin of 1.
__global__ void ccs_prep_mfma_kernel(const float* __restrict__ cent, const float* __restrict__ cnmax,
                                     float* __restrict__ aux_a, float* __restrict__ cnmax_pad, uint32_t CB,
                                     uint32_t C, uint32_t v)
{
    const uint32_t pair = blockIdx.x, lane = threadIdx.x;
    const uint32_t i = lane & 31, kh = lane >> 5;
    const uint32_t h = (i >> 2) & 1, r = (i & 3) + 4 * (i >> 3);
    const uint32_t cb = 2 * pair + h;
    const bool real = (cb < CB) && (r < C);
    const float* cp = cent + ((size_t)cb * C + r) * v;
    float cn = (float)r;
    if (real) {
        cn = 0.0f;
        for (uint32_t t = 0; t < v; ++t) cn = fmaf(cp[t], cp[t], cn);
    } else if (cb < CB) {
        cn = 3e38f;  // centroid ids past C never win
    }
    for (uint32_t q = 0; q <= v; ++q) {
        const uint32_t k = 2 * q + kh;
        float val = 0.0f;
        if (k < 2 * v) {
            if (real && k / v == h) val = -2.0f * cp[k % v];
        } else if (k == 2 * v) {
            val = cn;
        }
        aux_a[((size_t)pair * (v + 1) + q) * 64 + lane] = val;
    }
    if (lane < 2) {
        const uint32_t c2 = 2 * pair + lane;
        cnmax_pad[c2] = (c2 < CB) ? cnmax[c2] : 0.0f;
    }
}

template <int V>  // (v = 8 does not fit four waves per SIMD: asked for two, which is what the compiler reaches)
__global__ __launch_bounds__(CCS_THREADS, V == 8 ? 2 : 4) void ccs_mfma_kernel(const float* __restrict__ x,
                                                                 const float* __restrict__ cent,
                                                                 const float* __restrict__ aux_a,
                                                                 const float* __restrict__ cnmax_pad,
                                                                 uint8_t* __restrict__ idx, uint32_t N,
                                                                 uint32_t K, uint32_t CB, uint32_t C,
                                                                 uint32_t idx_row_bytes, int idx_tiled, int vec_ok,
                                                                 uint32_t tiles_cb, uint32_t total_tiles)
{
    using S = CcsMfmaShape<V>;
    constexpr int TF = S::TF, PITCH = S::PITCH, TT = S::TILE_TOKENS, NQ = S::NQ, CBW = S::CBW, TG = S::TG;
    constexpr int ITEMS = S::ITEMS;
    __shared__ __attribute__((aligned(16))) float tile[S::X_FLOATS];
    __shared__ __attribute__((aligned(16))) float cst[S::CENT_FLOATS];
    __shared__ __attribute__((aligned(16))) uint8_t ist[TT * (CBW / 2)];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t j = lane & 31, h = lane >> 5;  // token within a group, codebook of the pair

    constexpr int F4_PER_ROW = TF / 4;
    constexpr int ROWS_PER_PASS = CCS_THREADS / F4_PER_ROW;
    constexpr int PASSES = TT / ROWS_PER_PASS;
    static_assert(CCS_THREADS % F4_PER_ROW == 0 && TT % ROWS_PER_PASS == 0, "tile shape");
    const uint32_t fq = threadIdx.x % F4_PER_ROW;
    const uint32_t fr0 = threadIdx.x / F4_PER_ROW;
    auto fetch = [&](float4 (&pf)[PASSES], uint32_t tile_id) {
        const uint32_t t_tok0 = (tile_id / tiles_cb) * TT;
        const uint32_t col = (tile_id % tiles_cb) * TF + 4 * fq;
#pragma unroll
        for (int i = 0; i < PASSES; ++i) {
            uint32_t tok = t_tok0 + fr0 + i * ROWS_PER_PASS;
            if (tok >= N) tok = N - 1;  // rows past N repeat the last token; never stored
            const float* src = x + (size_t)tok * K + col;
            if (vec_ok && col + 4 <= K) {
                pf[i] = *reinterpret_cast<const float4*>(src);
            } else {
                pf[i].x = (col + 0 < K) ? src[0] : 0.0f;
                pf[i].y = (col + 1 < K) ? src[1] : 0.0f;
                pf[i].z = (col + 2 < K) ? src[2] : 0.0f;
                pf[i].w = (col + 3 < K) ? src[3] : 0.0f;
            }
        }
    };
    // operands of this lane inside the tile: row of token (32 tg + j), columns of pair (2 wave + pl)
    const float* brow0 = tile + j * PITCH + 2 * wave * 2 * V;
    const float b_last = (h == 0) ? 1.0f : 0.0f;

    float4 pf[PASSES];
    if (blockIdx.x < total_tiles) fetch(pf, blockIdx.x);

    for (uint32_t tile_id = blockIdx.x; tile_id < total_tiles; tile_id += gridDim.x) {
        const uint32_t tok0 = (tile_id / tiles_cb) * TT;
        const uint32_t tcb = tile_id % tiles_cb;          // codebooks 16 tcb .. 16 tcb + 15
        const uint32_t pair0 = tcb * (CBW / 2) + 2 * wave;  // first of this wave's two pairs

        float aq[2][NQ];
#pragma unroll
        for (int pl = 0; pl < 2; ++pl)
#pragma unroll
            for (int q = 0; q < NQ; ++q) aq[pl][q] = aux_a[((size_t)(pair0 + pl) * NQ + q) * 64 + lane];
        // every global load the search needs is issued here, ahead of the next tile's prefetch:
        // loads complete in order, so a later load would have to wait for the prefetch from HBM
        float cmax[2];
#pragma unroll
        for (int pl = 0; pl < 2; ++pl) cmax[pl] = cnmax_pad[2 * (pair0 + pl) + h];
        // raw centroids of the tile's codebooks, only read by exact replays
        const uint32_t cb_here = (CB - tcb * CBW < (uint32_t)CBW) ? CB - tcb * CBW : (uint32_t)CBW;
        const uint32_t cent_fl = cb_here * C * V;
        const float* csrc = cent + (size_t)tcb * CBW * C * V;  // 16-byte aligned: CBW * V * 4 bytes per c
#pragma unroll
        for (int i = 0; i < PASSES; ++i)
            *reinterpret_cast<float4*>(&tile[(fr0 + i * ROWS_PER_PASS) * PITCH + 4 * fq]) = pf[i];
        for (uint32_t i = threadIdx.x; i < cent_fl / 4; i += CCS_THREADS)
            reinterpret_cast<float4*>(cst)[i] = reinterpret_cast<const float4*>(csrc)[i];
        if (threadIdx.x < cent_fl % 4) cst[cent_fl - 1 - threadIdx.x] = csrc[cent_fl - 1 - threadIdx.x];
        __syncthreads();
        if (tile_id + gridDim.x < total_tiles) fetch(pf, tile_id + gridDim.x);

        auto scores = [&](floatx16& acc, int it) {
            const int pl = it / TG, tg = it % TG;
            const float* brow = brow0 + tg * 32 * PITCH + pl * 2 * V;
            acc = floatx16(0.0f);
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                const float b = (q < V) ? brow[2 * q + h] : b_last;
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(aq[pl][q], b, acc, 0, 0, 0);
            }
        };

        // words[tg / 2], 16 bits per token group: nibble of (pair pl, half h) at bit 8 pl + 4 h
        uint32_t words[TG / 2];
#pragma unroll
        for (int i = 0; i < TG / 2; ++i) words[i] = 0;
        uint32_t need = 0;  // bit it: item it must be replayed exactly by this lane

        floatx16 acc_cur, acc_nxt;
        scores(acc_cur, 0);
        static_for<ITEMS>([&](auto itc) {
            constexpr int it = decltype(itc)::value;
            constexpr int pl = it / TG, tg = it % TG;
            if constexpr (it + 1 < ITEMS) scores(acc_nxt, it + 1);
            // |x|^2 of this lane's own codebook, for the error bound
            const float* xo = brow0 + tg * 32 * PITCH + pl * 2 * V + V * h;
            float xx = xo[0] * xo[0];
#pragma unroll
            for (int t = 1; t < V; ++t) xx = fmaf(xo[t], xo[t], xx);
            // smallest (m1) and second smallest (m2) of the 16 id-tagged scores, 36 VALU operations:
            // five triples give (min3, med3) each; the overall second smallest is the smaller of
            // the second smallest of the six group minima and the smallest of the group medians.
            float key[16];
#pragma unroll
            for (int r = 0; r < 16; ++r)
                key[r] = __uint_as_float((__float_as_uint(acc_cur[r]) & ~15u) | (uint32_t)r);
            float lo[5], md[5];
#pragma unroll
            for (int i = 0; i < 5; ++i) {
                lo[i] = vmin3(key[3 * i], key[3 * i + 1], key[3 * i + 2]);
                md[i] = __builtin_amdgcn_fmed3f(key[3 * i], key[3 * i + 1], key[3 * i + 2]);
            }
            const float a1 = vmin3(lo[0], lo[1], lo[2]), a2 = __builtin_amdgcn_fmed3f(lo[0], lo[1], lo[2]);
            const float b1 = vmin3(lo[3], lo[4], key[15]), b2 = __builtin_amdgcn_fmed3f(lo[3], lo[4], key[15]);
            const float m1 = vmin(a1, b1);
            const float m2 = vmin3(vmin3(md[0], md[1], md[2]), vmin3(md[3], md[4], vmax(a1, b1)), vmin(a2, b2));
            const uint32_t bi = __float_as_uint(m1) & 15u;
            const float mag = xx + cmax[pl];
            constexpr float A2 = 2.0f * 2.0f * (5 * V + 8) * 5.9604645e-8f;  // 2 * [2 (5v+8) u]
            constexpr float B2 = 2.0f * 16.0f * 2.3841858e-7f;               // 2 * 2^(4-22)
            const float thr = fmaf(A2, mag, fmaf(B2, fabsf(m2), 1.001e-6f));
            // NaN anywhere makes a compare false, which counts as "not safe"
            const bool safe = ((m2 - m1) > thr) && (mag < 1e36f);
            need |= (safe ? 0u : 1u) << it;
            words[tg / 2] |= bi << (16 * (tg % 2) + 8 * pl + 4 * h);
            if constexpr (it + 1 < ITEMS) acc_cur = acc_nxt;
        });

        // ---- exact replay of the items that failed the margin test (rare, lane-divergent) -------
        if (__builtin_amdgcn_ballot_w64(need != 0) != 0) {
            // kept rolled on purpose: the replay is rare and must not cost the fast path registers
#pragma nounroll
            for (int it = 0; it < ITEMS; ++it) {
                if (!((need >> it) & 1u)) continue;
                const int pl = it / TG, tg = it % TG;
                const uint32_t cbl = 2 * (2 * wave + pl) + h;
                uint32_t bi = 0;
                if (tcb * CBW + cbl < CB) {
                    const float* xo = brow0 + tg * 32 * PITCH + pl * 2 * V + V * h;
                    const float* cp = cst + cbl * C * V;
                    float best = 0.0f;
#pragma nounroll
                    for (uint32_t c = 0; c < C; ++c) {
                        float diff = __fsub_rn(xo[0], cp[c * V + 0]);
                        float d = __fmul_rn(diff, diff);
#pragma unroll
                        for (int t = 1; t < V; ++t) {
                            diff = __fsub_rn(xo[t], cp[c * V + t]);
                            d = __fadd_rn(d, __fmul_rn(diff, diff));
                        }
                        const bool take = (c == 0) || (__fsub_rn(best, d) > 1e-6f);
                        best = take ? d : best;
                        bi = take ? c : bi;
                    }
                }
                const uint32_t sh = 16 * (tg % 2) + 8 * pl + 4 * h;
                uint32_t w = words[0];
#pragma unroll
                for (int i = 1; i < TG / 2; ++i) w = (tg / 2 == i) ? words[i] : w;
                w = (w & ~(15u << sh)) | (bi << sh);
#pragma unroll
                for (int i = 0; i < TG / 2; ++i) words[i] = (tg / 2 == i) ? w : words[i];
            }
        }

        // ---- merge the two codebooks of each pair (lanes l and l+32), gather the tile's index
        //      bytes in LDS, store 8 bytes per token ------------------------------------------------
#pragma unroll
        for (int i = 0; i < TG / 2; ++i) words[i] |= __shfl_xor(words[i], 32);
        if (h == 0) {
#pragma unroll
            for (int tg = 0; tg < TG; ++tg)
                *reinterpret_cast<uint16_t*>(&ist[(32 * tg + j) * (CBW / 2) + 2 * wave]) =
                    (uint16_t)(words[tg / 2] >> (16 * (tg % 2)));
        }
        __syncthreads();  // index bytes complete; every wave is done with the activation tile
        if (threadIdx.x < TT) {
            const uint32_t tok = tok0 + threadIdx.x;
            if (tok < N) {
                const uint2 w = *reinterpret_cast<const uint2*>(&ist[threadIdx.x * (CBW / 2)]);
                if (idx_tiled) {
                    *reinterpret_cast<uint32_t*>(idx + idx_offset(tok, tcb * (CBW / 2), idx_row_bytes, 1)) = w.x;
                    *reinterpret_cast<uint32_t*>(idx + idx_offset(tok, tcb * (CBW / 2) + 4, idx_row_bytes, 1)) = w.y;
                } else {
                    *reinterpret_cast<uint2*>(idx + (size_t)tok * idx_row_bytes + tcb * (CBW / 2)) = w;
                }
            }
        }
    }
}

// =============================================================================================
// bf16-split variant of the MFMA search for v in {2, 4, 8} (C <= 16).  The fp32 MFMA above shares the fp32
// units with the VALU, so its five instructions per item (147 ns) add to the ~50 VALU operations of
// the top-two search (100 ns).  v_mfma_f32_32x32x16_bf16 is twice as fast per K-slot and runs beside
// VALU work.  bf16 has 8 significand bits, so each fp32 value is cut into three bf16 pieces and six
// of the nine cross products are kept (see `scores` below); the score then carries a known error
// bound like the fp32 form's, only larger (A2 below), and everything after the scores -- tagged
// keys, tournament, margin test, exact replay -- is the same.  Operands:
//   aux_b [CB_pad/2 pairs][NM][64 lanes] uint4 A-operand images (bf16 pieces of -2c, by K-slot)
//   cn16  [CB_pad][16] float                   |c|^2 (r for padded codebooks, 3e38 for ids past C)
// =============================================================================================
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned int v6u __attribute__((ext_vector_type(6)));

// K-slot registers (two bf16 K-slots each, four registers per MFMA) of lane (row i, half kh).  The lane
// covers dims DL*kh .. DL*kh + DL-1 (DL = v/2) of both codebooks of the pair.
//   DL >= 2: three MFMAs per pair of dims (d, d+1); a register holds (piece of d | piece of d+1 << 16).  The
//            search kernel keeps six registers  xm(cb0) xm(cb1) xh(cb0) xh(cb1) xl(cb0) xl(cb1)  in a row and
//            hands the MFMAs windows of four of them, so that no piece is copied:
//              registers 0..3 against {ch, ch, ch, ch}   (xm*ch, xh*ch)
//              registers 0..3 against {cm, cm, cm, cm}   (xm*cm, xh*cm)
//              registers 2..5 against {cl, cl, ch, ch}   (xh*cl, xl*ch)
//            with the pieces of -2c of the row's own codebook in that codebook's registers;
//   DL == 1: codebook q owns registers 3q .. 3q+2 of the first two MFMAs: (ch | cm), (ch | cm), (cl | ch)
//            against (xh | xh), (xm | xm), (xh | xl).
// Registers of the other codebook, and registers past the last one used, hold zeros.
// WIDE (17..32 centroids): "pair" p is codebook p alone, its half h holds centroids 16h .. 16h+15, and both
// halves meet the same sub-vector (the search kernel feeds the activations of codebook p to both).
template <uint32_t V, bool WIDE>
__global__ void ccs_prep_bf16_kernel(const float* __restrict__ cent, uint4* __restrict__ aux_b,
                                     float* __restrict__ cn16, uint32_t CB, uint32_t C)
{
    constexpr uint32_t DL = V / 2, NM = ccs_bf16_nm(V);
    const uint32_t pair = blockIdx.x, lane = threadIdx.x;
    const uint32_t i = lane & 31, kh = lane >> 5;
    const uint32_t h = (i >> 2) & 1, r = (i & 3) + 4 * (i >> 3);
    const uint32_t cb = WIDE ? pair : 2 * pair + h;
    const uint32_t cid = WIDE ? 16 * h + r : r;  // centroid of row i
    const bool real = (cb < CB) && (cid < C);
    const float* cp = cent + ((size_t)cb * C + cid) * V;
    uint32_t pc[DL][3];  // bf16 pieces ch, cm, cl of -2c for the lane's dims
    for (uint32_t d = 0; d < DL; ++d) {
        const float a = real ? -2.0f * cp[DL * kh + d] : 0.0f;
        const uint32_t au = __float_as_uint(a);
        const float r1 = __fsub_rn(a, __uint_as_float(au & 0xffff0000u));
        const uint32_t r1u = __float_as_uint(r1);
        const float r2 = __fsub_rn(r1, __uint_as_float(r1u & 0xffff0000u));
        pc[d][0] = au >> 16;
        pc[d][1] = r1u >> 16;
        pc[d][2] = __float_as_uint(r2) >> 16;
    }
    for (uint32_t m = 0; m < NM; ++m) {
        uint32_t w[4];
        for (uint32_t q = 0; q < 4; ++q) {
            const uint32_t rho = 4 * m + q;
            uint32_t val = 0;
            if (DL == 1) {
                if (real && rho < 6 && rho / 3 == h)
                    val = rho % 3 == 2 ? (pc[0][2] | (pc[0][0] << 16)) : (pc[0][0] | (pc[0][1] << 16));
            } else if (real && (q & 1) == h) {
                const uint32_t dp = m / 3, kind = m % 3;
                const uint32_t t = kind == 2 ? (q < 2 ? 2u : 0u) : kind;  // ch, cm, or cl | ch
                val = pc[2 * dp][t] | (pc[2 * dp + 1][t] << 16);
            }
            w[q] = val;
        }
        aux_b[((size_t)pair * NM + m) * 64 + lane] = make_uint4(w[0], w[1], w[2], w[3]);
    }
    if (kh == 0) {
        float cn = (float)cid;  // a padded codebook scores r against centroid r: index 0 with a margin of 1
        if (real) {
            cn = 0.0f;
            for (uint32_t t = 0; t < V; ++t) cn = fmaf(cp[t], cp[t], cn);
        } else if (cb < CB) {
            cn = 3e38f;  // centroid ids past C never win
        }
        cn16[(size_t)(2 * pair + h) * 16 + r] = cn;
    }
}

// Register budget: three waves per SIMD (168 registers) but for v = 8 with 128-token tiles and up to 16 centroids,
// whose 64 prefetch registers do not fit: asked for three the compiler gives up and takes 288 (one workgroup per
// CU); asked for two it takes 237 without spills, and the 76 KB of LDS allow no more than two anyway.
template <int V, bool WIDE, int TTOK>
__global__ __launch_bounds__(CCS_THREADS, (V == 8 && !WIDE && TTOK == 128) ? 2 : 3) void ccs_bf16_kernel(const float* __restrict__ x,
                                                                 const float* __restrict__ cent,
                                                                 const uint4* __restrict__ aux_b,
                                                                 const float* __restrict__ cn16,
                                                                 const float* __restrict__ cnmax_pad,
                                                                 uint8_t* __restrict__ idx, uint32_t N,
                                                                 uint32_t K, uint32_t CB, uint32_t C,
                                                                 uint32_t idx_row_bytes, int idx_tiled, int vec_ok,
                                                                 uint32_t tiles_cb, uint32_t total_tiles, uint32_t tiles_x)
{
    // K is the length of an activation row.  tiles_x < tiles_cb: the codebooks are those of several operators
    // that read the same row (tiles_x codebook tiles each), so the activation columns wrap around.
    using S = CcsMfmaShape<V, WIDE, TTOK>;
    constexpr int TF = S::TF, PITCH = S::PITCH, TT = S::TILE_TOKENS, CBW = S::CBW, TG = S::TG, RCB = S::RCB;
    constexpr int XSTEP = WIDE ? V : 2 * V;  // activation floats per pair
    constexpr int NM = (int)ccs_bf16_nm(V);  // MFMAs per item: 2 codebooks x v dims x 6 cross products, 16 K-slots each
    constexpr int DL = V / 2;                // dims of each codebook this lane supplies
    constexpr int ITEMS = S::ITEMS;
    __shared__ __attribute__((aligned(16))) float tile[S::X_FLOATS];
    __shared__ __attribute__((aligned(16))) float cst[S::CENT_FLOATS];
    __shared__ __attribute__((aligned(16))) uint8_t ist[TT * (CBW / 2)];
    __shared__ __attribute__((aligned(16))) float cnl[CBW * 16];  // |c|^2 of the tile's centroids: the accumulators start from them
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t j = lane & 31, h = lane >> 5;  // token within a group, codebook of the pair

    constexpr int F4_PER_ROW = TF / 4;
    constexpr int ROWS_PER_PASS = CCS_THREADS / F4_PER_ROW;
    constexpr int PASSES = TT / ROWS_PER_PASS;
    static_assert(CCS_THREADS % F4_PER_ROW == 0 && TT % ROWS_PER_PASS == 0, "tile shape");
    const uint32_t fq = threadIdx.x % F4_PER_ROW;
    const uint32_t fr0 = threadIdx.x / F4_PER_ROW;
    auto fetch = [&](float4 (&pf)[PASSES], uint32_t tile_id) {
        const uint32_t t_tok0 = (tile_id / tiles_cb) * TT;
        const uint32_t col0 = ((tile_id % tiles_cb) % tiles_x) * TF;  // workgroup-uniform
        const uint32_t col = col0 + 4 * fq;
        // The whole tile inside the row and 16-byte aligned (every tile but a ragged last one): one 16-byte load
        // per pass, decided once for the workgroup.  Decided per lane instead, the compiler splits every load in
        // two and wraps each pass in a dozen exec-mask operations.
        if (vec_ok && col0 + TF <= K) {
#pragma unroll
            for (int i = 0; i < PASSES; ++i) {
                uint32_t tok = t_tok0 + fr0 + i * ROWS_PER_PASS;
                tok = tok < N ? tok : N - 1;  // rows past N repeat the last token; never stored
                pf[i] = *reinterpret_cast<const float4*>(x + (size_t)tok * K + col);
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < PASSES; ++i) {
            uint32_t tok = t_tok0 + fr0 + i * ROWS_PER_PASS;
            if (tok >= N) tok = N - 1;
            const float* src = x + (size_t)tok * K + col;
            pf[i].x = (col + 0 < K) ? src[0] : 0.0f;
            pf[i].y = (col + 1 < K) ? src[1] : 0.0f;
            pf[i].z = (col + 2 < K) ? src[2] : 0.0f;
            pf[i].w = (col + 3 < K) ? src[3] : 0.0f;
        }
    };
    // operands of this lane inside the tile: row of token (32 tg + j), columns of pair (2 wave + pl)
    const float* brow0 = tile + j * PITCH + 2 * wave * XSTEP;

    float4 pf[PASSES];
    if (blockIdx.x < total_tiles) fetch(pf, blockIdx.x);

    // The CU issues from its oldest waves first, so of the workgroups resident on a CU the first one
    // placed would finish its (equal) share of tiles well before the last and leave the CU half empty.
    // A wave's priority falls as its workgroup progresses through its share: whoever is behind goes first.
    const uint32_t my_tiles = (total_tiles - blockIdx.x + gridDim.x - 1) / gridDim.x;
    uint32_t tiles_done = 0;
    uint32_t tcb_loaded = 0xFFFFFFFFu;  // codebook tile whose operands are resident (registers and LDS)
    uint4 aq[2][NM];
    float cmax[2];
    for (uint32_t tile_id = blockIdx.x; tile_id < total_tiles; tile_id += gridDim.x) {
        switch (4 * tiles_done / my_tiles) {
            case 0: __builtin_amdgcn_s_setprio(3); break;
            case 1: __builtin_amdgcn_s_setprio(2); break;
            case 2: __builtin_amdgcn_s_setprio(1); break;
            default: __builtin_amdgcn_s_setprio(0); break;
        }
        ++tiles_done;
        const uint32_t tok0 = (tile_id / tiles_cb) * TT;
        const uint32_t tcb = tile_id % tiles_cb;          // codebooks 16 tcb .. 16 tcb + 15
        const uint32_t pair0 = tcb * (CBW / 2) + 2 * wave;  // first of this wave's two pairs

        // What depends on the codebooks alone stays from the previous tile when this one has the same codebooks
        // (a grid that is a multiple of the codebook tiles gives a workgroup the same ones every time).
        const bool new_cb = tcb != tcb_loaded;  // workgroup-uniform
        tcb_loaded = tcb;
        if (new_cb) {
#pragma unroll
            for (int pl = 0; pl < 2; ++pl)
#pragma unroll
                for (int m = 0; m < NM; ++m) aq[pl][m] = aux_b[((size_t)(pair0 + pl) * NM + m) * 64 + lane];
            // every global load the search needs is issued here, ahead of the next tile's prefetch:
            // loads complete in order, so a later load would have to wait for the prefetch from HBM
#pragma unroll
            for (int pl = 0; pl < 2; ++pl) cmax[pl] = cnmax_pad[WIDE ? pair0 + pl : 2 * (pair0 + pl) + h];
        }
#pragma unroll
        for (int i = 0; i < PASSES; ++i)
            *reinterpret_cast<float4*>(&tile[(fr0 + i * ROWS_PER_PASS) * PITCH + 4 * fq]) = pf[i];
        if (new_cb) {
            // raw centroids of the tile's codebooks, only read by exact replays
            const uint32_t cb_here = (CB - tcb * RCB < (uint32_t)RCB) ? CB - tcb * RCB : (uint32_t)RCB;
            const uint32_t cent_fl = cb_here * C * V;
            const float* csrc = cent + (size_t)tcb * RCB * C * V;  // 16-byte aligned: RCB * V * 4 bytes per c
            for (uint32_t i = threadIdx.x; i < cent_fl / 4; i += CCS_THREADS)
                reinterpret_cast<float4*>(cst)[i] = reinterpret_cast<const float4*>(csrc)[i];
            if (threadIdx.x < cent_fl % 4) cst[cent_fl - 1 - threadIdx.x] = csrc[cent_fl - 1 - threadIdx.x];
            if (threadIdx.x < CBW * 16 / 4)
                reinterpret_cast<float4*>(cnl)[threadIdx.x] = reinterpret_cast<const float4*>(cn16 + (size_t)tcb * CBW * 16)[threadIdx.x];
        }
        __syncthreads();
        if (tile_id + gridDim.x < total_tiles) fetch(pf, tile_id + gridDim.x);

        // Scores of item `it` (pair pl, token group tg) for this lane's token: this lane (half h) holds
        // dims DL*h .. DL*h + DL-1 of both codebooks of the pair.  Each value is cut into three bf16 pieces
        // by masking (x = xh + xm + xl exactly: 8 + 8 + 8 significand bits); the A operand holds the same
        // pieces of -2c, and the K-slots pair them as  xh*ch, xh*cm, xm*ch, xm*cm, xh*cl, xl*ch  (the three
        // omitted products are below 2^-20 |x||c|).  Products of bf16 values are exact in fp32; the
        // accumulators start from |c|^2.  xx_out: |x|^2 over the lane's own codebook (for the bound).
        // activations of item `it` for this lane; read two items ahead of their use (see the loop below)
        auto load_x = [&](float (&xs)[2][DL], int it) {
            const int pl = it / TG, tg = it % TG;
            const float* brow = brow0 + tg * 32 * PITCH + pl * XSTEP;
#pragma unroll
            for (int cbh = 0; cbh < 2; ++cbh) {
                const float* src = brow + (WIDE ? 0 : cbh * V) + DL * h;
                if constexpr (DL == 1) {
                    xs[cbh][0] = src[0];
                } else if constexpr (DL == 2) {
                    const float2 t2 = *reinterpret_cast<const float2*>(src);
                    xs[cbh][0] = t2.x;
                    xs[cbh][1] = t2.y;
                } else {
                    static_assert(DL == 4, "dims per lane");
                    const float4 t4 = *reinterpret_cast<const float4*>(src);
                    xs[cbh][0] = t4.x;
                    xs[cbh][1] = t4.y;
                    xs[cbh][2] = t4.z;
                    xs[cbh][3] = t4.w;
                }
            }
        };
        floatx16 cn_pl;  // |c|^2 of the lane's 16 centroids of the current pair: what every accumulator starts from
        auto scores = [&](floatx16& acc, float& xx_out, int it, const float (&xs)[2][DL]) {
            const int pl = it / TG;
            if (it % TG == 0) {  // (a constant once the item loop is unrolled) first token group of a pair
                const float4* cnp = reinterpret_cast<const float4*>(cnl + (2 * (2 * wave + pl) + h) * 16);
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    const float4 c4 = cnp[q4];
                    cn_pl[4 * q4 + 0] = c4.x;
                    cn_pl[4 * q4 + 1] = c4.y;
                    cn_pl[4 * q4 + 2] = c4.z;
                    cn_pl[4 * q4 + 3] = c4.w;
                }
            }
            // bf16 pieces of the lane's activations: x = xh + xm + xl exactly
            uint32_t xu[2][DL], r1u[2][DL], r2u[2][DL];
            float part[2];
#pragma unroll
            for (int cbh = 0; cbh < 2; ++cbh) {
                float sq = 0.0f;
#pragma unroll
                for (int d = 0; d < DL; ++d) {
                    const float a = xs[cbh][d];
                    xu[cbh][d] = __float_as_uint(a);
                    const float r1 = a - __uint_as_float(xu[cbh][d] & 0xffff0000u);
                    r1u[cbh][d] = __float_as_uint(r1);
                    r2u[cbh][d] = __float_as_uint(r1 - __uint_as_float(r1u[cbh][d] & 0xffff0000u));
                    sq = d == 0 ? a * a : fmaf(a, a, sq);
                }
                part[cbh] = sq;
            }
            // |x|^2 of codebook h: lanes l and l+32 each hold half of it for both codebooks
            const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(part[0]), __float_as_uint(part[1]), false, false);
            xx_out = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
            auto mfma = [&](int m, const v4u& b, bool first) {
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, aq[pl][m]), __builtin_bit_cast(bf16x8, b),
                                                              first ? cn_pl : acc, 0, 0, 0);
            };
            // __builtin_amdgcn_perm(p, q, 0x07060302) = (bf16 of q | bf16 of p << 16)
            if constexpr (DL == 1) {
                uint32_t breg[8];
#pragma unroll
                for (int cbh = 0; cbh < 2; ++cbh) {
                    breg[3 * cbh + 0] = __builtin_amdgcn_perm(xu[cbh][0], xu[cbh][0], 0x07060302u);    // (xh | xh)
                    breg[3 * cbh + 1] = __builtin_amdgcn_perm(r1u[cbh][0], r1u[cbh][0], 0x07060302u);  // (xm | xm)
                    breg[3 * cbh + 2] = __builtin_amdgcn_perm(r2u[cbh][0], xu[cbh][0], 0x07060302u);   // (xh | xl)
                }
                breg[6] = breg[7] = 0;
                mfma(0, v4u{breg[0], breg[1], breg[2], breg[3]}, true);
                mfma(1, v4u{breg[4], breg[5], breg[6], breg[7]}, false);
            } else {
#pragma unroll
                for (int dp = 0; dp < DL / 2; ++dp) {
                    // six registers in a row, the MFMAs read windows of four of them (see ccs_prep_bf16_kernel)
                    v6u s6;
#pragma unroll
                    for (int cbh = 0; cbh < 2; ++cbh) {
                        s6[0 + cbh] = __builtin_amdgcn_perm(r1u[cbh][2 * dp + 1], r1u[cbh][2 * dp], 0x07060302u);  // xm
                        s6[2 + cbh] = __builtin_amdgcn_perm(xu[cbh][2 * dp + 1], xu[cbh][2 * dp], 0x07060302u);    // xh
                        s6[4 + cbh] = __builtin_amdgcn_perm(r2u[cbh][2 * dp + 1], r2u[cbh][2 * dp], 0x07060302u);  // xl
                    }
                    const v4u lo = __builtin_shufflevector(s6, s6, 0, 1, 2, 3), hi = __builtin_shufflevector(s6, s6, 2, 3, 4, 5);
                    mfma(3 * dp + 0, lo, dp == 0);
                    mfma(3 * dp + 1, lo, false);
                    mfma(3 * dp + 2, hi, false);
                }
            }
        };

        // words[tg / 2], 16 bits per token group: nibble of (pair pl, half h) at bit 8 pl + 4 h
        uint32_t words[TG / 2];
#pragma unroll
        for (int i = 0; i < TG / 2; ++i) words[i] = 0;
        uint32_t need = 0;  // bit it: item it must be replayed exactly by this lane

        floatx16 acc_cur, acc_nxt;
        float xx_cur, xx_nxt;
        // The activations of item it + 2 are read from LDS before item it + 1 is scored and item it searched, and
        // the read is kept there: left to itself the compiler sinks it to a few instructions before its use and
        // the wave waits out the LDS latency once per item.
        float xs_ring[3][2][DL];
        load_x(xs_ring[0], 0);
        if constexpr (ITEMS > 1) load_x(xs_ring[1], 1);
        scores(acc_cur, xx_cur, 0, xs_ring[0]);
        static_for<ITEMS>([&](auto itc) {
            constexpr int it = decltype(itc)::value;
            constexpr int pl = it / TG, tg = it % TG;
            (void)tg;
            if constexpr (it + 2 < ITEMS) {
                load_x(xs_ring[(it + 2) % 3], it + 2);
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (it + 1 < ITEMS) scores(acc_nxt, xx_nxt, it + 1, xs_ring[(it + 1) % 3]);
            const float xx = xx_cur;
            // smallest (m1) and second smallest (m2) of the 16 id-tagged scores, 36 VALU operations:
            // five triples give (min3, med3) each; the overall second smallest is the smaller of
            // the second smallest of the six group minima and the smallest of the group medians.
            float key[16];
#pragma unroll
            for (int r = 0; r < 16; ++r)
                key[r] = __uint_as_float((__float_as_uint(acc_cur[r]) & ~15u) | (uint32_t)r);
            float lo[5], md[5];
#pragma unroll
            for (int i = 0; i < 5; ++i) {
                lo[i] = vmin3(key[3 * i], key[3 * i + 1], key[3 * i + 2]);
                md[i] = __builtin_amdgcn_fmed3f(key[3 * i], key[3 * i + 1], key[3 * i + 2]);
            }
            const float a1 = vmin3(lo[0], lo[1], lo[2]), a2 = __builtin_amdgcn_fmed3f(lo[0], lo[1], lo[2]);
            const float b1 = vmin3(lo[3], lo[4], key[15]), b2 = __builtin_amdgcn_fmed3f(lo[3], lo[4], key[15]);
            float m1 = vmin(a1, b1);
            float m2 = vmin3(vmin3(md[0], md[1], md[2]), vmin3(md[3], md[4], vmax(a1, b1)), vmin(a2, b2));
            uint32_t bi = __float_as_uint(m1) & 15u;
            if constexpr (WIDE) {
                // the other 16 centroids of the codebook were searched by lane l ^ 32: both lanes merge the
                // two (smallest, second smallest) pairs and reach the same outcome.  Equal tagged minima
                // give m2 == m1, which fails the margin test.
                const auto s1 = __builtin_amdgcn_permlane32_swap(__float_as_uint(m1), __float_as_uint(m1), false, false);
                const auto s2 = __builtin_amdgcn_permlane32_swap(__float_as_uint(m2), __float_as_uint(m2), false, false);
                const float m1lo = __uint_as_float(s1[0]), m1hi = __uint_as_float(s1[1]);
                const float m2lo = __uint_as_float(s2[0]), m2hi = __uint_as_float(s2[1]);
                m1 = vmin(m1lo, m1hi);
                m2 = vmin3(vmax(m1lo, m1hi), m2lo, m2hi);
                bi = (__float_as_uint(m1) & 15u) | (m1hi < m1lo ? 16u : 0u);
            }
            const float mag = xx + cmax[pl];
            // 2 * [ (v+1)u (|c|^2) + 16u (omitted products) + 2.02 (12v + NM) u (that many additions, each
            //       within u of a partial sum below 2.02 mag) + 2(v+2)u (the reference's own chain) ]
            //       = 2 * {80, 136, 251} u  for v = {2, 4, 8}
            constexpr float A2 = 2.0f * ((V + 1) + 16.0f + 2.02f * (12 * V + NM) + 2 * (V + 2)) * 5.9604645e-8f;
            constexpr float B2 = 2.0f * 16.0f * 2.3841858e-7f;               // 2 * 2^(4-22)
            const float thr = fmaf(A2, mag, fmaf(B2, fabsf(m2), 1.001e-6f));
            // NaN anywhere makes a compare false, which counts as "not safe"
            const bool safe = ((m2 - m1) > thr) && (mag < 1e36f);
            need |= (safe ? 0u : 1u) << it;
            if constexpr (WIDE)
                words[tg / 2] |= (h == 0 ? bi : 0u) << (16 * (tg % 2) + 8 * pl);  // one byte per codebook
            else
                words[tg / 2] |= bi << (16 * (tg % 2) + 8 * pl + 4 * h);
            if constexpr (it + 1 < ITEMS) {
                acc_cur = acc_nxt;
                xx_cur = xx_nxt;
            }
        });

        // ---- exact replay of the items that failed the margin test (rare) ---------------------------------
        // The reference's own arithmetic: per centroid the distance as a chain of single roundings, then one
        // pass over the centroids in order that moves to a centroid closer by more than 1e-6.
        const uint64_t replay_mask = __builtin_amdgcn_ballot_w64(need != 0);
        constexpr int COOP_MAX = V / 2;  // up to that many lanes: one at a time, by the whole wave (8 measured the same)
        if (replay_mask != 0 && __builtin_popcountll(WIDE ? (replay_mask & 0xFFFFFFFFull) : replay_mask) <= COOP_MAX) {
            // A lane's replay done by the wave: lane c computes the distance to centroid c, the pass over the
            // centroids reads them lane by lane.  A single lane doing all of it (below) keeps the other 63 waiting
            // for C x (3v + 4) operations; this is 3v + 5C.
            // wide: lanes l and l + 32 hold the same outcome, and lane l (h = 0) keeps the byte
            uint64_t mask = WIDE ? (replay_mask & 0xFFFFFFFFull) : replay_mask;
            const uint32_t wave_s = __builtin_amdgcn_readfirstlane(wave);
            while (mask) {
                const uint32_t l = (uint32_t)__builtin_ctzll(mask);
                mask &= mask - 1;
                uint32_t nd = __builtin_amdgcn_readlane(need, l);
                const uint32_t jl = l & 31, hl = l >> 5;
                while (nd) {
                    const uint32_t it = (uint32_t)__builtin_ctz(nd);
                    nd &= nd - 1;
                    const uint32_t pl = it / TG, tg = it % TG;
                    const uint32_t cbl = WIDE ? 2 * wave_s + pl : 2 * (2 * wave_s + pl) + hl;
                    uint32_t bi = 0;
                    if (tcb * RCB + cbl < CB) {
                        const float* xo = tile + (tg * 32 + jl) * PITCH + (2 * wave_s + pl) * XSTEP + (WIDE ? 0 : V * hl);
                        const uint32_t cl = lane < C ? lane : C - 1;  // lanes past the last centroid repeat it; never read
                        const float* cp = cst + (cbl * C + cl) * V;
                        float diff = __fsub_rn(xo[0], cp[0]);
                        float d = __fmul_rn(diff, diff);
#pragma unroll
                        for (int t = 1; t < V; ++t) {
                            diff = __fsub_rn(xo[t], cp[t]);
                            d = __fadd_rn(d, __fmul_rn(diff, diff));
                        }
                        float best = 0.0f;
                        for (uint32_t c = 0; c < C; ++c) {
                            const float dc = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(d), c));
                            const bool take = (c == 0) || (__fsub_rn(best, dc) > 1e-6f);
                            best = take ? dc : best;
                            bi = take ? c : bi;
                        }
                    }
                    const uint32_t sh = WIDE ? 16 * (tg % 2) + 8 * pl : 16 * (tg % 2) + 8 * pl + 4 * hl;
                    const uint32_t keep_mask = WIDE ? 255u : 15u;
                    const bool mine = lane == l;
#pragma unroll
                    for (int i = 0; i < TG / 2; ++i)
                        words[i] = (mine && tg / 2 == (uint32_t)i) ? ((words[i] & ~(keep_mask << sh)) | (bi << sh)) : words[i];
                }
            }
        } else if (replay_mask != 0) {
            // many lanes at once (ties: rows of zeros, repeated centroids): every lane replays its own items
            // kept rolled on purpose: the replay is rare and must not cost the fast path registers
#pragma nounroll
            for (int it = 0; it < ITEMS; ++it) {
                if (!((need >> it) & 1u)) continue;
                const int pl = it / TG, tg = it % TG;
                const uint32_t cbl = WIDE ? 2 * wave + pl : 2 * (2 * wave + pl) + h;  // codebook within the tile
                uint32_t bi = 0;
                if (tcb * RCB + cbl < CB) {
                    const float* xo = brow0 + tg * 32 * PITCH + pl * XSTEP + (WIDE ? 0 : V * h);
                    const float* cp = cst + cbl * C * V;
                    float best = 0.0f;
                    // eight centroids per trip: their rows are read from LDS together, and the wave waits for
                    // LDS once per trip instead of once per centroid (rolled, a replay took 1.5 us)
#pragma unroll 8
                    for (uint32_t c = 0; c < C; ++c) {
                        float diff = __fsub_rn(xo[0], cp[c * V + 0]);
                        float d = __fmul_rn(diff, diff);
#pragma unroll
                        for (int t = 1; t < V; ++t) {
                            diff = __fsub_rn(xo[t], cp[c * V + t]);
                            d = __fadd_rn(d, __fmul_rn(diff, diff));
                        }
                        const bool take = (c == 0) || (__fsub_rn(best, d) > 1e-6f);
                        best = take ? d : best;
                        bi = take ? c : bi;
                    }
                }
                // wide: both lanes of the pair replay all of the codebook's centroids; lane h = 0 keeps the byte
                const uint32_t sh = WIDE ? 16 * (tg % 2) + 8 * pl : 16 * (tg % 2) + 8 * pl + 4 * h;
                const uint32_t keep_mask = WIDE ? 255u : 15u;
                if (WIDE && h != 0) bi = 0;
                uint32_t w = words[0];
#pragma unroll
                for (int i = 1; i < TG / 2; ++i) w = (tg / 2 == i) ? words[i] : w;
                w = (w & ~(keep_mask << sh)) | (bi << sh);
#pragma unroll
                for (int i = 0; i < TG / 2; ++i) words[i] = (tg / 2 == i) ? w : words[i];
            }
        }

        // ---- merge the two codebooks of each pair (lanes l and l+32), gather the tile's index
        //      bytes in LDS, store 8 bytes per token ------------------------------------------------
#pragma unroll
        for (int i = 0; i < TG / 2; ++i) {  // lanes l and l + 32 exchange their words without going through LDS
            const auto sw = __builtin_amdgcn_permlane32_swap(words[i], words[i], false, false);
            words[i] = sw[0] | sw[1];
        }
        if (h == 0) {
#pragma unroll
            for (int tg = 0; tg < TG; ++tg)
                *reinterpret_cast<uint16_t*>(&ist[(32 * tg + j) * (CBW / 2) + 2 * wave]) =
                    (uint16_t)(words[tg / 2] >> (16 * (tg % 2)));
        }
        __syncthreads();  // index bytes complete; every wave is done with the activation tile
        if (threadIdx.x < TT) {
            const uint32_t tok = tok0 + threadIdx.x;
            if (tok < N) {
                const uint2 w = *reinterpret_cast<const uint2*>(&ist[threadIdx.x * (CBW / 2)]);
                if (idx_tiled) {
                    *reinterpret_cast<uint32_t*>(idx + idx_offset(tok, tcb * (CBW / 2), idx_row_bytes, 1)) = w.x;
                    *reinterpret_cast<uint32_t*>(idx + idx_offset(tok, tcb * (CBW / 2) + 4, idx_row_bytes, 1)) = w.y;
                } else {
                    *reinterpret_cast<uint2*>(idx + (size_t)tok * idx_row_bytes + tcb * (CBW / 2)) = w;
                }
            }
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
                                                         uint32_t idx_row_bytes, int idx_tiled)
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
    idx[idx_offset(tok, byte, idx_row_bytes, idx_tiled)] = (uint8_t)outv;
}

// packed indices -> uint16 at the reference's tiled offset (index_calc_host.cpp:41-49)
template <int IDX_BITS>
__global__ void unpack_idx_kernel(const uint8_t* __restrict__ idx, uint16_t* __restrict__ out,
                                  uint32_t N, uint32_t CB, uint32_t idx_row_bytes, int idx_tiled,
                                  uint32_t n_stile, uint32_t cb_mtile)
{
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)N * CB) return;
    const uint32_t n = gid / CB, cb = gid % CB;
    const uint8_t b = idx[idx_offset(n, cb * IDX_BITS / 8, idx_row_bytes, idx_tiled)];
    const uint16_t val = (IDX_BITS == 4) ? ((b >> (4 * (cb & 1))) & 0xF) : b;
    const uint64_t off = (uint64_t)(n / n_stile) * n_stile * CB + (uint64_t)(cb / cb_mtile) * n_stile * cb_mtile +
                         (uint64_t)(n % n_stile) * cb_mtile + (cb % cb_mtile);
    out[off] = val;
}

// uint16 centroid ids at the reference's tiled offset -> packed rows (padded codebooks get index 0)
template <int IDX_BITS>
__global__ void pack_idx_kernel(const uint16_t* __restrict__ in, uint8_t* __restrict__ idx, uint32_t N,
                                uint32_t CB, uint32_t idx_row_bytes, int idx_tiled, uint32_t n_stile,
                                uint32_t cb_mtile)
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
    idx[idx_offset(n, byte, idx_row_bytes, idx_tiled)] = (uint8_t)outv;
}

template <int V, int IDX_BITS>
int launch_ccs_t(Ctx* ctx, const AmmGeom& g, const float* d_x, const float* d_cent, uint8_t* d_idx, uint32_t n)
{
    using S = CcsShape<V>;
    const uint32_t cb_per_tile = S::WAVES * S::CBT;
    const uint32_t tiles_cb = (g.CB_pad + cb_per_tile - 1) / cb_per_tile;
    const uint64_t total64 = (uint64_t)((n + S::TILE_TOKENS - 1) / S::TILE_TOKENS) * tiles_cb;
    if (total64 > 0xFFFFFFFFull) return set_error(ctx, PIMDL_ERR_INVALID, "ccs: too many tiles");
    const uint32_t total = (uint32_t)total64;
    // persistent grid: as many workgroups as stay resident (LDS bound, at most 4 per CU)
    const uint32_t lds = S::LDS_BYTES;
    uint32_t per_cu = (uint32_t)(160 * 1024 / lds);
    if (per_cu > 4) per_cu = 4;
    if (per_cu < 1) per_cu = 1;
    const uint32_t slots = (uint32_t)ctx->prop.multiProcessorCount * per_cu;
    dim3 grid(total < slots ? total : slots);
    const int vec_ok = (g.K % 4 == 0) && ((reinterpret_cast<uintptr_t>(d_x) & 15) == 0);
    const float* aux = d_cent + (size_t)g.CB * g.C * g.v;
    const float* cnmax = aux + ccs_aux_floats(g);
    if (g.tune_search ? g.tune_search == PIMDL_SEARCH_SCAN : ccs_exact_only())
        hipLaunchKernelGGL((ccs_kernel<V, IDX_BITS, false>), grid, dim3(CCS_THREADS), 0, ctx->stream, d_x, d_cent,
                           aux, cnmax, d_idx, n, g.K, g.CB, g.C, g.idx_row_bytes, (int)g.idx_tiled, vec_ok, g.CB_pad, tiles_cb, total);
    else
        hipLaunchKernelGGL((ccs_kernel<V, IDX_BITS, true>), grid, dim3(CCS_THREADS), 0, ctx->stream, d_x, d_cent,
                           aux, cnmax, d_idx, n, g.K, g.CB, g.C, g.idx_row_bytes, (int)g.idx_tiled, vec_ok, g.CB_pad, tiles_cb, total);
    return hip_check(ctx, hipGetLastError(), "ccs_kernel launch");
}

template <int V>
int launch_ccs_mfma(Ctx* ctx, const AmmGeom& g, const float* d_x, const float* d_cent, uint8_t* d_idx, uint32_t n)
{
    using S = CcsMfmaShape<V>;
    const uint32_t tiles_cb = g.CB_pad / S::CBW;  // CB_pad is a multiple of 32
    const uint64_t total64 = (uint64_t)((n + S::TILE_TOKENS - 1) / S::TILE_TOKENS) * tiles_cb;
    if (total64 > 0xFFFFFFFFull) return set_error(ctx, PIMDL_ERR_INVALID, "ccs: too many tiles");
    const uint32_t total = (uint32_t)total64;
    // persistent grid: exactly the workgroups that are resident at once
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, ccs_mfma_kernel<V>, CCS_THREADS, 0) != hipSuccess ||
        per_cu < 1) {
        (void)hipGetLastError();
        per_cu = 1;
    }
    const uint32_t slots = (uint32_t)ctx->prop.multiProcessorCount * (uint32_t)per_cu;
    dim3 grid(total < slots ? total : slots);
    const int vec_ok = (g.K % 4 == 0) && ((reinterpret_cast<uintptr_t>(d_x) & 15) == 0);
    const float* aux = d_cent + (size_t)g.CB * g.C * g.v;
    const float* cnmax = aux + ccs_aux_floats(g);
    const float* aux_a = cnmax + g.CB;
    const float* cnmax_pad = aux_a + (size_t)(g.CB_pad / 2) * (g.v + 1) * 64;
    hipLaunchKernelGGL((ccs_mfma_kernel<V>), grid, dim3(CCS_THREADS), 0, ctx->stream, d_x, d_cent, aux_a, cnmax_pad,
                       d_idx, n, g.K, g.CB, g.C, g.idx_row_bytes, (int)g.idx_tiled, vec_ok, tiles_cb, total);
    return hip_check(ctx, hipGetLastError(), "ccs_mfma_kernel launch");
}

// PIMDL_CCS_F32=1 keeps the fp32 matrix-core search (same results; for comparison)
static bool ccs_f32_only()
{
    static const bool v = [] {
        const char* e = getenv("PIMDL_CCS_F32");
        return e && e[0] == '1';
    }();
    return v;
}

template <int V, bool WIDE, int TTOK>
int launch_ccs_bf16_tt(Ctx* ctx, const AmmGeom& g, const float* d_x, const float* d_cent, uint8_t* d_idx, uint32_t n,
                       uint32_t x_cols)
{
    using S = CcsMfmaShape<V, WIDE, TTOK>;
    const uint32_t tiles_cb = g.CB_pad / S::RCB;  // CB_pad is a multiple of 32
    const uint64_t total64 = (uint64_t)((n + S::TILE_TOKENS - 1) / S::TILE_TOKENS) * tiles_cb;
    if (total64 > 0xFFFFFFFFull) return set_error(ctx, PIMDL_ERR_INVALID, "ccs: too many tiles");
    const uint32_t total = (uint32_t)total64;
    // persistent grid: exactly the workgroups that are resident at once (asked once per kernel variant;
    // every device this library runs on is the same part)
    static int per_cu = 0;
    if (per_cu == 0) {
        int q = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&q, ccs_bf16_kernel<V, WIDE, TTOK>, CCS_THREADS, 0) != hipSuccess || q < 1) {
            (void)hipGetLastError();
            q = 1;
        }
        per_cu = q;
    }
    const uint32_t slots = (uint32_t)ctx->prop.multiProcessorCount * (uint32_t)per_cu;
    uint32_t grid_wgs = total < slots ? total : slots;
    // a grid that is a multiple of the codebook tiles gives every workgroup the same codebooks tile after tile,
    // and the kernel then keeps their operands; taken where it costs at most 4 % of the resident workgroups
    if (total > slots && tiles_cb <= slots && (slots / tiles_cb) * tiles_cb * 25 >= slots * 24) grid_wgs = (slots / tiles_cb) * tiles_cb;
    dim3 grid(grid_wgs);
    const uint32_t row = x_cols ? x_cols : g.K;  // floats per activation row
    const uint32_t tiles_x = x_cols ? x_cols / S::TF : tiles_cb;
    const int vec_ok = (row % 4 == 0) && ((reinterpret_cast<uintptr_t>(d_x) & 15) == 0);
    const float* aux = d_cent + (size_t)g.CB * g.C * g.v;
    const float* cnmax = aux + ccs_aux_floats(g);
    const float* cnmax_pad = cnmax + g.CB + (size_t)(g.CB_pad / 2) * (g.v + 1) * 64;
    const float* bf = d_cent + ccs_bf16_offset(g);
    const uint4* aux_b = reinterpret_cast<const uint4*>(bf);
    const float* cn16 = bf + ccs_bf16_units(g) * ccs_bf16_nm(V) * 64 * 4;
    hipLaunchKernelGGL((ccs_bf16_kernel<V, WIDE, TTOK>), grid, dim3(CCS_THREADS), 0, ctx->stream, d_x, d_cent, aux_b, cn16, cnmax_pad,
                       d_idx, n, row, g.CB, g.C, g.idx_row_bytes, (int)g.idx_tiled, vec_ok, tiles_cb, total, tiles_x);
    return hip_check(ctx, hipGetLastError(), "ccs_bf16_kernel launch");
}

// 128-token tiles amortise a tile's operand loads best, but a workgroup that gets only one or two of them
// cannot overlap a tile's loads with the previous tile's arithmetic: small batches use 64-token tiles.
template <int V, bool WIDE>
int launch_ccs_bf16(Ctx* ctx, const AmmGeom& g, const float* d_x, const float* d_cent, uint8_t* d_idx, uint32_t n,
                    uint32_t x_cols)
{
    const uint64_t tiles128 = (uint64_t)((n + 127) / 128) * (g.CB_pad / CcsMfmaShape<V, WIDE>::RCB);
    // 64-token tiles up to two 128-token tiles per resident workgroup: the grid fills more evenly, and since a
    // workgroup keeps the operands of its codebooks from tile to tile the extra tiles cost little (asking the
    // compiler for four workgroups per CU with them was measured slower: 10.9 against 10.1 us at K = 768)
    // (measured 64 / 128-token tiles, us: 6.1 / 8.7 at 192 tiles; 11.0 / 11.9 at 768; 14.8 / 15.5 at 1188;
    // 17.8 / 18.8 at 1536; 28.2 .. 31.5 / 28.2 .. 29.0 at 3072; 42.3 / 41.8 at 4752)
    // v = 8 with up to 16 centroids: the 128-token kernel (two workgroups per CU: 237 registers, 76 KB of LDS) beats
    // the 64-token one (three per CU, with spills) from half a tile per CU upwards (us, 64 / 128: 6.5 / 7.0 at 96
    // tiles, 8.3 / 7.0 at 192, 15.1 / 9.7 at 512, 26 / 24.5 at 1536, 35.7 / 33.5 at 2376)
    const uint64_t few = (V == 8 && !WIDE) ? ctx->prop.multiProcessorCount / 2 : 6ull * ctx->prop.multiProcessorCount;
    const bool small_tiles = g.tune_search_tile ? g.tune_search_tile == 64 : tiles128 <= few;
    if (small_tiles) return launch_ccs_bf16_tt<V, WIDE, 64>(ctx, g, d_x, d_cent, d_idx, n, x_cols);
    return launch_ccs_bf16_tt<V, WIDE, 128>(ctx, g, d_x, d_cent, d_idx, n, x_cols);
}

template <int IDX_BITS>
int launch_ccs_bits(Ctx* ctx, const AmmGeom& g, const float* d_x, const float* d_cent, uint8_t* d_idx, uint32_t n,
                    uint32_t x_cols)
{
    // the operator's own choice (pimdl_amm_tuning.search_kernel) comes before the environment's
    const bool exact = g.tune_search ? g.tune_search == PIMDL_SEARCH_SCAN : ccs_exact_only();
    const bool f32 = g.tune_search ? g.tune_search == PIMDL_SEARCH_MFMA_F32 : ccs_f32_only();
    if (IDX_BITS == 8 && g.C <= 32 && !exact && !f32) {
        switch (g.v) {
            case 2: return launch_ccs_bf16<2, true>(ctx, g, d_x, d_cent, d_idx, n, x_cols);
            case 4: return launch_ccs_bf16<4, true>(ctx, g, d_x, d_cent, d_idx, n, x_cols);
            case 8: return launch_ccs_bf16<8, true>(ctx, g, d_x, d_cent, d_idx, n, x_cols);
            default: break;
        }
    }
    if (IDX_BITS == 4 && !exact) {
        if (!f32) {
            switch (g.v) {
                case 2: return launch_ccs_bf16<2, false>(ctx, g, d_x, d_cent, d_idx, n, x_cols);
                case 4: return launch_ccs_bf16<4, false>(ctx, g, d_x, d_cent, d_idx, n, x_cols);
                case 8: return launch_ccs_bf16<8, false>(ctx, g, d_x, d_cent, d_idx, n, x_cols);
                default: break;
            }
        }
    }
    if (x_cols) return set_error(ctx, PIMDL_ERR_UNSUPPORTED, "shared-input search needs the matrix-core search kernel");
    if (IDX_BITS == 4 && !exact) {
        switch (g.v) {
            case 2: return launch_ccs_mfma<2>(ctx, g, d_x, d_cent, d_idx, n);
            case 4: return launch_ccs_mfma<4>(ctx, g, d_x, d_cent, d_idx, n);
            case 8: return launch_ccs_mfma<8>(ctx, g, d_x, d_cent, d_idx, n);
            default: break;
        }
    }
    switch (g.v) {
        case 2: return launch_ccs_t<2, IDX_BITS>(ctx, g, d_x, d_cent, d_idx, n);
        case 4: return launch_ccs_t<4, IDX_BITS>(ctx, g, d_x, d_cent, d_idx, n);
        case 8: return launch_ccs_t<8, IDX_BITS>(ctx, g, d_x, d_cent, d_idx, n);
        case 10: return launch_ccs_t<10, IDX_BITS>(ctx, g, d_x, d_cent, d_idx, n);  // the reference's hidden-dim sweep:
        case 16: return launch_ccs_t<16, IDX_BITS>(ctx, g, d_x, d_cent, d_idx, n);
        case 20: return launch_ccs_t<20, IDX_BITS>(ctx, g, d_x, d_cent, d_idx, n);  // token_dim 2560 and 5120 over 256 codebooks
        case 32: return launch_ccs_t<32, IDX_BITS>(ctx, g, d_x, d_cent, d_idx, n);
        default: {
            const uint64_t total = (uint64_t)n * (g.CB_pad / (8 / IDX_BITS));
            dim3 grid((uint32_t)((total + 255) / 256));
            hipLaunchKernelGGL((ccs_generic_kernel<IDX_BITS>), grid, dim3(256), 0, ctx->stream, d_x, d_cent, d_idx,
                               n, g.K, g.v, g.CB, g.CB_pad, g.C, g.idx_row_bytes, (int)g.idx_tiled);
            return hip_check(ctx, hipGetLastError(), "ccs_generic_kernel launch");
        }
    }
}

}  // namespace

// Measures what the bf16-split search assumes about the matrix core: a chain of three
// v_mfma_f32_32x32x16_bf16 (48 products + the initial accumulator) against the exact sum, over random
// operands whose pieces differ in magnitude like xh/xm/xl do.  Reports max |D - exact| / (u * sum|terms|).
// The search kernel's bound allows 2.02 (12 v + NM) u per partial sum, i.e. 51 in this unit for v = 4.
namespace {
__global__ void mfma_error_kernel(const uint4* __restrict__ a, const uint4* __restrict__ b, const float* __restrict__ c,
                                  float* __restrict__ d, int chain)
{
    const int l = threadIdx.x;
    a += (size_t)blockIdx.x * chain * 64;
    b += (size_t)blockIdx.x * chain * 64;
    c += (size_t)blockIdx.x * 1024;
    d += (size_t)blockIdx.x * 1024;
    floatx16 acc;
    for (int r = 0; r < 16; ++r) acc[r] = c[(8 * (r / 4) + 4 * (l / 32) + r % 4) * 32 + (l % 32)];
    for (int m = 0; m < chain; ++m)
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[m * 64 + l]),
                                                      __builtin_bit_cast(bf16x8, b[m * 64 + l]), acc, 0, 0, 0);
    for (int r = 0; r < 16; ++r) d[(8 * (r / 4) + 4 * (l / 32) + r % 4) * 32 + (l % 32)] = acc[r];
}
}  // namespace

// crafted: instead of random operands, chains built to make an accumulator lose as much as it can: an
// accumulator of 1.0 that receives 48 equal products just below / just above a half, one and two units in its
// last place (a sequential adder that rounds to nearest drops every product of the first kind, one that
// truncates also drops the larger ones), of either sign, and products whose magnitudes fall by a factor of
// four from slot to slot (bits shifted out when the terms of one instruction are aligned).  `trials` is
// ignored then.
constexpr uint32_t MFMA_CRAFTED_TRIALS = 14;
int launch_diag_mfma_error(Ctx* ctx, uint32_t trials, bool crafted, float* max_err_u)
{
    constexpr int CHAIN = 3;
    if (crafted) trials = MFMA_CRAFTED_TRIALS;
    if (trials == 0 || trials > 4096) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_diag_mfma_error: trials must be in 1..4096");
    std::vector<uint16_t> A((size_t)trials * CHAIN * 32 * 16), B((size_t)trials * CHAIN * 16 * 32);
    std::vector<float> C((size_t)trials * 1024), D((size_t)trials * 1024);
    uint64_t st = 0x9E3779B97F4A7C15ull;
    auto next = [&]() {  // splitmix64
        uint64_t z = (st += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    };
    auto unif = [&]() { return (float)((double)(next() >> 11) / 9007199254740992.0 * 2.0 - 1.0); };
    auto to_bf16 = [](float f) { uint32_t u; memcpy(&u, &f, 4); return (uint16_t)(u >> 16); };
    auto from_bf16 = [](uint16_t h) { uint32_t u = (uint32_t)h << 16; float f; memcpy(&f, &u, 4); return f; };
    for (uint32_t t = 0; crafted && t < trials; ++t) {
        static const float mags[6] = {0.4921875f, 0.5078125f, 0.9921875f, 1.0078125f, 1.984375f, 2.015625f};  // 8-bit significands
        const float sign = (t & 1) ? -1.0f : 1.0f;
        for (int m = 0; m < CHAIN; ++m)
            for (int r = 0; r < 32; ++r)
                for (int kk = 0; kk < 16; ++kk) {
                    // A[r][kk] * B[kk][r]: 2^-12 * (sign * mag * 2^-12) = sign * mag * 2^-24, or the falling staircase
                    const float a = t < 12 ? ldexpf(1.0f, -12) : 1.0f;
                    const float b = t < 12 ? sign * ldexpf(mags[t / 2], -12) : sign * ldexpf(1.9921875f, -2 * kk - 1);
                    A[((size_t)(t * CHAIN + m) * 32 + r) * 16 + kk] = to_bf16(a);
                    B[((size_t)(t * CHAIN + m) * 16 + kk) * 32 + r] = to_bf16(b);
                }
        for (size_t i = 0; i < 1024; ++i) C[(size_t)t * 1024 + i] = 1.0f;
    }
    for (uint32_t t = 0; !crafted && t < trials; ++t) {
        const float small = ldexpf(1.0f, (int)(t % 5) * 6 - 24);
        for (size_t i = 0; i < (size_t)CHAIN * 512; ++i) {
            A[(size_t)t * CHAIN * 512 + i] = to_bf16(3.0f * unif() * ((next() & 1) ? 1.0f : small));
            B[(size_t)t * CHAIN * 512 + i] = to_bf16(3.0f * unif() * ((next() & 3) ? 1.0f : small));
        }
        for (size_t i = 0; i < 1024; ++i) C[(size_t)t * 1024 + i] = 8.0f * unif();
    }
    std::vector<uint4> ha((size_t)trials * CHAIN * 64), hb((size_t)trials * CHAIN * 64);
    for (uint32_t t = 0; t < trials; ++t)
        for (int m = 0; m < CHAIN; ++m)
            for (int l = 0; l < 64; ++l) {
                uint16_t pa[8], pb[8];
                for (int e = 0; e < 8; ++e) {
                    const int kk = 8 * (l / 32) + e;
                    pa[e] = A[((size_t)(t * CHAIN + m) * 32 + l % 32) * 16 + kk];
                    pb[e] = B[((size_t)(t * CHAIN + m) * 16 + kk) * 32 + l % 32];
                }
                memcpy(&ha[(size_t)(t * CHAIN + m) * 64 + l], pa, 16);
                memcpy(&hb[(size_t)(t * CHAIN + m) * 64 + l], pb, 16);
            }
    uint4 *da = nullptr, *db = nullptr;
    float *dc = nullptr, *dd = nullptr;
    int rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&da), ha.size() * 16), "hipMalloc(diag)");
    if (!rc) rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&db), hb.size() * 16), "hipMalloc(diag)");
    if (!rc) rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&dc), C.size() * 4), "hipMalloc(diag)");
    if (!rc) rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&dd), D.size() * 4), "hipMalloc(diag)");
    if (!rc) rc = hip_check(ctx, hipMemcpy(da, ha.data(), ha.size() * 16, hipMemcpyHostToDevice), "H2D diag");
    if (!rc) rc = hip_check(ctx, hipMemcpy(db, hb.data(), hb.size() * 16, hipMemcpyHostToDevice), "H2D diag");
    if (!rc) rc = hip_check(ctx, hipMemcpy(dc, C.data(), C.size() * 4, hipMemcpyHostToDevice), "H2D diag");
    if (!rc) {
        hipLaunchKernelGGL(mfma_error_kernel, dim3(trials), dim3(64), 0, ctx->stream, da, db, dc, dd, CHAIN);
        rc = hip_check(ctx, hipGetLastError(), "mfma_error_kernel launch");
    }
    if (!rc) rc = hip_check(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    if (!rc) rc = hip_check(ctx, hipMemcpy(D.data(), dd, D.size() * 4, hipMemcpyDeviceToHost), "D2H diag");
    (void)hipFree(da);
    (void)hipFree(db);
    (void)hipFree(dc);
    (void)hipFree(dd);
    if (rc) return rc;
    double worst = 0.0;
    for (uint32_t t = 0; t < trials; ++t)
        for (int i = 0; i < 32; ++i)
            for (int j = 0; j < 32; ++j) {
                double ex = C[(size_t)t * 1024 + i * 32 + j], sabs = fabs(ex);
                for (int m = 0; m < CHAIN; ++m)
                    for (int kk = 0; kk < 16; ++kk) {
                        const double p = (double)from_bf16(A[((size_t)(t * CHAIN + m) * 32 + i) * 16 + kk]) *
                                         (double)from_bf16(B[((size_t)(t * CHAIN + m) * 16 + kk) * 32 + j]);
                        ex += p;
                        sabs += fabs(p);
                    }
                const double e = fabs((double)D[(size_t)t * 1024 + i * 32 + j] - ex) / (5.9604644775390625e-8 * sabs);
                if (e > worst) worst = e;
            }
    *max_err_u = (float)worst;
    return PIMDL_OK;
}

// PIMDL_CCS_EXACT=1 in the environment switches the two-speed search off (every pair takes the
// reference's scan); the results are the same by construction, so this is a debugging aid only.
bool ccs_exact_only()
{
    static const bool v = [] {
        const char* e = getenv("PIMDL_CCS_EXACT");
        return e && e[0] == '1';
    }();
    return v;
}

size_t ccs_centroid_bytes(const AmmGeom& g)
{
    return (ccs_bf16_offset(g) + ccs_bf16_floats(g)) * sizeof(float);
}

int launch_ccs_prep(Ctx* ctx, const AmmGeom& g, float* d_cent)
{
    float* aux = d_cent + (size_t)g.CB * g.C * g.v;
    float* cnmax = aux + ccs_aux_floats(g);
    hipLaunchKernelGGL(ccs_prep_kernel, dim3(g.CB), dim3(64), 0, ctx->stream,
                       d_cent, aux, cnmax, g.C, g.v);
    int rc = hip_check(ctx, hipGetLastError(), "ccs_prep_kernel launch");
    if (rc) return rc;
    float* aux_a = cnmax + g.CB;
    hipLaunchKernelGGL(ccs_prep_mfma_kernel, dim3(g.CB_pad / 2), dim3(64), 0, ctx->stream, d_cent, cnmax, aux_a,
                       aux_a + (size_t)(g.CB_pad / 2) * (g.v + 1) * 64, g.CB, g.C, g.v);
    rc = hip_check(ctx, hipGetLastError(), "ccs_prep_mfma_kernel launch");
    if (rc || !ccs_has_bf16(g)) return rc;
    float* bf = d_cent + ccs_bf16_offset(g);
    uint4* aux_b = reinterpret_cast<uint4*>(bf);
    float* cn16 = bf + ccs_bf16_units(g) * ccs_bf16_nm(g.v) * 64 * 4;
    const dim3 pg((uint32_t)ccs_bf16_units(g)), pb(64);
    const bool wide = ccs_bf16_wide(g);
#define PIMDL_PREP_BF16(V_)                                                                                        \
    if (wide) hipLaunchKernelGGL((ccs_prep_bf16_kernel<V_, true>), pg, pb, 0, ctx->stream, d_cent, aux_b, cn16, g.CB, g.C); \
    else hipLaunchKernelGGL((ccs_prep_bf16_kernel<V_, false>), pg, pb, 0, ctx->stream, d_cent, aux_b, cn16, g.CB, g.C);
    switch (g.v) {
        case 2: PIMDL_PREP_BF16(2) break;
        case 4: PIMDL_PREP_BF16(4) break;
        default: PIMDL_PREP_BF16(8) break;
    }
#undef PIMDL_PREP_BF16
    return hip_check(ctx, hipGetLastError(), "ccs_prep_bf16_kernel launch");
}

uint32_t ccs_cb_per_wg(uint32_t v)
{
    switch (v) {
        case 2: return CcsShape<2>::WAVES * CcsShape<2>::CBT;
        case 4: return CcsShape<4>::WAVES * CcsShape<4>::CBT;
        case 8: return CcsShape<8>::WAVES * CcsShape<8>::CBT;
        case 10: return CcsShape<10>::WAVES * CcsShape<10>::CBT;
        case 16: return CcsShape<16>::WAVES * CcsShape<16>::CBT;
        case 20: return CcsShape<20>::WAVES * CcsShape<20>::CBT;
        case 32: return CcsShape<32>::WAVES * CcsShape<32>::CBT;
        default: return 0;
    }
}

int launch_ccs(Ctx* ctx, const AmmGeom& g, const float* d_x, const float* d_cent, uint8_t* d_idx, uint32_t n,
               uint32_t x_cols)
{
    if (n == 0) return PIMDL_OK;
    return g.idx_bits == 4 ? launch_ccs_bits<4>(ctx, g, d_x, d_cent, d_idx, n, x_cols)
                           : launch_ccs_bits<8>(ctx, g, d_x, d_cent, d_idx, n, x_cols);
}

// Can launch_ccs search the codebooks of several operators that read rows of x_cols floats?  Needs the
// matrix-core kernel and whole codebook tiles per operator.
bool ccs_supports_shared_input(const AmmGeom& g, uint32_t x_cols)
{
    if (!ccs_has_bf16(g)) return false;
    if (g.tune_search ? g.tune_search != PIMDL_SEARCH_MFMA_BF16 : (ccs_exact_only() || ccs_f32_only())) return false;
    const uint32_t tf = (ccs_bf16_wide(g) ? 8 : 16) * g.v;
    return x_cols % tf == 0;
}

int launch_unpack_idx(Ctx* ctx, const AmmGeom& g, const uint8_t* d_idx, uint16_t* d_idx16, uint32_t n,
                      uint32_t n_stile, uint32_t cb_mtile)
{
    if (n == 0) return PIMDL_OK;
    const uint64_t total = (uint64_t)n * g.CB;
    dim3 grid((uint32_t)((total + 255) / 256));
    if (g.idx_bits == 4)
        hipLaunchKernelGGL((unpack_idx_kernel<4>), grid, dim3(256), 0, ctx->stream, d_idx, d_idx16, n, g.CB,
                           g.idx_row_bytes, (int)g.idx_tiled, n_stile, cb_mtile);
    else
        hipLaunchKernelGGL((unpack_idx_kernel<8>), grid, dim3(256), 0, ctx->stream, d_idx, d_idx16, n, g.CB,
                           g.idx_row_bytes, (int)g.idx_tiled, n_stile, cb_mtile);
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
                           g.idx_row_bytes, (int)g.idx_tiled, n_stile, cb_mtile);
    else
        hipLaunchKernelGGL((pack_idx_kernel<8>), grid, dim3(256), 0, ctx->stream, d_idx16, d_idx, n, g.CB,
                           g.idx_row_bytes, (int)g.idx_tiled, n_stile, cb_mtile);
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
