// Pieces shared by the gather kernels of libpimdl (gfx950 only): the epilogue's parameters and arithmetic,
// the dealing of work items to the XCDs, and the inline-assembly LDS reads whose completion the kernels
// wait for by hand.
#pragma once
#include <type_traits>

#include "pimdl_internal.h"

namespace pimdl {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

struct Epilogue {
    float scale;
    float lut_bias_term;  // lut_bias or lut_bias*CB, already rounded to fp32 like the reference does
    const float* bias;    // [M] or nullptr
    uint32_t act;         // pimdl_activation
    // Several operators side by side in one launch (one-hot kernel only): column tiles
    // k * op_col_tiles .. (k+1) * op_col_tiles - 1 belong to operator k, which has its own scale and whose
    // index bytes start op_idx_stride * k bytes into the index buffer.  op_col_tiles == 0: one operator.
    const float* op_scales;
    uint32_t op_col_tiles, op_idx_stride;
};

// Time of a launch whose persistent grid of `slots` workgroups (two per CU) shares `items` equal items, in units
// of a full round.  Whole rounds cost 1 each.  A partly filled round costs less than a full one, because a
// workgroup that has a CU to itself runs faster (one item per CU: 0.65 of the time two per CU take, measured with
// the sparse kernel's 256-token items at 768 -> 3072: 256 items 13.7 us, 512 items 20.9 us after the launch's
// fixed 4.4 us), and after the first round the stragglers of a round also overlap with the round before
// (640 items 1.40, 768 items 1.48, 1024 items 2.0 rounds).
inline double grid_rounds(uint64_t items, uint64_t slots)
{
    const uint64_t full = items / slots, rem = items % slots;
    if (rem == 0) return (double)full;
    if (2 * rem > slots) return (double)full + 0.9;
    return (double)full + (full == 0 ? 0.65 : 0.5);
}
// Time of one item of the matrix-core gathers relative to a 256-token x 96-column one (same number of codebooks):
// 64- and 48-column tiles read the one-hot operand for fewer column groups (measured per round at 768 -> 3072,
// N = 8192, launch overhead taken off: 21.5 / 14.7 / 13.1 us; 27.9 / 19.2 at 1024 -> 4096; the 64-column figure is
// set a little above the measured 0.68 .. 0.72 so that near ties go to the wider tile, which won them: 768 -> 3072
// at N = 12608 with 32 centroids, 131.8 against 139.3 us); a 128-token item takes 0.62 of a 256-token one.
inline double item_cost(uint32_t tn, bool small_item) { return (tn >= 6 ? 1.0 : tn == 4 ? 0.72 : 0.61) * (small_item ? 0.62 : 1.0); }
// 128-token items instead of 256-token ones where that is the shorter launch by the two figures above.
inline bool prefer_small_items(uint64_t items256, uint64_t items128, uint64_t slots)
{
    return grid_rounds(items128, slots) * 0.62 < grid_rounds(items256, slots);
}

// How the items (column tile x token tile) of a gather are dealt to the 8 XCDs.  Workgroup b takes
// positions b, b + grid, ... of the item sequence and the hardware places workgroups on the XCDs
// round-robin, so (for a grid that is a multiple of 8) positions congruent mod 8 run on one XCD, each
// with an L2 of its own.  XCD x = cx + col_split * tx then owns the column tiles congruent to cx mod
// col_split and the token tiles congruent to tx mod tok_split (col_split * tok_split = 8), and its L2
// fetches only that share of the LUT and of the index buffer instead of all of both.
// col_split = 0: plain order, position p = column tile p / n_token_tiles, token tile p % n_token_tiles.
struct XcdMap {
    uint32_t col_split, tok_split, tok_per_xcd;  // tok_per_xcd = n_token_tiles / tok_split
    __device__ __forceinline__ void decode(uint32_t p, uint32_t n_token_tiles, uint32_t& col, uint32_t& tok) const
    {
        if (col_split == 0) {
            col = p / n_token_tiles;
            tok = p % n_token_tiles;
        } else {
            const uint32_t x = p % 8, q = p / 8;
            col = x % col_split + col_split * (q / tok_per_xcd);
            tok = x / col_split + tok_split * (q % tok_per_xcd);
        }
    }
};

// Picks the split with the least L2 fill traffic: 8 * (lut_bytes / col_split + idx_bytes / tok_split).
// forced: the caller's column split (pimdl_amm_tuning.xcd_col_split), used when it divides the tile counts
inline XcdMap choose_xcd_map(uint32_t n_col_tiles, uint32_t n_token_tiles, uint32_t grid, uint64_t lut_bytes,
                             uint64_t idx_bytes, uint32_t forced = 0)
{
    XcdMap best{0, 0, 0};
    if (grid % 8 != 0 || forced == PIMDL_XCD_PLAIN) return best;
    if (forced && n_col_tiles % forced == 0 && n_token_tiles % (8 / forced) == 0)
        return XcdMap{forced, 8 / forced, n_token_tiles / (8 / forced)};
    uint64_t best_cost = lut_bytes + idx_bytes / 8 + 1;  // plain order: every XCD reads the whole LUT
    best_cost *= 8;
    for (uint32_t cs = 8; cs >= 1; cs /= 2) {
        const uint32_t ts = 8 / cs;
        if (n_col_tiles % cs != 0 || n_token_tiles % ts != 0) continue;
        const uint64_t cost = 8 * (lut_bytes / cs + idx_bytes / ts);
        if (cost < best_cost) {
            best_cost = cost;
            best = XcdMap{cs, ts, n_token_tiles / ts};
        }
    }
    return best;
}

constexpr int GATHER_WAVES = 8;
constexpr int GATHER_THREADS = GATHER_WAVES * 64;

// The tanh form of GELU, 0.5 y (1 + tanh u) with u = sqrt(2/pi) (y + 0.044715 y^3), evaluated as
// y * sigmoid(2u) = y / (1 + exp(-2u)): no cancellation of 1 + tanh u for negative y, exp overflow gives
// y / inf = -0, and one v_exp_f32 plus one v_rcp_f32 (1 ulp each) keep it within 1e-6 relative.
__device__ __forceinline__ float gelu_tanh(float y)
{
    constexpr float k0 = -2.0f * 0.7978845608028654f * 1.4426950408889634f;  // -2 sqrt(2/pi) log2(e)
    constexpr float k1 = k0 * 0.044715f;
    const float w = y * __builtin_fmaf(y * y, k1, k0);  // -2u log2(e)
    return y * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(w));
}

__device__ __forceinline__ float activate(float y, uint32_t act)  // act is uniform over the launch
{
    return act == PIMDL_ACT_GELU_TANH ? gelu_tanh(y) : y;
}

// ACT: the epilogues are compiled once per activation and chosen by a (uniform) branch; as a select the
// activation's arithmetic would run for every element of every launch
template <bool ACT>
__device__ __forceinline__ float dequant(int32_t acc, const Epilogue& ep, float b)
{
    // ((float)acc * scale + lut_bias_term) + bias[f]   -- three separately rounded fp32 operations
    const float y = __fadd_rn(__fadd_rn(__fmul_rn((float)acc, ep.scale), ep.lut_bias_term), b);
    return ACT ? gelu_tanh(y) : y;
}

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

template <int OFF>
__device__ __forceinline__ void lds_read(v4i& slot, uint32_t addr)
{
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(slot) : "v"(addr), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ void lds_read32(uint32_t& dst, uint32_t addr)
{
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}

template <int OFF>
__device__ __forceinline__ void lds_read_u8(uint32_t& dst, uint32_t addr)
{
    asm volatile("ds_read_u8 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}

// Loads through the scalar data cache (read only) of wave-uniform addresses; they count on the
// scalar/LDS counter, not on the vector-memory counter.
typedef float floatx16 __attribute__((ext_vector_type(16)));
__device__ __forceinline__ floatx16 scalar_load16(const float* p)  // p: 4-byte aligned, wave-uniform
{
    floatx16 r;
    asm volatile("s_load_dwordx16 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(r) : "s"(p) : "memory");
    return r;
}
__device__ __forceinline__ float scalar_load1(const float* p)
{
    float r;
    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(r) : "s"(p) : "memory");
    return r;
}

}  // namespace
}  // namespace pimdl
