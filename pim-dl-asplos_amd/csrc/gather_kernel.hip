// LUT gather-accumulate for gfx950 (MI355X).
//
// Replaces the DPU kernel of the reference (inference-engine/src/dpu/pim_lut_kernel.c:97-2296; its
// row-major statement is inference-engine/test/test_amm.cpp:164-175) and the host epilogue
// (inference-engine/src/host/pim_lut_host.cpp:190-203 / test_amm.cpp:178-181):
//     acc[n][f] = sum over cb of lut[cb][idx[n][cb]][f]          (int8 table, int32 sum, exact)
//     out[n][f] = (float)acc * scale + lut_bias(*CB) + bias[f]   (fp32, left to right, unfused)
//
// The path is bound by LDS read bandwidth: every gathered LUT byte is read once from LDS
// (N*CB*M bytes), while HBM only sees the packed indices, the LUT slices and the output.
//
// int8 kernel.  A workgroup owns a tile of tokens x one column block (16*Q columns) and walks the
// codebooks in slices that are staged into LDS (double buffered; the next slice is fetched into
// registers while the current one is consumed).  Inside a wave, lane l = 16*g + j works for token j
// of a 16-token group and for the g-th quarter of the slice's codebooks: it turns its 4/8-bit index
// into an LDS row address and issues one ds_read_b128 per 16-column chunk.  The four lane groups
// therefore hold 16-byte row pieces of four different codebooks for the same 16 tokens -- which is
// exactly the B operand (K=64 x N=16, 16 consecutive K per lane) of v_mfma_i32_16x16x64_i8.  With a
// constant A operand A[i][16*g + b] = (b == i), the MFMA computes
//     D[i][j] += sum over g of byte_i(row piece of lane (j, g)),
// i.e. it adds the four gathered bytes of column i for token j into an int32 accumulator: the matrix
// core is used as a 1024-bytes-per-instruction byte adder, the VALU only forms addresses, and the
// sum stays exact.  (This is not the one-hot GEMM formulation: no work is multiplied by C.)
// D leaves the MFMA as 4 consecutive columns per lane, so the epilogue stores float4.
//
// Bank conflicts.  gfx950 serves a ds_read_b128 in four passes of 16 lanes over 64 four-byte banks,
// and the 16 lanes of a pass are NOT consecutive: the passes are lanes {0-3,12-15,20-27},
// {4-11,16-19,28-31}, {32-35,44-47,52-59}, {36-43,48-51,60-63} (measured with a pairwise probe).
// Each pass therefore holds all 16 tokens of the group but lanes of two MFMA K-blocks.  The MFMA
// only needs the four lanes (j, 0..3) of a token to cover four different codebooks, in any order,
// so a lane takes the codebook quarter of its *pass* (K-block g, flipped in bit 0 for tokens 4..11)
// and every pass reads one codebook only.  LDS rows are pitched 16*Q + 16 bytes: with an odd number
// of 16-byte units per row the 16 rows of a codebook start in 16 different bank quads, so a pass
// never conflicts whatever the indices are (equal indices read the same address and broadcast).
//
// fp32 kernel.  Same staging; one lane owns one token and adds rows in ascending codebook order
// (bit-identical to a sequential CPU sum).
#include <type_traits>

#include "pimdl_internal.h"

namespace pimdl {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

struct Epilogue {
    float scale;
    float lut_bias_term;  // lut_bias or lut_bias*CB, already rounded to fp32 like the reference does
    const float* bias;    // [M] or nullptr
};

constexpr int GATHER_WAVES = 8;
constexpr int GATHER_THREADS = GATHER_WAVES * 64;

__device__ __forceinline__ float dequant(int32_t acc, float scale, float lut_bias_term, float b)
{
    // ((float)acc * scale + lut_bias_term) + bias[f]   -- three separately rounded fp32 operations
    return __fadd_rn(__fadd_rn(__fmul_rn((float)acc, scale), lut_bias_term), b);
}

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// The three building blocks of the gather pipeline.  They are inline assembly because the order
// "wait for the oldest read, feed it to the matrix core, re-arm the slot with the next read" is the
// whole point, and the compiler's scheduler serialises the equivalent C++ (one read in flight).
template <int OFF>
__device__ __forceinline__ void lds_read(v4i& slot, uint32_t addr)
{
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(slot) : "v"(addr), "n"(OFF));
}
template <int OFF, int WAIT>
__device__ __forceinline__ void mfma_then_read(v4i& acc, v4i& slot, const v4i& a, uint32_t addr)
{
    asm volatile(
        "s_waitcnt lgkmcnt(%4)\n\t"
        "v_mfma_i32_16x16x64_i8 %0, %2, %1, %0\n\t"
        "ds_read_b128 %1, %3 offset:%5"
        : "+v"(acc), "+v"(slot)
        : "v"(a), "v"(addr), "n"(WAIT), "n"(OFF));
}
template <int WAIT>
__device__ __forceinline__ void mfma_last(v4i& acc, const v4i& slot, const v4i& a)
{
    asm volatile(
        "s_waitcnt lgkmcnt(%3)\n\t"
        "v_mfma_i32_16x16x64_i8 %0, %2, %1, %0"
        : "+v"(acc)
        : "v"(slot), "v"(a), "n"(WAIT));
}

// C_T: centroid rows per codebook in the tiled LUT (power of two >= C)
// Q:   16-byte chunks per row (column block = 16*Q)
// GQ:  codebooks per lane group per slice (slice = 4*GQ codebooks)
// TG:  16-token groups per wave (tokens per workgroup = 8 waves * TG * 16)
template <int C_T, int Q, int GQ, int TG, int IDX_BITS>
__global__ __launch_bounds__(GATHER_THREADS) void gather_i8_kernel(
    const uint8_t* __restrict__ idx, const int8_t* __restrict__ lut, float* __restrict__ out,
    int32_t* __restrict__ acc_out, uint32_t N, uint32_t M, uint32_t CB_pad, uint32_t idx_row_bytes,
    Epilogue ep)
{
    constexpr int G = 4 * GQ;                     // codebooks per slice
    constexpr int FB = 16 * Q;                    // columns (= bytes) per row
    constexpr int PITCH = FB + 16;                // LDS row pitch
    constexpr int CB_BYTES = C_T * PITCH;         // LDS bytes per codebook
    constexpr int SLICE_LDS = G * CB_BYTES;
    constexpr int SLICE_UNITS = G * C_T * Q;      // 16-byte units per slice in HBM
    constexpr int UPT = (SLICE_UNITS + GATHER_THREADS - 1) / GATHER_THREADS;
    constexpr int IDX_BYTES = GQ * IDX_BITS / 8;  // index bytes one lane needs per slice and token
    static_assert(IDX_BYTES == 1 || IDX_BYTES == 2 || IDX_BYTES == 4, "index fetch width");
    static_assert((GQ - 1) * CB_BYTES + (Q - 1) * 16 < 65536, "ds_read immediate offset range");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t j = lane & 15;  // token within the 16-token group (MFMA column)
    const uint32_t g = lane >> 4;  // MFMA K-block of this lane; also selects its 4 output columns
    // codebook quarter = index of the LDS pass this lane is served in (see "Bank conflicts" above)
    const uint32_t gq = g ^ (((j + 4) >> 3) & 1);
    const uint32_t tok0 = blockIdx.x * (GATHER_WAVES * TG * 16) + wave * (TG * 16);
    const uint32_t colblk = blockIdx.y;
    const uint32_t nslices = CB_pad / G;

    const uint4* __restrict__ lut_blk =
        reinterpret_cast<const uint4*>(lut) + (size_t)colblk * CB_pad * C_T * Q;

    // constant A operand: byte (lane % 16) of the lane's 16 bytes is 1
    const int one_hot = 1 << (8 * (j & 3));
    const v4i a_sel = {(j >> 2) == 0 ? one_hot : 0, (j >> 2) == 1 ? one_hot : 0, (j >> 2) == 2 ? one_hot : 0,
                       (j >> 2) == 3 ? one_hot : 0};

    // per token group: pointer to this lane's index bytes of slice 0
    const uint8_t* idx_ptr[TG];
#pragma unroll
    for (int t = 0; t < TG; ++t) {
        uint32_t tok = tok0 + t * 16 + j;
        if (tok >= N) tok = N - 1;  // clamp: results of such lanes are never stored
        idx_ptr[t] = idx + (size_t)tok * idx_row_bytes + (size_t)(gq * GQ) * IDX_BITS / 8;
    }
    auto load_idx = [](const uint8_t* base, uint32_t s) -> uint32_t {
        const uint8_t* p = base + (size_t)s * G * IDX_BITS / 8;
        if constexpr (IDX_BYTES == 4) return *reinterpret_cast<const uint32_t*>(p);
        else if constexpr (IDX_BYTES == 2) return *reinterpret_cast<const uint16_t*>(p);
        else return *p;
    };

    v4i acc[TG][Q], slot[TG][Q];
#pragma unroll
    for (int t = 0; t < TG; ++t)
#pragma unroll
        for (int c = 0; c < Q; ++c) acc[t][c] = (v4i){0, 0, 0, 0};

    // ---- main loop: the next slice travels HBM -> registers while the current one is consumed ----
    uint4 stage[UPT];
    uint32_t idx_cur[TG], idx_nxt[TG];
#define PIMDL_FETCH_SLICE(S)                                                                        \
    {                                                                                               \
        const uint4* src_ = lut_blk + (size_t)(S) * SLICE_UNITS;                                    \
        _Pragma("unroll") for (int u = 0; u < UPT; ++u)                                             \
        {                                                                                           \
            const uint32_t unit_ = threadIdx.x + u * GATHER_THREADS;                                \
            stage[u] = (SLICE_UNITS % GATHER_THREADS == 0 || unit_ < SLICE_UNITS) ? src_[unit_]     \
                                                                                  : make_uint4(0, 0, 0, 0); \
        }                                                                                           \
    }
#define PIMDL_COMMIT_SLICE(BUF)                                                                     \
    {                                                                                               \
        unsigned char* dst_ = smem + (BUF) * SLICE_LDS;                                             \
        _Pragma("unroll") for (int u = 0; u < UPT; ++u)                                             \
        {                                                                                           \
            const uint32_t unit_ = threadIdx.x + u * GATHER_THREADS;                                \
            if (SLICE_UNITS % GATHER_THREADS == 0 || unit_ < SLICE_UNITS)                           \
                *reinterpret_cast<uint4*>(dst_ + (unit_ / Q) * PITCH + (unit_ % Q) * 16) = stage[u]; \
        }                                                                                           \
    }
    PIMDL_FETCH_SLICE(0)
#pragma unroll
    for (int t = 0; t < TG; ++t) idx_cur[t] = load_idx(idx_ptr[t], 0);
    PIMDL_COMMIT_SLICE(0)
    __syncthreads();

    const uint32_t lane_base = gq * GQ * CB_BYTES;
    for (uint32_t s = 0; s < nslices; ++s) {
        // the last iteration re-fetches its own slice (into the idle buffer) instead of branching
        const uint32_t sn = s + 1 < nslices ? s + 1 : s;
        PIMDL_FETCH_SLICE(sn)
#pragma unroll
        for (int t = 0; t < TG; ++t) idx_nxt[t] = load_idx(idx_ptr[t], sn);
        // keep the prefetch of the next slice (and of its indices) at the top of the iteration
        __builtin_amdgcn_sched_barrier(0);
        const uint32_t buf = (s & 1) * SLICE_LDS + lane_base;
        // LDS byte address of the row each token group gathers from, for every codebook of the quarter
        uint32_t row_addr[GQ][TG];
#pragma unroll
        for (int q = 0; q < GQ; ++q)
#pragma unroll
            for (int t = 0; t < TG; ++t)
                row_addr[q][t] = buf + ((idx_cur[t] >> (IDX_BITS * q)) & ((1u << IDX_BITS) - 1)) * PITCH;
        // Rolling pipeline, one register slot per accumulator: the row piece for (q+1, t, c) is
        // requested into the slot as soon as the MFMA for (q, t, c) has consumed it, so TG*Q reads
        // stay in flight behind the matrix core.  Waits are explicit: LDS returns in order, and
        // lgkmcnt(TG*Q-1) before an MFMA means "the oldest outstanding read has landed".
        static_for<0, TG * Q>([&](auto i) {
            constexpr int t = i / Q, c = i % Q;
            lds_read<c * 16>(slot[t][c], row_addr[0][t]);
        });
        static_for<0, GQ - 1>([&](auto q) {
            static_for<0, TG * Q>([&](auto i) {
                constexpr int t = i / Q, c = i % Q;
                mfma_then_read<(q + 1) * CB_BYTES + c * 16, TG * Q - 1>(acc[t][c], slot[t][c], a_sel,
                                                                       row_addr[q + 1][t]);
            });
        });
        static_for<0, TG * Q>([&](auto i) {
            constexpr int t = i / Q, c = i % Q;
            mfma_last<TG * Q - 1 - i>(acc[t][c], slot[t][c], a_sel);
        });
        PIMDL_COMMIT_SLICE((s + 1) & 1)
#pragma unroll
        for (int t = 0; t < TG; ++t) idx_cur[t] = idx_nxt[t];
        __syncthreads();
    }
#undef PIMDL_FETCH_SLICE
#undef PIMDL_COMMIT_SLICE

    // ---- epilogue: lane (j, g) holds columns 4*g .. 4*g+3 of every 16-column chunk for token j ----
    const bool vec_store = (M % 4 == 0);
#pragma unroll
    for (int t = 0; t < TG; ++t) {
        const uint32_t tok = tok0 + t * 16 + j;
        if (tok >= N) continue;
#pragma unroll
        for (int c = 0; c < Q; ++c) {
            const uint32_t f = colblk * FB + c * 16 + 4 * g;
            if (f >= M) continue;
            const v4i a = acc[t][c];
            if (vec_store) {  // M % 4 == 0 and f % 4 == 0: the whole float4 is in range and aligned
                float4 bv = make_float4(0.f, 0.f, 0.f, 0.f);
                if (ep.bias) bv = *reinterpret_cast<const float4*>(ep.bias + f);
                float4 o;
                o.x = dequant(a[0], ep.scale, ep.lut_bias_term, bv.x);
                o.y = dequant(a[1], ep.scale, ep.lut_bias_term, bv.y);
                o.z = dequant(a[2], ep.scale, ep.lut_bias_term, bv.z);
                o.w = dequant(a[3], ep.scale, ep.lut_bias_term, bv.w);
                *reinterpret_cast<float4*>(out + (size_t)tok * M + f) = o;
                if (acc_out) *reinterpret_cast<v4i*>(acc_out + (size_t)tok * M + f) = a;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (f + e < M) {
                        const float b = ep.bias ? ep.bias[f + e] : 0.0f;
                        out[(size_t)tok * M + f + e] = dequant(a[e], ep.scale, ep.lut_bias_term, b);
                        if (acc_out) acc_out[(size_t)tok * M + f + e] = a[e];
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// fp32 LUT: out[n][f] = (sum over cb ascending, fp32) lut[cb][idx][f] + bias[f]
// One lane = one token; a workgroup = 256 tokens x 4*Q columns; slices of GS codebooks in LDS.
// ---------------------------------------------------------------------------------------------
constexpr int GF_THREADS = 256;

template <int C_T, int Q, int GS, int IDX_BITS>
__global__ __launch_bounds__(GF_THREADS) void gather_f32_kernel(const uint8_t* __restrict__ idx,
                                                               const float* __restrict__ lut,
                                                               float* __restrict__ out, uint32_t N,
                                                               uint32_t M, uint32_t CB_pad,
                                                               uint32_t idx_row_bytes,
                                                               const float* __restrict__ bias)
{
    constexpr int FB = 4 * Q;             // columns per row
    constexpr int PITCH = 16 * Q + 16;    // bytes
    constexpr int CB_BYTES = C_T * PITCH;
    constexpr int SLICE_LDS = GS * CB_BYTES;
    constexpr int SLICE_UNITS = GS * C_T * Q;
    constexpr int UPT = (SLICE_UNITS + GF_THREADS - 1) / GF_THREADS;
    constexpr int IDX_BYTES = GS * IDX_BITS / 8;
    constexpr int IDX_WORDS = (IDX_BYTES + 3) / 4;
    static_assert(IDX_BYTES % 4 == 0, "index fetch is in dwords");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t tok = blockIdx.x * GF_THREADS + threadIdx.x;
    const uint32_t tokc = tok < N ? tok : N - 1;
    const uint32_t colblk = blockIdx.y;
    const uint32_t nslices = CB_pad / GS;
    const uint4* __restrict__ lut_blk = reinterpret_cast<const uint4*>(lut) + (size_t)colblk * CB_pad * C_T * Q;
    const uint32_t* idx_row = reinterpret_cast<const uint32_t*>(idx + (size_t)tokc * idx_row_bytes);

    float acc[FB];
#pragma unroll
    for (int i = 0; i < FB; ++i) acc[i] = 0.0f;

    uint4 stage[UPT];
    uint32_t idx_cur[IDX_WORDS], idx_nxt[IDX_WORDS];
#define PIMDL_FETCH_SLICE(S)                                                                        \
    {                                                                                               \
        const uint4* src_ = lut_blk + (size_t)(S) * SLICE_UNITS;                                    \
        _Pragma("unroll") for (int u = 0; u < UPT; ++u)                                             \
        {                                                                                           \
            const uint32_t unit_ = threadIdx.x + u * GF_THREADS;                                    \
            stage[u] = (SLICE_UNITS % GF_THREADS == 0 || unit_ < SLICE_UNITS) ? src_[unit_]         \
                                                                              : make_uint4(0, 0, 0, 0); \
        }                                                                                           \
    }
#define PIMDL_COMMIT_SLICE(BUF)                                                                     \
    {                                                                                               \
        unsigned char* dst_ = smem + (BUF) * SLICE_LDS;                                             \
        _Pragma("unroll") for (int u = 0; u < UPT; ++u)                                             \
        {                                                                                           \
            const uint32_t unit_ = threadIdx.x + u * GF_THREADS;                                    \
            if (SLICE_UNITS % GF_THREADS == 0 || unit_ < SLICE_UNITS)                               \
                *reinterpret_cast<uint4*>(dst_ + (unit_ / Q) * PITCH + (unit_ % Q) * 16) = stage[u]; \
        }                                                                                           \
    }
    PIMDL_FETCH_SLICE(0)
#pragma unroll
    for (int w = 0; w < IDX_WORDS; ++w) idx_cur[w] = idx_row[w];
    PIMDL_COMMIT_SLICE(0)
    __syncthreads();

    constexpr int per_word = 32 / IDX_BITS;
    for (uint32_t s = 0; s < nslices; ++s) {
        const uint32_t sn = s + 1 < nslices ? s + 1 : s;
        PIMDL_FETCH_SLICE(sn)
#pragma unroll
        for (int w = 0; w < IDX_WORDS; ++w) idx_nxt[w] = idx_row[sn * IDX_WORDS + w];
        const unsigned char* cbbase = smem + (s & 1) * SLICE_LDS;
#pragma unroll
        for (int w = 0; w < IDX_WORDS; ++w) {
            uint32_t word = idx_cur[w];
            // ascending codebook order; partial unroll keeps the loads in flight within the VGPR budget
#pragma unroll 4
            for (int h = 0; h < per_word; ++h) {
                const uint32_t r = word & ((1u << IDX_BITS) - 1);
                word >>= IDX_BITS;
                const unsigned char* row = cbbase + r * PITCH;
                cbbase += CB_BYTES;
#pragma unroll
                for (int c = 0; c < Q; ++c) {
                    const float4 vv = *reinterpret_cast<const float4*>(row + c * 16);
                    acc[4 * c + 0] = __fadd_rn(acc[4 * c + 0], vv.x);
                    acc[4 * c + 1] = __fadd_rn(acc[4 * c + 1], vv.y);
                    acc[4 * c + 2] = __fadd_rn(acc[4 * c + 2], vv.z);
                    acc[4 * c + 3] = __fadd_rn(acc[4 * c + 3], vv.w);
                }
            }
        }
        PIMDL_COMMIT_SLICE((s + 1) & 1)
#pragma unroll
        for (int w = 0; w < IDX_WORDS; ++w) idx_cur[w] = idx_nxt[w];
        __syncthreads();
    }
#undef PIMDL_FETCH_SLICE
#undef PIMDL_COMMIT_SLICE

    if (tok < N) {
#pragma unroll
        for (int i = 0; i < FB; ++i) {
            const uint32_t f = colblk * FB + i;
            if (f < M) out[(size_t)tok * M + f] = __fadd_rn(acc[i], bias ? bias[f] : 0.0f);
        }
    }
}

template <int C_T, int Q, int GQ, int TG, int IDX_BITS>
int launch_i8(Ctx* ctx, const Amm& a, const uint8_t* d_idx, float* d_out, int32_t* d_acc, uint32_t n,
              const Epilogue& ep)
{
    constexpr int TOK_WG = GATHER_WAVES * TG * 16;
    constexpr int LDS = 2 * 4 * GQ * C_T * (16 * Q + 16);
    auto kern = gather_i8_kernel<C_T, Q, GQ, TG, IDX_BITS>;
    static bool attr_set = false;
    if (!attr_set) {
        int rc = hip_check(ctx, hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, LDS),
                           "hipFuncSetAttribute(gather_i8)");
        if (rc) return rc;
        attr_set = true;
    }
    dim3 grid((n + TOK_WG - 1) / TOK_WG, a.g.M_pad / (16 * Q));
    hipLaunchKernelGGL(kern, grid, dim3(GATHER_THREADS), LDS, ctx->stream, d_idx,
                       reinterpret_cast<const int8_t*>(a.d_lut), d_out, d_acc, n, a.g.M, a.g.CB_pad,
                       a.g.idx_row_bytes, ep);
    return hip_check(ctx, hipGetLastError(), "gather_i8_kernel launch");
}

template <int C_T, int Q, int GS, int IDX_BITS>
int launch_f32(Ctx* ctx, const Amm& a, const uint8_t* d_idx, float* d_out, uint32_t n)
{
    constexpr int LDS = 2 * GS * C_T * (16 * Q + 16);
    auto kern = gather_f32_kernel<C_T, Q, GS, IDX_BITS>;
    static bool attr_set = false;
    if (!attr_set) {
        int rc = hip_check(ctx, hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, LDS),
                           "hipFuncSetAttribute(gather_f32)");
        if (rc) return rc;
        attr_set = true;
    }
    dim3 grid((n + GF_THREADS - 1) / GF_THREADS, a.g.M_pad / (4 * Q));
    hipLaunchKernelGGL(kern, grid, dim3(GF_THREADS), LDS, ctx->stream, d_idx,
                       reinterpret_cast<const float*>(a.d_lut), d_out, n, a.g.M, a.g.CB_pad, a.g.idx_row_bytes,
                       a.d_bias);
    return hip_check(ctx, hipGetLastError(), "gather_f32_kernel launch");
}

}  // namespace

// Tiling choices per centroid count.  int8: slice = 4*GQ codebooks, rows of 64 bytes (Q=4) except for
// the largest tables; two slices must fit the 160 KB LDS.  fp32: rows of 16 floats (Q=4).
//   C_T   int8 (Q, GQ) -> slice bytes        fp32 (Q, GS) -> slice bytes
//   8     (4, 8)  20 KB                      (4, 32) 20 KB
//   16    (4, 8)  40 KB                      (4, 32) 40 KB
//   32    (4, 4)  40 KB                      (4, 16) 40 KB
//   64    (4, 2)  40 KB                      (4, 8)  40 KB
//   128   (2, 2)  48 KB                      (2, 8)  48 KB
//   256   (2, 1)  48 KB                      (2, 4)  48 KB
bool plan_geometry(const pimdl_amm_desc& d, AmmGeom* g, std::string* why)
{
    const uint32_t K = d.input_feature_len, v = d.sub_vec_len, C = d.num_centroid, M = d.output_feature_len;
    if (!K || !v || !C || !M || !d.max_n) { *why = "zero-sized dimension"; return false; }
    if (K % v) { *why = "input_feature_len is not a multiple of sub_vec_len"; return false; }
    if (C < 1 || C > 256) { *why = "num_centroid must be in 1..256"; return false; }
    if (d.lut_dtype != PIMDL_LUT_I8 && d.lut_dtype != PIMDL_LUT_F32) { *why = "unknown lut_dtype"; return false; }
    if (d.bias_mode != PIMDL_BIAS_ONCE && d.bias_mode != PIMDL_BIAS_TIMES_CB) { *why = "unknown bias_mode"; return false; }
    g->K = K; g->v = v; g->CB = K / v; g->C = C; g->M = M;
    g->CB_pad = (g->CB + 31) / 32 * 32;
    uint32_t ct = 8;
    while (ct < C) ct *= 2;
    g->C_tile = ct;
    g->idx_bits = C <= 16 ? 4 : 8;
    g->idx_row_bytes = g->CB_pad * g->idx_bits / 8;
    const bool i8 = d.lut_dtype == PIMDL_LUT_I8;
    g->q = ct >= 128 ? 2 : 4;
    if (i8) {
        g->gq = ct <= 16 ? 8 : ct == 32 ? 4 : ct <= 128 ? 2 : 1;
        g->cb_per_slice = 4 * g->gq;
        g->col_block = 16 * g->q;
        g->gather_threads = GATHER_THREADS;
        g->tokens_per_wg = GATHER_WAVES * 2 * 16;
    } else {
        g->gq = 0;
        g->cb_per_slice = ct <= 16 ? 32 : ct == 32 ? 16 : ct <= 128 ? 8 : 4;
        g->col_block = 4 * g->q;
        g->gather_threads = GF_THREADS;
        g->tokens_per_wg = GF_THREADS;
    }
    g->row_pitch = 16 * g->q + 16;
    g->gather_lds_bytes = 2 * g->cb_per_slice * ct * g->row_pitch;
    g->M_pad = (M + g->col_block - 1) / g->col_block * g->col_block;
    g->ccs_cb_per_wg = ccs_cb_per_wg(v);
    g->ccs_row_floats = g->ccs_cb_per_wg * v;
    g->ccs_lds_bytes = g->ccs_cb_per_wg ? 256 * (g->ccs_row_floats + 4) * 4 : 0;
    return true;
}

int launch_gather(Ctx* ctx, const Amm& a, const uint8_t* d_idx, float* d_out, int32_t* d_acc, uint32_t n)
{
    if (n == 0) return PIMDL_OK;
    const AmmGeom& g = a.g;
    if (a.desc.lut_dtype == PIMDL_LUT_I8) {
        Epilogue ep;
        ep.scale = a.h_scale0;
        ep.lut_bias_term = a.desc.bias_mode == PIMDL_BIAS_TIMES_CB ? a.desc.lut_bias * (float)g.CB : a.desc.lut_bias;
        ep.bias = a.d_bias;
        switch (g.C_tile) {
            case 8: return launch_i8<8, 4, 8, 2, 4>(ctx, a, d_idx, d_out, d_acc, n, ep);
            case 16: return launch_i8<16, 4, 8, 2, 4>(ctx, a, d_idx, d_out, d_acc, n, ep);
            case 32: return launch_i8<32, 4, 4, 2, 8>(ctx, a, d_idx, d_out, d_acc, n, ep);
            case 64: return launch_i8<64, 4, 2, 2, 8>(ctx, a, d_idx, d_out, d_acc, n, ep);
            case 128: return launch_i8<128, 2, 2, 2, 8>(ctx, a, d_idx, d_out, d_acc, n, ep);
            case 256: return launch_i8<256, 2, 1, 2, 8>(ctx, a, d_idx, d_out, d_acc, n, ep);
        }
    } else {
        switch (g.C_tile) {
            case 8: return launch_f32<8, 4, 32, 4>(ctx, a, d_idx, d_out, n);
            case 16: return launch_f32<16, 4, 32, 4>(ctx, a, d_idx, d_out, n);
            case 32: return launch_f32<32, 4, 16, 8>(ctx, a, d_idx, d_out, n);
            case 64: return launch_f32<64, 4, 8, 8>(ctx, a, d_idx, d_out, n);
            case 128: return launch_f32<128, 2, 8, 8>(ctx, a, d_idx, d_out, n);
            case 256: return launch_f32<256, 2, 4, 8>(ctx, a, d_idx, d_out, n);
        }
    }
    return set_error(ctx, PIMDL_ERR_UNSUPPORTED, "no gather kernel for C_tile=%u", g.C_tile);
}

}  // namespace pimdl
