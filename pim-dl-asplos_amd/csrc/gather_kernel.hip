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
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

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

// One v_mad_u32_u24: the compiler otherwise splits r*PITCH + base into a multiply and an or, and
// every VALU instruction beyond about one per MFMA takes issue cycles away from the matrix core.
__device__ __forceinline__ uint32_t mad24(uint32_t a, uint32_t b, uint32_t c)
{
    uint32_t d;
    asm("v_mad_u32_u24 %0, %1, %2, %3" : "=v"(d) : "v"(a), "s"(b), "v"(c));
    return d;
}

// Move one 16-byte staging unit: the register holds LUT data fetched during the previous slice and
// is written to LDS; the same register is then re-armed with the unit of the slice after next.
// (ds_write reads its data operand at issue; the load's result lands hundreds of cycles later.)
__device__ __forceinline__ void stage_xfer(v4u& reg, uint32_t lds_addr, const v4u* gptr)
{
    asm volatile(
        "ds_write_b128 %1, %0\n\t"
        "global_load_dwordx4 %0, %2, off"
        : "+v"(reg)
        : "v"(lds_addr), "v"(gptr)
        : "memory");
}

// index fetch of 1, 2 or 4 bytes (zero-extended) that the compiler does not know is in flight
template <int BYTES>
__device__ __forceinline__ void load_idx_async(uint32_t& reg, const void* gptr)
{
    if constexpr (BYTES == 4) asm volatile("global_load_dword %0, %1, off" : "=v"(reg) : "v"(gptr) : "memory");
    else if constexpr (BYTES == 2) asm volatile("global_load_ushort %0, %1, off" : "=v"(reg) : "v"(gptr) : "memory");
    else asm volatile("global_load_ubyte %0, %1, off" : "=v"(reg) : "v"(gptr) : "memory");
}

// C_T: centroid rows per codebook in the tiled LUT (power of two >= C)
// Q:   16-byte chunks per row (column block = 16*Q)
// GQ:  codebooks per lane group per slice (slice = 4*GQ codebooks)
// TG:  16-token groups per wave (tokens per work item = 8 waves * TG * 16)
//
// Persistent: the grid is a fixed number of workgroups (two per CU); workgroup w processes the work
// items w, w + gridDim.x, ... where an item is (column block, token tile).  The loop over
// (item, codebook slice) is one flat stream k = 0, 1, ...: while slice k is consumed from one LDS
// buffer, the registers holding slice k+1 are written to the other buffer and re-armed with global
// loads of slice k+2, one 16-byte unit at a time *between* groups of MFMAs, so neither the texture
// path nor the LDS write port ever sees a burst, no wave ever stalls on issue, and the only
// synchronisation is one barrier per slice between waves that all did identical work.
template <int C_T, int Q, int GQ, int TG, int IDX_BITS>
__global__ __launch_bounds__(GATHER_THREADS, 4) void gather_i8_kernel(
    const uint8_t* __restrict__ idx, const int8_t* __restrict__ lut, float* __restrict__ out,
    int32_t* __restrict__ acc_out, uint32_t N, uint32_t M, uint32_t CB_pad, uint32_t idx_row_bytes,
    uint32_t n_token_tiles, uint32_t n_items, Epilogue ep)
{
    constexpr int G = 4 * GQ;                     // codebooks per slice
    constexpr int FB = 16 * Q;                    // columns (= bytes) per row
    constexpr int PITCH = 16 * (Q | 1);           // LDS row pitch: an odd number of 16-byte units
    constexpr int CB_BYTES = C_T * PITCH;         // LDS bytes per codebook
    constexpr int SLICE_LDS = G * CB_BYTES;
    constexpr int SLICE_UNITS = G * C_T * Q;      // 16-byte units per slice in HBM
    constexpr int UPT = (SLICE_UNITS + GATHER_THREADS - 1) / GATHER_THREADS;
    constexpr int IDX_BYTES = GQ * IDX_BITS / 8;  // index bytes one lane needs per slice and token
    constexpr int TOK_ITEM = GATHER_WAVES * TG * 16;
    static_assert(IDX_BYTES == 1 || IDX_BYTES == 2 || IDX_BYTES == 4, "index fetch width");
    static_assert((GQ - 1) * CB_BYTES + (Q - 1) * 16 < 65536, "ds_read immediate offset range");
    static_assert(PITCH >= FB && (PITCH / 16) % 2 == 1, "row pitch");
    static_assert(SLICE_UNITS % GATHER_THREADS == 0, "every lane moves the same number of staging units");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t j = lane & 15;  // token within the 16-token group (MFMA column)
    const uint32_t g = lane >> 4;  // MFMA K-block of this lane; also selects its 4 output columns
    // codebook quarter = index of the LDS pass this lane is served in (see "Bank conflicts" above)
    const uint32_t gq = g ^ (((j + 4) >> 3) & 1);
    const uint32_t nslices = CB_pad / G;
    if (blockIdx.x >= n_items) return;  // whole workgroup
    const uint32_t my_items = (n_items - blockIdx.x + gridDim.x - 1) / gridDim.x;
    const uint32_t total = my_items * nslices;  // length of this workgroup's (item, slice) stream

    // constant A operand: byte (lane % 16) of the lane's 16 bytes is 1
    const int one_hot = 1 << (8 * (j & 3));
    const v4i a_sel = {(j >> 2) == 0 ? one_hot : 0, (j >> 2) == 1 ? one_hot : 0, (j >> 2) == 2 ? one_hot : 0,
                       (j >> 2) == 3 ? one_hot : 0};

    auto load_idx = [](const uint8_t* base, uint32_t s) -> uint32_t {
        const uint8_t* p = base + (size_t)s * G * IDX_BITS / 8;
        if constexpr (IDX_BYTES == 4) return *reinterpret_cast<const uint32_t*>(p);
        else if constexpr (IDX_BYTES == 2) return *reinterpret_cast<const uint16_t*>(p);
        else return *p;
    };
    // this lane's index bytes of slice 0 of an item, per token group
    auto locate_idx = [&](uint32_t item, const uint8_t* (&ptr)[TG]) {
        const uint32_t tok0 = (item % n_token_tiles) * TOK_ITEM + wave * (TG * 16);
#pragma unroll
        for (int t = 0; t < TG; ++t) {
            uint32_t tok = tok0 + t * 16 + j;
            if (tok >= N) tok = N - 1;  // clamp: results of such lanes are never stored
            ptr[t] = idx + (size_t)tok * idx_row_bytes + (size_t)(gq * GQ) * IDX_BITS / 8;
        }
    };
    // this lane's first staging unit of slice s of an item (the others follow GATHER_THREADS units apart)
    auto locate_lut = [&](uint32_t item, uint32_t s) -> const v4u* {
        return reinterpret_cast<const v4u*>(lut) + ((size_t)(item / n_token_tiles) * CB_pad * C_T * Q) +
               (size_t)s * SLICE_UNITS + threadIdx.x;
    };
    // LDS byte offset (within a slice buffer) of this lane's staging unit u
    uint32_t stage_lds[UPT];
#pragma unroll
    for (int u = 0; u < UPT; ++u) {
        const uint32_t unit = threadIdx.x + u * GATHER_THREADS;
        stage_lds[u] = (unit / Q) * PITCH + (unit % Q) * 16;
    }

    v4i acc[TG][Q], slot[TG][Q];
#pragma unroll
    for (int t = 0; t < TG; ++t)
#pragma unroll
        for (int c = 0; c < Q; ++c) acc[t][c] = (v4i){0, 0, 0, 0};

    // stream positions: p0 is consumed, p1 is written to LDS, p2 is fetched from HBM/L2
    uint32_t item0 = blockIdx.x, s0 = 0;
    uint32_t item1 = item0, s1 = 0, item2, s2;
    auto advance = [&](uint32_t& item, uint32_t& s) {
        if (++s == nslices) {
            s = 0;
            item += gridDim.x;
        }
    };
    advance(item1, s1);
    item2 = item1;
    s2 = s1;
    advance(item2, s2);

    // ---- prologue: slice 0 into LDS buffer 0, slice 1 into the staging registers ----------------
    v4u stage[UPT];
    uint32_t idx_cur[TG], idx_nxt[TG];
    const uint8_t* idx_base[TG];  // of the item p1 belongs to
    {
        const v4u* src = locate_lut(item0, 0);
#pragma unroll
        for (int u = 0; u < UPT; ++u) stage[u] = src[u * GATHER_THREADS];
        locate_idx(item0, idx_base);
#pragma unroll
        for (int t = 0; t < TG; ++t) idx_nxt[t] = load_idx(idx_base[t], 0);  // moved to idx_cur at the top of k = 0
#pragma unroll
        for (int u = 0; u < UPT; ++u) *reinterpret_cast<v4u*>(smem + stage_lds[u]) = stage[u];
        const bool valid1 = 1 < total;
        src = valid1 ? locate_lut(item1, s1) : locate_lut(item0, 0);
#pragma unroll
        for (int u = 0; u < UPT; ++u) stage[u] = src[u * GATHER_THREADS];
        if (valid1 && s1 == 0) locate_idx(item1, idx_base);
    }
    __syncthreads();

    const uint32_t lane_base = gq * GQ * CB_BYTES;
    bool pending_epilogue = false;
    uint32_t epilogue_item = 0;

    // De-quantise and store one finished item, then clear the accumulators.  Lane (j, g) holds columns
    // 4*g .. 4*g+3 of every 16-column chunk for token j.  It runs right after a top-of-slice wait, so
    // its stores have a whole slice to drain before anything waits on the memory counter again; the
    // bias values are fetched first so that no store sits between a load and its use.
    auto epilogue = [&](uint32_t item) {
        const uint32_t colblk = item / n_token_tiles;
        const uint32_t tok0 = (item % n_token_tiles) * TOK_ITEM + wave * (TG * 16);
        const bool vec_store = (M % 4 == 0);
        float4 bv[Q];
#pragma unroll
        for (int c = 0; c < Q; ++c) {
            const uint32_t f = colblk * FB + c * 16 + 4 * g;
            bv[c] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (ep.bias && f < M) {
                if (vec_store) {
                    bv[c] = *reinterpret_cast<const float4*>(ep.bias + f);
                } else {
                    bv[c].x = ep.bias[f];
                    if (f + 1 < M) bv[c].y = ep.bias[f + 1];
                    if (f + 2 < M) bv[c].z = ep.bias[f + 2];
                    if (f + 3 < M) bv[c].w = ep.bias[f + 3];
                }
            }
        }
#pragma unroll
        for (int t = 0; t < TG; ++t) {
            const uint32_t tok = tok0 + t * 16 + j;
#pragma unroll
            for (int c = 0; c < Q; ++c) {
                const uint32_t f = colblk * FB + c * 16 + 4 * g;
                const v4i a = acc[t][c];
                acc[t][c] = (v4i){0, 0, 0, 0};
                if (tok >= N || f >= M) continue;
                float4 o;
                o.x = dequant(a[0], ep.scale, ep.lut_bias_term, bv[c].x);
                o.y = dequant(a[1], ep.scale, ep.lut_bias_term, bv[c].y);
                o.z = dequant(a[2], ep.scale, ep.lut_bias_term, bv[c].z);
                o.w = dequant(a[3], ep.scale, ep.lut_bias_term, bv[c].w);
                if (vec_store) {  // M % 4 == 0 and f % 4 == 0: the whole float4 is in range and aligned
                    *reinterpret_cast<float4*>(out + (size_t)tok * M + f) = o;
                    if (acc_out) *reinterpret_cast<v4i*>(acc_out + (size_t)tok * M + f) = a;
                } else {
                    const float ov[4] = {o.x, o.y, o.z, o.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (f + e < M) {
                            out[(size_t)tok * M + f + e] = ov[e];
                            if (acc_out) acc_out[(size_t)tok * M + f + e] = a[e];
                        }
                    }
                }
            }
        }
    };

    for (uint32_t k = 0; k < total; ++k) {
        // everything this lane has in flight is at least one slice old: the staging registers hold
        // slice k+1, the indices fetched during the previous iteration have landed
        // (the indices move out of their in-flight registers inside the asm, behind the wait, so the
        // compiler never holds a value it could copy before it has landed)
        static_assert(TG == 1 || TG == 2, "operand list of the wait below");
        if constexpr (TG == 2)
            asm volatile("s_waitcnt vmcnt(0)\n\tv_mov_b32 %0, %2\n\tv_mov_b32 %1, %3"
                         : "=&v"(idx_cur[0]), "=&v"(idx_cur[1])
                         : "v"(idx_nxt[0]), "v"(idx_nxt[1])
                         : "memory");
        else
            asm volatile("s_waitcnt vmcnt(0)\n\tv_mov_b32 %0, %1" : "=&v"(idx_cur[0]) : "v"(idx_nxt[0]) : "memory");
        if (pending_epilogue) {  // workgroup-uniform
            epilogue(epilogue_item);
            pending_epilogue = false;
        }

        const bool valid1 = k + 1 < total, valid2 = k + 2 < total;  // workgroup-uniform
#pragma unroll
        for (int t = 0; t < TG; ++t)
            load_idx_async<IDX_BYTES>(idx_nxt[t], idx_base[t] + (size_t)(valid1 ? s1 : 0) * G * IDX_BITS / 8);
        const v4u* fetch_ptr = valid2 ? locate_lut(item2, s2) : locate_lut(item0, s0);

        const uint32_t buf = (k & 1) * SLICE_LDS + lane_base;
        const uint32_t wbuf = ((k + 1) & 1) * SLICE_LDS;
        // LDS byte address of the row each token group gathers from, per codebook of the quarter
        uint32_t row_addr[GQ][TG];
#pragma unroll
        for (int q = 0; q < GQ; ++q)
#pragma unroll
            for (int t = 0; t < TG; ++t)
                row_addr[q][t] = mad24((idx_cur[t] >> (IDX_BITS * q)) & ((1u << IDX_BITS) - 1), PITCH, buf);

        // Rolling pipeline, one register slot per accumulator: the row piece for (q+1, t, c) is
        // requested into the slot as soon as the MFMA for (q, t, c) has consumed it, so TG*Q reads
        // stay in flight behind the matrix core.  Waits are explicit: LDS operations complete in
        // order, and lgkmcnt(TG*Q-1) before an MFMA means "the oldest outstanding read has landed"
        // (an interleaved staging write only makes that wait stricter).
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
            // staging: one unit after each of the first steps (the rest after the last interior step),
            // so that the re-armed loads have most of a slice to land
            static_for<(q < UPT ? q : UPT), (q + 1 == GQ - 1 ? UPT : (q + 1 < UPT ? q + 1 : UPT))>([&](auto u) {
                stage_xfer(stage[u], wbuf + stage_lds[u], fetch_ptr + u * GATHER_THREADS);
            });
        });
        if constexpr (GQ == 1) {
            static_for<0, UPT>([&](auto u) {
                stage_xfer(stage[u], wbuf + stage_lds[u], fetch_ptr + u * GATHER_THREADS);
            });
        }
        static_for<0, TG * Q>([&](auto i) {
            constexpr int t = i / Q, c = i % Q;
            mfma_last<TG * Q - 1 - i>(acc[t][c], slot[t][c], a_sel);
        });

        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this lane's staging writes are in LDS
        __syncthreads();

        if (s0 + 1 == nslices) {  // item finished: its epilogue runs after the next top-of-slice wait
            pending_epilogue = true;
            epilogue_item = item0;
        }

        // advance the three stream positions
        item0 = item1;
        s0 = s1;
        item1 = item2;
        s1 = s2;
        advance(item2, s2);
        if (k + 2 < total && s1 == 0) locate_idx(item1, idx_base);  // p1 entered a new item
    }
    // drain the loads armed by the last iterations before the registers die, then the last item
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (pending_epilogue) epilogue(epilogue_item);
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
    constexpr int TOK_ITEM = GATHER_WAVES * TG * 16;
    constexpr int PITCH = 16 * (Q | 1);
    constexpr int LDS = 2 * 4 * GQ * C_T * PITCH;
    auto kern = gather_i8_kernel<C_T, Q, GQ, TG, IDX_BITS>;
    static bool attr_set = false;
    if (!attr_set) {
        int rc = hip_check(ctx, hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, LDS),
                           "hipFuncSetAttribute(gather_i8)");
        if (rc) return rc;
        attr_set = true;
    }
    const uint32_t n_token_tiles = (n + TOK_ITEM - 1) / TOK_ITEM;
    const uint32_t n_items = n_token_tiles * (a.g.M_pad / (16 * Q));
    // persistent grid: as many workgroups as fit at once (LDS-limited), never more than there are items
    const uint32_t per_cu = LDS > 0 ? (uint32_t)(ctx->prop.maxSharedMemoryPerMultiProcessor / LDS) : 1;
    uint32_t grid = ctx->prop.multiProcessorCount * (per_cu < 1 ? 1 : per_cu > 2 ? 2 : per_cu);
    if (grid > n_items) grid = n_items;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(GATHER_THREADS), LDS, ctx->stream, d_idx,
                       reinterpret_cast<const int8_t*>(a.d_lut), d_out, d_acc, n, a.g.M, a.g.CB_pad,
                       a.g.idx_row_bytes, n_token_tiles, n_items, ep);
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
bool plan_geometry(const pimdl_amm_desc& d, uint32_t num_cus, AmmGeom* g, std::string* why)
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
    if (i8 && ct >= 16 && ct <= 64) {
        // Column block of 64 or 48 columns: take the one that fills the persistent grid (two
        // workgroups per CU) more evenly for the largest batch this operator will see.  An item is
        // 256 tokens x one column block; all items cost the same.
        const uint32_t slots = 2 * (num_cus ? num_cus : 256);
        const uint32_t tiles = (d.max_n + 255) / 256;
        double best = -1.0;
        for (uint32_t q : {4u, 3u}) {
            const uint32_t blocks = (M + 16 * q - 1) / (16 * q);
            const uint64_t items = (uint64_t)tiles * blocks;
            const uint64_t rounds = (items + slots - 1) / slots;
            const double eff = (double)items / (double)(rounds * slots) * (double)M / (double)(blocks * 16 * q);
            if (eff > best + 1e-9) {
                best = eff;
                g->q = q;
            }
        }
    }
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
    g->row_pitch = 16 * (g->q | 1);
    g->gather_lds_bytes = 2 * g->cb_per_slice * ct * g->row_pitch;
    g->M_pad = (M + g->col_block - 1) / g->col_block * g->col_block;
    g->ccs_cb_per_wg = ccs_cb_per_wg(v);
    g->ccs_row_floats = g->ccs_cb_per_wg * v;
    g->ccs_lds_bytes = g->ccs_cb_per_wg ? 64 * (g->ccs_row_floats + 4) * 4 : 0;
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
            case 16:
                return g.q == 3 ? launch_i8<16, 3, 8, 2, 4>(ctx, a, d_idx, d_out, d_acc, n, ep)
                                : launch_i8<16, 4, 8, 2, 4>(ctx, a, d_idx, d_out, d_acc, n, ep);
            case 32:
                return g.q == 3 ? launch_i8<32, 3, 4, 2, 8>(ctx, a, d_idx, d_out, d_acc, n, ep)
                                : launch_i8<32, 4, 4, 2, 8>(ctx, a, d_idx, d_out, d_acc, n, ep);
            case 64:
                return g.q == 3 ? launch_i8<64, 3, 2, 2, 8>(ctx, a, d_idx, d_out, d_acc, n, ep)
                                : launch_i8<64, 4, 2, 2, 8>(ctx, a, d_idx, d_out, d_acc, n, ep);
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
