// LUT gather-accumulate for gfx950 (MI355X).
//
// Replaces the DPU kernel of the reference (inference-engine/src/dpu/pim_lut_kernel.c:97-2296; its
// row-major statement is inference-engine/test/test_amm.cpp:164-175) and the host epilogue
// (inference-engine/src/host/pim_lut_host.cpp:190-203 / test_amm.cpp:178-181):
//     acc[n][f] = sum over cb of lut[cb][idx[n][cb]][f]          (int8 table, int32 sum, exact)
//     out[n][f] = (float)acc * scale + lut_bias(*CB) + bias[f]   (fp32, left to right, unfused)
//
// Three kernels: the one-hot matrix-core gather for int8 tables with up to 16 centroids (further down,
// the one the benchmark shapes run), the byte adder below for int8 tables with more centroids, and the
// fp32-table gather (also used for int8 tables with one scale per group of codebooks).
//
// The byte adder and the fp32 gather are bound by LDS read bandwidth: every gathered LUT byte is read
// once from LDS (N*CB*M bytes), while HBM only sees the packed indices, the LUT slices and the output.
//
// int8 byte adder.  A workgroup owns a tile of tokens x one column block (16*Q columns) and walks the
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
#include <stdlib.h>

#include <stdio.h>

#include "gather_common.h"

namespace pimdl {

namespace {

// The three building blocks of the gather pipeline.  They are inline assembly because the order
// "wait for the oldest read, feed it to the matrix core, re-arm the slot with the next read" is the
// whole point, and the compiler's scheduler serialises the equivalent C++ (one read in flight).
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
__global__ __launch_bounds__(GATHER_THREADS, TG == 4 ? 2 : 4) void gather_i8_kernel(
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
    // (always_inline: called from two places; as a real function it would take the accumulators, and
    // registers whose loads are still in flight, through memory)
    auto epilogue_as = [&](uint32_t item, auto actc) __attribute__((always_inline)) {
        constexpr bool ACT = decltype(actc)::value;
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
                o.x = dequant<ACT>(a[0], ep, bv[c].x);
                o.y = dequant<ACT>(a[1], ep, bv[c].y);
                o.z = dequant<ACT>(a[2], ep, bv[c].z);
                o.w = dequant<ACT>(a[3], ep, bv[c].w);
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
    auto epilogue = [&](uint32_t item) __attribute__((always_inline)) {
        if (ep.act == PIMDL_ACT_GELU_TANH) epilogue_as(item, std::true_type{});
        else epilogue_as(item, std::false_type{});
    };

    for (uint32_t k = 0; k < total; ++k) {
        // everything this lane has in flight is at least one slice old: the staging registers hold
        // slice k+1, the indices fetched during the previous iteration have landed
        // (the indices move out of their in-flight registers inside the asm, behind the wait, so the
        // compiler never holds a value it could copy before it has landed)
        static_assert(TG == 1 || TG == 2 || TG == 4, "operand list of the wait below");
        if constexpr (TG == 4)
            asm volatile("s_waitcnt vmcnt(0)\n\tv_mov_b32 %0, %4\n\tv_mov_b32 %1, %5\n\tv_mov_b32 %2, %6\n\tv_mov_b32 %3, %7"
                         : "=&v"(idx_cur[0]), "=&v"(idx_cur[1]), "=&v"(idx_cur[2]), "=&v"(idx_cur[3])
                         : "v"(idx_nxt[0]), "v"(idx_nxt[1]), "v"(idx_nxt[2]), "v"(idx_nxt[3])
                         : "memory");
        else if constexpr (TG == 2)
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


// =============================================================================================
// One-hot matrix-core gather for C <= 16 (int8 LUT, 4-bit indices).
//
// The byte-adder kernel above reads every gathered row piece from LDS once per token: N*CB*M
// bytes, which ties it to LDS read bandwidth and leaves the matrix core waiting.  For C <= 16 the
// same v_mfma_i32_16x16x64_i8 does the same amount of gathering per instruction (16 tokens x 16
// columns x 4 codebooks) in the reference's own definition of the operator
// (model-calibration/LUTNeuro/LUTLinear_t.py:78, bmm(one_hot, lut)):
//     A[i][16 g + c] = lut[cb_g][c][column i]        (the 16 centroid rows of 4 codebooks)
//     B[16 g + c][j] = (idx[token j][cb_g] == c)     (one-hot of token j's index)
//     D[i][j] += sum over g of lut[cb_g][idx[j][cb_g]][i]
// Both operands are now shared: one A operand serves every token of the tile, one B operand every
// column, so a wave that keeps TM token groups x TN column groups of accumulators issues TM*TN
// MFMAs per TM+TN LDS reads (0.42 reads per MFMA at 4 x 6 instead of 1), and the kernel is bound by
// the matrix core.  The sum is still an exact int32 sum of int8 entries.
//
// LUT layout for this kernel (HBM and LDS alike): [column tile][codebook][column][16 centroids],
// so a lane's A operand is 16 consecutive bytes, lanes of a column group read consecutive 16-byte
// units (no bank conflicts), and a slice of 16 codebooks is one contiguous block that goes from
// L2 to LDS with global_load_lds (no registers, no ds_write).
// The one-hot operand comes from a 256-byte table in LDS (entry c = 16 bytes with byte c set):
// lanes with equal indices read the same address (broadcast), others hit different banks.
//
// A workgroup is four waves; wave w owns tokens 64 w .. 64 w + 63 of a 256-token tile (TM = 4)
// and all 16*TN columns of the tile.  Workgroups are persistent over a flat (item, slice) stream,
// double-buffered in LDS, one barrier per slice.
// =============================================================================================
constexpr int OH_WAVES = 4;
constexpr int OH_THREADS = OH_WAVES * 64;
// 16-token groups per wave (TM): 4 (256-token items) where the batch offers enough items to put two
// workgroups on every CU, else 2 (128-token items, twice as many of them)
constexpr int oh_tok_item(int tm) { return OH_WAVES * tm * 16; }

// codebooks per slice (4 per MFMA K-step)
constexpr int oh_slice_cbs(int, int gs = 16) { return gs; }
// LUT slice buffers in LDS (prefetch distance = buffers - 1); two workgroups must fit in a CU's LDS
constexpr int oh_nbuf(int, int gs = 16) { return gs > 16 ? 2 : 3; }
// Up to 8 centroids ("paired"): two codebooks share the 16 K-slots of a lane, so a slice entry is a pair of
// codebooks, its index is the whole byte (one nibble per codebook) and the table holds two-hot vectors.
constexpr int oh_table_bytes(bool p8) { return p8 ? 4096 : 256; }
constexpr int oh_iwords(int tn, bool p8, int gs = 16) { return p8 ? oh_slice_cbs(tn, gs) / 4 : oh_slice_cbs(tn, gs) / 8; }
// one-hot table + LUT slice buffers + index buffers
constexpr int oh_lds_bytes(int tn, bool p8 = false, int gs = 16)
{
    // (every wave keeps the index words of a whole 64-token block, whatever part of it it owns)
    return oh_table_bytes(p8) + oh_nbuf(tn, gs) * oh_slice_cbs(tn, gs) * 16 * tn * 16 +
           oh_nbuf(tn, gs) * OH_WAVES * 64 * 4 * oh_iwords(tn, p8, gs);
}

// all operands of one K-step have landed; the registers pass through (empty, ordered) asm statements
// so that no consumer can be scheduled ahead of the wait
template <int TN, int TM>
__device__ __forceinline__ void oh_wait(v4i (&a)[TN], v4i (&b)[TM])
{
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < TN; ++i) asm volatile("" : "+v"(a[i]));
#pragma unroll
    for (int i = 0; i < TM; ++i) asm volatile("" : "+v"(b[i]));
}

// A workgroup is four waves; wave w owns tokens 64 w .. 64 w + 63 of a 256-token tile (TM = 4) and
// all 16*TN columns of the tile; two workgroups per CU put two waves on every SIMD (one wave alone
// can only issue an MFMA every ~30 cycles; two keep the matrix core at its ~21).  Smaller wave
// tiles with more waves were slower: a K-step must hold enough MFMAs (TM*TN) to cover the LDS
// latency of the next K-step's operands.
template <int TN, int TM, bool P8, int GS>
__global__ __launch_bounds__(OH_THREADS, 2) void gather_onehot_kernel(
    const uint8_t* __restrict__ idx, const int8_t* __restrict__ lut, float* __restrict__ out,
    int32_t* __restrict__ acc_out, uint32_t N, uint32_t M, uint32_t CB_pad, uint32_t idx_row_bytes,
    uint32_t n_token_tiles, uint32_t n_items, Epilogue ep, XcdMap xmap)
{
    constexpr int OH_TOK_ITEM = oh_tok_item(TM);
    static_assert(TM == 4 || TM == 2, "a wave owns a whole or half a 64-token index block");
    constexpr int WN = 16 * TN;                    // columns per item
    constexpr int G = oh_slice_cbs(TN, GS);       // codebooks per slice
    constexpr int SLICE = G * WN * 16;             // bytes of one codebook slice
    constexpr int KSTEPS = G / 4;
    constexpr int IWORDS = oh_iwords(TN, P8, GS); // 32-bit index words per token and slice
    constexpr int NBLK = SLICE / 1024;             // 1 KB blocks (one copy instruction of a wave) per slice
    constexpr int DMA_PER_WAVE = (NBLK + OH_WAVES - 1) / OH_WAVES;

    // LDS: one-hot table (256 B) | NBUF LUT slice buffers | NIBUF index buffers
    // (index words k+1 .. k+PD+1 are live while slice k is consumed; words k are in registers)
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    constexpr int NBUF = oh_nbuf(TN, GS), NIBUF = NBUF;
    constexpr int PD = NBUF - 1;  // prefetch distance of the LUT stream, in slices
    constexpr uint32_t BUF0 = oh_table_bytes(P8);  // the table sits at LDS offset 0: entry address = nibble (byte) * 16
    constexpr uint32_t IBUF0 = BUF0 + NBUF * SLICE;
    constexpr uint32_t IBYTES = OH_WAVES * 64 * 4 * IWORDS;   // index bytes of one slice (a 64-token block per wave)
    constexpr uint32_t IWAVE = 64 * 4 * IWORDS;               // ... of one wave's 64 tokens
    constexpr int IX_OPS = IWORDS;                            // 64 lanes x 4 B = 64 tokens x 1 word
    constexpr int DMA_OPS = DMA_PER_WAVE + IX_OPS;            // memory operations per wave and slice

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar: addresses below stay in SGPRs
    const uint32_t j = lane & 15;  // column within a group (A operand) / token within a group (B operand)
    const uint32_t g = lane >> 4;  // codebook of the K-step
    if (blockIdx.x >= n_items) return;  // whole workgroup
    const uint32_t nslices = CB_pad / G;
    const uint32_t my_items = (n_items - blockIdx.x + gridDim.x - 1) / gridDim.x;
    const uint32_t total = my_items * nslices;

    if constexpr (P8) {
        // entry e (index byte: codebook 2k in the low nibble, 2k+1 in the high one) = 16 bytes with byte
        // (e & 15) and byte 8 + (e >> 4) set; a nibble of 8 or more (no such centroid) sets nothing
        static_assert(OH_THREADS == 256, "one table entry per thread");
        const uint32_t lo = threadIdx.x & 15, hi = threadIdx.x >> 4;
        uint32_t w[4];
#pragma unroll
        for (uint32_t q = 0; q < 4; ++q)
            w[q] = ((lo < 8 && (lo >> 2) == q) ? (1u << (8 * (lo & 3))) : 0u) |
                   ((hi < 8 && 2 + (hi >> 2) == q) ? (1u << (8 * (hi & 3))) : 0u);
        reinterpret_cast<uint4*>(smem)[threadIdx.x] = make_uint4(w[0], w[1], w[2], w[3]);
    } else if (threadIdx.x < 64) {  // entry e = 16 bytes, byte e is 1
        const uint32_t e = threadIdx.x >> 2, w = threadIdx.x & 3;
        reinterpret_cast<uint32_t*>(smem)[threadIdx.x] = ((e >> 2) == w) ? (1u << (8 * (e & 3))) : 0u;
    }

    // Everything comes in through global_load_lds, so the only memory-counter waits in the loop are
    // the explicit ones.  Two independent stream positions step through the (item, slice) sequence:
    // the LUT position runs PD slices ahead of the one being consumed, the index position PD+1
    // (the index words of slice k+1 are unpacked while slice k is multiplied).
    //   LUT:   wave w copies DMA_PER_WAVE consecutive 1 KB blocks of a slice.  All of a slice's operations
    //          share one global address (per lane) and one LDS address; the block is chosen by the
    //          instruction's immediate offset, which the hardware adds to both (the field reaches 4 KB, so
    //          blocks beyond the fourth go through a second address pair 4 KB further on).
    //   index: lane L of wave w copies index word i of token 64 w + L with its i-th operation,
    //          into [wave][word][64 tokens]; only the wave itself reads them back.
    // Addresses are kept as a wave-uniform 64-bit base (scalar registers) plus a 32-bit per-lane
    // offset, the form the copy instructions take directly.
    auto col_of = [&](uint32_t p) { uint32_t c, t; xmap.decode(p, n_token_tiles, c, t); return c; };
    auto tok_tile_of = [&](uint32_t p) { uint32_t c, t; xmap.decode(p, n_token_tiles, c, t); return t; };
    uint32_t lut_item = blockIdx.x, lut_s = 0, ix_item = blockIdx.x, ix_s = 0;
    static_assert(NBLK % OH_WAVES == 0 && DMA_PER_WAVE <= 8, "whole blocks per wave, two address pairs");
    const int8_t* dma_base;   // uniform: start of the slice at the LUT stream position
    const uint32_t dma_wave = wave * (DMA_PER_WAVE * 1024);
    const uint32_t dma_lane = dma_wave + lane * 16;
    const uint8_t* ix_base;   // uniform: the 256-byte block of index words at the index stream position
    uint32_t ix_lane_off;     // per lane: its token's word inside a block
    auto locate_lut = [&]() {
        dma_base = lut + (size_t)col_of(lut_item) * CB_pad * (WN * 16);
    };
    // Index words live as [N/64][row words][64 tokens]: the word of a slice for this wave's 64 tokens
    // is one contiguous 256-byte block (see idx_offset).
    const uint32_t last_block = (N - 1) / 64;
    auto locate_ix = [&]() {
        // TM = 4: wave w owns block w of the tile; TM = 2: waves 2p and 2p+1 each copy block p and own half of it
        uint32_t blk = (tok_tile_of(ix_item) * OH_TOK_ITEM + wave * (TM * 16)) / 64;
        if (blk > last_block) blk = last_block;  // clamp: results of such tokens are never stored
        const uint32_t op = ep.op_col_tiles ? col_of(ix_item) / ep.op_col_tiles : 0u;
        ix_base = idx + (size_t)op * ep.op_idx_stride + (size_t)blk * idx_row_bytes * 64;
        ix_lane_off = lane * 4;
    };
    // fetch = false (past the end of the stream): the operations re-copy the first slice of the
    // LUT into a buffer nobody reads any more, so that every slice issues the same number of
    // operations and the waits can count them
    const int8_t* lut_src = nullptr;  // this slice's source for this lane
    uint32_t lut_dst = 0;             // ... and the wave's destination in LDS
    auto lut_begin = [&](uint32_t buf, bool fetch) {
        lut_src = (fetch ? dma_base : lut) + dma_lane;
        lut_dst = BUF0 + buf * SLICE + dma_wave;
    };
    auto lut_op = [&](auto uc) {
        constexpr int u = decltype(uc)::value, hi = u / 4, lo = u % 4;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(lut_src + hi * 4096),
                                         (__attribute__((address_space(3))) void*)(smem + lut_dst + hi * 4096), 16, lo * 1024, 0);
    };
    auto lut_advance = [&]() {
        dma_base += SLICE;
        if (++lut_s == nslices) {
            lut_s = 0;
            lut_item += gridDim.x;
            locate_lut();  // may point past the last item; never dereferenced then
        }
    };
    auto stage_lut = [&](uint32_t buf) {
        lut_begin(buf, true);
        static_for<0, DMA_PER_WAVE>([&](auto uc) { lut_op(uc); });
        lut_advance();
    };
    // index words: the same scheme, 256 bytes (64 tokens x one word) per operation; fetch = false: as above,
    // into an index buffer nobody will unpack (from the start of the index buffer: any 64 tokens' words)
    const uint8_t* ix_src = nullptr;
    uint32_t ix_dst = 0;
    auto ix_begin = [&](uint32_t ibuf, bool fetch) {
        ix_src = (fetch ? ix_base : idx) + ix_lane_off;
        ix_dst = IBUF0 + ibuf * IBYTES + wave * IWAVE;
    };
    auto ix_op = [&](auto ic) {
        constexpr int i = decltype(ic)::value;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)ix_src,
                                         (__attribute__((address_space(3))) void*)(smem + ix_dst), 4, 256 * i, 0);
    };
    auto ix_advance = [&]() {
        ix_base += IWORDS * 256;
        if (++ix_s == nslices) {
            ix_s = 0;
            ix_item += gridDim.x;
            if (ix_item < n_items) locate_ix();
        }
    };
    auto stage_ix = [&](uint32_t ibuf) {
        ix_begin(ibuf, true);
        static_for<0, IX_OPS>([&](auto ic) { ix_op(ic); });
        ix_advance();
    };
    // This lane's nibble of K-step ks is nibble 4 (ks & 1) + g of index word ks / 2.  Shifting the
    // word left by 4 for even g puts that nibble into the high half of byte 2 (ks & 1) + g / 2, so
    // after masking, one v_bfe_u32 yields nibble * 16: the byte offset of the one-hot table entry.
    const uint32_t pre_shift = (g & 1) ? 0u : 4u;
    const uint32_t byte_shift = 8 * (g >> 1);
    const uint32_t rot8 = (8 * g + 28) & 31;  // rotate right by 8g - 4
    const uint32_t ix_lane = IBUF0 + wave * IWAVE + (((wave * (TM * 16)) & 63) + j) * 4;
    // The index words are read with inline assembly: the compiler cannot tell these reads from the
    // LDS ranges the copy operations in flight are writing, and would wait for all of them first.
    auto read_ix = [&](uint32_t (&raw)[TM][IWORDS], uint32_t ibuf) {
        const uint32_t addr = ix_lane + ibuf * IBYTES;
        static_for<0, TM * IWORDS>([&](auto ec) {
            constexpr int t = decltype(ec)::value / IWORDS, i = decltype(ec)::value % IWORDS;
            lds_read32<(i * 64 + t * 16) * 4>(raw[t][i], addr);
        });
    };
    auto unpack_ix = [&](uint32_t (&iwm)[TM][IWORDS], uint32_t (&raw)[TM][IWORDS]) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int t = 0; t < TM; ++t)
#pragma unroll
            for (int i = 0; i < IWORDS; ++i) asm volatile("" : "+v"(raw[t][i]));
#pragma unroll
        for (int t = 0; t < TM; ++t)
#pragma unroll
            for (int i = 0; i < IWORDS; ++i) {
                // paired: word i belongs to K-step i and this lane's pair is byte g of it; rotating that
                // byte to bits 4..11 leaves byte * 16, the table entry's offset
                if constexpr (P8) iwm[t][i] = __builtin_amdgcn_alignbit(raw[t][i], raw[t][i], rot8) & 0xFF0u;
                else iwm[t][i] = (raw[t][i] << pre_shift) & 0xF0F0F0F0u;
            }
    };

    v4i acc[TM][TN];
#pragma unroll
    for (int t = 0; t < TM; ++t)
#pragma unroll
        for (int c = 0; c < TN; ++c) acc[t][c] = (v4i){0, 0, 0, 0};

    // The bias values come in through scalar loads (wave-uniform addresses, the scalar counter): a
    // vector load here would make the compiler wait on the vector-memory counter before its first
    // use, i.e. for every output store issued so far and for the slices being prefetched, once per
    // group of stores.  With scalar loads the epilogue contains no such wait and its stores leave
    // back to back.
    auto epilogue_as = [&](uint32_t item, auto actc) __attribute__((always_inline)) -> bool {
        constexpr bool ACT = decltype(actc)::value;
        // j and g pass through an opaque asm so that none of the address arithmetic below is
        // loop-invariant for the compiler: hoisted out of the slice loop it would occupy dozens of
        // registers for the whole kernel
        uint32_t je = j, ge = g;
        asm volatile("" : "+v"(je), "+v"(ge));
        const uint32_t colblk = col_of(item);
        Epilogue epl = ep;
        if (ep.op_col_tiles) epl.scale = scalar_load1(ep.op_scales + colblk / ep.op_col_tiles);
        const uint32_t tile_tok0 = tok_tile_of(item) * OH_TOK_ITEM;
        const uint32_t tok0 = tile_tok0 + wave * (TM * 16);
        const bool vec_store = (M % 4 == 0);
        const bool full = vec_store && !acc_out && tile_tok0 + OH_TOK_ITEM <= N && (colblk + 1) * WN <= M;
#pragma unroll
        for (int c = 0; c < TN; ++c) {
            const uint32_t f0 = colblk * WN + c * 16;  // wave-uniform
            const uint32_t f = f0 + 4 * ge;
            floatx16 b16;
            if (ep.bias && f0 + 16 <= M) {
                b16 = scalar_load16(ep.bias + f0);
            } else {
#pragma unroll
                for (int e = 0; e < 16; ++e) b16[e] = (ep.bias && f0 + e < M) ? scalar_load1(ep.bias + f0 + e) : 0.0f;
            }
            float4 bv;
            bv.x = ge == 0 ? b16[0] : ge == 1 ? b16[4] : ge == 2 ? b16[8] : b16[12];
            bv.y = ge == 0 ? b16[1] : ge == 1 ? b16[5] : ge == 2 ? b16[9] : b16[13];
            bv.z = ge == 0 ? b16[2] : ge == 1 ? b16[6] : ge == 2 ? b16[10] : b16[14];
            bv.w = ge == 0 ? b16[3] : ge == 1 ? b16[7] : ge == 2 ? b16[11] : b16[15];
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                const uint32_t tok = tok0 + t * 16 + je;
                const v4i a = acc[t][c];
                acc[t][c] = (v4i){0, 0, 0, 0};
                float4 o;
                o.x = dequant<ACT>(a[0], epl, bv.x);
                o.y = dequant<ACT>(a[1], epl, bv.y);
                o.z = dequant<ACT>(a[2], epl, bv.z);
                o.w = dequant<ACT>(a[3], epl, bv.w);
                if (full) {  // workgroup-uniform: every token and column of the tile exists
                    // streaming store: the output is not read again by this kernel
                    typedef float v4f __attribute__((ext_vector_type(4)));
                    __builtin_nontemporal_store((v4f){o.x, o.y, o.z, o.w}, reinterpret_cast<v4f*>(out + (size_t)tok * M + f));
                    continue;
                }
                if (tok >= N || f >= M) continue;
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
        return full;
    };
    auto epilogue = [&](uint32_t item) __attribute__((always_inline)) -> bool {
        return ep.act == PIMDL_ACT_GELU_TANH ? epilogue_as(item, std::true_type{}) : epilogue_as(item, std::false_type{});
    };

    // ---- prologue: slices 0 .. PD-1, index words 0 .. PD ------------------------------------------
    locate_lut();
    locate_ix();
    static_for<0, PD + 1>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if (i < total) stage_ix(i);
    });
    static_for<0, PD>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if (i < total) stage_lut(i);
    });
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // also: the one-hot table is complete
    uint32_t iwm[TM][IWORDS], iw_raw[TM][IWORDS];
    read_ix(iw_raw, 0);
    unpack_ix(iwm, iw_raw);

    uint32_t item0 = blockIdx.x;  // the item being consumed
    const uint32_t a_lane = BUF0 + (g * WN + j) * 16;
    uint32_t buf = 0, ibuf_next = 1;  // k % NBUF and (k + 1) % NIBUF
    uint32_t k = 0;                   // position in the flat (item, slice) stream
    // number of stores a wave issues in the epilogue of a full tile (no tail in tokens or columns,
    // float4 stores, no accumulator dump): then, and only then, the count is the same for every wave
    constexpr int EPI_STORES = TM * TN;
    static_assert((PD - 1) * DMA_OPS + EPI_STORES <= 63, "memory counter range");
    bool stores_behind = false;       // the previous item's EPI_STORES stores were issued after its last copy operations

    for (uint32_t it = 0; it < my_items; ++it, item0 += gridDim.x) {
    for (uint32_t s0 = 0; s0 < nslices; ++s0, ++k) {
        // Loads complete in order, so "at most the (PD-1)*DMA_OPS operations issued during the
        // previous PD-1 slices are outstanding" means this wave's share of slice k (and of index
        // words k+1) has landed.  After the barrier everybody's has, and everybody is done with
        // slice k-1, whose buffer slice k+PD goes into.  The copy operations are issued for every
        // slice, also past the end of the stream, so the count never changes -- except that the
        // stores of an item's epilogue sit behind them at the first slice of the next item: when
        // their number is known they are allowed to stay outstanding (they have had no time to
        // drain yet), otherwise the wait is simply stricter than necessary.
        if (k != 0) {
            if (stores_behind) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((PD - 1) * DMA_OPS + EPI_STORES) : "memory");
            else asm volatile("s_waitcnt vmcnt(%0)" ::"n"((PD - 1) * DMA_OPS) : "memory");
            stores_behind = false;
            __syncthreads();
        }
        // This slice's DMA_OPS copy operations (slice k+PD of the LUT, index words k+PD+1) are
        // issued a few at a time between the K-steps: issued together right after the barrier they
        // would hold every wave of the CU at the memory pipeline's queue while the matrix core idles.
        const bool fetch = k + PD < total;            // workgroup-uniform
        const bool fetch_ix = k + PD + 1 < total;     // workgroup-uniform
        const uint32_t lbp = buf >= 1 ? buf - 1 : NBUF - 1;               // (k + PD) % NBUF = (k - 1) % NBUF
        const uint32_t ibp = ibuf_next >= 1 ? ibuf_next - 1 : NIBUF - 1;  // (k + PD + 1) % NIBUF = k % NIBUF
        const uint32_t abase = buf * SLICE + a_lane;
        lut_begin(lbp, fetch);
        ix_begin(ibp, fetch_ix);

        v4i a_op[2][TN], b_op[2][TM];
        // K-step ks covers codebooks 4 ks .. 4 ks + 3 of the slice; this lane's is 4 ks + g.
        // The operands of K-step ks+1 are requested before the MFMAs of K-step ks are issued.
        auto issue_reads = [&](auto ksc) {
            constexpr int ks = decltype(ksc)::value;
            static_for<0, TN>([&](auto cc) {
                constexpr int c = decltype(cc)::value;
                lds_read<(4 * ks * WN + c * 16) * 16>(a_op[ks & 1][c], abase);
            });
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                uint32_t entry;
                if constexpr (P8) entry = iwm[t][ks];
                else entry = __builtin_amdgcn_ubfe(iwm[t][ks / 2], 16 * (ks & 1) + byte_shift, 8);
                lds_read<0>(b_op[ks & 1][t], entry);
            }
        };
        issue_reads(std::integral_constant<int, 0>{});
        static_for<0, KSTEPS>([&](auto ksc) {
            constexpr int ks = decltype(ksc)::value;
            oh_wait<TN, TM>(a_op[ks & 1], b_op[ks & 1]);
            if constexpr (ks + 1 < KSTEPS) issue_reads(std::integral_constant<int, ks + 1>{});
            // the next slice's index words (this wave's own copy, landed before the wait above)
            if constexpr (ks == KSTEPS - 1) read_ix(iw_raw, ibuf_next);
            // (with a prefetch distance of one slice the copies go out in the first half of the K-steps, so
            // that the last of them has half a slice to land)
            constexpr int IK = PD == 1 ? KSTEPS / 2 : KSTEPS;
            static_for<(ks < IK ? ks : IK) * DMA_OPS / IK, (ks + 1 < IK ? ks + 1 : IK) * DMA_OPS / IK>([&](auto oc) {
                constexpr int o = decltype(oc)::value;
                if constexpr (o < DMA_PER_WAVE) lut_op(std::integral_constant<int, o>{});
                else ix_op(std::integral_constant<int, o - DMA_PER_WAVE>{});
            });
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < TM; ++t)
#pragma unroll
                for (int c = 0; c < TN; ++c)
                    acc[t][c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_op[ks & 1][c], b_op[ks & 1][t], acc[t][c], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        });
        if (fetch) {
            lut_advance();
            if (fetch_ix) ix_advance();
        }
        unpack_ix(iwm, iw_raw);

        buf = buf + 1 == NBUF ? 0 : buf + 1;
        ibuf_next = ibuf_next + 1 == NIBUF ? 0 : ibuf_next + 1;
    }
    stores_behind = epilogue(item0);
    }
}

template <int TN, int TM, bool P8, int GS = 16>
int launch_onehot_tm(Ctx* ctx, const Amm& a, const uint8_t* d_idx, float* d_out, int32_t* d_acc, uint32_t n,
                     const Epilogue& ep)
{
    constexpr int LDS = oh_lds_bytes(TN, P8, GS);
    static_assert(2 * LDS <= 160 * 1024, "two workgroups per CU");
    constexpr int OH_TOK_ITEM = oh_tok_item(TM);
    auto kern = gather_onehot_kernel<TN, TM, P8, GS>;
    if (int rc = allow_dynamic_lds(ctx, reinterpret_cast<const void*>(kern), LDS, "hipFuncSetAttribute(gather_onehot)")) return rc;
    const uint32_t n_token_tiles = (n + OH_TOK_ITEM - 1) / OH_TOK_ITEM;
    const uint32_t n_items = n_token_tiles * (a.g.M_pad / (16 * TN));
    uint32_t grid = ctx->prop.multiProcessorCount * 2;  // two workgroups per CU, see plan_geometry
    if (grid > n_items) grid = n_items;
    const uint32_t slice_entries = P8 ? a.g.CB_pad / 2 : a.g.CB_pad;  // codebooks, or pairs of them
    const XcdMap xmap = choose_xcd_map(a.g.M_pad / (16 * TN), n_token_tiles, grid,
                                       (uint64_t)slice_entries * 16 * a.g.M_pad, (uint64_t)n * a.g.idx_row_bytes,
                                       a.g.tune_xcd_col_split);
    snprintf(a.last_gather, sizeof(a.last_gather), "gather_onehot_kernel<%d, %d, %s, %d>", TN, TM, P8 ? "true" : "false", GS);
    a.note_launch(GS, LDS, OH_TOK_ITEM, OH_THREADS);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(OH_THREADS), LDS, ctx->stream, d_idx,
                       reinterpret_cast<const int8_t*>(a.d_lut), d_out, d_acc, n, a.g.M, slice_entries,
                       a.g.idx_row_bytes, n_token_tiles, n_items, ep, xmap);
    return hip_check(ctx, hipGetLastError(), "gather_onehot_kernel launch");
}

// 256-token items (TM = 4) need fewer LDS reads and copies per MFMA; 128-token items (TM = 2) fill the grid
// of a small batch better.  The item size that needs the shorter time wins: rounds of the persistent grid,
// partly filled ones counted for what they cost (grid_rounds), x the cost of an item.
template <int TN, bool P8>
int launch_onehot(Ctx* ctx, const Amm& a, const uint8_t* d_idx, float* d_out, int32_t* d_acc, uint32_t n,
                  const Epilogue& ep)
{
    const uint64_t items4 = (uint64_t)((n + oh_tok_item(4) - 1) / oh_tok_item(4)) * (a.g.M_pad / (16 * TN));
    // Slices of 32 codebooks in two buffers instead of 16 in three, where two workgroups still fit a CU: the
    // per-slice costs (barrier, first operand reads, bookkeeping) are paid half as often.  Measured 3-9 %
    // faster for 48- and 64-column tiles; 96-column tiles only have room for 24, which gained nothing.
    constexpr int GSB = (TN == 3 || (TN == 4 && !P8)) ? 32 : 16;
    const uint64_t slots = 2ull * ctx->prop.multiProcessorCount;
    const uint64_t items2 = (uint64_t)((n + oh_tok_item(2) - 1) / oh_tok_item(2)) * (a.g.M_pad / (16 * TN));
    bool small_items = prefer_small_items(items4, items2, slots);
    if (a.g.tune_token_item) small_items = a.g.tune_token_item == 128;
    if constexpr (GSB != 16) {
        const uint32_t entries = P8 ? a.g.CB_pad / 2 : a.g.CB_pad;
        if (entries % GSB == 0 && a.g.tune_cb_per_slice != 16) {
            if (small_items) return launch_onehot_tm<TN, 2, P8, GSB>(ctx, a, d_idx, d_out, d_acc, n, ep);
            return launch_onehot_tm<TN, 4, P8, GSB>(ctx, a, d_idx, d_out, d_acc, n, ep);
        }
    }
    if (small_items) return launch_onehot_tm<TN, 2, P8>(ctx, a, d_idx, d_out, d_acc, n, ep);
    return launch_onehot_tm<TN, 4, P8>(ctx, a, d_idx, d_out, d_acc, n, ep);
}

// ---------------------------------------------------------------------------------------------
// fp32 LUT: out[n][f] = (sum over cb ascending, fp32) lut[cb][idx][f] + bias[f]
// One lane = one token; a workgroup = 256 tokens x 4*Q columns; slices of GS codebooks in LDS.
//
// GROUPED (int8 table with one scale per `group` consecutive codebooks; not in the reference): the
// table holds the int8 entries converted to fp32, so the sum inside a group is an exact integer
// (|sum| <= 128 * group < 2^24 is checked at creation); at the end of each group
//     tot = tot + (float)acc_g * scale[g]      (two separately rounded operations, groups ascending)
// and out = tot + bias[f].
// ---------------------------------------------------------------------------------------------
constexpr int GF_THREADS = 256;

template <int C_T, int Q, int GS, int IDX_BITS, bool GROUPED, int TPL>
__global__ __launch_bounds__(GF_THREADS) void gather_f32_kernel(const uint8_t* __restrict__ idx,
                                                               const float* __restrict__ lut,
                                                               float* __restrict__ out, uint32_t N,
                                                               uint32_t M, uint32_t CB_pad,
                                                               uint32_t idx_row_bytes,
                                                               const float* __restrict__ bias,
                                                               const float* __restrict__ scales,
                                                               uint32_t CB, uint32_t group, uint32_t act,
                                                               uint32_t n_token_tiles, uint32_t by_xcd)
{
    constexpr int FB = 4 * Q;             // columns per row
    // 32 rows of 16-byte pieces cover the 64 banks twice: two lanes of a ds_read_b128 pass that want
    // different rows 16 apart collide (measured 1.7x the conflict-free time).  8-byte pieces of 32 rows
    // cover the banks exactly once, and a ds_read_b64 takes half the time of a b128: the table for 32
    // centroids is therefore kept as [codebook][8-byte chunk][row], read with twice as many b64 reads
    // and no conflicts (the same layout in HBM, so that staging stays a flat copy).
    constexpr bool CHUNKED = f32_lut_chunked(C_T, Q);
    constexpr int PITCH = CHUNKED ? 16 * Q : 16 * Q + 16;    // bytes
    constexpr int CB_BYTES = C_T * PITCH;
    constexpr int SLICE_LDS = GS * CB_BYTES;
    constexpr int SLICE_UNITS = GS * C_T * Q;
    constexpr int UPT = (SLICE_UNITS + GF_THREADS - 1) / GF_THREADS;
    constexpr int IDX_BYTES = GS * IDX_BITS / 8;
    constexpr int IDX_WORDS = (IDX_BYTES + 3) / 4;
    static_assert(IDX_BYTES % 4 == 0, "index fetch is in dwords");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    // TPL tokens per lane: the staged slice serves TPL * 256 tokens, so the table is streamed from L2
    // 1/TPL as often
    uint32_t tok[TPL];
    // Workgroup p of the 1-D grid: column block p / n_token_tiles, token tile p % n_token_tiles -- or, by_xcd
    // (column blocks a multiple of 8): workgroups go to the 8 XCDs round-robin, and XCD p % 8 takes every token
    // tile of the column blocks congruent to it, so that a column block's part of the table is streamed
    // through one L2 instead of all eight.
    const uint32_t pq = by_xcd ? blockIdx.x / 8 : blockIdx.x;
    const uint32_t tile = pq % n_token_tiles;
    const uint32_t colblk = by_xcd ? blockIdx.x % 8 + 8 * (pq / n_token_tiles) : pq / n_token_tiles;
#pragma unroll
    for (int t = 0; t < TPL; ++t) tok[t] = (tile * TPL + t) * GF_THREADS + threadIdx.x;
    const uint32_t nslices = CB_pad / GS;
    const uint4* __restrict__ lut_blk = reinterpret_cast<const uint4*>(lut) + (size_t)colblk * CB_pad * C_T * Q;
    const uint32_t* idx_row[TPL];
#pragma unroll
    for (int t = 0; t < TPL; ++t)
        idx_row[t] = reinterpret_cast<const uint32_t*>(idx + (size_t)(tok[t] < N ? tok[t] : N - 1) * idx_row_bytes);

    float acc[TPL][FB];
    float tot[TPL][GROUPED ? FB : 1];
#pragma unroll
    for (int t = 0; t < TPL; ++t) {
#pragma unroll
        for (int i = 0; i < FB; ++i) acc[t][i] = 0.0f;
#pragma unroll
        for (int i = 0; i < (GROUPED ? FB : 1); ++i) tot[t][i] = 0.0f;
    }
    uint32_t cb = 0, in_group = 0, gi = 0;  // workgroup-uniform position in the codebook sequence

    uint4 stage[UPT];
    uint32_t idx_cur[TPL][IDX_WORDS], idx_nxt[TPL][IDX_WORDS];
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
                *reinterpret_cast<uint4*>(dst_ + (CHUNKED ? unit_ * 16 : (unit_ / Q) * PITCH + (unit_ % Q) * 16)) = stage[u]; \
        }                                                                                           \
    }
    PIMDL_FETCH_SLICE(0)
#pragma unroll
    for (int t = 0; t < TPL; ++t)
#pragma unroll
        for (int w = 0; w < IDX_WORDS; ++w) idx_cur[t][w] = idx_row[t][w];
    PIMDL_COMMIT_SLICE(0)
    __syncthreads();

    constexpr int per_word = 32 / IDX_BITS;
    for (uint32_t s = 0; s < nslices; ++s) {
        const uint32_t sn = s + 1 < nslices ? s + 1 : s;
        PIMDL_FETCH_SLICE(sn)
#pragma unroll
        for (int t = 0; t < TPL; ++t)
#pragma unroll
            for (int w = 0; w < IDX_WORDS; ++w) idx_nxt[t][w] = idx_row[t][sn * IDX_WORDS + w];
        const unsigned char* cbbase = smem + (s & 1) * SLICE_LDS;
#pragma unroll
        for (int w = 0; w < IDX_WORDS; ++w) {
            uint32_t word[TPL];
#pragma unroll
            for (int t = 0; t < TPL; ++t) word[t] = idx_cur[t][w];
            // ascending codebook order; partial unroll keeps the loads in flight within the VGPR budget
#pragma unroll 2
            for (int h = 0; h < per_word; ++h) {
#pragma unroll
                for (int t = 0; t < TPL; ++t) {
                    const uint32_t r = word[t] & ((1u << IDX_BITS) - 1);
                    word[t] >>= IDX_BITS;
                    if constexpr (CHUNKED) {
                        const unsigned char* row = cbbase + r * 8;
#pragma unroll
                        for (int c = 0; c < 2 * Q; ++c) {
                            // volatile: keeps the compiler from pairing two chunks into one ds_read2_b64, whose
                            // halves (256 bytes apart) would meet in the same banks
                            typedef float v2f __attribute__((ext_vector_type(2)));
                            const v2f vv = *(const volatile __attribute__((address_space(3))) v2f*)(row + c * (C_T * 8));
                            acc[t][2 * c + 0] = __fadd_rn(acc[t][2 * c + 0], vv[0]);
                            acc[t][2 * c + 1] = __fadd_rn(acc[t][2 * c + 1], vv[1]);
                        }
                    } else {
                        const unsigned char* row = cbbase + r * PITCH;
#pragma unroll
                        for (int c = 0; c < Q; ++c) {
                            const float4 vv = *reinterpret_cast<const float4*>(row + c * 16);
                            acc[t][4 * c + 0] = __fadd_rn(acc[t][4 * c + 0], vv.x);
                            acc[t][4 * c + 1] = __fadd_rn(acc[t][4 * c + 1], vv.y);
                            acc[t][4 * c + 2] = __fadd_rn(acc[t][4 * c + 2], vv.z);
                            acc[t][4 * c + 3] = __fadd_rn(acc[t][4 * c + 3], vv.w);
                        }
                    }
                }
                cbbase += CB_BYTES;
                if constexpr (GROUPED) {
                    // codebooks past CB are padding (zero rows) and belong to no group
                    if (cb < CB && (++in_group == group || cb + 1 == CB)) {
                        const float sc = scales[gi];
#pragma unroll
                        for (int t = 0; t < TPL; ++t)
#pragma unroll
                            for (int i = 0; i < FB; ++i) {
                                tot[t][i] = __fadd_rn(tot[t][i], __fmul_rn(acc[t][i], sc));
                                acc[t][i] = 0.0f;
                            }
                        ++gi;
                        in_group = 0;
                    }
                    ++cb;
                }
            }
        }
        PIMDL_COMMIT_SLICE((s + 1) & 1)
#pragma unroll
        for (int t = 0; t < TPL; ++t)
#pragma unroll
            for (int w = 0; w < IDX_WORDS; ++w) idx_cur[t][w] = idx_nxt[t][w];
        __syncthreads();
    }
#undef PIMDL_FETCH_SLICE
#undef PIMDL_COMMIT_SLICE

    const bool vec_store = (M % 4 == 0);  // then every 4-column piece is whole and 16-byte aligned
#pragma unroll
    for (int t = 0; t < TPL; ++t) {
        if (tok[t] >= N) continue;
#pragma unroll
        for (int c = 0; c < Q; ++c) {
            const uint32_t f = colblk * FB + 4 * c;
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
                o[e] = activate(__fadd_rn(GROUPED ? tot[t][4 * c + e] : acc[t][4 * c + e], (bias && f + e < M) ? bias[f + e] : 0.0f), act);
            if (vec_store) {
                if (f < M) *reinterpret_cast<float4*>(out + (size_t)tok[t] * M + f) = make_float4(o[0], o[1], o[2], o[3]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (f + e < M) out[(size_t)tok[t] * M + f + e] = o[e];
            }
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
    if (int rc = allow_dynamic_lds(ctx, reinterpret_cast<const void*>(kern), LDS, "hipFuncSetAttribute(gather_i8)")) return rc;
    const uint32_t n_token_tiles = (n + TOK_ITEM - 1) / TOK_ITEM;
    const uint32_t n_items = n_token_tiles * (a.g.M_pad / (16 * Q));
    // persistent grid: as many workgroups as fit at once (LDS-limited), never more than there are items
    const uint32_t per_cu = LDS > 0 ? (uint32_t)(ctx->prop.maxSharedMemoryPerMultiProcessor / LDS) : 1;
    uint32_t grid = ctx->prop.multiProcessorCount * (per_cu < 1 ? 1 : per_cu > 2 ? 2 : per_cu);
    if (grid > n_items) grid = n_items;
    snprintf(a.last_gather, sizeof(a.last_gather), "gather_i8_kernel<%d, %d, %d, %d, %d>", C_T, Q, GQ, TG, IDX_BITS);
    a.note_launch(4 * GQ, LDS, TOK_ITEM, GATHER_THREADS);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(GATHER_THREADS), LDS, ctx->stream, d_idx,
                       reinterpret_cast<const int8_t*>(a.d_lut), d_out, d_acc, n, a.g.M, a.g.CB_pad,
                       a.g.idx_row_bytes, n_token_tiles, n_items, ep);
    return hip_check(ctx, hipGetLastError(), "gather_i8_kernel launch");
}

template <int C_T, int Q, int GS, int IDX_BITS, bool GROUPED, int TPL>
int launch_f32_impl(Ctx* ctx, const Amm& a, const uint8_t* d_idx, float* d_out, uint32_t n)
{
    constexpr int LDS = 2 * GS * C_T * (f32_lut_chunked(C_T, Q) ? 16 * Q : 16 * Q + 16);
    auto kern = gather_f32_kernel<C_T, Q, GS, IDX_BITS, GROUPED, TPL>;
    if (int rc = allow_dynamic_lds(ctx, reinterpret_cast<const void*>(kern), LDS, "hipFuncSetAttribute(gather_f32)")) return rc;
    const uint32_t n_token_tiles = (n + GF_THREADS * TPL - 1) / (GF_THREADS * TPL), colblocks = a.g.M_pad / (4 * Q);
    const uint64_t wgs = (uint64_t)n_token_tiles * colblocks;
    if (wgs > 0x7FFFFFFFull) return set_error(ctx, PIMDL_ERR_UNSUPPORTED, "gather: %llu workgroups", (unsigned long long)wgs);
    const uint32_t by_xcd = colblocks % 8 == 0 ? 1u : 0u;
    snprintf(a.last_gather, sizeof(a.last_gather), "gather_f32_kernel<%d, %d, %d, %d, %s, %d>", C_T, Q, GS, IDX_BITS, GROUPED ? "true" : "false", TPL);
    a.note_launch(GS, LDS, GF_THREADS * TPL, GF_THREADS);
    hipLaunchKernelGGL(kern, dim3((uint32_t)wgs), dim3(GF_THREADS), LDS, ctx->stream, d_idx,
                       reinterpret_cast<const float*>(a.d_lut), d_out, n, a.g.M, a.g.CB_pad, a.g.idx_row_bytes,
                       a.d_bias, a.d_scales, a.g.CB, a.desc.scale_group, a.desc.activation, n_token_tiles, by_xcd);
    return hip_check(ctx, hipGetLastError(), "gather_f32_kernel launch");
}

// workgroups of gather_f32_kernel that one CU holds at a time (asked once per variant)
template <int C_T, int Q, int GS, int IDX_BITS, bool GROUPED, int TPL>
int f32_wgs_per_cu()
{
    static int cached = 0;
    if (cached == 0) {
        constexpr int LDS = 2 * GS * C_T * (f32_lut_chunked(C_T, Q) ? 16 * Q : 16 * Q + 16);
        int q = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&q, gather_f32_kernel<C_T, Q, GS, IDX_BITS, GROUPED, TPL>, GF_THREADS,
                                                         LDS) != hipSuccess || q < 1) {
            (void)hipGetLastError();
            q = 1;
        }
        cached = q;
    }
    return cached;
}

template <int C_T, int Q, int GS, int IDX_BITS, bool GROUPED>
int launch_f32_tpl(Ctx* ctx, const Amm& a, const uint8_t* d_idx, float* d_out, uint32_t n)
{
    // Two tokens per lane halve the table traffic from L2 for batches that still give every CU two workgroups.
    // The grid is not persistent, so a batch pays for whole rounds of resident workgroups, and workgroups of
    // two tokens per lane are twice as long: for tables beyond the caches (where the ViT-Base sweep at
    // N = 12608 measured it to matter: 5 of 6 shapes 10-28 % faster, one 7 % slower) the variant with the
    // shorter rounds x length is taken, one token per lane counted 6 % dearer per token for its extra staging.
    const uint64_t cus = ctx->prop.multiProcessorCount, colblocks = a.g.M_pad / (4 * Q);
    const uint64_t wgs2 = (uint64_t)((n + 2 * GF_THREADS - 1) / (2 * GF_THREADS)) * colblocks;
    bool two = wgs2 >= 2 * cus;
    if (two && a.lut_bytes > (64ull << 20)) {
        const uint64_t wgs1 = (uint64_t)((n + GF_THREADS - 1) / GF_THREADS) * colblocks;
        const uint64_t slots1 = cus * (uint64_t)f32_wgs_per_cu<C_T, Q, GS, IDX_BITS, GROUPED, 1>();
        const uint64_t slots2 = cus * (uint64_t)f32_wgs_per_cu<C_T, Q, GS, IDX_BITS, GROUPED, 2>();
        two = 200 * ((wgs2 + slots2 - 1) / slots2) <= 106 * ((wgs1 + slots1 - 1) / slots1);
    }
    if (two) return launch_f32_impl<C_T, Q, GS, IDX_BITS, GROUPED, 2>(ctx, a, d_idx, d_out, n);
    return launch_f32_impl<C_T, Q, GS, IDX_BITS, GROUPED, 1>(ctx, a, d_idx, d_out, n);
}

template <int C_T, int Q, int GS, int IDX_BITS>
int launch_f32(Ctx* ctx, const Amm& a, const uint8_t* d_idx, float* d_out, uint32_t n)
{
    return a.grouped && !a.prescaled ? launch_f32_tpl<C_T, Q, GS, IDX_BITS, true>(ctx, a, d_idx, d_out, n)
                     : launch_f32_tpl<C_T, Q, GS, IDX_BITS, false>(ctx, a, d_idx, d_out, n);
}

}  // namespace

// Tiling choices per centroid count.  int8: slice = 4*GQ codebooks, rows of 64 bytes (Q=4) except for
// the largest tables; two slices must fit the 160 KB LDS.  fp32: rows of 16 floats (Q=4).
//   C_T   int8 (Q, GQ) -> slice bytes        fp32 (Q, GS) -> slice bytes
//   8     (4, 8)  20 KB                      (4, 32) 20 KB
//   16    (4, 8)  40 KB                      (4, 16) 20 KB
//   32    (4, 4)  40 KB                      (4, 8)  20 KB
//   64    (4, 2)  40 KB                      (4, 8)  40 KB
//   128   (2, 2)  48 KB                      (2, 8)  48 KB
//   256   (2, 1)  48 KB                      (2, 4)  48 KB
// PIMDL_GATHER_ROWS=1 in the environment keeps the byte-adder kernel for every shape (the one-hot
// kernel gives the same bits; this is for comparing the two).
bool gather_rows_only()
{
    static const bool v = [] {
        const char* e = getenv("PIMDL_GATHER_ROWS");
        return e && e[0] == '1';
    }();
    return v;
}

// PIMDL_GATHER_DENSE=1 in the environment keeps the dense one-hot kernel where the sparse-instruction kernel
// would run (same bits; for comparing the two).
bool gather_dense_only()
{
    static const bool v = [] {
        const char* e = getenv("PIMDL_GATHER_DENSE");
        return e && e[0] == '1';
    }();
    return v;
}

bool apply_runtime_tuning(AmmGeom* g, const pimdl_amm_tuning& t, std::string* why)
{
    const bool matrix_core = g->gather_kind != 0;
    const bool eight_waves = t.token_item == 512 && g->gather_kind == 2 && g->C_tile != 32;  // one workgroup of eight waves per CU
    if (t.token_item && (!matrix_core || (t.token_item != 128 && t.token_item != 256 && !eight_waves))) {
        *why = "token_item must be 128 or 256 (512 for the sparse kernel up to 16 centroids), and only the matrix-core gathers (int8, up to 32 centroids) have it";
        return false;
    }
    if (t.cb_per_slice) {
        const uint32_t entries = g->C_tile == 8 ? g->CB_pad / 2 : g->C_tile == 32 ? 2 * g->CB_pad : g->CB_pad;  // table entries of 16 slots
        const bool has32 = eight_waves || (g->gather_kind == 2 ? g->q <= 4 : (g->q == 3 || (g->q == 4 && g->C_tile != 8)));
        // 64-codebook slices: eight waves, either 512-token items or 256-token items whose two waves of a SIMD
        // split the slice between them
        const bool has64 = g->q == 3 && (eight_waves || (t.token_item == 256 && g->gather_kind == 2 && g->C_tile != 32));
        if (!matrix_core || (t.cb_per_slice == 16 && eight_waves && g->q == 3) ||
            (t.cb_per_slice != 16 && !(t.cb_per_slice == 32 && has32 && entries % 32 == 0) &&
                             !(t.cb_per_slice == 64 && has64 && entries % 64 == 0))) {
            *why = "cb_per_slice must be 16, or 32 / 64 where the operator's kernel has that variant";
            return false;
        }
    }
    if (t.xcd_col_split && t.xcd_col_split != PIMDL_XCD_PLAIN &&
        (!matrix_core || (t.xcd_col_split != 1 && t.xcd_col_split != 2 && t.xcd_col_split != 4 && t.xcd_col_split != 8))) {
        *why = "xcd_col_split must be 1, 2, 4, 8 or PIMDL_XCD_PLAIN, and only the matrix-core gathers have it";
        return false;
    }
    if (t.search_kernel > PIMDL_SEARCH_MFMA_BF16) { *why = "unknown search_kernel"; return false; }
    const bool v248 = g->v == 2 || g->v == 4 || g->v == 8;
    if (t.search_kernel == PIMDL_SEARCH_MFMA_F32 && !(g->C <= 16 && v248)) {
        *why = "the fp32 matrix-core search needs up to 16 centroids and sub_vec_len 2, 4 or 8";
        return false;
    }
    if (t.search_kernel == PIMDL_SEARCH_MFMA_BF16 && !(g->C <= 32 && v248)) {
        *why = "the bf16 matrix-core search needs up to 32 centroids and sub_vec_len 2, 4 or 8";
        return false;
    }
    if (t.search_token_tile && t.search_token_tile != 64 && t.search_token_tile != 128) {
        *why = "search_token_tile must be 64 or 128";
        return false;
    }
    g->tune_search_tile = t.search_token_tile;
    g->tune_token_item = t.token_item;
    g->tune_cb_per_slice = t.cb_per_slice;
    g->tune_xcd_col_split = t.xcd_col_split;
    g->tune_search = t.search_kernel;
    return true;
}

bool plan_geometry(const pimdl_amm_desc& d, uint32_t num_cus, AmmGeom* g, std::string* why, const pimdl_amm_tuning* tuning)
{
    const pimdl_amm_tuning none = {0, 0, 0, 0, 0, 0, 0};
    const pimdl_amm_tuning& tune = tuning ? *tuning : none;
    const uint32_t col_block_hint = tune.col_block;
    const uint32_t K = d.input_feature_len, v = d.sub_vec_len, C = d.num_centroid, M = d.output_feature_len;
    if (!K || !v || !C || !M || !d.max_n) { *why = "zero-sized dimension"; return false; }
    if (K % v) { *why = "input_feature_len is not a multiple of sub_vec_len"; return false; }
    if (C < 1 || C > 256) { *why = "num_centroid must be in 1..256"; return false; }
    if (d.lut_dtype != PIMDL_LUT_I8 && d.lut_dtype != PIMDL_LUT_F32) { *why = "unknown lut_dtype"; return false; }
    if (d.bias_mode != PIMDL_BIAS_ONCE && d.bias_mode != PIMDL_BIAS_TIMES_CB) { *why = "unknown bias_mode"; return false; }
    if (d.activation != PIMDL_ACT_NONE && d.activation != PIMDL_ACT_GELU_TANH) { *why = "unknown activation"; return false; }
    g->K = K; g->v = v; g->CB = K / v; g->C = C; g->M = M;
    g->CB_pad = (g->CB + 31) / 32 * 32;
    uint32_t ct = 8;
    while (ct < C) ct *= 2;
    g->C_tile = ct;
    g->idx_bits = C <= 16 ? 4 : 8;
    g->idx_row_bytes = g->CB_pad * g->idx_bits / 8;
    const bool i8 = d.lut_dtype == PIMDL_LUT_I8;
    g->q = ct >= 128 ? 2 : 4;
    g->gather_kind = (i8 && C <= 16 && !gather_rows_only()) ? 1 : 0;
    if (g->gather_kind == 1 && C > 8 && !gather_dense_only()) g->gather_kind = 2;
    // 17..32 centroids: the sparse kernel with every codebook as two of 16
    if (i8 && C > 16 && C <= 32 && !gather_rows_only() && !gather_dense_only()) g->gather_kind = 2;
    switch (tune.gather_kernel) {
        case PIMDL_GATHER_AUTO: break;
        case PIMDL_GATHER_ROWS:
            g->gather_kind = 0;
            break;
        case PIMDL_GATHER_ONEHOT:
            if (!(i8 && C <= 16)) { *why = "the one-hot gather needs an int8 table with up to 16 centroids"; return false; }
            g->gather_kind = 1;
            break;
        case PIMDL_GATHER_SPARSE:
            if (!(i8 && C <= 32)) { *why = "the sparse one-hot gather needs an int8 table with up to 32 centroids"; return false; }
            g->gather_kind = 2;
            break;
        default: *why = "unknown gather_kernel"; return false;
    }
    g->idx_tiled = g->gather_kind != 0;
    if (g->gather_kind != 0) {
        // One-hot matrix-core kernel: an item is 256 tokens x 16*TN columns.  Take the TN with the shortest
        // launch for the largest batch this operator will see: rounds of the persistent grid (two workgroups
        // per CU; grid_rounds) x the cost of an item of that width; among equals the widest.
        // up to 8 centroids: two codebooks share a lane's 16 K-slots (C_tile 8); 96-column tiles then do not
        // leave room for two workgroups per CU
        const uint32_t slots = 2 * (num_cus ? num_cus : 256);
        const uint32_t tiles = (d.max_n + 255) / 256;
        auto pick_tn = [&](bool paired_layout) {
            double best = 1e300;
            uint32_t pick = 0;
            for (uint32_t tn : {6u, 4u, 3u}) {
                if (paired_layout && tn == 6) continue;
                if (col_block_hint && col_block_hint != 16 * tn) continue;
                const uint32_t blocks = (M + 16 * tn - 1) / (16 * tn);
                const uint64_t items = (uint64_t)tiles * blocks;
                const uint64_t items_small = (uint64_t)((d.max_n + 127) / 128) * blocks;
                const double t256 = grid_rounds(items, slots) * item_cost(tn, false);
                const double t128 = grid_rounds(items_small, slots) * item_cost(tn, true);
                const double t = t128 < t256 ? t128 : t256;  // the launcher takes the better item size
                if (t < best - 1e-9) {
                    best = t;
                    pick = tn;
                }
            }
            return pick;
        };
        // Up to 8 centroids, kernel not named by the caller: the paired dense kernel has the cheaper K-loop, the
        // sparse kernel (the table as 16 centroids with empty rows) the cheaper epilogue and the 96-column tile.
        // Measured over N 2048..12608, K and M 768..4096, vec_len 2..8: the sparse kernel is 3 to 38 % faster where
        // the launch is large against its codebook count (tokens x columns >= 65536 x codebooks) and either
        // 96-column tiles are its best launch or there are at most 128 codebooks; elsewhere 0 to 20 % slower.
        if (C <= 8 && g->gather_kind == 1 && tune.gather_kernel == PIMDL_GATHER_AUTO && !gather_dense_only() &&
            (col_block_hint == 96 ||  // (only the sparse kernel has that tile)
             ((uint64_t)d.max_n * M >= 65536ull * g->CB && (pick_tn(false) == 6 || g->CB <= 128))))
            g->gather_kind = 2;
        const bool paired = C <= 8 && g->gather_kind == 1;
        g->C_tile = paired ? 8 : C > 16 ? 32 : 16;
        if (col_block_hint && col_block_hint != 64 && col_block_hint != 48 && (paired || col_block_hint != 96)) {
            *why = paired ? "column tile hint must be 48 or 64 for this operator"
                          : "column tile hint must be 48, 64 or 96 for this operator";
            return false;
        }
        g->q = pick_tn(paired);
        g->gq = 4;
        g->cb_per_slice = 16;
        g->col_block = 16 * g->q;
        g->gather_threads = 256;
        g->tokens_per_wg = 256;
        g->row_pitch = 16;
        g->gather_lds_bytes = g->gather_kind == 2 ? sparse_lds_bytes(g->q, C > 16) : (uint32_t)oh_lds_bytes((int)g->q, paired);
        g->M_pad = (M + g->col_block - 1) / g->col_block * g->col_block;
        g->ccs_cb_per_wg = ccs_cb_per_wg(v);
        g->ccs_row_floats = g->ccs_cb_per_wg * v;
        g->ccs_lds_bytes = g->ccs_cb_per_wg ? 64 * (g->ccs_row_floats + 4) * 4 : 0;
        return apply_runtime_tuning(g, tune, why);
    }
    if (i8 && ct >= 16 && ct <= 64) {
        // Column block of 64 or 48 columns: take the one that fills the persistent grid (two
        // workgroups per CU) more evenly for the largest batch this operator will see.  An item is
        // 256 tokens x one column block; all items cost the same.
        const uint32_t slots = 2 * (num_cus ? num_cus : 256);
        const uint32_t tiles = (d.max_n + 255) / 256;
        double best = -1.0;
        if (col_block_hint && col_block_hint != 64 && col_block_hint != 48) {
            *why = "column tile hint must be 48 or 64 for this operator";
            return false;
        }
        for (uint32_t q : {4u, 3u}) {
            if (col_block_hint && col_block_hint != 16 * q) continue;
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
        g->cb_per_slice = ct == 8 ? 32 : ct == 16 ? 16 : ct <= 128 ? 8 : 4;
        g->col_block = 4 * g->q;
        g->gather_threads = GF_THREADS;
        g->tokens_per_wg = GF_THREADS;
    }
    g->lut_chunked = !i8 && f32_lut_chunked((int)ct, (int)g->q);
    g->row_pitch = g->lut_chunked ? 16 * g->q : 16 * (g->q | 1);
    g->gather_lds_bytes = 2 * g->cb_per_slice * ct * g->row_pitch;
    g->M_pad = (M + g->col_block - 1) / g->col_block * g->col_block;
    g->ccs_cb_per_wg = ccs_cb_per_wg(v);
    g->ccs_row_floats = g->ccs_cb_per_wg * v;
    g->ccs_lds_bytes = g->ccs_cb_per_wg ? 64 * (g->ccs_row_floats + 4) * 4 : 0;
    if (col_block_hint && !i8) { *why = "fp32 tables have one column block width"; return false; }
    return apply_runtime_tuning(g, tune, why);
}

int launch_gather(Ctx* ctx, const Amm& a, const uint8_t* d_idx, float* d_out, int32_t* d_acc, uint32_t n)
{
    if (n == 0) return PIMDL_OK;
    const AmmGeom& g = a.g;
    if (a.desc.lut_dtype == PIMDL_LUT_I8 && !a.grouped) {
        Epilogue ep;
        ep.scale = a.h_scale0;
        ep.lut_bias_term = a.desc.bias_mode == PIMDL_BIAS_TIMES_CB ? a.desc.lut_bias * (float)g.CB : a.desc.lut_bias;
        ep.bias = a.d_bias;
        ep.act = a.desc.activation;
        ep.op_scales = a.d_op_scales;
        ep.op_col_tiles = a.op_col_tiles;
        ep.op_idx_stride = a.op_idx_stride;
        if (g.gather_kind == 2) return launch_gather_sparse(ctx, a, d_idx, d_out, d_acc, n, ep.scale, ep.lut_bias_term);
        if (g.gather_kind == 1) {
            if (g.C_tile == 8) {
                switch (g.q) {
                    case 3: return launch_onehot<3, true>(ctx, a, d_idx, d_out, d_acc, n, ep);
                    case 4: return launch_onehot<4, true>(ctx, a, d_idx, d_out, d_acc, n, ep);
                }
            } else {
                switch (g.q) {
                    case 3: return launch_onehot<3, false>(ctx, a, d_idx, d_out, d_acc, n, ep);
                    case 4: return launch_onehot<4, false>(ctx, a, d_idx, d_out, d_acc, n, ep);
                    case 6: return launch_onehot<6, false>(ctx, a, d_idx, d_out, d_acc, n, ep);
                }
            }
            return set_error(ctx, PIMDL_ERR_UNSUPPORTED, "no one-hot gather kernel for %u column groups", g.q);
        }
        // 64 centroids and more: a slice holds few codebooks (8, 8, 4), so an item's time goes to its slices'
        // barriers and staging as much as to its reads; four token groups per wave (items of 8 waves x 64 = 512
        // tokens instead of 256) halve the slices per token where the batch still gives every resident workgroup
        // (two per CU) such an item (measured at N = 8192, 768 -> 3072: C = 64 145 -> 140 us, C = 128 237 -> 186,
        // C = 256 416 -> 338; with fewer items, 3072 -> 768 at C = 256, 407 -> 434)
        constexpr uint32_t TOK_ITEM4 = GATHER_WAVES * 4 * 16;
        const uint64_t items4 = (uint64_t)((n + TOK_ITEM4 - 1) / TOK_ITEM4) * (g.M_pad / g.col_block);
        const bool tg4 = g.C_tile >= 64 && items4 >= 2ull * ctx->prop.multiProcessorCount;
        switch (g.C_tile) {
            case 8: return launch_i8<8, 4, 8, 2, 4>(ctx, a, d_idx, d_out, d_acc, n, ep);
            case 16:
                return g.q == 3 ? launch_i8<16, 3, 8, 2, 4>(ctx, a, d_idx, d_out, d_acc, n, ep)
                                : launch_i8<16, 4, 8, 2, 4>(ctx, a, d_idx, d_out, d_acc, n, ep);
            case 32:
                return g.q == 3 ? launch_i8<32, 3, 4, 2, 8>(ctx, a, d_idx, d_out, d_acc, n, ep)
                                : launch_i8<32, 4, 4, 2, 8>(ctx, a, d_idx, d_out, d_acc, n, ep);
            case 64:
                if (tg4)
                    return g.q == 3 ? launch_i8<64, 3, 2, 4, 8>(ctx, a, d_idx, d_out, d_acc, n, ep)
                                    : launch_i8<64, 4, 2, 4, 8>(ctx, a, d_idx, d_out, d_acc, n, ep);
                return g.q == 3 ? launch_i8<64, 3, 2, 2, 8>(ctx, a, d_idx, d_out, d_acc, n, ep)
                                : launch_i8<64, 4, 2, 2, 8>(ctx, a, d_idx, d_out, d_acc, n, ep);
            case 128:
                return tg4 ? launch_i8<128, 2, 2, 4, 8>(ctx, a, d_idx, d_out, d_acc, n, ep)
                           : launch_i8<128, 2, 2, 2, 8>(ctx, a, d_idx, d_out, d_acc, n, ep);
            case 256:
                return tg4 ? launch_i8<256, 2, 1, 4, 8>(ctx, a, d_idx, d_out, d_acc, n, ep)
                           : launch_i8<256, 2, 1, 2, 8>(ctx, a, d_idx, d_out, d_acc, n, ep);
        }
    } else {
        switch (g.C_tile) {
            case 8: return launch_f32<8, 4, 32, 4>(ctx, a, d_idx, d_out, n);
            case 16: return launch_f32<16, 4, 16, 4>(ctx, a, d_idx, d_out, n);
            case 32: return launch_f32<32, 4, 8, 8>(ctx, a, d_idx, d_out, n);
            case 64: return launch_f32<64, 4, 8, 8>(ctx, a, d_idx, d_out, n);
            case 128: return launch_f32<128, 2, 8, 8>(ctx, a, d_idx, d_out, n);
            case 256: return launch_f32<256, 2, 4, 8>(ctx, a, d_idx, d_out, n);
        }
    }
    return set_error(ctx, PIMDL_ERR_UNSUPPORTED, "no gather kernel for C_tile=%u", g.C_tile);
}

}  // namespace pimdl
