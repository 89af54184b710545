// LUT gather-accumulate on the sparse matrix instruction (gfx950), int8 tables with up to 32 centroids
// (9..32 always; up to 8 where the launch rule of plan_geometry prefers it to the paired dense kernel).
//
// Same operator as the other gather kernels (inference-engine/src/dpu/pim_lut_kernel.c:97-2296, row-major
// statement inference-engine/test/test_amm.cpp:164-175, epilogue inference-engine/src/host/pim_lut_host.cpp:190-203):
//     acc[n][f] = sum over cb of lut[cb][idx[n][cb]][f]          (int8 table, int32 sum, exact)
// in the reference's own matrix form (model-calibration/LUTNeuro/LUTLinear_t.py:78, bmm(one_hot, lut)).
//
// A one-hot row over the 16 centroids of a codebook has at most one non-zero in every group of four
// positions, which is a valid 2:4 structured-sparse operand.  v_smfmac_i32_16x16x128_i8 multiplies a
// 16 x 128 matrix given in that compressed form (per lane: 16 value bytes + 16 two-bit positions) by a dense
// 128 x 16 one: with the one-hot as the sparse operand, ONE instruction gathers and adds 8 codebooks for
// 16 tokens x 16 columns, twice what the dense v_mfma_i32_16x16x64_i8 form of the one-hot product does, at
// the same issue rate (measured: 16.5 clocks per instruction and SIMD for either).
//
// Operands of one instruction (K-step = 8 codebooks b = 0..7 of a slice), lane l = 16 g + i:
//   sparse A (tokens x K)  lane (g, i) holds, for token i of the 16-token group, codebooks 2g (value bytes
//             0..7) and 2g+1 (value bytes 8..15): each codebook is four groups of two value slots; the group
//             that contains the token's centroid c (group c / 4) has value 1 in its first slot with position
//             c % 4, everything else is 0.  Both codebooks' nibbles are one byte of the packed index row.
//             The 8 value bytes of a nibble are the 64-bit number 1 << 16 (c / 4): one shift.  (With 17..32
//             centroids they come from a table in LDS, entry c 16 bytes apart: 8-byte reads of such entries do
//             not meet in a bank.)  The lane's whole position word (16 bits per nibble) comes from a second
//             table with one 4-byte word per value of the index byte.
//   dense B (K x columns)  lane (g, j) holds column j's 16 centroid entries of codebook g (bytes 0..15) and
//             of codebook g + 4 (bytes 16..31): two 16-byte reads of the tiled table, whose layout is that
//             of the dense one-hot kernel ([column tile][codebook][column][16 centroids]).
//   D (tokens x columns)   lane (g, j) holds tokens 4g..4g+3 of the group for column j.
// (This pairing of lane groups and codebooks was read off the instruction on the device with one-hot probes.)
//
// A lane thus ends up with four tokens of ONE column per 16-column group.  So that its stores are still
// 16 bytes wide, the columns of a tile are dealt to the 16-column groups in pieces: the first 4 * (TN / 4)
// groups in fours (group c of a four holds columns 4 j + c: a lane's four accumulator tiles are four
// consecutive columns), then a pair (columns 2 j + c), then a single group.  The permutation is applied once
// when the table is tiled at upload (sparse_tile_column); reads of the table from LDS stay consecutive.
//
// Work decomposition, staging through LDS with global_load_lds, the dealing of items to the XCDs, the fused
// de-quantisation / bias / GELU epilogue and operator groups are those of the dense one-hot kernel.
//
// 17..32 centroids (WIDE): a codebook of 32 centroids is two of 16 side by side, of which the token's centroid
// lies in one and the other contributes nothing.  The table is tiled as 2 CB codebooks of 16 (centroids 0..15,
// then 16..31), the index row holds one byte per codebook where the 16-centroid form holds two nibbles, and the
// lane looks its byte up in two 32-entry tables: the first has the one-hot entries for bytes 0..15 and zero
// entries for 16..31, the second the other way round.  Everything else is the same kernel; one instruction then
// covers 4 codebooks.
#include "gather_common.h"

namespace pimdl {

// column (within its tile of 16 * tn columns) stored at position s = 16 c + j of the tile
uint32_t sparse_tile_column(uint32_t tn, uint32_t s)
{
    const uint32_t c = s / 16, j = s % 16;
    const uint32_t n4 = tn / 4 * 4;                 // groups dealt in fours
    const uint32_t n2 = n4 + (tn % 4) / 2 * 2;      // ... then a pair
    if (c < n4) return 16 * (c / 4 * 4) + 4 * j + c % 4;
    if (c < n2) return 16 * n4 + 2 * j + (c - n4);
    return 16 * c + j;
}

namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v2i __attribute__((ext_vector_type(2)));

// Waves per workgroup (NW): 4, two workgroups per CU -- or 8, one workgroup per CU: the same two waves per
// SIMD, but a LUT slice is copied into LDS once for 512 tokens instead of 256 and the CU's whole LDS belongs
// to one workgroup (slices twice as deep, half as many barriers).
constexpr int sp_tok_item(int tm, int nw = 4) { return nw * tm * 16; }
// workgroups per CU: two of four waves or one of eight, two waves per SIMD either way.  (Eight waves of 32 tokens
// each, two such workgroups per CU -- four waves per SIMD on 128 registers -- were measured 17 % slower on 64-column
// tiles: a wave then re-reads every table entry for two token groups instead of four, and 96-column tiles spill.)
constexpr int sp_wgs_per_cu(int, int nw) { return nw == 4 ? 2 : 1; }
// 64-token index blocks a workgroup keeps per slice: a wave of 32 tokens shares its block with its neighbour (both
// copy the same bytes to the same place)
constexpr int sp_ix_blocks(int tm, int nw) { return nw * tm * 16 / 64; }
constexpr int sp_nbuf(int gs) { return gs > 16 ? 2 : 3; }
// value tables (17..32 centroids only: two tables of 32 entries of 16 bytes); then the position words, one per index byte
constexpr int sp_value_table_bytes(bool wide) { return wide ? 1024 : 0; }
constexpr int sp_table_bytes(bool wide) { return sp_value_table_bytes(wide) + 1024; }
constexpr int sp_lds_bytes(int tn, int gs, int nw = 4, bool wide = false)
{
    return sp_table_bytes(wide) + sp_nbuf(gs) * gs * 16 * tn * 16 + sp_nbuf(gs) * nw * 64 * 4 * (gs / 8);
}
// ks: waves that share a token block and split the codebooks of a slice between them (1 or 2)
constexpr int sp_lds_bytes_tm(int tn, int tm, int gs, int nw, bool wide, int ks = 1)
{
    return sp_table_bytes(wide) + sp_nbuf(gs) * gs * 16 * tn * 16 + sp_nbuf(gs) * sp_ix_blocks(tm, nw / ks) * 64 * 4 * (gs / 8);
}

template <int OFF>
__device__ __forceinline__ void lds_read64(v2i& dst, uint32_t addr)
{
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ void lds_read32(int& dst, uint32_t addr)
{
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
template <int N>
__device__ __forceinline__ void lgkm_wait()
{
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N < 15 ? N : 15) : "memory");
}

// a pointer that is the same in every lane, moved to scalar registers
template <class T>
__device__ __forceinline__ T* uniform_ptr(T* p)
{
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<T*>(((uint64_t)hi << 32) | lo);
}

// CB_pad: codebooks of 16 centroids in the tiled table (twice the operator's for WIDE)
// KS = 2 (eight waves): waves w and w + 4 hold the same 64 tokens and take one half of every slice's codebooks each;
// the halves are added through LDS before the epilogue.  An item is then 256 tokens: a launch too small to give
// every CU a 512-token item still fills the chip with TM = 4 tiles and copies a slice once per 256 tokens.
template <int TN, int TM, int GS, int NW, bool WIDE, int KS = 1>
__global__ __launch_bounds__(NW * 64, sp_wgs_per_cu(TM, NW) * NW / 4 /* waves per SIMD */) void gather_sparse_kernel(
    const uint8_t* __restrict__ idx, const int8_t* __restrict__ lut, float* __restrict__ out,
    int32_t* __restrict__ acc_out, uint32_t N, uint32_t M, uint32_t CB_pad, uint32_t idx_row_bytes,
    uint32_t n_token_tiles, uint32_t n_items, Epilogue ep, XcdMap xmap)
{
    constexpr int SP_WAVES = NW;
    constexpr int NWT = NW / KS;                   // waves with tokens of their own
    static_assert(KS == 1 || (KS == 2 && NW == 8), "the codebook split is between the two waves of a SIMD");
    constexpr int TOK_ITEM = sp_tok_item(TM, NWT);
    static_assert(TM == 4 || TM == 2, "a wave owns a whole or half a 64-token index block");
    constexpr int WN = 16 * TN;                    // columns per item
    constexpr int G = GS;                          // codebooks per slice
    constexpr int SLICE = G * WN * 16;             // bytes of one codebook slice
    constexpr int KSTEPS = G / 8 / KS;             // one instruction covers 8 codebooks (this wave's share of a slice)
    constexpr int IWORDS = G / 8 / KS;             // 32-bit index words per token and slice (8 nibbles each), this wave's
    constexpr int IWORDS_ALL = G / 8;
    constexpr int NBLK = SLICE / 1024;             // 1 KB blocks (one copy instruction of a wave) per slice
    constexpr int DMA_PER_WAVE = (NBLK + SP_WAVES - 1) / SP_WAVES;
    static_assert(KSTEPS >= 2, "the operand pipeline below re-arms inside a slice");

    // LDS: value table(s) | position words (1 KB) | NBUF LUT slice buffers | NIBUF index buffers
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    constexpr int NBUF = sp_nbuf(GS), NIBUF = NBUF;
    constexpr int PD = NBUF - 1;  // prefetch distance of the LUT stream, in slices
    constexpr uint32_t POS0 = sp_value_table_bytes(WIDE);  // position words
    constexpr uint32_t BUF0 = sp_table_bytes(WIDE);
    constexpr uint32_t IBUF0 = BUF0 + NBUF * SLICE;
    constexpr uint32_t IBYTES = sp_ix_blocks(TM, NWT) * 64 * 4 * IWORDS_ALL;   // index bytes of one slice (64-token blocks)
    constexpr uint32_t IWAVE = 64 * 4 * IWORDS_ALL;           // ... of one 64-token block
    // index words: one operation copies one word of 64 tokens (64 lanes x 4 B) or, where a slice has a multiple of
    // four words, four of them (64 lanes x 16 B: consecutive words of a 64-token block are consecutive 256-byte
    // pieces in the tiled index buffer and in LDS alike); fewer instructions, the same time (measured)
    constexpr bool IX_WIDE = IWORDS % 4 == 0;
    constexpr int IX_OPS = IX_WIDE ? IWORDS / 4 : IWORDS;
    constexpr int DMA_OPS = DMA_PER_WAVE + IX_OPS;            // memory operations per wave and slice
    // Up to 16 centroids: the value bytes of a nibble are 1 << 16 (c / 4) as a 64-bit number, made by one shift
    // instead of read from a table (one LDS read per token group and K-step instead of three; measured 1 - 7 %
    // of the kernel, most on narrow column tiles).
    constexpr bool VALU_VALUES = !WIDE;
    constexpr int A_OPS = VALU_VALUES ? 1 : 3;                // LDS reads per token group for the sparse operand

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t tw = KS == 1 ? wave : wave % NWT;  // which tokens of the item
    const uint32_t kh = KS == 1 ? 0u : wave / NWT;    // which part of a slice's codebooks
    const uint32_t j = lane & 15;  // token within a group (sparse operand) / column within a group (dense operand, result)
    const uint32_t g = lane >> 4;
    if (blockIdx.x >= n_items) return;  // whole workgroup
    const uint32_t nslices = CB_pad / G;
    const uint32_t my_items = (n_items - blockIdx.x + gridDim.x - 1) / gridDim.x;
    const uint32_t total = my_items * nslices;

    // Table entry c (16 bytes): value bytes of a codebook whose centroid is c (first slot of group c / 4 is 1).
    // Position table, word b: the position bits of both codebooks of index byte b (c % 4 at value slot 2 (c / 4),
    // two bits per slot; low nibble in the low half of the word, high nibble in the high half).
    // WIDE: table h (h = 0, 1; 512 bytes each) has entry c at byte b = 16 h + c and zero entries elsewhere.
    static_assert(NW * 64 >= 256, "one table word per thread");
    if (WIDE && threadIdx.x < 256) {
        const uint32_t b = (threadIdx.x >> 2) & 31, table = threadIdx.x >> 7;
        const uint32_t c = b & 15, w = threadIdx.x & 3, grp = c >> 2;
        uint32_t word;
        if (w < 2) word = (grp >> 1) == w ? (1u << (16 * (grp & 1))) : 0u;  // value bytes 0..3 / 4..7: slot 2 grp
        else word = 0;
        if (WIDE && (b >> 4) != table) word = 0;
        reinterpret_cast<uint32_t*>(smem)[threadIdx.x] = word;
    }
    if (threadIdx.x < 256) {
        const uint32_t b = threadIdx.x;
        auto pos_bits = [](uint32_t c) { return (c & 3u) << (4 * (c >> 2)); };
        // WIDE: the byte is one centroid of 32; its bits belong to the half its table is looked up for
        const uint32_t word = WIDE ? pos_bits(b & 15) << (16 * ((b >> 4) & 1)) : pos_bits(b & 15) | (pos_bits(b >> 4) << 16);
        reinterpret_cast<uint32_t*>(smem + POS0)[b] = word;
    }

    auto col_of = [&](uint32_t p) { uint32_t c, t; xmap.decode(p, n_token_tiles, c, t); return c; };
    auto tok_tile_of = [&](uint32_t p) { uint32_t c, t; xmap.decode(p, n_token_tiles, c, t); return t; };
    uint32_t lut_item = blockIdx.x, lut_s = 0, ix_item = blockIdx.x, ix_s = 0;
    const int8_t* dma_base;   // uniform: start of the slice at the LUT stream position
    const uint8_t* ix_base;   // uniform: the 256-byte block of index words at the index stream position
    uint32_t ix_lane_off;
    auto locate_lut = [&]() { dma_base = lut + (size_t)col_of(lut_item) * CB_pad * (WN * 16); };
    const uint32_t last_block = (N - 1) / 64;
    auto locate_ix = [&]() {
        uint32_t blk = (tok_tile_of(ix_item) * TOK_ITEM + tw * (TM * 16)) / 64;
        if (blk > last_block) blk = last_block;  // clamp: results of such tokens are never stored
        const uint32_t op = ep.op_col_tiles ? col_of(ix_item) / ep.op_col_tiles : 0u;
        ix_base = idx + (size_t)op * ep.op_idx_stride + (size_t)blk * idx_row_bytes * 64;
        ix_lane_off = lane * (IX_WIDE ? 16 : 4) + kh * (IWORDS * 256);  // this wave's words of the block
    };
    // A wave copies DMA_PER_WAVE consecutive 1 KB blocks of a slice.  All of a slice's operations share one
    // global address (the wave's part of the slice, per lane) and one LDS address; the block is chosen by the
    // instruction's immediate offset, which the hardware adds to both.  The offset field reaches 4 KB, so blocks
    // beyond the fourth go through a second address pair 4 KB further on.
    // fetch = false (past the end of the stream): the operations re-copy the first slice of the table into a
    // buffer nobody reads any more, so that every slice issues the same number of operations and the waits
    // can count them.
    static_assert(NBLK % SP_WAVES == 0 && DMA_PER_WAVE <= 8, "whole blocks per wave, two address pairs");
    const uint32_t dma_wave = wave * (DMA_PER_WAVE * 1024);
    const uint32_t dma_lane = dma_wave + lane * 16;
    const int8_t* lut_src = nullptr;  // this slice's source for this lane
    uint32_t lut_dst = 0;             // ... and the wave's destination in LDS
    // buf_off: byte offset of the destination buffer among the slice buffers
    auto lut_begin = [&](uint32_t buf_off, bool fetch) {
        // the choice is uniform: made once on the scalar side, not per lane
        const int8_t* base = uniform_ptr(fetch ? dma_base : lut);
        lut_src = base + dma_lane;
        lut_dst = BUF0 + buf_off + dma_wave;
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
        lut_begin(buf * SLICE, true);
        static_for<0, DMA_PER_WAVE>([&](auto uc) { lut_op(uc); });
        lut_advance();
    };
    // index words: the same scheme, 256 bytes (64 tokens x one word) per operation
    const uint8_t* ix_src = nullptr;
    uint32_t ix_dst = 0;
    auto ix_begin = [&](uint32_t ibuf_off, bool fetch) {
        const uint8_t* base = uniform_ptr(fetch ? ix_base : idx);  // idx itself: any 64 tokens' words, never read
        ix_src = base + ix_lane_off;
        ix_dst = IBUF0 + ibuf_off + (tw * (TM * 16) / 64) * IWAVE + kh * (IWORDS * 256);
    };
    auto ix_op = [&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if constexpr (IX_WIDE)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)ix_src,
                                             (__attribute__((address_space(3))) void*)(smem + ix_dst), 16, 1024 * i, 0);
        else
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)ix_src,
                                             (__attribute__((address_space(3))) void*)(smem + ix_dst), 4, 256 * i, 0);
    };
    auto ix_advance = [&]() {
        ix_base += IWORDS_ALL * 256;
        if (++ix_s == nslices) {
            ix_s = 0;
            ix_item += gridDim.x;
            if (ix_item < n_items) locate_ix();
        }
    };
    auto stage_ix = [&](uint32_t ibuf) {
        ix_begin(ibuf * IBYTES, true);
        static_for<0, IX_OPS>([&](auto ic) { ix_op(ic); });
        ix_advance();
    };
    // Index word k of a token holds the nibbles of codebooks 8k .. 8k+7 of the slice; this lane's two are byte g,
    // which it reads on its own (the four lane groups read the four bytes of the same word: one bank, broadcast).
    // Kept as the two table offsets, nibble * 16.
    const uint32_t ix_lane = IBUF0 + (tw * (TM * 16) / 64) * IWAVE + kh * (IWORDS * 256) + (((tw * (TM * 16)) & 63) + j) * 4 + g;
    auto read_ix = [&](uint32_t (&raw)[TM][IWORDS], uint32_t ibuf_off) {
        const uint32_t addr = ix_lane + ibuf_off;
        static_for<0, TM * IWORDS>([&](auto ec) {
            constexpr int t = decltype(ec)::value / IWORDS, i = decltype(ec)::value % IWORDS;
            lds_read_u8<(i * 64 + t * 16) * 4>(raw[t][i], addr);
        });
    };
    // the index bytes requested by read_ix have landed (the registers pass through the wait)
    auto wait_ix = [&](uint32_t (&raw)[TM][IWORDS]) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int t = 0; t < TM; ++t)
#pragma unroll
            for (int i = 0; i < IWORDS; ++i) asm volatile("" : "+v"(raw[t][i]));
    };

    v4i acc[TM][TN];
#pragma unroll
    for (int t = 0; t < TM; ++t)
#pragma unroll
        for (int c = 0; c < TN; ++c) acc[t][c] = (v4i){0, 0, 0, 0};

    // ---- epilogue ------------------------------------------------------------------------------------
    // Lane (g, j) holds acc[t][c][r] = sum for token 16 t + 4 g + r and the column that sparse_tile_column
    // assigns to position 16 c + j.  Pieces of W = 4, 2 or 1 groups give W consecutive columns per lane.
    constexpr int N4 = TN / 4 * 4, N2 = N4 + (TN % 4) / 2 * 2;
    constexpr int NPIECES = TN / 4 + (TN % 4) / 2 + TN % 2;
    constexpr int EPI_STORES = TM * 4 * NPIECES;  // stores of a wave in the epilogue of a full tile
    auto epilogue_as = [&](uint32_t item, auto actc) __attribute__((always_inline)) -> bool {
        constexpr bool ACT = decltype(actc)::value;
        uint32_t je = j, ge = g;
        asm volatile("" : "+v"(je), "+v"(ge));  // keeps the address arithmetic below out of the slice loop
        const uint32_t colblk = col_of(item);
        Epilogue epl = ep;
        if (ep.op_col_tiles) epl.scale = scalar_load1(ep.op_scales + colblk / ep.op_col_tiles);
        const uint32_t tile_tok0 = tok_tile_of(item) * TOK_ITEM;
        const uint32_t tok0 = tile_tok0 + tw * (TM * 16) + 4 * ge;
        const bool vec_ok = (M % 4 == 0);
        const bool full = vec_ok && !acc_out && tile_tok0 + TOK_ITEM <= N && (colblk + 1) * WN <= M;
        auto piece = [&](auto c0c, auto wc) __attribute__((always_inline)) {
            constexpr int c0 = decltype(c0c)::value, W = decltype(wc)::value;
            const uint32_t f = colblk * WN + 16 * c0 + W * je;  // first of this lane's W columns
            float bv[W];
#pragma unroll
            for (int e = 0; e < W; ++e) bv[e] = (ep.bias && f + e < M) ? ep.bias[f + e] : 0.0f;
#pragma unroll
            for (int t = 0; t < TM; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t tok = tok0 + t * 16 + r;
                    float o[W];
                    int32_t a[W];
#pragma unroll
                    for (int e = 0; e < W; ++e) {
                        a[e] = acc[t][c0 + e][r];
                        o[e] = dequant<ACT>(a[e], epl, bv[e]);
                    }
                    float* dst = out + (size_t)tok * M + f;
                    if (full) {  // workgroup-uniform: every token and column of the tile exists
                        if constexpr (W == 4) {
                            typedef float v4f __attribute__((ext_vector_type(4)));
                            // 96-column tiles (the widest outputs): plain stores, which the caches may hold for the
                            // operator that reads the output next; measured 0.7 us faster at 768 -> 3072, N = 8192
                            // (100 MB), while the 25 MB of 3072 -> 768 are 1.4 us faster with streaming stores
                            if constexpr (TN == 6) *reinterpret_cast<v4f*>(dst) = (v4f){o[0], o[1], o[2], o[3]};
                            else __builtin_nontemporal_store((v4f){o[0], o[1], o[2], o[3]}, reinterpret_cast<v4f*>(dst));
                        } else if constexpr (W == 2) {
                            typedef float v2f __attribute__((ext_vector_type(2)));
                            __builtin_nontemporal_store((v2f){o[0], o[1]}, reinterpret_cast<v2f*>(dst));
                        } else {
                            __builtin_nontemporal_store(o[0], dst);
                        }
                        continue;
                    }
                    if (tok >= N) continue;
#pragma unroll
                    for (int e = 0; e < W; ++e)
                        if (f + e < M) {
                            dst[e] = o[e];
                            if (acc_out) acc_out[(size_t)tok * M + f + e] = a[e];
                        }
                }
        };
        static_for<0, TN / 4>([&](auto pc) { piece(std::integral_constant<int, 4 * decltype(pc)::value>{}, std::integral_constant<int, 4>{}); });
        if constexpr (N2 > N4) piece(std::integral_constant<int, N4>{}, std::integral_constant<int, 2>{});
        if constexpr (TN > N2) piece(std::integral_constant<int, N2>{}, std::integral_constant<int, 1>{});
#pragma unroll
        for (int t = 0; t < TM; ++t)
#pragma unroll
            for (int c = 0; c < TN; ++c) acc[t][c] = (v4i){0, 0, 0, 0};
        return full;
    };
    auto epilogue = [&](uint32_t item) __attribute__((always_inline)) -> bool {
        return ep.act == PIMDL_ACT_GELU_TANH ? epilogue_as(item, std::true_type{}) : epilogue_as(item, std::false_type{});
    };

    // ---- prologue: slices 0 .. PD-1, index words 0 .. PD ------------------------------------------------
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
    __syncthreads();  // also: the table is complete
    uint32_t iw_raw[TM][IWORDS];
    read_ix(iw_raw, 0);
    wait_ix(iw_raw);

    uint32_t item0 = blockIdx.x;
    // this lane's 16 bytes of codebook g (of this wave's share of the slice), column position j
    const uint32_t b_lane = BUF0 + (g * WN + j) * 16 + kh * (KSTEPS * 8 * WN * 16);
    // byte offsets of the buffers in their rings: the slice being read and the one its copies go into (the
    // slice before), the index words read next and the ones copied into
    uint32_t cur_off = 0, copy_off = (NBUF - 1) * SLICE, ixn_off = IBYTES, ixc_off = 0;
    uint32_t k = 0;
    bool stores_behind = false;
    constexpr bool COUNT_STORES = (PD - 1) * DMA_OPS + EPI_STORES <= 63;  // memory counter range

    for (uint32_t it = 0; it < my_items; ++it, item0 += gridDim.x) {
    for (uint32_t s0 = 0; s0 < nslices; ++s0, ++k) {
        // at most the operations issued during the previous PD-1 slices are outstanding: this wave's share of
        // slice k (and of index words k+1) has landed; after the barrier everybody's has, and everybody is
        // done with slice k-1, whose buffer slice k+PD goes into
        if (k != 0) {
            if (COUNT_STORES && stores_behind) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(COUNT_STORES ? (PD - 1) * DMA_OPS + EPI_STORES : 0) : "memory");
            else asm volatile("s_waitcnt vmcnt(%0)" ::"n"((PD - 1) * DMA_OPS) : "memory");
            stores_behind = false;
            __syncthreads();
        }
        const bool fetch = k + PD < total;
        const bool fetch_ix = k + PD + 1 < total;
        const uint32_t bbase = cur_off + b_lane;
        lut_begin(copy_off, fetch);
        ix_begin(ixc_off, fetch_ix);

        // Operand registers: the dense operand of a column group is re-armed with the next K-step's bytes as
        // soon as its TM instructions have been issued; the sparse operand is double buffered.
        v4i b_lo[TN], b_hi[TN];
        v2i a_lo[2][TM], a_hi[2][TM];
        int pw[2][TM];  // the lane's position word
        auto issue_b = [&](auto ksc, auto cc) {
            constexpr int ks = decltype(ksc)::value, c = decltype(cc)::value;
            lds_read<((8 * ks) * WN + c * 16) * 16>(b_lo[c], bbase);
            lds_read<((8 * ks + 4) * WN + c * 16) * 16>(b_hi[c], bbase);
        };
        // The sparse operand of K-step ks from the index bytes: what a byte turns into is worked out here, between the
        // matrix instructions of the K-step before (a few vector operations per token group in their shadow), not for
        // the whole slice at its boundary, where a wave would spend them alone.
        auto issue_a = [&](auto ksc) {
            constexpr int ks = decltype(ksc)::value;
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                const uint32_t raw = iw_raw[t][ks];
                const uint32_t pa = raw << 2;  // its position word
                if constexpr (VALU_VALUES) {
                    // the shift that makes the value bytes: 16 bits per group of four centroids
                    const uint64_t v0 = 1ull << (pa & 0x30u), v1 = 1ull << ((raw >> 2) & 0x30u);
                    a_lo[ks & 1][t] = (v2i){(int)(uint32_t)v0, (int)(uint32_t)(v0 >> 32)};
                    a_hi[ks & 1][t] = (v2i){(int)(uint32_t)v1, (int)(uint32_t)(v1 >> 32)};
                } else {
                    // (17..32 centroids) the byte is one codebook's centroid: its entry in the first and in the second table
                    const uint32_t e0 = raw << 4;
                    lds_read64<0>(a_lo[ks & 1][t], e0);
                    lds_read64<512>(a_hi[ks & 1][t], e0);
                }
                lds_read32<POS0>(pw[ks & 1][t], pa);
            }
        };
        // slice prologue: sparse operand first, then the dense operand of every column group, in this order
        issue_a(std::integral_constant<int, 0>{});
        static_for<0, TN>([&](auto cc) { issue_b(std::integral_constant<int, 0>{}, cc); });

        static_for<0, KSTEPS>([&](auto ksc) {
            constexpr int ks = decltype(ksc)::value;
            constexpr bool LAST = ks + 1 == KSTEPS;
            constexpr int RI = TM * IWORDS;  // index-word reads issued after column group 0 of the last K-step
            static_for<0, TN>([&](auto cc) {
                constexpr int c = decltype(cc)::value;
                // LDS operations complete in order; the count is the number of operations issued after the
                // ones this column group needs (see the issue order above and below)
                if constexpr (c == 0) lgkm_wait<2 * (TN - 1)>();
                else if constexpr (LAST) lgkm_wait<2 * (TN - 1 - c) + RI>();
                else lgkm_wait<2 * TN + A_OPS * TM - 2>();
                if constexpr (c == 0) {
#pragma unroll
                    for (int t = 0; t < TM; ++t)
                        asm volatile("" : "+v"(a_lo[ks & 1][t]), "+v"(a_hi[ks & 1][t]), "+v"(pw[ks & 1][t]));
                }
                asm volatile("" : "+v"(b_lo[c]), "+v"(b_hi[c]));
                __builtin_amdgcn_sched_barrier(0);
                const v8i bb = {b_lo[c][0], b_lo[c][1], b_lo[c][2], b_lo[c][3], b_hi[c][0], b_hi[c][1], b_hi[c][2], b_hi[c][3]};
#pragma unroll
                for (int t = 0; t < TM; ++t) {
                    const v4i aa = {a_lo[ks & 1][t][0], a_lo[ks & 1][t][1], a_hi[ks & 1][t][0], a_hi[ks & 1][t][1]};
                    acc[t][c] = __builtin_amdgcn_smfmac_i32_16x16x128_i8(aa, bb, acc[t][c], pw[ks & 1][t], 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (!LAST) {
                    issue_b(std::integral_constant<int, ks + 1>{}, cc);
                    if constexpr (c == 0) issue_a(std::integral_constant<int, ks + 1>{});
                } else if constexpr (c == 0) {
                    read_ix(iw_raw, ixn_off);  // the next slice's index words (this wave's own copy, landed)
                }
                // this slice's copy operations (slice k+PD of the table, index words k+PD+1), a few per column group
                constexpr int IK = PD == 1 ? KSTEPS * TN / 2 : KSTEPS * TN;
                constexpr int pos = ks * TN + c;
                static_for<(pos < IK ? pos : IK) * DMA_OPS / IK, (pos + 1 < IK ? pos + 1 : IK) * DMA_OPS / IK>([&](auto oc) {
                    constexpr int o = decltype(oc)::value;
                    if constexpr (o < DMA_PER_WAVE) lut_op(std::integral_constant<int, o>{});
                    else ix_op(std::integral_constant<int, o - DMA_PER_WAVE>{});
                });
                __builtin_amdgcn_sched_barrier(0);
            });
        });
        if (fetch) {
            lut_advance();
            if (fetch_ix) ix_advance();
        }
        wait_ix(iw_raw);

        copy_off = cur_off;
        cur_off = cur_off + SLICE == NBUF * SLICE ? 0 : cur_off + SLICE;
        ixc_off = ixn_off;
        ixn_off = ixn_off + IBYTES == NIBUF * IBYTES ? 0 : ixn_off + IBYTES;
    }
    if constexpr (KS == 2) {
        // the two halves of every sum meet in the slice buffer read last (nothing is copied into it before the next
        // slice's barrier): waves 4..7 put their accumulators there, waves 0..3 add them to their own
        static_assert(NWT * 64 * TM * TN * 16 <= SLICE, "the accumulators of half the waves fit a slice buffer");
        v4i* cbuf = reinterpret_cast<v4i*>(smem + BUF0 + copy_off) + tw * (TM * TN * 64) + lane;
        __syncthreads();  // every wave is done reading that buffer
        if (kh == 1) {
#pragma unroll
            for (int t = 0; t < TM; ++t)
#pragma unroll
                for (int c = 0; c < TN; ++c) {
                    cbuf[(t * TN + c) * 64] = acc[t][c];
                    acc[t][c] = (v4i){0, 0, 0, 0};
                }
        }
        __syncthreads();
        if (kh == 0) {
#pragma unroll
            for (int t = 0; t < TM; ++t)
#pragma unroll
                for (int c = 0; c < TN; ++c) acc[t][c] += cbuf[(t * TN + c) * 64];
            stores_behind = epilogue(item0);
        }
    } else {
        stores_behind = epilogue(item0);
    }
    }
}

template <int TN, int TM, int GS, int NW = 4, bool WIDE = false, int KS = 1>
int launch_sparse_tm(Ctx* ctx, const Amm& a, const uint8_t* d_idx, float* d_out, int32_t* d_acc, uint32_t n,
                     const Epilogue& ep)
{
    constexpr int LDS = sp_lds_bytes_tm(TN, TM, GS, NW, WIDE, KS);
    static_assert(sp_wgs_per_cu(TM, NW) * LDS <= 160 * 1024, "the CU's LDS holds the workgroups that its registers hold");
    constexpr int TOK_ITEM = sp_tok_item(TM, NW / KS);
    auto kern = gather_sparse_kernel<TN, TM, GS, NW, WIDE, KS>;
    const uint32_t cb16 = sparse_codebooks(a.g);  // codebooks of 16 centroids in the tiled table
    if (int rc = allow_dynamic_lds(ctx, reinterpret_cast<const void*>(kern), LDS, "hipFuncSetAttribute(gather_sparse)")) return rc;
    const uint32_t n_token_tiles = (n + TOK_ITEM - 1) / TOK_ITEM;
    const uint32_t n_items = n_token_tiles * (a.g.M_pad / (16 * TN));
    uint32_t grid = ctx->prop.multiProcessorCount * sp_wgs_per_cu(TM, NW);
    if (grid > n_items) grid = n_items;
    const XcdMap xmap = choose_xcd_map(a.g.M_pad / (16 * TN), n_token_tiles, grid, (uint64_t)cb16 * 16 * a.g.M_pad,
                                       (uint64_t)n * a.g.idx_row_bytes, a.g.tune_xcd_col_split);
    if (KS == 1) snprintf(a.last_gather, sizeof(a.last_gather), "gather_sparse_kernel<%d, %d, %d, %d, %s>", TN, TM, GS, NW, WIDE ? "true" : "false");
    else snprintf(a.last_gather, sizeof(a.last_gather), "gather_sparse_kernel<%d, %d, %d, %d, %s, %d>", TN, TM, GS, NW, WIDE ? "true" : "false", KS);
    a.note_launch(GS, LDS, TOK_ITEM, NW * 64);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NW * 64), LDS, ctx->stream, d_idx, reinterpret_cast<const int8_t*>(a.d_lut),
                       d_out, d_acc, n, a.g.M, cb16, a.g.idx_row_bytes, n_token_tiles, n_items, ep, xmap);
    return hip_check(ctx, hipGetLastError(), "gather_sparse_kernel launch");
}

// 256- or 128-token items, whichever gives the shorter launch (the rule of the dense kernel)
template <int TN, bool WIDE>
int launch_sparse_tn(Ctx* ctx, const Amm& a, const uint8_t* d_idx, float* d_out, int32_t* d_acc, uint32_t n, const Epilogue& ep)
{
    const uint32_t cb16 = sparse_codebooks(a.g);
    const uint64_t col_tiles = a.g.M_pad / (16 * TN);
    const uint64_t items4 = (uint64_t)((n + sp_tok_item(4) - 1) / sp_tok_item(4)) * col_tiles;
    const uint64_t items2 = (uint64_t)((n + sp_tok_item(2) - 1) / sp_tok_item(2)) * col_tiles;
    const uint64_t slots = 2ull * ctx->prop.multiProcessorCount;
    bool small_items = prefer_small_items(items4, items2, slots);
    if (a.g.tune_token_item) small_items = a.g.tune_token_item == 128;
    // 48-column tiles read the sparse operand of a token group for three column groups only, so the copies and
    // the per-slice costs weigh most there: with eight waves per workgroup a slice is copied once per 512 tokens
    // and can be 64 codebooks deep (measured 44.1 -> 42.4 us at 3072 -> 768, N = 8192; the 96-column kernel
    // loses 3 us the same way, its two waves of a SIMD then waiting at the same barrier).  Taken where it gives the
    // shorter launch: a round of 512-token items takes 0.96 of a round of twice as many 256-token items, but a partly
    // filled last round costs a whole one (its workgroups are alone on their CUs either way), where four-wave
    // workgroups speed up (grid_rounds): the fused Q/K/V gather at N = 4096 (1.5 rounds) takes 21.7 us with four
    // waves and 27.4 us with eight.
    if constexpr (TN == 3 && !WIDE) {
        const uint64_t cus = ctx->prop.multiProcessorCount;
        const uint64_t items8 = (uint64_t)((n + sp_tok_item(4, 8) - 1) / sp_tok_item(4, 8)) * col_tiles;
        if (!a.g.tune_token_item && !a.g.tune_cb_per_slice && cb16 % 64 == 0 && !small_items && items8 >= cus &&
            0.96 * (double)((items8 + cus - 1) / cus) < grid_rounds(items4, slots))
            return launch_sparse_tm<TN, 4, 64, 8>(ctx, a, d_idx, d_out, d_acc, n, ep);
        // A launch of long sums that offers about one 256-token item per CU: 128-token items would fill the chip's
        // workgroup slots but copy every slice twice as often and re-read every table entry for two token groups
        // instead of four; with the codebooks of a slice split between the two waves of a SIMD the 256-token item
        // keeps both (3072 -> 768: N = 4096 26.3 -> 23.1 us, N = 3072 24.6 -> 22.6; half a round of such items
        // (N = 2048) or more than one (N = 6144), and sums of 192 codebooks, are not faster that way).
        if ((a.g.tune_token_item == 256 && a.g.tune_cb_per_slice == 64 && cb16 % 64 == 0) ||
            (!a.g.tune_token_item && !a.g.tune_cb_per_slice && cb16 % 64 == 0 && cb16 >= 384 && items4 <= cus &&
             10 * items4 >= 7 * cus))
            return launch_sparse_tm<TN, 4, 64, 8, false, 2>(ctx, a, d_idx, d_out, d_acc, n, ep);
    }
    if constexpr (!WIDE) if (a.g.tune_token_item == 512) {  // one workgroup of eight waves per CU
        if constexpr (TN == 3) {
            if (cb16 % 64 == 0 && a.g.tune_cb_per_slice == 64) return launch_sparse_tm<TN, 4, 64, 8>(ctx, a, d_idx, d_out, d_acc, n, ep);
        }
        // (CB_pad is a multiple of 32; 48-column tiles have no 16-codebook variant here: 12 blocks for 8 waves)
        if (TN == 3 || a.g.tune_cb_per_slice != 16) return launch_sparse_tm<TN, 4, 32, 8>(ctx, a, d_idx, d_out, d_acc, n, ep);
        if constexpr (TN != 3) return launch_sparse_tm<TN, 4, 16, 8>(ctx, a, d_idx, d_out, d_acc, n, ep);
    }
    constexpr int GSB = TN <= 4 ? 32 : 16;  // 32-codebook slices in two buffers where two workgroups still fit a CU
    if constexpr (GSB != 16) {
        if (cb16 % GSB == 0 && a.g.tune_cb_per_slice != 16) {
            if (small_items) return launch_sparse_tm<TN, 2, GSB, 4, WIDE>(ctx, a, d_idx, d_out, d_acc, n, ep);
            return launch_sparse_tm<TN, 4, GSB, 4, WIDE>(ctx, a, d_idx, d_out, d_acc, n, ep);
        }
    }
    if (small_items) return launch_sparse_tm<TN, 2, 16, 4, WIDE>(ctx, a, d_idx, d_out, d_acc, n, ep);
    return launch_sparse_tm<TN, 4, 16, 4, WIDE>(ctx, a, d_idx, d_out, d_acc, n, ep);
}

}  // namespace

uint32_t sparse_lds_bytes(uint32_t tn, bool wide) { return (uint32_t)sp_lds_bytes((int)tn, 16, 4, wide); }

int launch_gather_sparse(Ctx* ctx, const Amm& a, const uint8_t* d_idx, float* d_out, int32_t* d_acc, uint32_t n,
                         float scale, float lut_bias_term)
{
    Epilogue ep;
    ep.scale = scale;
    ep.lut_bias_term = lut_bias_term;
    ep.bias = a.d_bias;
    ep.act = a.desc.activation;
    ep.op_scales = a.d_op_scales;
    ep.op_col_tiles = a.op_col_tiles;
    ep.op_idx_stride = a.op_idx_stride;
    if (a.g.C_tile == 32) {
        switch (a.g.q) {
            case 3: return launch_sparse_tn<3, true>(ctx, a, d_idx, d_out, d_acc, n, ep);
            case 4: return launch_sparse_tn<4, true>(ctx, a, d_idx, d_out, d_acc, n, ep);
            case 6: return launch_sparse_tn<6, true>(ctx, a, d_idx, d_out, d_acc, n, ep);
        }
    } else {
        switch (a.g.q) {
            case 3: return launch_sparse_tn<3, false>(ctx, a, d_idx, d_out, d_acc, n, ep);
            case 4: return launch_sparse_tn<4, false>(ctx, a, d_idx, d_out, d_acc, n, ep);
            case 6: return launch_sparse_tn<6, false>(ctx, a, d_idx, d_out, d_acc, n, ep);
        }
    }
    return set_error(ctx, PIMDL_ERR_UNSUPPORTED, "no sparse gather kernel for %u column groups", a.g.q);
}

}  // namespace pimdl
