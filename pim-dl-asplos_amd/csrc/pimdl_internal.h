// Internal declarations shared by the HIP translation units of libpimdl (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>
#include <vector>

#include "pimdl.h"

namespace pimdl {

// ---------------------------------------------------------------------------------------------
// Geometry of one AMM operator as the kernels see it.
//
// Index rows   [N][idx_row_bytes] bytes; IDX_BITS = 4 (C <= 16, codebook 2k in the low nibble
//              of byte k) or 8.  Codebooks are padded to a multiple of 32 with index 0.
//              idx_tiled (operators served by the one-hot gather): the same bytes stored as
//              [N/64][idx_row_bytes/4][64 tokens][4 bytes], so that the 32-bit index words one
//              wave needs for one codebook slice (64 tokens x 1 word) are 256 contiguous bytes;
//              the buffer covers N rounded up to 64 tokens.
// int8 LUT     gather_kind 0: tiled [M_pad / col_block][CB_pad][C_tile][col_block] bytes
//              (col_block = 16*Q); gather_kind 1: [M_pad / col_block][CB_pad][col_block][16] bytes
//              (the 16 centroid entries of a column are contiguous).  Either way one (column block,
//              codebook range) slice is contiguous, so staging it into LDS is a flat copy.  Padded
//              codebooks / centroid rows / columns hold zeros.
// fp32 LUT     tiled the same way with col_block floats per row.
// ---------------------------------------------------------------------------------------------
struct AmmGeom {
    uint32_t K, v, CB, CB_pad, C, C_tile, M, M_pad;
    uint32_t idx_bits, idx_row_bytes;
    uint32_t idx_tiled;     // layout of the packed index buffer, see above
    uint32_t lut_chunked;   // fp32 table of 32 centroids: [column block][codebook][8-byte chunk][row][2 floats]
    // gather kernel
    uint32_t gather_kind;   // 0: byte-adder rows kernel, 1: one-hot matrix-core kernel (int8, C <= 16),
                            // 2: one-hot on the sparse matrix instruction (int8, C <= 32: a codebook of 17..32
                            //    centroids is two of 16 side by side; table laid out as for 1, with the columns
                            //    of a tile permuted by sparse_tile_column)
    uint32_t q;             // 16-byte chunks per LUT row in LDS
    uint32_t col_block;     // columns per workgroup (int8: 16*q, fp32: 4*q)
    uint32_t row_pitch;     // bytes between LUT rows in LDS (16*q + 16: bank-conflict-free b128 gathers)
    uint32_t gq;            // int8: codebooks per lane group per slice; slice = 4*gq codebooks
    uint32_t cb_per_slice;
    uint32_t gather_threads, tokens_per_wg, gather_lds_bytes;
    // ccs kernel
    uint32_t ccs_row_floats, ccs_cb_per_wg, ccs_lds_bytes;
    // choices a caller has taken over from the library (pimdl_amm_tuning; 0 = the library decides)
    uint32_t tune_search, tune_search_tile, tune_token_item, tune_cb_per_slice, tune_xcd_col_split;
};

// fp32 tables whose rows are read in 8-byte chunks (see gather_f32_kernel)
constexpr bool f32_lut_chunked(int c_tile, int q) { return c_tile == 32 && q == 4; }

// bytes of a packed index buffer for n tokens
inline size_t idx_buffer_bytes(const AmmGeom& g, uint32_t n)
{
    return (size_t)(g.idx_tiled ? (n + 63) / 64 * 64 : n) * g.idx_row_bytes;
}

#ifdef __HIPCC__
// byte offset of byte `byte` of token `tok`'s index row (aligned groups of 4 bytes stay contiguous)
__device__ __forceinline__ size_t idx_offset(uint32_t tok, uint32_t byte, uint32_t row_bytes, int tiled)
{
    return tiled ? ((size_t)(tok >> 6) * (row_bytes >> 2) + (byte >> 2)) * 256 + ((tok & 63) << 2) + (byte & 3)
                 : (size_t)tok * row_bytes + byte;
}
#endif

struct Ctx;

struct Amm {
    Ctx* ctx;
    pimdl_amm_desc desc;
    AmmGeom g;
    float* d_centroids;  // [CB][C][v], then the derived search data (ccs_centroid_bytes)
    void* d_lut;         // tiled
    size_t lut_bytes;
    float* d_scales;     // int8: scales
    uint32_t nscales;
    float* d_bias;       // [M]
    std::vector<float> h_bias;  // what d_bias holds (pimdl_amm_set_bias skips the copy when nothing changed)
    float h_scale0;
    bool grouped;        // int8 LUT with scale_group > 0: resident as fp32 integers, fp32 gather kernel
    bool prescaled;      // ... with scale_group == 1: resident already multiplied by its codebook's scale (the one
                         // rounding the grouped kernel would apply per entry), gathered like an fp32 table: same bits
    // several one-hot operators laid side by side along the columns (see Epilogue in gather_kernel.hip)
    float* d_op_scales;
    uint32_t op_col_tiles, op_idx_stride;
    // name (with template arguments) of the gather kernel the operator's last launch used: what a profile lists
    mutable char last_gather[80];
    // shape of that launch (0 before the first one): codebooks per slice, LDS bytes, tokens and threads per workgroup
    mutable uint32_t last_cb_per_slice = 0, last_lds_bytes = 0, last_tokens_per_wg = 0, last_threads = 0;
    void note_launch(uint32_t cb_per_slice, uint32_t lds_bytes, uint32_t tokens_per_wg, uint32_t threads) const
    {
        last_cb_per_slice = cb_per_slice;
        last_lds_bytes = lds_bytes;
        last_tokens_per_wg = tokens_per_wg;
        last_threads = threads;
    }
};

// Pinned staging ring of the host-buffer path (pimdl_capi.hip): SLOTS chunks of tokens in flight, each with a
// pinned and a device buffer per direction, so that the caller's copy into pinned memory, the transfer to the
// device, the two kernels, the transfer back and the copy out of pinned memory of different chunks overlap.
struct HostPipe {
    static constexpr int SLOTS = 4;
    hipStream_t s_in = nullptr, s_out = nullptr;       // transfers; the kernels run on the context's stream
    hipEvent_t ev_in[SLOTS] = {}, ev_run[SLOTS] = {}, ev_out[SLOTS] = {};
    bool used_in[SLOTS] = {}, used_run[SLOTS] = {}, used_out[SLOTS] = {};  // the event has been recorded at least once
    void* pin_in[SLOTS] = {};
    void* pin_out[SLOTS] = {};
    float* d_in[SLOTS] = {};
    float* d_out[SLOTS] = {};
    size_t in_bytes = 0, out_bytes = 0;                // per slot
};

struct Ctx {
    int device;
    hipStream_t own_stream;
    hipStream_t stream;
    hipDeviceProp_t prop;
    std::string err;
    // Grow-only device scratch.  A buffer that has to grow is replaced, and the old one is kept until the
    // context is destroyed (`retired`): a HIP graph captured from earlier calls holds its address.
    std::vector<void*> retired;
    uint8_t* d_static_scratch;  // this device's copy of the allocation-free entry point's file-scope array
    float* d_in;
    size_t in_bytes;
    float* d_out;
    size_t out_bytes;
    uint8_t* d_idx;
    size_t idx_bytes;
    int32_t* d_acc;
    size_t acc_bytes;
    uint16_t* d_idx16;
    size_t idx16_bytes;
    float* d_tmp;        // row-major output before re-tiling
    size_t tmp_bytes;
    float* d_cent;       // centroids of a context-level pimdl_index_calculation call
    size_t cent_bytes;
    hipEvent_t ev[4];
    HostPipe* pipe;      // created by the first call that hands over a host buffer
};

int set_error(Ctx* ctx, int code, const char* fmt, ...);
int hip_check(Ctx* ctx, hipError_t e, const char* what);
// Raises a kernel's dynamic LDS limit to `lds_bytes`, once per (device of ctx, kernel); safe from several threads.
int allow_dynamic_lds(Ctx* ctx, const void* kernel, int lds_bytes, const char* what);

// kernels (launchers validate nothing: callers have already checked shapes against AmmGeom)
// x_cols != 0: the geometry's codebooks are those of several operators that all read rows of x_cols
// floats (g.K = operators * x_cols); only where ccs_supports_shared_input() says so.
int launch_ccs(Ctx* ctx, const AmmGeom& g, const float* d_x, const float* d_cent, uint8_t* d_idx,
               uint32_t n, uint32_t x_cols = 0);
bool ccs_supports_shared_input(const AmmGeom& g, uint32_t x_cols);
// A centroid buffer holds the raw [CB][C][v] floats followed by data derived from them for the
// search kernel; allocate ccs_centroid_bytes() and run launch_ccs_prep() after every upload.
size_t ccs_centroid_bytes(const AmmGeom& g);
int launch_ccs_prep(Ctx* ctx, const AmmGeom& g, float* d_cent);
bool ccs_exact_only();
int launch_gather(Ctx* ctx, const Amm& a, const uint8_t* d_idx, float* d_out, int32_t* d_acc_or_null,
                  uint32_t n);
int launch_unpack_idx(Ctx* ctx, const AmmGeom& g, const uint8_t* d_idx, uint16_t* d_idx16, uint32_t n,
                      uint32_t n_stile, uint32_t cb_mtile);
int launch_pack_idx(Ctx* ctx, const AmmGeom& g, const uint16_t* d_idx16, uint8_t* d_idx, uint32_t n,
                    uint32_t n_stile, uint32_t cb_mtile);
int launch_retile_output(Ctx* ctx, const float* d_rowmajor, float* d_tiled, uint32_t n, uint32_t M,
                         uint32_t n_stile, uint32_t f_stile, uint32_t f_mtile);
int launch_lutgen_f32(Ctx* ctx, const float* d_cent, const float* d_w, float* d_lut, uint32_t CB,
                      uint32_t C, uint32_t v, uint32_t M, bool ordered = false);
int launch_lut_quant(Ctx* ctx, const float* d_lut, int8_t* d_q, float* d_scales, uint32_t CB, uint32_t C,
                     uint32_t M, uint32_t scale_group);
int launch_layer_norm(Ctx* ctx, const float* d_x, const float* d_w, const float* d_b, const float* d_residual,
                      float* d_out, uint32_t n, uint32_t d, float eps);
int launch_attention_hd64(Ctx* ctx, const float* d_q, const float* d_k, const float* d_v, float* d_out, uint32_t batch,
                          uint32_t seq, uint32_t heads, uint32_t in_stride, uint32_t out_stride, float scale);
int launch_diag(Ctx* ctx, uint64_t bytes, float* copy_gbps, float* lds_gbps);
int launch_diag_mfma_error(Ctx* ctx, uint32_t trials, bool crafted, float* max_err_u);

// the sparse one-hot gather (gather_sp_kernel.hip)
int launch_gather_sparse(Ctx* ctx, const Amm& a, const uint8_t* d_idx, float* d_out, int32_t* d_acc_or_null,
                         uint32_t n, float scale, float lut_bias_term);
uint32_t sparse_tile_column(uint32_t tn, uint32_t s);  // column of a tile stored at position s of the tile
uint32_t sparse_lds_bytes(uint32_t tn, bool wide);
// codebooks of 16 centroids in the table of the sparse one-hot gather: a codebook of 17..32 centroids is two
inline uint32_t sparse_codebooks(const AmmGeom& g) { return g.C_tile == 32 ? 2 * g.CB_pad : g.CB_pad; }
bool gather_dense_only();

uint32_t ccs_cb_per_wg(uint32_t v);  // codebooks one ccs workgroup covers (0: generic kernel)
bool gather_rows_only();
// tuning: choices taken over by the caller (nullptr: none); an error if the shape has no kernel for one
bool plan_geometry(const pimdl_amm_desc& d, uint32_t num_cus, AmmGeom* g, std::string* why,
                   const pimdl_amm_tuning* tuning = nullptr);
// checks the run-time fields of a tuning against a planned geometry and stores them in it
bool apply_runtime_tuning(AmmGeom* g, const pimdl_amm_tuning& t, std::string* why);

}  // namespace pimdl
