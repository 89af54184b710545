/*
 * pimdl.h -- C ABI of the MI355X (gfx950) LUT-AMM engine.
 *
 * One data-parallel path: closest-centroid search over activation sub-vectors, gather of
 * pre-computed centroid x weight LUT rows by those indices, sum across codebooks, de-quantise.
 * Plain pointers and sizes only; no C++ or torch types cross this boundary.  Every entry point
 * returns PIMDL_OK (0) or a negative pimdl_status; pimdl_last_error() gives the text.
 *
 * Each entry point names the interface of the reference (PIM-DL, paths under its
 * inference-engine/ or model-calibration/ trees) that it replaces.
 *
 * Conventions
 *   N tokens, K = input_feature_len, v = sub_vec_len, CB = K / v codebooks, C = num_centroid,
 *   M = output_feature_len.
 *   centroids  fp32 [CB][C][v]                     (src/host/index_calc_host.cpp:23)
 *   LUT        int8 or fp32 [CB][C][M], canonical  (test/test_amm.cpp:173; the .npz
 *                                                   "<op>.lut.tensor" written by
 *                                                   pim_weight_converter.py:89-94)
 *   input      fp32 [N][K] row-major, output fp32 [N][M] row-major.
 *   "dev" pointers are HIP device pointers; "host" pointers are ordinary host memory.
 *   pimdl_amm_run() accepts either kind for input and output and finds out which by itself.
 */
#ifndef PIMDL_H
#define PIMDL_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(PIMDL_BUILD)
#define PIMDL_API __attribute__((visibility("default")))
#else
#define PIMDL_API
#endif

typedef enum pimdl_status {
    PIMDL_OK = 0,
    PIMDL_ERR_INVALID = -1,     /* null pointer, zero size, K % v != 0, n > max_n ... */
    PIMDL_ERR_UNSUPPORTED = -2, /* shape outside what the kernels are built for */
    PIMDL_ERR_HIP = -3,         /* a HIP runtime call failed (text has hipGetErrorString) */
    PIMDL_ERR_NOMEM = -4,
    PIMDL_ERR_NO_DEVICE = -5    /* no gfx950 device visible: there is no CPU fallback */
} pimdl_status;

typedef enum pimdl_lut_dtype { PIMDL_LUT_I8 = 0, PIMDL_LUT_F32 = 1 } pimdl_lut_dtype;

/* How the epilogue adds the scalar LUT bias (both exist in the reference and differ unless
 * the bias is 0, which is all its converter ever writes):
 *   PIMDL_BIAS_ONCE       out = acc*scale + lut_bias      + bias[f]   test/test_amm.cpp:181
 *   PIMDL_BIAS_TIMES_CB   out = acc*scale + lut_bias*CB   + bias[f]   src/host/pim_lut_host.cpp:201 */
typedef enum pimdl_bias_mode { PIMDL_BIAS_ONCE = 0, PIMDL_BIAS_TIMES_CB = 1 } pimdl_bias_mode;

/* Function applied to every output element by the gather kernel's epilogue, after the bias.
 *   PIMDL_ACT_NONE        out = y                                   amm_host as in the reference
 *   PIMDL_ACT_GELU_TANH   out = 0.5 y (1 + tanh(sqrt(2/pi) (y + 0.044715 y^3)))
 * The reference's layer applies GELU to the first feed-forward AMM's output in a pass of its own
 * (ggml_gelu_inplace, src/host/transformer_layer.cpp:499-556); folding it into the epilogue saves
 * one read and one write of the [N][ffn_hidden_dim] tensor.  fp32, within 1e-6 relative of the
 * formula (evaluated as y / (1 + exp(-2u)), which does not cancel for negative y). */
typedef enum pimdl_activation { PIMDL_ACT_NONE = 0, PIMDL_ACT_GELU_TANH = 1 } pimdl_activation;

typedef struct pimdl_ctx pimdl_ctx; /* one device + one stream + scratch */
typedef struct pimdl_amm pimdl_amm; /* one linear layer's centroids + LUT + bias, resident in HBM */

/* Shape and numeric mode of one AMM operator.  Mirrors the shape fields of IndexCalcParams and
 * LUTParams (src/host/defines.h:12-50); the DPU tiling fields have no meaning on a GPU. */
typedef struct pimdl_amm_desc {
    uint32_t max_n;             /* largest N a run may pass */
    uint32_t input_feature_len; /* K */
    uint32_t sub_vec_len;       /* v */
    uint32_t num_centroid;      /* C, 2..256 */
    uint32_t output_feature_len;/* M */
    uint32_t lut_dtype;         /* pimdl_lut_dtype */
    uint32_t scale_group;       /* int8 only. 0: one scale for the tensor (the reference,
                                   LUTParams.scale).  g > 0 (extension, no counterpart in the
                                   reference): one scale per g consecutive codebooks; the sum
                                   inside a group is exact, then out = (sum over groups
                                   ascending, fp32, from 0) (float)acc_g * scale[g] + bias[f].
                                   Needs lut_bias == 0; runs on the fp32-table gather kernel
                                   (the table is resident as fp32 integers, 4 bytes/entry). */
    uint32_t bias_mode;         /* pimdl_bias_mode */
    float lut_bias;             /* LUTParams.bias */
    uint32_t activation;        /* pimdl_activation */
} pimdl_amm_desc;

typedef struct pimdl_amm_group pimdl_amm_group; /* operators that read the same input rows */

/* Timing of the last profiled run, milliseconds on the device (HIP events on the context's
 * stream, averaged over `iters` launches of each kernel on its own). */
typedef struct pimdl_amm_timing {
    float ccs_ms;    /* closest-centroid search kernel */
    float gather_ms; /* LUT gather-accumulate (+ epilogue) kernel */
    float total_ms;  /* both, back to back, as pimdl_amm_run issues them */
} pimdl_amm_timing;

/* ---- context ---------------------------------------------------------------------------
 * Replaces allocate_dpu / allocate_rank / load_binary / free_dpu_set
 * (src/host/dpu_common.h:11-54): the opaque device handle every call takes. */
PIMDL_API int pimdl_init(int device, pimdl_ctx** out);
PIMDL_API int pimdl_destroy(pimdl_ctx* ctx);
/* Text of the last error on this context (or of the last failed pimdl_init when ctx is NULL). */
PIMDL_API const char* pimdl_last_error(const pimdl_ctx* ctx);
/* Run this context's kernels on a caller-owned hipStream_t (NULL: back to the context's own).
 * Lets a caller that already has a stream (e.g. torch's current stream) order and time work. */
PIMDL_API int pimdl_set_stream(pimdl_ctx* ctx, void* hip_stream);
PIMDL_API int pimdl_synchronize(pimdl_ctx* ctx);

/* ---- operator: upload once, run many times ---------------------------------------------
 * Replaces prepare_lut_table (src/host/pim_lut_host.cpp:26-37), which re-sends the LUT to the
 * DPUs on every call, and the per-op load_binary before each amm_host in
 * src/host/transformer_layer.cpp:300,430,499,555.  All pointers are HOST pointers; the data is
 * copied (the LUT is re-tiled into column blocks for LDS staging) and may be freed on return.
 *   centroids  fp32 [CB][C][v]
 *   lut        int8 or fp32 [CB][C][M], canonical layout
 *   scales     int8: 1 float (scale_group 0) or ceil(CB/scale_group) floats; fp32 LUT: NULL
 *   bias       fp32 [M] or NULL (treated as zeros)                                        */
PIMDL_API int pimdl_amm_create(pimdl_ctx* ctx, const pimdl_amm_desc* desc, const float* centroids,
                               const void* lut, const float* scales, const float* bias,
                               pimdl_amm** out);
/* The same with the width of the gather kernel's column tile given by the caller (48, 64 or 96 output
 * columns; 0 = let the library choose by load balance, which is what pimdl_amm_create does).  This is the
 * knob a measured tile search turns -- the counterpart of the tile parameters the reference's auto-tuner
 * writes into its YAML (inference-engine/src/tuner/auto_tuner.cpp:552-603), found by timing instead of by a latency model.
 * PIMDL_ERR_INVALID if the operator's kernel has no variant of that width. */
PIMDL_API int pimdl_amm_create_tuned(pimdl_ctx* ctx, const pimdl_amm_desc* desc, const float* centroids,
                                     const void* lut, const float* scales, const float* bias,
                                     uint32_t col_block, pimdl_amm** out);
/* Every choice the library makes for an operator, open to a measured search (the tile autotuner).  The
 * counterpart of the kernel_params the reference's auto-tuner enumerates -- sub-tile sizes, load tile sizes,
 * LUT load type and loop order (inference-engine/src/tuner/auto_tuner.cpp:368-603) -- for this hardware:
 * the token tile, the column block, the codebook group staged at a time, and the way entries are
 * accumulated (which kernel).  0 in a field = the library's own choice.  Results do not depend on any of
 * them (every kernel gives the same bits); only the time does. */
typedef enum pimdl_gather_kernel {
    PIMDL_GATHER_AUTO = 0,
    PIMDL_GATHER_ROWS = 1,   /* byte adder: gathered row pieces summed by an identity matrix product; any C */
    PIMDL_GATHER_ONEHOT = 2, /* one-hot x table on the dense int8 matrix instruction; C <= 16 */
    PIMDL_GATHER_SPARSE = 3  /* one-hot as a 2:4 sparse operand, 8 codebooks per instruction; C <= 32 (17..32 as two codebooks of 16, up to 8 as 16 with empty rows) */
} pimdl_gather_kernel;
typedef enum pimdl_search_kernel {
    PIMDL_SEARCH_AUTO = 0,
    PIMDL_SEARCH_SCAN = 1,      /* one lane per token, the reference's scan for every pair */
    PIMDL_SEARCH_MFMA_F32 = 2,  /* scores on the fp32 matrix instruction, exact replay of near ties; C <= 16 */
    PIMDL_SEARCH_MFMA_BF16 = 3  /* scores from three bf16 pieces per value; C <= 32, sub_vec_len 2, 4, 8 */
} pimdl_search_kernel;
typedef struct pimdl_amm_tuning {
    uint32_t col_block;      /* output columns per work item of the gather: 48, 64 or 96 (what the kernel offers) */
    uint32_t gather_kernel;  /* pimdl_gather_kernel; fixes the layout of the resident table */
    uint32_t token_item;     /* tokens per work item of the matrix-core gathers: 128 or 256; the sparse kernel
                                also 512 (one workgroup of eight waves per CU instead of two of four) */
    uint32_t cb_per_slice;   /* codebooks staged in LDS at a time by the matrix-core gathers: 16 or 32
                                (32 needs col_block <= 64, or 512-token items); 64 with col_block 48 and
                                num_codebook padded to a multiple of 64, for 512-token items or for 256-token
                                items (eight waves either way; with 256 tokens the two waves of a SIMD share
                                their tokens and split the slice's codebooks) */
    uint32_t xcd_col_split;  /* how the 8 XCDs (each with its own L2) share the work items of the matrix-core
                                gathers: 1, 2, 4 or 8 of them along the column tiles, the rest along the token
                                tiles; PIMDL_XCD_PLAIN = no dealing.  A split that does not divide a launch's
                                tile counts is replaced by the library's choice for that launch. */
    uint32_t search_kernel;  /* pimdl_search_kernel */
    uint32_t search_token_tile; /* tokens per tile of the bf16 matrix-core search: 64 or 128 */
} pimdl_amm_tuning;
#define PIMDL_XCD_PLAIN 0xFFFFFFFFu
/* pimdl_amm_create with these choices made by the caller (tuning NULL or all zero: pimdl_amm_create).
 * PIMDL_ERR_INVALID when the operator's shape has no kernel for a choice. */
PIMDL_API int pimdl_amm_create_with(pimdl_ctx* ctx, const pimdl_amm_desc* desc, const float* centroids,
                                    const void* lut, const float* scales, const float* bias,
                                    const pimdl_amm_tuning* tuning, pimdl_amm** out);
/* Changes the choices that do not touch resident data (token_item, cb_per_slice, xcd_col_split,
 * search_kernel, search_token_tile) on an existing operator, so that a search need not upload the table once per candidate;
 * col_block and gather_kernel must be 0 or what the operator was created with.  pimdl_amm_get_tuning
 * reports the operator's current settings (0 where the library still chooses per launch). */
PIMDL_API int pimdl_amm_set_tuning(pimdl_amm* amm, const pimdl_amm_tuning* tuning);
PIMDL_API int pimdl_amm_get_tuning(const pimdl_amm* amm, pimdl_amm_tuning* tuning);
/* Replaces the operator's bias [M] (HOST pointer; NULL = zeros).  The reference's pim_lut reads
 * bias_tensor anew on every call (src/host/pim_lut_host.cpp:201), so a caller may refill that buffer between
 * calls; the C++ layer sends it through here each time.  Ordered behind the launches already queued on the
 * context's stream; synchronous.  A fused group (pimdl_amm_group_run_fused) keeps the biases its members had
 * when it was created. */
PIMDL_API int pimdl_amm_set_bias(pimdl_amm* amm, const float* bias);
PIMDL_API int pimdl_amm_destroy(pimdl_amm* amm);

/* The AMM itself.  Replaces amm_host (src/host/amm_host.h:8-10, amm_host.cpp:10-30) =
 * index_calculation + pim_lut, with row-major input and output.
 *   in   fp32 [n][K], host or device
 *   out  fp32 [n][M], host or device
 * Synchronous for host pointers.  For device pointers the kernels are queued on the context's
 * stream and the call returns at once; use pimdl_synchronize() or stream ordering.
 * Host buffers may be ordinary pageable memory: the batch is cut into chunks of tokens that are copied into
 * pinned staging buffers by a pool of host threads (PIMDL_COPY_THREADS, default 8), transferred, searched,
 * gathered, transferred back and copied out with four chunks in flight, so the copies overlap each other and
 * the kernels; the output bits are those of one launch over the whole batch.  With `out` on the device and
 * `in` on the host the call returns once `in` has been copied (it may be reused); the rest is stream-ordered. */
PIMDL_API int pimdl_amm_run(pimdl_amm* amm, const float* in, uint32_t n, float* out);

/* pimdl_amm_run for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  It calls no hipMalloc, hipFree
 * or other allocating routine: the packed centroid indices that travel from the search kernel to the gather
 * kernel live in a fixed array of PIMDL_NOALLOC_SCRATCH_BYTES inside the library's device image (each GPU
 * the library runs on holds its copy until the process ends) instead of the context's grow-only scratch.
 *   in_dev, out_dev  DEVICE pointers, fp32 [n][K] and [n][M]; queued on the context's stream, returns at once.
 *   PIMDL_ERR_INVALID when a pointer is a host pointer, or when n tokens need more index bytes than the array
 *   holds: n rounded up to 64, times num_codebook rounded up to 32, times 1/2 byte (up to 16 centroids) or
 *   1 byte (more).  BERT-base's 3072 -> 768 matrix at n = 8192 needs 3 MiB.
 * Output bits are those of pimdl_amm_run.  Every call on one GPU, from any context or thread, shares that
 * GPU's array: calls that overlap in time on one GPU race (calls queued on one stream do not overlap). */
#define PIMDL_NOALLOC_SCRATCH_BYTES (8u << 20)
PIMDL_API int pimdl_amm_run_noalloc(pimdl_amm* amm, const float* in_dev, uint32_t n, float* out_dev);

/* As pimdl_amm_run, plus the two intermediates that make the bit-exact claims checkable:
 *   idx_out  host uint16 [n][CB] centroid ids (what index_calculation writes under the
 *            identity tiling, src/host/index_calc_host.cpp:41-49), or NULL
 *   acc_out  host int32 [n][M] accumulators before de-quantisation (int8 LUT, scale_group 0
 *            only; the DPU's output_data, src/host/pim_lut_host.cpp:173-181), or NULL
 * Always synchronous. */
PIMDL_API int pimdl_amm_run_debug(pimdl_amm* amm, const float* in, uint32_t n, float* out,
                                  uint16_t* idx_out, int32_t* acc_out);

/* Operators that read the same rows: the reference's layer calls amm_host three times on one input for
 * the separate Q, K and V projections (src/host/transformer_layer.cpp:335-343), searching the same
 * activations against three sets of centroids.  A group searches the codebooks of all its operators
 * in ONE launch (the input is read once and the launch's fixed cost is paid once), then runs each
 * operator's gather; results are bit for bit those of pimdl_amm_run on each operator.
 *   Conditions: same context, input_feature_len, sub_vec_len (2, 4 or 8) and num_centroid (<= 32), the same
 *   LUT type, num_codebook a multiple of 32; otherwise PIMDL_ERR_UNSUPPORTED / PIMDL_ERR_INVALID and the
 *   caller runs the operators one by one.  The group borrows its operators: destroy it before them.
 *   outs[i]: fp32 [n][M_i] of operator i, host or device; n <= the smallest max_n. */
PIMDL_API int pimdl_amm_group_create(pimdl_ctx* ctx, pimdl_amm* const* amms, uint32_t count,
                                     pimdl_amm_group** out);
PIMDL_API int pimdl_amm_group_run(pimdl_amm_group* group, const float* in, uint32_t n, float* const* outs);
PIMDL_API int pimdl_amm_group_destroy(pimdl_amm_group* group);
/* When the members are int8 operators of one shape served by the matrix-core gather (up to 16
 * centroids, output_feature_len a multiple of the column tile, same LUT bias and activation), the
 * group can also run ONE gather launch over all of them and write one buffer
 *   out fp32 [n][count * M], operator i in columns i*M .. (i+1)*M - 1
 * (the layout of the reference's fused qkv output, src/host/transformer_layer.cpp:301), each column
 * bit for bit that of the operator run alone.  pimdl_amm_group_fused_cols gives count * M, or 0 when
 * the members do not allow it (pimdl_amm_group_run_fused then returns PIMDL_ERR_UNSUPPORTED). */
PIMDL_API int pimdl_amm_group_fused_cols(const pimdl_amm_group* group, uint32_t* cols);
PIMDL_API int pimdl_amm_group_run_fused(pimdl_amm_group* group, const float* in, uint32_t n, float* out);

/* Runs the two kernels `iters` times each on device-resident buffers and reports the average
 * device time of each.  in/out must be DEVICE pointers. */
PIMDL_API int pimdl_amm_profile(pimdl_amm* amm, const float* in_dev, uint32_t n, float* out_dev,
                                uint32_t warmup, uint32_t iters, pimdl_amm_timing* timing);

/* ---- the two halves on their own ---------------------------------------------------------
 * pimdl_index_calculation replaces index_calculation (src/host/index_calc_host.h:5,
 * index_calc_host.cpp:8-53) with its own argument list: in is host or device fp32 [n][K],
 * centroids is HOST fp32 [K/v][C][v] (uploaded on every call, as the reference reads it on every
 * call), idx_out is HOST uint16, written at the reference's tiled offset
 * (index_calc_host.cpp:41-49); n_stile_size == n and cb_mtile_size == K/v give row-major. */
PIMDL_API int pimdl_index_calculation(pimdl_ctx* ctx, const float* in, const float* centroids,
                                      uint32_t n, uint32_t input_feature_len, uint32_t sub_vec_len,
                                      uint32_t num_centroid, uint16_t* idx_out,
                                      uint32_t n_stile_size, uint32_t cb_mtile_size);
/* The same with an operator's resident centroids (no upload). */
PIMDL_API int pimdl_amm_index_calculation(pimdl_amm* amm, const float* in, uint32_t n,
                                          uint16_t* idx_out, uint32_t n_stile_size,
                                          uint32_t cb_mtile_size);
/* pimdl_lut_gather replaces pim_lut (src/host/pim_lut_host.h:13-14, pim_lut_host.cpp:121-222):
 * idx is HOST uint16 row-major [n][CB] holding centroid ids; out is host or device fp32 [n][M].
 * PIMDL_ERR_INVALID (the text names token and codebook) when an entry is not below num_centroid, e.g. a
 * buffer that pim_lut has already rewritten into table offsets (pim_lut_host.cpp:40-104). */
PIMDL_API int pimdl_lut_gather(pimdl_amm* amm, const uint16_t* idx, uint32_t n, float* out);

/* ---- the reference's DPU tile orders ---------------------------------------------------------
 * The reference's amm_host / pim_lut hand back the output in the order the DPUs produced it, and
 * pim_lut takes the index buffer in the order index_calculation wrote it.  These variants keep
 * those orders so the C++ layer with the reference's signatures can sit on this ABI.
 *   index offset  (n / ns)*ns*CB + (cb / cm)*ns*cm + (n % ns)*cm + cb % cm
 *                 ns = n_stile_size, cm = cb_mtile_size          (index_calc_host.cpp:41-49)
 *   output offset dpu*ns*fs + ((f % fs) / fm)*ns*fm + (n % ns)*fm + (f % fs) % fm,
 *                 dpu = (n / ns)*(M / fs) + f / fs, fs = feature_stile_size,
 *                 fm = feature_mtile_size                         (test/test_amm.cpp:193-202)
 * A zero field means "identity" (ns = n, cm = CB, fs = fm = M), i.e. row-major. */
typedef struct pimdl_tiling {
    uint32_t n_stile_size, cb_mtile_size, feature_stile_size, feature_mtile_size;
} pimdl_tiling;
/* amm_host with the reference's output order.  in host or device; out host or device. */
PIMDL_API int pimdl_amm_run_tiled(pimdl_amm* amm, const float* in, uint32_t n, float* out,
                                  const pimdl_tiling* tiling);
/* pimdl_amm_run_tiled with the phases run one after the other and waited for, and their wall-clock seconds
 * ADDED to *acc: the counterpart of the reference's AMM_BREAKDOWN build, which accumulates
 * "index calculation time" (src/host/amm_host.cpp:14-26) and "other / data transfer / pim kernel latency"
 * (src/host/pim_lut_host.cpp:124-212) the same way, with a dpu_sync between phases.  Slower than
 * pimdl_amm_run_tiled (nothing overlaps); same output bits. */
typedef struct pimdl_amm_breakdown {
    double h2d_s;    /* input to the device (staging included) */
    double search_s; /* closest-centroid search kernel: the reference's index calculation */
    double gather_s; /* LUT gather-accumulate kernel (+ output re-tiling): the reference's pim kernel */
    double d2h_s;    /* output back to the host */
} pimdl_amm_breakdown;
PIMDL_API int pimdl_amm_run_breakdown(pimdl_amm* amm, const float* in, uint32_t n, float* out,
                                      const pimdl_tiling* tiling, pimdl_amm_breakdown* acc);
/* pim_lut with the reference's index and output orders.  idx is HOST uint16 centroid ids. */
PIMDL_API int pimdl_lut_gather_tiled(pimdl_amm* amm, const uint16_t* idx, uint32_t n, float* out,
                                     const pimdl_tiling* tiling);

/* ---- LUT construction ----------------------------------------------------------------------
 * Replaces model-calibration/pim_weight_converter.py:82-91 (bmm of centroids with the weight)
 * and lut_quant (:21-35).  All pointers are HOST pointers.
 *   centroids fp32 [CB][C][v];  weight fp32 [K][M] (the transposed nn.Linear weight)
 *   lut_dtype PIMDL_LUT_F32: lut_out fp32 [CB][C][M], scales_out untouched
 *   lut_dtype PIMDL_LUT_I8 : lut_out int8 [CB][C][M]; scale_group 0: scales_out[0] =
 *             max|lut|/127 over the tensor (the reference); g > 0: one per g codebooks. */
PIMDL_API int pimdl_lutgen(pimdl_ctx* ctx, const float* centroids, const float* weight,
                           uint32_t num_codebook, uint32_t num_centroid, uint32_t sub_vec_len,
                           uint32_t output_feature_len, uint32_t lut_dtype, uint32_t scale_group,
                           void* lut_out, float* scales_out);

/* The same with the summation order of the product chosen by the caller:
 *   PIMDL_LUTGEN_MFMA     matrix instruction (what pimdl_lutgen does): the v products of an entry are added
 *                         in the matrix core's order; entries are within 1e-5 relative of any other order,
 *                         int8 tables within one quantisation step
 *   PIMDL_LUTGEN_ORDERED  ascending over the sub-vector from 0.0f, every multiplication and addition rounded
 *                         on its own: the result of a plain scalar loop, reproducible bit for bit on a CPU
 *                         (the reference's torch.bmm, pim_weight_converter.py:86-90, fixes no order).
 * Both read W once and write the table once; the work is memory bound either way. */
typedef enum pimdl_lutgen_order { PIMDL_LUTGEN_MFMA = 0, PIMDL_LUTGEN_ORDERED = 1 } pimdl_lutgen_order;
PIMDL_API int pimdl_lutgen_mode(pimdl_ctx* ctx, const float* centroids, const float* weight,
                                uint32_t num_codebook, uint32_t num_centroid, uint32_t sub_vec_len,
                                uint32_t output_feature_len, uint32_t lut_dtype, uint32_t scale_group,
                                uint32_t mode, void* lut_out, float* scales_out);

/* ---- layer normalisation of the transformer layer ---------------------------------------------
 * Replaces norm() (src/host/transformer_layer.cpp:50-90) and, when `residual` is not NULL, the
 * residual add that follows it in the layer (:476-486, :601-611):
 *     out[r][i] = residual[r][i] + ((x[r][i] - mean_r) * (1 / sqrtf(var_r + eps))) * weight[i] + bias[i]
 * mean and variance accumulated in double and rounded to float, every other operation a separately
 * rounded fp32 operation, as in the reference (which uses eps = 1e-6).  x, residual, out: [n][d];
 * weight, bias: [d]; host or device pointers; out may alias residual but not x. */
PIMDL_API int pimdl_layer_norm(pimdl_ctx* ctx, const float* x, const float* weight, const float* bias,
                               const float* residual, float* out, uint32_t n, uint32_t d, float eps);

/* ---- attention of the transformer layer ---------------------------------------------------------
 * Replaces step 2 of the reference's attention (src/host/transformer_layer.cpp:211-230: K Q, scale,
 * soft_max, V KQ, permute back), unmasked, fp32:  out = softmax(q k^T * scale) v  per (batch, head).
 *   q, k, v  DEVICE fp32 [batch*seq][in_stride], head h in columns 64 h .. 64 h + 63 (three column
 *            ranges of one fused [n][3*token_dim] buffer are fine: pass the three start addresses)
 *   out      DEVICE fp32 [batch*seq][out_stride], same column order: no head transposes
 * head_dim must be 64 (PIMDL_ERR_UNSUPPORTED otherwise: the caller keeps its own attention then).
 * Queued on the context's stream. */
PIMDL_API int pimdl_attention(pimdl_ctx* ctx, const float* q, const float* k, const float* v, float* out,
                              uint32_t batch, uint32_t seq, uint32_t heads, uint32_t head_dim,
                              uint32_t in_stride, uint32_t out_stride, float scale);

/* ---- introspection ---------------------------------------------------------------------------
 * No reference counterpart: figures a benchmark needs to place a kernel on its roofline. */
typedef struct pimdl_device_info {
    char name[64];
    char arch[32];            /* "gfx950..." */
    uint32_t compute_units;
    uint32_t clock_khz;
    uint32_t lds_bytes_per_cu;
    uint64_t hbm_bytes;
} pimdl_device_info;
PIMDL_API int pimdl_get_device_info(pimdl_ctx* ctx, pimdl_device_info* info);
/* Geometry of the operator's kernels (for documentation of a measurement).  The gather launcher picks the slice
 * depth, the tokens per workgroup and with them the LDS bytes and threads by the batch it is given:
 * cb_per_slice, lds_bytes, tokens_per_wg and gather_threads are those of the last launch, or the plan's defaults
 * before the first. */
typedef struct pimdl_amm_geometry {
    uint32_t num_codebook, num_codebook_padded, idx_bits, idx_row_bytes;
    uint32_t col_block, row_pitch, cb_per_slice, lds_bytes, tokens_per_wg, gather_threads;
    uint32_t ccs_tokens_per_wg, ccs_cb_per_wg, ccs_threads, ccs_lds_bytes;
} pimdl_amm_geometry;
PIMDL_API int pimdl_amm_get_geometry(const pimdl_amm* amm, pimdl_amm_geometry* g);
/* Name, with template arguments, of the gather kernel the operator's last launch used ("" before the first
 * launch): the name a profile of that launch lists, so that a benchmark can tell which kernel its counters
 * belong to. */
PIMDL_API int pimdl_amm_last_gather_kernel(const pimdl_amm* amm, char* name, size_t len);
/* Achieved bandwidth, GB/s, of (a) a plain device-to-device copy kernel of `bytes` bytes and
 * (b) a ds_read_b128 loop that keeps every CU's LDS busy.  Either pointer may be NULL. */
PIMDL_API int pimdl_diag_bandwidth(pimdl_ctx* ctx, uint64_t bytes, float* copy_gbps,
                                   float* lds_gbps);
/* Rates of the four legs of the host-buffer path over `bytes` bytes, GB/s: the host thread pool's copy from pageable
 * into pinned memory and back, and the transfers between pinned memory and the device.  A measuring aid. */
PIMDL_API int pimdl_diag_host_copy(pimdl_ctx* ctx, uint64_t bytes, float* to_pinned_gbps, float* from_pinned_gbps,
                                   float* h2d_gbps, float* d2h_gbps);
/* Checks on this device what the bf16-split closest-centroid search takes for granted about the
 * matrix core: runs `trials` (1..4096) chains of three v_mfma_f32_32x32x16_bf16 on random operands of
 * mixed magnitude and reports the largest |result - exact sum| in units of 2^-24 * sum|terms|.  The
 * search kernel's margin allows 51 of these units (sub_vec_len 4); index_calculation itself
 * (src/host/index_calc_host.cpp:8-53) has no counterpart of this: it is a property of this port. */
PIMDL_API int pimdl_diag_mfma_error(pimdl_ctx* ctx, uint32_t trials, float* max_err_u);
/* The same measurement on operands built to make an accumulator lose as much as it can, instead of random
 * ones: an accumulator of 1.0 that receives 48 equal products just below or just above 1/2, 1 and 2 units in its
 * last place, of either sign (an adder that rounds to nearest after every product drops all of the first kind,
 * 24 units in all; one that truncates would drop up to 96), and products that fall by a factor of four from
 * slot to slot (bits shifted out when the terms of one instruction are aligned).  The margin allows 51. */
PIMDL_API int pimdl_diag_mfma_error_crafted(pimdl_ctx* ctx, float* max_err_u);

#ifdef __cplusplus
}
#endif
#endif /* PIMDL_H */
