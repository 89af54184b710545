// The reference's C++ operator API for the LUT-AMM path, on an MI355X.
//
// Same names, argument order and argument meaning as
//   amm_host           inference-engine/src/host/amm_host.h:8-10
//   index_calculation  inference-engine/src/host/index_calc_host.h:5
//   pim_lut            inference-engine/src/host/pim_lut_host.h:13-14
//   allocate_dpu / allocate_rank / free_dpu_set / load_binary
//                      inference-engine/src/host/dpu_common.h:11-54
// so a caller of the reference (its test_amm.cpp:295, transformer_layer.cpp:301,431,500,556) links
// against libpimdl.so instead of libhost.so + the UPMEM SDK.  `dpu_set_t` is UPMEM's device-set
// handle; here it is an opaque struct that owns a GPU context (C ABI: include/pimdl.h).
//
// Buffer orders are the reference's:
//   index buffer  (n/ns)*ns*CB + (cb/cm)*ns*cm + (n%ns)*cm + cb%cm      index_calc_host.cpp:41-49
//   lut_table     [f_tile][cb][c][f_in_tile], tile = feature_stile_size when lut_load_type is
//                 STATIC, else feature_load_tile_size                   test/test_amm.cpp:71-121
//   output        dpu*ns*fs + ((f%fs)/fm)*ns*fm + (n%ns)*fm + (f%fs)%fm  test/test_amm.cpp:193-202
// With n_stile_size = n, cb_mtile_size = num_codebook and feature_*_size = output_feature_len all
// three are plain row-major / canonical.
//
// Differences from the reference, all deliberate:
//   * the LUT and the centroids are uploaded to the device once per (pointer, shape) and reused; the
//     reference re-sends the LUT on every call (pim_lut_host.cpp:143).  Every call hashes both buffers
//     in full (one pass over host memory, on the library's host threads) and uploads again when anything
//     behind the pointers has changed (PimdlHostOptions::assume_unchanged skips the hash); bias_tensor is
//     compared with the device's copy on every call and sent when it differs (the reference reads it on
//     every call, :201).
//     pimdl_host_invalidate(lut_table) drops the device copy explicitly.
//   * failures throw std::runtime_error (the reference aborts through DPU_ASSERT);
//   * nothing is leaked per call (the reference leaks its index and int32 buffers,
//     amm_host.cpp:19, pim_lut_host.cpp:133).
//   * pim_lut() rewrites the caller's index buffer in place exactly as the reference's
//     prepare_input_index does (pim_lut_host.cpp:40-104) unless
//     pimdl_host_options().mutate_index_buffer is cleared.
//   * the epilogue adds bias*num_codebook like pim_lut (pim_lut_host.cpp:201), not bias like the
//     test-only amm_cpu (test_amm.cpp:181); the two agree for bias == 0.
#pragma once
#include <string>

#include "defines.h"

struct dpu_set_t {
    void* impl;  // pimdl_ctx*
};

uint32_t allocate_dpu(dpu_set_t* dpu_set, uint32_t dpu_num);    // dpu_common.h:11-20; returns dpu_num
uint32_t allocate_rank(dpu_set_t* dpu_set, uint32_t rank_num);  // dpu_common.h:22-31; returns 64*rank_num
void free_dpu_set(dpu_set_t* dpu_set);                          // dpu_common.h:33-36
void load_binary(dpu_set_t* dpu_set, std::string binary_name = "");  // dpu_common.h:38-54; no-op

void index_calculation(float* input_tensor, float* centroid_tensor, index_data_type* lut_input_index,
                       IndexCalcParams index_params);

void pim_lut(LUTParams lut_params, dpu_set_t* dpu_set, index_data_type* input_index, lut_data_type* lut_table,
             float* bias_tensor, float* output_tensor);

void amm_host(dpu_set_t* dpu_set, float* input_tensor, float* centroid_tensor, lut_data_type* lut_table,
              float* bias_tensor, float* output_tensor, IndexCalcParams index_params, LUTParams lut_params);

// ---- additions (no counterpart in the reference) --------------------------------------------------
struct PimdlHostOptions {
    bool mutate_index_buffer = true;  // pim_lut(): reproduce the reference's in-place index rewrite
    int device = 0;                   // GPU used by allocate_dpu / by index_calculation's implicit context
    // amm_host / pim_lut: trust the device copy of a LUT and its centroids once they have been uploaded for a
    // (pointer, shape) and skip the per-call hash of both buffers.  Off by default: the reference re-sends the LUT
    // on every call (pim_lut_host.cpp:143), so in-place edits must be seen.  With it on, edits behind the same
    // pointers go unnoticed until pimdl_host_invalidate(lut_table).
    bool assume_unchanged = false;
    // amm_host: run the phases one after the other, add their wall-clock seconds to pimdl_host_profiles() and
    // print the two lines of the reference's AMM_BREAKDOWN build (amm_host.cpp:14-26, pim_lut_host.cpp:211).
    bool breakdown = false;
};
PimdlHostOptions& pimdl_host_options();
// The reference's amm_profiles (utils.h:37-40), seconds, cumulative: index calculation = the search kernel,
// kernel = the gather kernel, data transfer = input to and output from the device, other = the rest of the call.
struct PimdlHostProfiles {
    double index_calc_latency = 0, other_latency = 0, data_transfer_latency = 0, kernel_latency = 0;
};
PimdlHostProfiles& pimdl_host_profiles();
// Forget the device copy of a LUT (and its centroids) cached under this host pointer.
void pimdl_host_invalidate(const void* lut_table);
