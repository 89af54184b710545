// C entry point around the reference's index_calculation so that ctypes can call it.
// Compiled together with <reference>/inference-engine/src/host/index_calc_host.cpp by
// oracle/Makefile; the declaration comes from the reference's own header
// (inference-engine/src/host/index_calc_host.h:5, params struct defines.h:12-23).
// Test infrastructure only.
#include "index_calc_host.h"

extern "C" __attribute__((visibility("default")))
void ref_index_calculation(float* input, float* centroids, uint16_t* index_out,
                           uint32_t n, uint32_t input_feature_len, uint32_t sub_vec_len,
                           uint32_t num_codebook, uint32_t num_centroid, uint32_t num_threads,
                           uint32_t n_stile_size, uint32_t cb_mtile_size)
{
    IndexCalcParams p;
    p.n = n;
    p.input_feature_len = input_feature_len;
    p.sub_vec_len = sub_vec_len;
    p.num_codebook = num_codebook;
    p.num_centroid = num_centroid;
    p.num_threads = num_threads;
    p.n_stile_size = n_stile_size;
    p.cb_mtile_size = cb_mtile_size;
    index_calculation(input, centroids, index_out, p);
}
