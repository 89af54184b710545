// Parameter structs and element types of the LUT-AMM operator API, field for field as in the
// reference (inference-engine/src/host/defines.h:5-56), so that code written against the
// reference's amm_host / index_calculation / pim_lut compiles against this library unchanged.
// The DPU tiling fields are honoured for index/LUT/output *layout* (they define the order of the
// buffers crossing the API); they do not steer the GPU kernels.
#pragma once
#include <stdint.h>

typedef int8_t lut_data_type;      // defines.h:5
typedef uint16_t index_data_type;  // defines.h:6
typedef int32_t output_data_type;  // defines.h:7

enum LUTLoadType { STATIC, FINE_GRAIN, COARSE_GRAIN };  // defines.h:10

struct IndexCalcParams {  // defines.h:12-23
    uint32_t n;
    uint32_t input_feature_len;
    uint32_t sub_vec_len;
    uint32_t num_codebook;
    uint32_t num_centroid;
    uint32_t num_threads;  // CPU threads in the reference; unused here

    uint32_t n_stile_size;   // index buffer order, see index_calculation()
    uint32_t cb_mtile_size;
};

struct LUTParams {  // defines.h:25-50
    uint32_t n;
    uint32_t output_feature_len;
    uint32_t num_codebook;
    uint32_t num_centroid;

    float scale;
    float bias;

    uint32_t num_threads;  // unused
    uint32_t dpu_num;      // unused

    uint32_t input_parallelism;
    uint32_t lut_parallelism;
    uint32_t feature_stile_size;
    uint32_t n_stile_size;

    uint32_t n_mtile_size;  // unused (DPU micro-kernel tile)
    uint32_t feature_mtile_size;
    uint32_t cb_mtile_size;
    LUTLoadType lut_load_type;
    uint32_t feature_load_tile_size;
    uint32_t cb_load_tile_size;
};

struct AMMParams {  // defines.h:52-56
    IndexCalcParams index_params;
    LUTParams lut_params;
};
