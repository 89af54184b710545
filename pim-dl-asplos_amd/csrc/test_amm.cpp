// Single-AMM driver: the counterpart of the reference's inference-engine/test/test_amm.cpp
// (what `python run_amm.py --amm_config_file X.yaml` ends up running).
//
//   test_amm <kernel_config.yaml> [dpu_binary_path (ignored)] [--dump FILE] [--rounds WARMUP RECORD]
//            [--split] [--load-type 0|1|2] [--refill] [--breakdown] [--assume-unchanged]
//
//   --breakdown  every amm_host call prints the two lines of the reference's AMM_BREAKDOWN build, cumulative seconds:
//                "index calculation time" (amm_host.cpp:24) and "other latency ..., data transfer latency ..., pim
//                kernel latency ..." (pim_lut_host.cpp:211); the phases then run one after the other
//   --assume-unchanged  skip the per-call hash of LUT and centroids (PimdlHostOptions::assume_unchanged); with
//                --refill the in-place changes of LUT and centroids then go unnoticed (the bias is still compared on
//                every call), and the dump holds the LUT and the centroids as they were uploaded
//   --split      every round calls index_calculation() and then pim_lut() (the two halves amm_host is made of,
//                amm_host.cpp:10-30) instead of amm_host(); the dump then also holds the index buffer as
//                pim_lut leaves it (rewritten in place, pim_lut_host.cpp:40-104)
//   --load-type  overrides kernel_params.lut_load_type (0 static, 1 fine grain, 2 coarse grain)
//   --refill     before the last round the bias, one LUT entry per row and one centroid are changed IN PLACE
//                (same buffers, same pointers), as a caller of the reference may do between calls; the dump
//                holds the changed inputs, so its output must be the one they give
//
// Reads the reference's YAML keys (src/host/parser.cpp:22-47): amm_shape_params.{num_codebook,
// num_centroid, n, input_feature_len, output_feature_len, scale, bias}, system_params.{num_threads,
// dpu_num, nr_tasklets} and kernel_params.{n_stile_size, feature_stile_size, n_mtile_size,
// feature_mtile_size, cb_mtile_size, feature_load_tile_size, cb_load_tile_size, lut_load_type,
// loop_order}.  A missing kernel_params section means the identity tiling (row-major buffers).
// Data generation follows test_amm.cpp:26-67 (mt19937(233); inputs U(-5,5), centroids and bias
// U(-10,10), LUT uniform int8) but single-threaded, so it is reproducible.  10 warm-up and 20 timed
// rounds of amm_host, "PIM AMM time" per round and the average, as the reference prints them
// (test_amm.cpp:21-22,290-314).  --dump writes inputs and the output so a test can check them.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <chrono>
#include <fstream>
#include <iostream>
#include <map>
#include <random>
#include <sstream>
#include <string>
#include <vector>

#include "pimdl/amm_host.h"

using namespace std;

// "section.key" -> scalar text, for the two-level block YAML the reference's configs use
static map<string, string> load_yaml(const string& path)
{
    map<string, string> kv;
    ifstream f(path);
    if (!f) {
        cerr << "Config File Not Open" << endl;  // parser.cpp:16
        return kv;
    }
    string line, section;
    while (getline(f, line)) {
        size_t hash = line.find('#');
        if (hash != string::npos) line.erase(hash);
        size_t first = line.find_first_not_of(" \t\r");
        if (first == string::npos) continue;
        size_t colon = line.find(':');
        if (colon == string::npos) continue;
        string key = line.substr(first, colon - first);
        string val = line.substr(colon + 1);
        size_t vb = val.find_first_not_of(" \t\r"), ve = val.find_last_not_of(" \t\r");
        val = vb == string::npos ? "" : val.substr(vb, ve - vb + 1);
        if (first == 0) {
            section = key;
            if (!val.empty()) kv[key] = val;
        } else {
            kv[section + "." + key] = val;
        }
    }
    return kv;
}

static bool has(const map<string, string>& kv, const string& k) { return kv.count(k) != 0; }
static uint32_t get_u32(const map<string, string>& kv, const string& k, uint32_t dflt)
{
    return has(kv, k) ? (uint32_t)strtoul(kv.at(k).c_str(), nullptr, 10) : dflt;
}
static float get_f32(const map<string, string>& kv, const string& k, float dflt)
{
    return has(kv, k) ? strtof(kv.at(k).c_str(), nullptr) : dflt;
}

static bool parse_amm_configs(AMMParams& p, const string& path, uint32_t* nr_tasklets)
{
    map<string, string> kv = load_yaml(path);
    const char* req[] = {"amm_shape_params.n", "amm_shape_params.input_feature_len", "amm_shape_params.num_codebook",
                         "amm_shape_params.num_centroid", "amm_shape_params.output_feature_len"};
    for (const char* r : req)
        if (!has(kv, r)) {
            cerr << "Error in parsing configs: missing " << r << endl;
            return false;
        }
    IndexCalcParams& ip = p.index_params;
    LUTParams& lp = p.lut_params;
    ip.n = get_u32(kv, "amm_shape_params.n", 0);
    ip.input_feature_len = get_u32(kv, "amm_shape_params.input_feature_len", 0);
    ip.num_codebook = get_u32(kv, "amm_shape_params.num_codebook", 0);
    ip.num_centroid = get_u32(kv, "amm_shape_params.num_centroid", 0);
    if (!ip.num_codebook || ip.input_feature_len % ip.num_codebook) {
        cerr << "input_feature_len must be a multiple of num_codebook" << endl;  // parser.cpp:57
        return false;
    }
    ip.sub_vec_len = ip.input_feature_len / ip.num_codebook;
    ip.num_threads = get_u32(kv, "system_params.num_threads", 1);
    ip.n_stile_size = get_u32(kv, "kernel_params.n_stile_size", ip.n);
    ip.cb_mtile_size = get_u32(kv, "kernel_params.cb_mtile_size", ip.num_codebook);

    lp.n = ip.n;
    lp.output_feature_len = get_u32(kv, "amm_shape_params.output_feature_len", 0);
    lp.num_codebook = ip.num_codebook;
    lp.num_centroid = ip.num_centroid;
    lp.scale = get_f32(kv, "amm_shape_params.scale", 1.0f);
    lp.bias = get_f32(kv, "amm_shape_params.bias", 0.0f);
    lp.num_threads = ip.num_threads;
    lp.dpu_num = get_u32(kv, "system_params.dpu_num", 1);
    lp.n_stile_size = ip.n_stile_size;
    lp.feature_stile_size = get_u32(kv, "kernel_params.feature_stile_size", lp.output_feature_len);
    lp.input_parallelism = lp.n / lp.n_stile_size;
    lp.lut_parallelism = lp.output_feature_len / lp.feature_stile_size;
    lp.n_mtile_size = get_u32(kv, "kernel_params.n_mtile_size", lp.n_stile_size);
    lp.feature_mtile_size = get_u32(kv, "kernel_params.feature_mtile_size", lp.feature_stile_size);
    lp.cb_mtile_size = ip.cb_mtile_size;
    lp.feature_load_tile_size = get_u32(kv, "kernel_params.feature_load_tile_size", lp.feature_mtile_size);
    lp.cb_load_tile_size = get_u32(kv, "kernel_params.cb_load_tile_size", lp.cb_mtile_size);
    lp.lut_load_type = LUTLoadType(get_u32(kv, "kernel_params.lut_load_type", 0));
    *nr_tasklets = get_u32(kv, "system_params.nr_tasklets", 16);

    // the shape checks of parser.cpp:56-66 that still mean something without DPUs
    bool ok = lp.n == lp.n_stile_size * lp.input_parallelism &&
              lp.output_feature_len == lp.feature_stile_size * lp.lut_parallelism &&
              lp.feature_stile_size % lp.feature_mtile_size == 0 && lp.num_codebook % lp.cb_mtile_size == 0 &&
              lp.feature_mtile_size % lp.feature_load_tile_size == 0 && lp.cb_mtile_size % lp.cb_load_tile_size == 0;
    if (!ok) {
        cerr << "tiling parameters do not divide the shape" << endl;
        return false;
    }
    cout << "------ amm shape params ------\n";
    cout << "num codebook " << ip.num_codebook << ", num centroid " << ip.num_centroid << endl;
    cout << "n " << ip.n << ", input feature len " << ip.input_feature_len << ", output feature len "
         << lp.output_feature_len << endl;
    cout << "scale " << lp.scale << ", bias " << lp.bias << endl;
    cout << "------ kernel params ------\n";
    cout << "n stile size " << lp.n_stile_size << ", feature stile size " << lp.feature_stile_size << endl;
    cout << "feature mtile size " << lp.feature_mtile_size << ", cb mtile size " << lp.cb_mtile_size << endl;
    cout << "lut load type " << (int)lp.lut_load_type << ", feature load tile size " << lp.feature_load_tile_size << endl;
    cout << "sub vec len " << ip.sub_vec_len << endl;
    return true;
}

// canonical [cb][c][M] -> the order amm_host expects (the job of reorder_pim_lut, test_amm.cpp:71-121)
static void to_dpu_lut_order(const vector<lut_data_type>& canon, vector<lut_data_type>& dpu, const LUTParams& lp)
{
    const uint32_t ft = lp.lut_load_type == STATIC ? lp.feature_stile_size : lp.feature_load_tile_size;
    const uint32_t CB = lp.num_codebook, C = lp.num_centroid, M = lp.output_feature_len;
    for (uint32_t cb = 0; cb < CB; ++cb)
        for (uint32_t c = 0; c < C; ++c)
            for (uint32_t f = 0; f < M; ++f)
                dpu[(size_t)(f / ft) * CB * C * ft + ((size_t)cb * C + c) * ft + f % ft] = canon[((size_t)cb * C + c) * M + f];
}

static double now_s()
{
    return chrono::duration<double>(chrono::steady_clock::now().time_since_epoch()).count();
}

int main(int argc, char** argv)
{
    if (argc < 2) {
        printf("usage: %s kernel_config_yaml_path [dpu_binary_path] [--dump FILE] [--rounds WARMUP RECORD] [--split] "
               "[--load-type T] [--refill] [--breakdown] [--assume-unchanged]\n", argv[0]);
        return -1;
    }
    string dump_path;
    int warmup = 10, record = 20;  // test_amm.cpp:21-22
    bool split = false, refill = false;
    int load_type = -1;
    for (int i = 2; i < argc; ++i) {
        if (!strcmp(argv[i], "--dump") && i + 1 < argc) dump_path = argv[++i];
        else if (!strcmp(argv[i], "--split")) split = true;
        else if (!strcmp(argv[i], "--refill")) refill = true;
        else if (!strcmp(argv[i], "--breakdown")) pimdl_host_options().breakdown = true;
        else if (!strcmp(argv[i], "--assume-unchanged")) pimdl_host_options().assume_unchanged = true;
        else if (!strcmp(argv[i], "--load-type") && i + 1 < argc) load_type = atoi(argv[++i]);
        else if (!strcmp(argv[i], "--rounds") && i + 2 < argc) {
            warmup = atoi(argv[++i]);
            record = atoi(argv[++i]);
        }
    }
    AMMParams amm;
    uint32_t nr_tasklets;
    if (!parse_amm_configs(amm, argv[1], &nr_tasklets)) return -1;
    if (load_type >= 0) amm.lut_params.lut_load_type = LUTLoadType(load_type);
    const IndexCalcParams& ip = amm.index_params;
    const LUTParams& lp = amm.lut_params;

    vector<float> input((size_t)ip.n * ip.input_feature_len);
    vector<float> centroids((size_t)ip.num_codebook * ip.num_centroid * ip.sub_vec_len);
    vector<float> bias(lp.output_feature_len);
    vector<lut_data_type> cpu_lut((size_t)lp.num_codebook * lp.num_centroid * lp.output_feature_len), dpu_lut(cpu_lut.size());
    vector<float> output((size_t)lp.n * lp.output_feature_len, 0.0f);
    {
        mt19937 gen(233);
        uniform_real_distribution<float> di(-5.0f, 5.0f);
        for (auto& x : input) x = di(gen);
    }
    {
        mt19937 gen(233);
        uniform_real_distribution<float> dc(-10.0f, 10.0f);
        for (auto& x : centroids) x = dc(gen);
    }
    {
        mt19937 gen(233);
        uniform_int_distribution<int> dl(-128, 127);
        for (auto& x : cpu_lut) x = (lut_data_type)dl(gen);
    }
    {
        mt19937 gen(233);
        uniform_real_distribution<float> db(-10.0f, 10.0f);
        for (auto& x : bias) x = db(gen);
    }
    to_dpu_lut_order(cpu_lut, dpu_lut, lp);
    cout << "data generation finished" << endl;

    double t1 = now_s();
    dpu_set_t dpu_set;
    allocate_dpu(&dpu_set, lp.dpu_num);
    cout << "dpu allocate time is " << now_s() - t1 << endl;
    t1 = now_s();
    load_binary(&dpu_set, argc > 2 && argv[2][0] != '-' ? argv[2] : "");
    cout << "binary load time is " << now_s() - t1 << endl;

    const bool assume_unchanged = pimdl_host_options().assume_unchanged;
    const vector<lut_data_type> uploaded_lut = assume_unchanged ? cpu_lut : vector<lut_data_type>();
    const vector<float> uploaded_centroids = assume_unchanged ? centroids : vector<float>();
    vector<index_data_type> index_buffer(split ? (size_t)ip.n * ip.num_codebook : 0);
    double total = 0.0;
    for (int round = 0; round < warmup + record; ++round) {
        cout << "---------- ROUND " << round << " ----------" << endl;
        if (refill && round + 1 == warmup + record && round > 0) {
            for (auto& b : bias) b = -0.5f * b + 1.0f;
            // one entry per table row; the DPU-ordered copy is what the call reads
            for (size_t row = 0; row < (size_t)lp.num_codebook * lp.num_centroid; ++row) {
                lut_data_type& e = cpu_lut[row * lp.output_feature_len + (row * 7 + 3) % lp.output_feature_len];
                e = (lut_data_type)(e == 127 ? -128 : e + 1);
            }
            to_dpu_lut_order(cpu_lut, dpu_lut, lp);
            centroids[centroids.size() / 2] += 3.0f;
            cout << "inputs changed in place" << endl;
        }
        t1 = now_s();
        if (split) {
            // amm_host.cpp:19-29: a zeroed index buffer, index_calculation, pim_lut
            fill(index_buffer.begin(), index_buffer.end(), (index_data_type)0);
            index_calculation(input.data(), centroids.data(), index_buffer.data(), ip);
            pim_lut(lp, &dpu_set, index_buffer.data(), dpu_lut.data(), bias.data(), output.data());
        } else {
            amm_host(&dpu_set, input.data(), centroids.data(), dpu_lut.data(), bias.data(), output.data(), ip, lp);
        }
        double dt = now_s() - t1;
        cout << "PIM AMM time " << dt << endl;
        if (round >= warmup) total += dt;
    }
    cout << "warm up rounds " << warmup << ", record rounds " << record << endl;
    if (record > 0) cout << "PIM AVG AMM time " << total / record << endl;

    if (!dump_path.empty()) {
        FILE* fp = fopen(dump_path.c_str(), "wb");
        if (!fp) {
            perror("dump");
            return -1;
        }
        uint32_t hdr[12] = {ip.n, ip.input_feature_len, ip.sub_vec_len, ip.num_centroid, lp.output_feature_len,
                            lp.n_stile_size, lp.cb_mtile_size, lp.feature_stile_size, lp.feature_mtile_size,
                            (uint32_t)lp.lut_load_type, lp.feature_load_tile_size, lp.cb_load_tile_size};
        fwrite(hdr, 4, 12, fp);
        fwrite(&lp.scale, 4, 1, fp);
        fwrite(&lp.bias, 4, 1, fp);
        fwrite(input.data(), 4, input.size(), fp);
        fwrite(assume_unchanged ? uploaded_centroids.data() : centroids.data(), 4, centroids.size(), fp);
        fwrite(assume_unchanged ? uploaded_lut.data() : cpu_lut.data(), 1, cpu_lut.size(), fp);
        fwrite(bias.data(), 4, bias.size(), fp);
        fwrite(output.data(), 4, output.size(), fp);
        if (split) fwrite(index_buffer.data(), sizeof(index_data_type), index_buffer.size(), fp);
        fclose(fp);
        cout << "dumped to " << dump_path << endl;
    }
    free_dpu_set(&dpu_set);
    return 0;
}
