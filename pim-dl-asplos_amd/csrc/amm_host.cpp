// C++ host layer with the reference's operator API (include/pimdl/amm_host.h) on top of the C ABI.
// Plain host code: everything that touches the GPU goes through include/pimdl.h.
#include "pimdl/amm_host.h"

#include <stdio.h>
#include <string.h>

#include <chrono>
#include <map>
#include <mutex>
#include <stdexcept>
#include <tuple>
#include <vector>

#include "host_pool.h"
#include "pimdl.h"

#define PIMDL_HOST_API __attribute__((visibility("default")))

namespace {

struct Cached {
    pimdl_amm* amm;
    uint64_t fingerprint;
    uint32_t max_n;
};

// key: lut pointer, centroid pointer, N-independent shape, layout, scale, LUT bias.  The bias tensor is not part
// of it: it is sent to the device on every call, as the reference reads it on every call.
typedef std::tuple<const void*, const void*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t> Key;

std::mutex g_mu;
std::map<std::pair<pimdl_ctx*, Key>, Cached> g_cache;
pimdl_ctx* g_implicit_ctx = nullptr;
PimdlHostOptions g_opts;
PimdlHostProfiles g_profiles;

double now_s() { return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count(); }

[[noreturn]] void fail(pimdl_ctx* ctx, const char* what)
{
    throw std::runtime_error(std::string(what) + ": " + pimdl_last_error(ctx));
}

pimdl_ctx* ctx_of(dpu_set_t* s)
{
    if (!s || !s->impl) throw std::runtime_error("dpu_set_t is not allocated (call allocate_dpu / allocate_rank first)");
    return static_cast<pimdl_ctx*>(s->impl);
}

pimdl_ctx* implicit_ctx()
{
    if (!g_implicit_ctx && pimdl_init(g_opts.device, &g_implicit_ctx)) fail(nullptr, "pimdl_init");
    return g_implicit_ctx;
}

// Hash of every byte (four independent multiply-xor lanes over 32-byte blocks, then the tail): one pass over
// memory, a fraction of the host-to-device copy that it saves.  The reference re-sends LUT and centroids on
// every call, so whatever the caller changed behind the same pointers must be noticed here.
uint64_t fingerprint_piece(const void* p, size_t bytes);

// The pieces of a large buffer are hashed side by side on the host thread pool and their hashes combined in order.
uint64_t fingerprint(const void* p, size_t bytes)
{
    constexpr size_t PIECE = 1u << 20;
    if (bytes <= PIECE) return fingerprint_piece(p, bytes);
    const size_t pieces = (bytes + PIECE - 1) / PIECE;
    std::vector<uint64_t> h(pieces);
    const int width = pimdl::host_pool().width();
    pimdl::host_pool().run(width, [&](int w) {
        for (size_t i = w; i < pieces; i += width) {
            const size_t off = i * PIECE, len = off + PIECE <= bytes ? PIECE : bytes - off;
            h[i] = fingerprint_piece(static_cast<const unsigned char*>(p) + off, len);
        }
    });
    return fingerprint_piece(h.data(), pieces * sizeof(uint64_t)) ^ bytes;
}

uint64_t fingerprint_piece(const void* p, size_t bytes)
{
    const unsigned char* b = static_cast<const unsigned char*>(p);
    const uint64_t m = 0x9E3779B97F4A7C15ull;
    uint64_t h[4] = {bytes ^ 0x243F6A8885A308D3ull, 0x13198A2E03707344ull, 0xA4093822299F31D0ull, 0x082EFA98EC4E6C89ull};
    size_t off = 0;
    for (; off + 32 <= bytes; off += 32) {
        uint64_t w[4];
        memcpy(w, b + off, 32);
        for (int i = 0; i < 4; ++i) {
            h[i] = (h[i] ^ w[i]) * m;
            h[i] ^= h[i] >> 29;
        }
    }
    uint64_t tail[4] = {0, 0, 0, 0};
    memcpy(tail, b + off, bytes - off);
    for (int i = 0; i < 4; ++i) h[i] = (h[i] ^ tail[i]) * m;
    uint64_t r = 0;
    for (int i = 0; i < 4; ++i) r = (r ^ h[i] ^ (h[i] >> 32)) * m;
    return r;
}

uint32_t lut_tile(const LUTParams& lp)
{
    return lp.lut_load_type == STATIC ? lp.feature_stile_size : lp.feature_load_tile_size;
}

// [f_tile][cb][c][f_in_tile] (test_amm.cpp:82-92,106-116) -> canonical [cb][c][M]
void untile_lut(const lut_data_type* dpu_lut, lut_data_type* canon, uint32_t CB, uint32_t C, uint32_t M, uint32_t ft)
{
    const uint32_t ntile = M / ft;
    for (uint32_t t = 0; t < ntile; ++t)
        for (uint32_t cb = 0; cb < CB; ++cb)
            for (uint32_t c = 0; c < C; ++c)
                memcpy(canon + ((size_t)cb * C + c) * M + (size_t)t * ft,
                       dpu_lut + (size_t)t * CB * C * ft + ((size_t)cb * C + c) * ft, ft);
}

pimdl_amm* get_operator(pimdl_ctx* ctx, const float* centroids, uint32_t K, uint32_t v, const lut_data_type* lut,
                        const float* bias, const LUTParams& lp)
{
    const uint32_t CB = lp.num_codebook, C = lp.num_centroid, M = lp.output_feature_len;
    uint32_t ft = lut_tile(lp);
    if (ft == 0 || ft > M) ft = M;
    if (M % ft) throw std::runtime_error("LUT feature tile does not divide output_feature_len");
    uint32_t scale_bits, bias_bits;
    memcpy(&scale_bits, &lp.scale, 4);
    memcpy(&bias_bits, &lp.bias, 4);
    const Key key(lut, centroids, K, v, C, M, ft, scale_bits, bias_bits);
    const size_t lut_bytes = (size_t)CB * C * M;

    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_cache.find(std::make_pair(ctx, key));
    // assume_unchanged: a cached operator is trusted without reading the caller's tables again
    const bool trust = g_opts.assume_unchanged && it != g_cache.end();
    const uint64_t fp = trust ? it->second.fingerprint
                              : fingerprint(lut, lut_bytes) ^ (centroids ? fingerprint(centroids, (size_t)CB * C * v * 4) : 0);
    uint32_t max_n = lp.n;
    if (it != g_cache.end()) {
        if (it->second.fingerprint == fp && it->second.max_n >= lp.n) {
            if (pimdl_amm_set_bias(it->second.amm, bias)) fail(ctx, "pimdl_amm_set_bias");  // a no-op unless it changed
            return it->second.amm;
        }
        // a batch that creeps upwards: room for half as much again, so that operators are rebuilt (and the
        // table sent again) a logarithmic number of times
        if (it->second.fingerprint == fp && it->second.max_n < lp.n && it->second.max_n + it->second.max_n / 2 > lp.n)
            max_n = it->second.max_n + it->second.max_n / 2;
        pimdl_amm_destroy(it->second.amm);
        g_cache.erase(it);
    }
    std::vector<lut_data_type> canon;
    const lut_data_type* canon_ptr = lut;
    if (ft != M) {
        canon.resize(lut_bytes);
        untile_lut(lut, canon.data(), CB, C, M, ft);
        canon_ptr = canon.data();
    }
    std::vector<float> dummy_centroids;
    if (!centroids) {  // pim_lut() alone never searches centroids
        dummy_centroids.assign((size_t)CB * C * v, 0.0f);
        centroids = dummy_centroids.data();
    }
    pimdl_amm_desc d;
    memset(&d, 0, sizeof(d));
    d.max_n = max_n;
    d.input_feature_len = K;
    d.sub_vec_len = v;
    d.num_centroid = C;
    d.output_feature_len = M;
    d.lut_dtype = PIMDL_LUT_I8;
    d.scale_group = 0;
    d.bias_mode = PIMDL_BIAS_TIMES_CB;  // pim_lut_host.cpp:201
    d.lut_bias = lp.bias;
    pimdl_amm* amm = nullptr;
    if (pimdl_amm_create(ctx, &d, centroids, canon_ptr, &lp.scale, bias, &amm)) fail(ctx, "pimdl_amm_create");
    g_cache[std::make_pair(ctx, key)] = Cached{amm, fp, max_n};
    return amm;
}

pimdl_tiling tiling_of(const LUTParams& lp)
{
    pimdl_tiling t;
    t.n_stile_size = lp.n_stile_size;
    t.cb_mtile_size = lp.cb_mtile_size;
    t.feature_stile_size = lp.feature_stile_size;
    t.feature_mtile_size = lp.feature_mtile_size;
    return t;
}

// pim_lut_host.cpp:40-104: the in-place rewrite of centroid ids into DPU table offsets
void mutate_index(const LUTParams& lp, index_data_type* idx)
{
    const uint32_t ns = lp.n_stile_size ? lp.n_stile_size : lp.n;
    const uint32_t cm = lp.cb_mtile_size ? lp.cb_mtile_size : lp.num_codebook;
    for (uint32_t n = 0; n < lp.n; ++n)
        for (uint32_t cb = 0; cb < lp.num_codebook; ++cb) {
            const uint32_t ci = cb % cm;
            const size_t off = (size_t)(n / ns) * ns * lp.num_codebook + (size_t)(cb / cm) * ns * cm +
                               (size_t)(n % ns) * cm + ci;
            if (lp.lut_load_type == STATIC)
                idx[off] = (index_data_type)(idx[off] * lp.feature_stile_size);
            else if (lp.lut_load_type == FINE_GRAIN)
                idx[off] = (index_data_type)(idx[off] * lp.feature_load_tile_size);
            else
                idx[off] = (index_data_type)((ci % lp.cb_load_tile_size) * lp.num_centroid * lp.feature_load_tile_size +
                                             idx[off] * lp.feature_load_tile_size);
        }
}

}  // namespace

PIMDL_HOST_API PimdlHostOptions& pimdl_host_options() { return g_opts; }
PIMDL_HOST_API PimdlHostProfiles& pimdl_host_profiles() { return g_profiles; }

PIMDL_HOST_API void pimdl_host_invalidate(const void* lut_table)
{
    std::lock_guard<std::mutex> lock(g_mu);
    for (auto it = g_cache.begin(); it != g_cache.end();) {
        if (std::get<0>(it->first.second) == lut_table) {
            pimdl_amm_destroy(it->second.amm);
            it = g_cache.erase(it);
        } else {
            ++it;
        }
    }
}

PIMDL_HOST_API uint32_t allocate_dpu(dpu_set_t* dpu_set, uint32_t dpu_num)
{
    pimdl_ctx* ctx = nullptr;
    if (pimdl_init(g_opts.device, &ctx)) fail(nullptr, "allocate_dpu: pimdl_init");
    dpu_set->impl = ctx;
    return dpu_num;
}

PIMDL_HOST_API uint32_t allocate_rank(dpu_set_t* dpu_set, uint32_t rank_num)
{
    allocate_dpu(dpu_set, rank_num * 64);
    return rank_num * 64;  // NR_DPUS_PER_RANK
}

PIMDL_HOST_API void free_dpu_set(dpu_set_t* dpu_set)
{
    if (!dpu_set || !dpu_set->impl) return;
    pimdl_ctx* ctx = static_cast<pimdl_ctx*>(dpu_set->impl);
    {
        std::lock_guard<std::mutex> lock(g_mu);
        for (auto it = g_cache.begin(); it != g_cache.end();) {
            if (it->first.first == ctx) {
                pimdl_amm_destroy(it->second.amm);
                it = g_cache.erase(it);
            } else {
                ++it;
            }
        }
    }
    pimdl_destroy(ctx);
    dpu_set->impl = nullptr;
}

PIMDL_HOST_API void load_binary(dpu_set_t*, std::string) {}  // the kernels live in the library

PIMDL_HOST_API void index_calculation(float* input_tensor, float* centroid_tensor, index_data_type* lut_input_index,
                                      IndexCalcParams p)
{
    pimdl_ctx* ctx = implicit_ctx();
    if (pimdl_index_calculation(ctx, input_tensor, centroid_tensor, p.n, p.input_feature_len, p.sub_vec_len,
                                p.num_centroid, lut_input_index, p.n_stile_size, p.cb_mtile_size))
        fail(ctx, "index_calculation");
}

PIMDL_HOST_API void pim_lut(LUTParams lp, dpu_set_t* dpu_set, index_data_type* input_index, lut_data_type* lut_table,
                            float* bias_tensor, float* output_tensor)
{
    pimdl_ctx* ctx = ctx_of(dpu_set);
    // K and v are irrelevant to the gather; the operator is keyed with v = 1, K = num_codebook
    pimdl_amm* amm = get_operator(ctx, nullptr, lp.num_codebook, 1, lut_table, bias_tensor, lp);
    const pimdl_tiling t = tiling_of(lp);
    if (pimdl_lut_gather_tiled(amm, input_index, lp.n, output_tensor, &t)) fail(ctx, "pim_lut");
    if (g_opts.mutate_index_buffer) mutate_index(lp, input_index);
}

PIMDL_HOST_API void amm_host(dpu_set_t* dpu_set, float* input_tensor, float* centroid_tensor, lut_data_type* lut_table,
                             float* bias_tensor, float* output_tensor, IndexCalcParams ip, LUTParams lp)
{
    pimdl_ctx* ctx = ctx_of(dpu_set);
    if (ip.n != lp.n || ip.num_codebook != lp.num_codebook || ip.num_centroid != lp.num_centroid ||
        ip.input_feature_len != ip.num_codebook * ip.sub_vec_len)
        throw std::runtime_error("amm_host: index_params and lut_params disagree");
    const double t0 = g_opts.breakdown ? now_s() : 0.0;
    pimdl_amm* amm = get_operator(ctx, centroid_tensor, ip.input_feature_len, ip.sub_vec_len, lut_table, bias_tensor, lp);
    const pimdl_tiling t = tiling_of(lp);
    if (!g_opts.breakdown) {
        if (pimdl_amm_run_tiled(amm, input_tensor, lp.n, output_tensor, &t)) fail(ctx, "amm_host");
        return;
    }
    // The reference's AMM_BREAKDOWN build (amm_host.cpp:14-26, pim_lut_host.cpp:124-212): cumulative buckets,
    // printed on every call in the reference's own words.
    pimdl_amm_breakdown b = {0, 0, 0, 0};
    if (pimdl_amm_run_breakdown(amm, input_tensor, lp.n, output_tensor, &t, &b)) fail(ctx, "amm_host");
    const double total = now_s() - t0;
    g_profiles.index_calc_latency += b.search_s;
    g_profiles.data_transfer_latency += b.h2d_s + b.d2h_s;
    g_profiles.kernel_latency += b.gather_s;
    g_profiles.other_latency += total - (b.search_s + b.h2d_s + b.d2h_s + b.gather_s);
    printf("index calculation time %.6f\n", g_profiles.index_calc_latency);
    printf("other latency %.6f, data transfer latency %.6f, pim kernel latency %.6f\n", g_profiles.other_latency,
           g_profiles.data_transfer_latency, g_profiles.kernel_latency);
}
