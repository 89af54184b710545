// C ABI of libpimdl (see include/pimdl.h).  Host-side plumbing only: shape checks, uploads,
// scratch buffers, pointer classification, kernel sequencing.  There is no CPU compute path:
// without a gfx950 device pimdl_init fails and nothing else can be called.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <new>

#include <algorithm>
#include <chrono>
#include <mutex>
#include <set>
#include <utility>
#include <vector>

#include "host_pool.h"
#include "pimdl_internal.h"

// Scratch of pimdl_amm_run_noalloc: the packed centroid indices that the search kernel writes and the gather
// kernel reads.  A file-scope device array, so the entry point never allocates; every GPU the library runs on
// holds its own copy until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress: kernels and memory calls get the device address that call returned (kept per device in
// g_scratch_ptr, and per context in Ctx::d_static_scratch).
static __device__ __align__(256) unsigned char scratch[PIMDL_NOALLOC_SCRATCH_BYTES];

namespace pimdl {

static thread_local std::string g_init_error;

constexpr int MAX_DEVICES = 64;
static std::mutex g_scratch_mutex;
static unsigned char* g_scratch_ptr[MAX_DEVICES];  // device address of `scratch` on each device, once asked for

// Address of this device's copy of `scratch` (the device must be current).
static int static_scratch_address(Ctx* ctx, int device, unsigned char** out)
{
    if (device < 0 || device >= MAX_DEVICES) return set_error(ctx, PIMDL_ERR_UNSUPPORTED, "device %d: at most %d devices", device, MAX_DEVICES);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        unsigned char* p = nullptr;
        int rc = hip_check(ctx, hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)");
        if (rc) return rc;
        if (!p) return set_error(ctx, PIMDL_ERR_HIP, "hipGetSymbolAddress(scratch) returned a null address");
        g_scratch_ptr[device] = p;
    }
    *out = g_scratch_ptr[device];
    return PIMDL_OK;
}

int set_error(Ctx* ctx, int code, const char* fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    if (ctx) ctx->err = buf;
    else g_init_error = buf;
    return code;
}

int hip_check(Ctx* ctx, hipError_t e, const char* what)
{
    if (e == hipSuccess) return PIMDL_OK;
    return set_error(ctx, e == hipErrorOutOfMemory ? PIMDL_ERR_NOMEM : PIMDL_ERR_HIP, "%s: %s", what,
                     hipGetErrorString(e));
}

int allow_dynamic_lds(Ctx* ctx, const void* kernel, int lds_bytes, const char* what)
{
    static std::mutex mu;
    static std::set<std::pair<int, const void*>> done;  // the attribute belongs to the kernel's code object on one device
    std::lock_guard<std::mutex> lock(mu);
    const std::pair<int, const void*> key(ctx->device, kernel);
    if (done.count(key)) return PIMDL_OK;
    int rc = hip_check(ctx, hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes), what);
    if (!rc) done.insert(key);
    return rc;
}

static bool is_device_ptr(const void* p)
{
    hipPointerAttribute_t attr;
    memset(&attr, 0, sizeof(attr));
    hipError_t e = hipPointerGetAttributes(&attr, p);
    if (e != hipSuccess) {
        (void)hipGetLastError();  // ordinary host memory is reported as an error; clear it
        return false;
    }
    return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged;
}

// Grow-only scratch.  A buffer that is too small is replaced by a larger one; the old one stays allocated until
// the context is destroyed, because a HIP graph captured from earlier calls on this context holds its address
// (both kernels of a captured AMM were given the same buffer, so a replay stays consistent with itself).
// A buffer that grows does so by at least half its size, so that a caller whose batch creeps upwards goes through
// a geometric series of buffers: the retired ones together stay below twice the size of the live one.
// While the stream is being captured nothing may be allocated: the call is refused instead.
template <typename T>
static int ensure(Ctx* ctx, T** buf, size_t* have, size_t need, const char* what)
{
    if (*have >= need) return PIMDL_OK;
    if (*have && need < *have + *have / 2) need = *have + *have / 2;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(ctx->stream, &cap) != hipSuccess) (void)hipGetLastError();
    if (cap != hipStreamCaptureStatusNone)
        return set_error(ctx, PIMDL_ERR_INVALID,
                         "%s: the stream is being captured and the context's scratch (%zu bytes) would have to grow to "
                         "%zu: run the call once outside the capture first", what, *have, need);
    void* fresh = nullptr;
    int rc = hip_check(ctx, hipMalloc(&fresh, need), what);
    if (rc) return rc;
    if (*buf) {
        try {
            ctx->retired.push_back(*buf);
        } catch (...) {
            (void)hipFree(fresh);
            return set_error(ctx, PIMDL_ERR_NOMEM, "%s: out of host memory", what);
        }
    }
    *buf = static_cast<T*>(fresh);
    *have = need;
    return PIMDL_OK;
}

static int activate(Ctx* ctx) { return hip_check(ctx, hipSetDevice(ctx->device), "hipSetDevice"); }

// input/output staging common to run / run_debug / the two halves
struct IoPlan {
    const float* d_in;
    float* d_out;
    bool out_is_host;
};

static int stage_input(Ctx* ctx, const AmmGeom& g, const float* in, uint32_t n, const float** d_in)
{
    if (is_device_ptr(in)) {
        *d_in = in;
        return PIMDL_OK;
    }
    const size_t bytes = (size_t)n * g.K * sizeof(float);
    int rc = ensure(ctx, &ctx->d_in, &ctx->in_bytes, bytes, "hipMalloc(input scratch)");
    if (rc) return rc;
    rc = hip_check(ctx, hipMemcpyAsync(ctx->d_in, in, bytes, hipMemcpyHostToDevice, ctx->stream), "H2D input");
    *d_in = ctx->d_in;
    return rc;
}

static int stage_output(Ctx* ctx, const AmmGeom& g, float* out, uint32_t n, float** d_out, bool* host)
{
    if (is_device_ptr(out)) {
        *d_out = out;
        *host = false;
        return PIMDL_OK;
    }
    const size_t bytes = (size_t)n * g.M * sizeof(float);
    int rc = ensure(ctx, &ctx->d_out, &ctx->out_bytes, bytes, "hipMalloc(output scratch)");
    *d_out = ctx->d_out;
    *host = true;
    return rc;
}

static int finish_output(Ctx* ctx, const AmmGeom& g, float* out, uint32_t n, bool host)
{
    if (!host) return PIMDL_OK;
    int rc = hip_check(ctx, hipMemcpyAsync(out, ctx->d_out, (size_t)n * g.M * sizeof(float), hipMemcpyDeviceToHost,
                                           ctx->stream), "D2H output");
    if (rc) return rc;
    return hip_check(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
}

// ---- host buffers: the pinned staging ring ------------------------------------------------------------------
// The reference's amm_host takes and returns ordinary (pageable) host memory.  A transfer straight from such
// memory goes through the runtime's own single-threaded staging at about a fifth of the link's rate, so the
// library stages by itself: the batch is cut into chunks of tokens (rows are independent), each chunk is copied
// into a pinned buffer by the host thread pool, sent, searched and gathered on its own, sent back and copied out,
// with HostPipe::SLOTS chunks in flight on three streams of equal priority.
static void pipe_destroy(Ctx* ctx)
{
    HostPipe* hp = ctx->pipe;
    if (!hp) return;
    if (hp->s_in) (void)hipStreamSynchronize(hp->s_in);
    if (hp->s_out) (void)hipStreamSynchronize(hp->s_out);
    for (int s = 0; s < HostPipe::SLOTS; ++s) {
        if (hp->pin_in[s]) (void)hipHostFree(hp->pin_in[s]);
        if (hp->pin_out[s]) (void)hipHostFree(hp->pin_out[s]);
        (void)hipFree(hp->d_in[s]);
        (void)hipFree(hp->d_out[s]);
        if (hp->ev_in[s]) (void)hipEventDestroy(hp->ev_in[s]);
        if (hp->ev_run[s]) (void)hipEventDestroy(hp->ev_run[s]);
        if (hp->ev_out[s]) (void)hipEventDestroy(hp->ev_out[s]);
    }
    if (hp->s_in) (void)hipStreamDestroy(hp->s_in);
    if (hp->s_out) (void)hipStreamDestroy(hp->s_out);
    delete hp;
    ctx->pipe = nullptr;
}

static int pipe_get(Ctx* ctx, HostPipe** out)
{
    if (!ctx->pipe) {
        HostPipe* hp = new (std::nothrow) HostPipe();
        if (!hp) return set_error(ctx, PIMDL_ERR_NOMEM, "host staging: out of host memory");
        ctx->pipe = hp;
        int rc = hip_check(ctx, hipStreamCreateWithFlags(&hp->s_in, hipStreamNonBlocking), "hipStreamCreate(staging in)");
        if (!rc) rc = hip_check(ctx, hipStreamCreateWithFlags(&hp->s_out, hipStreamNonBlocking), "hipStreamCreate(staging out)");
        for (int s = 0; s < HostPipe::SLOTS && !rc; ++s) {
            rc = hip_check(ctx, hipEventCreateWithFlags(&hp->ev_in[s], hipEventDisableTiming), "hipEventCreate");
            if (!rc) rc = hip_check(ctx, hipEventCreateWithFlags(&hp->ev_run[s], hipEventDisableTiming), "hipEventCreate");
            if (!rc) rc = hip_check(ctx, hipEventCreateWithFlags(&hp->ev_out[s], hipEventDisableTiming), "hipEventCreate");
        }
        if (rc) {
            pipe_destroy(ctx);
            return rc;
        }
    }
    *out = ctx->pipe;
    return PIMDL_OK;
}

// Per-slot buffers of at least the given sizes (0: that direction is not staged).  Only called while the ring is
// idle (every call that uses it drains it before it returns or before it touches a slot again).
static int pipe_reserve(Ctx* ctx, HostPipe* hp, size_t in_bytes, size_t out_bytes)
{
    int rc = PIMDL_OK;
    if (in_bytes > hp->in_bytes) {
        if ((rc = hip_check(ctx, hipStreamSynchronize(hp->s_in), "hipStreamSynchronize(staging in)"))) return rc;
        if ((rc = hip_check(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize"))) return rc;
        for (int s = 0; s < HostPipe::SLOTS; ++s) {
            if (hp->pin_in[s]) (void)hipHostFree(hp->pin_in[s]);
            (void)hipFree(hp->d_in[s]);
            hp->pin_in[s] = nullptr;
            hp->d_in[s] = nullptr;
        }
        hp->in_bytes = 0;
        for (int s = 0; s < HostPipe::SLOTS && !rc; ++s) {
            rc = hip_check(ctx, hipHostMalloc(&hp->pin_in[s], in_bytes, hipHostMallocDefault), "hipHostMalloc(staging in)");
            if (!rc) rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&hp->d_in[s]), in_bytes), "hipMalloc(staging in)");
        }
        if (rc) return rc;
        hp->in_bytes = in_bytes;
    }
    if (out_bytes > hp->out_bytes) {
        if ((rc = hip_check(ctx, hipStreamSynchronize(hp->s_out), "hipStreamSynchronize(staging out)"))) return rc;
        if ((rc = hip_check(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize"))) return rc;
        for (int s = 0; s < HostPipe::SLOTS; ++s) {
            if (hp->pin_out[s]) (void)hipHostFree(hp->pin_out[s]);
            (void)hipFree(hp->d_out[s]);
            hp->pin_out[s] = nullptr;
            hp->d_out[s] = nullptr;
        }
        hp->out_bytes = 0;
        for (int s = 0; s < HostPipe::SLOTS && !rc; ++s) {
            rc = hip_check(ctx, hipHostMalloc(&hp->pin_out[s], out_bytes, hipHostMallocDefault), "hipHostMalloc(staging out)");
            if (!rc) rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&hp->d_out[s]), out_bytes), "hipMalloc(staging out)");
        }
        if (rc) return rc;
        hp->out_bytes = out_bytes;
    }
    return PIMDL_OK;
}

// Chunk boundaries (first token of each chunk, then n).  Chunks hold about 12 MiB of the wider staged side, in
// multiples of 256 tokens (whole items of the gathers); the first two and the last two are a quarter and a half of
// that, so that the device starts early and little is left to come back and be copied out after the last kernel.
static std::vector<uint32_t> pipe_chunks(uint32_t n, size_t row_bytes)
{
    const char* e = getenv("PIMDL_HOST_CHUNK_TOKENS");
    const uint64_t forced = e ? strtoull(e, nullptr, 10) : 0;
    uint64_t base = forced ? forced : (12u << 20) / (row_bytes ? row_bytes : 1);
    base = base / 256 * 256;
    if (base < 256) base = 256;
    std::vector<uint32_t> b;
    const bool ramp = !forced && base >= 1024 && n >= 4 * base;
    const uint32_t head[2] = {(uint32_t)base / 4, (uint32_t)base / 2};
    uint32_t at = 0;
    b.push_back(0);
    if (ramp)
        for (uint32_t h : head) b.push_back(at += h);
    const uint32_t tail = ramp ? head[0] + head[1] : 0;
    while (n - at > base + tail) b.push_back(at += (uint32_t)base);
    if (ramp) {
        const uint32_t rest = n - at - tail;  // 1 .. base tokens
        if (rest) b.push_back(at += rest);
        b.push_back(at += head[1]);
    }
    b.push_back(n);
    return b;
}

// One AMM with at least one of in / out in host memory.  `run_chunk(d_in, d_out, tokens)` queues the kernels of
// one chunk on the context's stream.  Synchronous when out is a host buffer; with a device `out` the call returns
// once `in` has been copied to pinned memory (the caller may reuse it), the rest is ordered on the streams.
template <class RunChunk>
static int run_piped(Ctx* ctx, uint32_t K, uint32_t M, const float* in, bool in_host, float* out, bool out_host,
                     uint32_t n, RunChunk run_chunk)
{
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(ctx->stream, &cap) != hipSuccess) (void)hipGetLastError();
    if (cap != hipStreamCaptureStatusNone)
        return set_error(ctx, PIMDL_ERR_INVALID, "host buffers cannot be staged while the stream is being captured: pass device pointers");
    HostPipe* hp;
    int rc = pipe_get(ctx, &hp);
    if (rc) return rc;
    constexpr int SLOTS = HostPipe::SLOTS, LAG = SLOTS - 1;
    const size_t in_row = (size_t)K * sizeof(float), out_row = (size_t)M * sizeof(float);
    const size_t wide = (in_host ? in_row : 0) > (out_host ? out_row : 0) ? in_row : out_row;
    std::vector<uint32_t> first;  // chunk c holds tokens first[c] .. first[c + 1] - 1
    try {
        first = pipe_chunks(n, wide);
    } catch (...) {
        return set_error(ctx, PIMDL_ERR_NOMEM, "host staging: out of host memory");
    }
    const uint32_t nchunks = (uint32_t)first.size() - 1;
    uint32_t chunk = 0;  // the largest
    for (uint32_t c = 0; c < nchunks; ++c) chunk = std::max(chunk, first[c + 1] - first[c]);
    if ((rc = pipe_reserve(ctx, hp, in_host ? chunk * in_row : 0, out_host ? chunk * out_row : 0))) return rc;

    auto fail = [&](int code) {  // nothing may stay in flight towards buffers the caller owns
        (void)hipStreamSynchronize(hp->s_in);
        (void)hipStreamSynchronize(ctx->stream);
        (void)hipStreamSynchronize(hp->s_out);
        return code;
    };
    auto tokens_of = [&](uint32_t c) { return first[c + 1] - first[c]; };
    for (uint32_t c = 0; c < nchunks + (out_host ? LAG : 0); ++c) {
        if (c < nchunks) {
            const int s = c % SLOTS;
            const uint32_t tok = tokens_of(c);
            const float* d_in = in + (size_t)first[c] * K;
            float* d_out = out + (size_t)first[c] * M;
            if (in_host) {
                // the slot's pinned buffer is free once its last transfer has left it
                if (hp->used_in[s] && (rc = hip_check(ctx, hipEventSynchronize(hp->ev_in[s]), "hipEventSynchronize(staging in)"))) return fail(rc);
                parallel_copy(hp->pin_in[s], d_in, tok * in_row);
                // ... and its device buffer once the kernels that read it are done
                if (hp->used_run[s] && (rc = hip_check(ctx, hipStreamWaitEvent(hp->s_in, hp->ev_run[s], 0), "hipStreamWaitEvent"))) return fail(rc);
                if ((rc = hip_check(ctx, hipMemcpyAsync(hp->d_in[s], hp->pin_in[s], tok * in_row, hipMemcpyHostToDevice, hp->s_in), "H2D input chunk"))) return fail(rc);
                if ((rc = hip_check(ctx, hipEventRecord(hp->ev_in[s], hp->s_in), "hipEventRecord"))) return fail(rc);
                hp->used_in[s] = true;
                if ((rc = hip_check(ctx, hipStreamWaitEvent(ctx->stream, hp->ev_in[s], 0), "hipStreamWaitEvent"))) return fail(rc);
                d_in = hp->d_in[s];
            }
            if (out_host) {
                // the slot's device output is free once its last transfer back has read it
                if (hp->used_out[s] && (rc = hip_check(ctx, hipStreamWaitEvent(ctx->stream, hp->ev_out[s], 0), "hipStreamWaitEvent"))) return fail(rc);
                d_out = hp->d_out[s];
            }
            if ((rc = run_chunk(d_in, d_out, tok))) return fail(rc);
            if ((rc = hip_check(ctx, hipEventRecord(hp->ev_run[s], ctx->stream), "hipEventRecord"))) return fail(rc);
            hp->used_run[s] = true;
            if (out_host) {
                if ((rc = hip_check(ctx, hipStreamWaitEvent(hp->s_out, hp->ev_run[s], 0), "hipStreamWaitEvent"))) return fail(rc);
                if ((rc = hip_check(ctx, hipMemcpyAsync(hp->pin_out[s], hp->d_out[s], tok * out_row, hipMemcpyDeviceToHost, hp->s_out), "D2H output chunk"))) return fail(rc);
                if ((rc = hip_check(ctx, hipEventRecord(hp->ev_out[s], hp->s_out), "hipEventRecord"))) return fail(rc);
                hp->used_out[s] = true;
            }
        }
        if (out_host && c >= (uint32_t)LAG) {  // chunk c - LAG has had LAG iterations to come back
            const uint32_t r = c - LAG;
            const int s = r % SLOTS;
            if ((rc = hip_check(ctx, hipEventSynchronize(hp->ev_out[s]), "hipEventSynchronize(staging out)"))) return fail(rc);
            parallel_copy(out + (size_t)first[r] * M, hp->pin_out[s], tokens_of(r) * out_row);
        }
    }
    return PIMDL_OK;
}

static int check_run_args(Amm* amm, const void* a, const void* b, uint32_t n)
{
    if (!amm) return PIMDL_ERR_INVALID;
    if (!a || !b) return set_error(amm->ctx, PIMDL_ERR_INVALID, "null buffer");
    if (n > amm->desc.max_n)
        return set_error(amm->ctx, PIMDL_ERR_INVALID, "n=%u exceeds max_n=%u of this operator", n, amm->desc.max_n);
    return activate(amm->ctx);
}

template <typename T>
static void retile_lut(const T* lut, T* tiled, const AmmGeom& g, uint32_t row_elems)
{
    // canonical [CB][C][M] -> [M_pad/row_elems][CB_pad][C_tile][row_elems], zero padded;
    // chunked fp32 tables: [M_pad/row_elems][CB_pad][row_elems/2][C_tile][2]
    const uint32_t nblk = g.M_pad / row_elems;
    const bool chunked = sizeof(T) == 4 && g.lut_chunked;
    for (uint32_t b = 0; b < nblk; ++b)
        for (uint32_t cb = 0; cb < g.CB; ++cb)
            for (uint32_t c = 0; c < g.C; ++c) {
                const T* src = lut + ((size_t)cb * g.C + c) * g.M + (size_t)b * row_elems;
                const uint32_t cnt = (b + 1) * row_elems <= g.M ? row_elems : g.M - b * row_elems;
                if (chunked) {
                    T* blk = tiled + ((size_t)b * g.CB_pad + cb) * g.C_tile * row_elems;
                    for (uint32_t e = 0; e < cnt; ++e) blk[((size_t)(e / 2) * g.C_tile + c) * 2 + e % 2] = src[e];
                    continue;
                }
                T* dst = tiled + (((size_t)b * g.CB_pad + cb) * g.C_tile + c) * row_elems;
                memcpy(dst, src, sizeof(T) * cnt);
            }
}

// canonical [CB][C][M] -> [M_pad/col_block][CB_pad][col_block][16], zero padded (C <= 16);
// C_tile 8 (C <= 8): [M_pad/col_block][CB_pad/2][col_block][2][8], codebooks 2k and 2k+1 side by side
static void retile_lut_onehot(const int8_t* lut, int8_t* tiled, const AmmGeom& g)
{
    const uint32_t wn = g.col_block;
    const bool paired = g.C_tile == 8, wide = g.C_tile == 32;
    // position of column f % wn inside its tile: the sparse-instruction kernel deals a tile's columns to its
    // 16-column groups so that a lane's accumulators are consecutive columns
    std::vector<uint32_t> where(wn);
    for (uint32_t s = 0; s < wn; ++s) where[g.gather_kind == 2 ? sparse_tile_column(wn / 16, s) : s] = s;
    for (uint32_t cb = 0; cb < g.CB; ++cb)
        for (uint32_t c = 0; c < g.C; ++c) {
            const int8_t* src = lut + ((size_t)cb * g.C + c) * g.M;
            // an entry is 16 slots: a codebook; two codebooks of up to 8 centroids; half a codebook of 17..32
            const uint32_t entry = paired ? cb / 2 : wide ? 2 * cb + c / 16 : cb;
            const uint32_t entries = paired ? g.CB_pad / 2 : wide ? 2 * g.CB_pad : g.CB_pad;
            const uint32_t slot = paired ? 8 * (cb & 1) + c : c % 16;
            for (uint32_t f = 0; f < g.M; ++f)
                tiled[((((size_t)(f / wn) * entries + entry) * wn) + where[f % wn]) * 16 + slot] = src[f];
        }
}

}  // namespace pimdl

using namespace pimdl;

struct pimdl_ctx : Ctx {};
struct pimdl_amm : Amm {};
// Operators that read the same input rows, searched by one launch over all their codebooks.
struct pimdl_amm_group {
    Ctx* ctx;
    std::vector<pimdl_amm*> members;
    AmmGeom g;            // search geometry: the members' codebooks side by side (K = members * K of one)
    float* d_centroids;   // the members' centroids, concatenated, + derived search data
    uint32_t x_cols;      // floats per input row (one member's K)
    uint32_t max_n;
    // Members that are matrix-core gathers of one shape also run as ONE gather launch over their column
    // tiles side by side, into one [n][members * M] output (pimdl_amm_group_run_fused): `merged` borrows the
    // members' geometry and owns concatenated copies of their tables, biases and scales.
    bool has_merged;
    Amm merged;
};

extern "C" {

int pimdl_init(int device, pimdl_ctx** out)
{
    if (!out) return set_error(nullptr, PIMDL_ERR_INVALID, "pimdl_init: out is null");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0) {
        (void)hipGetLastError();
        return set_error(nullptr, PIMDL_ERR_NO_DEVICE,
                         "pimdl_init: no HIP device visible (%s); this library has no CPU fallback",
                         e == hipSuccess ? "device count 0" : hipGetErrorString(e));
    }
    if (device < 0 || device >= count)
        return set_error(nullptr, PIMDL_ERR_INVALID, "pimdl_init: device %d out of range (0..%d)", device, count - 1);
    pimdl_ctx* ctx = new pimdl_ctx();
    ctx->device = device;
    ctx->own_stream = nullptr;
    ctx->stream = nullptr;
    ctx->d_in = nullptr; ctx->in_bytes = 0;
    ctx->d_out = nullptr; ctx->out_bytes = 0;
    ctx->d_idx = nullptr; ctx->idx_bytes = 0;
    ctx->d_acc = nullptr; ctx->acc_bytes = 0;
    ctx->d_idx16 = nullptr; ctx->idx16_bytes = 0;
    ctx->d_tmp = nullptr; ctx->tmp_bytes = 0;
    ctx->d_cent = nullptr; ctx->cent_bytes = 0;
    ctx->d_static_scratch = nullptr;
    ctx->pipe = nullptr;
    for (auto& ev : ctx->ev) ev = nullptr;
    int rc = hip_check(ctx, hipSetDevice(device), "hipSetDevice");
    if (!rc) rc = hip_check(ctx, hipGetDeviceProperties(&ctx->prop, device), "hipGetDeviceProperties");
    if (!rc && strncmp(ctx->prop.gcnArchName, "gfx950", 6) != 0)
        rc = set_error(ctx, PIMDL_ERR_UNSUPPORTED, "pimdl_init: device %d is %s; the kernels are built for gfx950 only",
                       device, ctx->prop.gcnArchName);
    // (after the check above: on another device the library's code object, and with it the symbol, does not exist)
    if (!rc) rc = static_scratch_address(ctx, device, &ctx->d_static_scratch);
    if (!rc) rc = hip_check(ctx, hipStreamCreate(&ctx->own_stream), "hipStreamCreate");
    for (auto& ev : ctx->ev)
        if (!rc) rc = hip_check(ctx, hipEventCreate(&ev), "hipEventCreate");
    if (rc) {
        g_init_error = ctx->err;
        pimdl_destroy(ctx);
        return rc;
    }
    ctx->stream = ctx->own_stream;
    *out = ctx;
    return PIMDL_OK;
}

int pimdl_destroy(pimdl_ctx* ctx)
{
    if (!ctx) return PIMDL_OK;
    (void)hipSetDevice(ctx->device);
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    pipe_destroy(ctx);
    (void)hipFree(ctx->d_in);
    (void)hipFree(ctx->d_out);
    (void)hipFree(ctx->d_idx);
    (void)hipFree(ctx->d_acc);
    (void)hipFree(ctx->d_idx16);
    (void)hipFree(ctx->d_tmp);
    (void)hipFree(ctx->d_cent);
    for (void* p : ctx->retired) (void)hipFree(p);
    for (auto& ev : ctx->ev)
        if (ev) (void)hipEventDestroy(ev);
    if (ctx->own_stream) (void)hipStreamDestroy(ctx->own_stream);
    delete ctx;
    return PIMDL_OK;
}

const char* pimdl_last_error(const pimdl_ctx* ctx) { return ctx ? ctx->err.c_str() : g_init_error.c_str(); }

int pimdl_set_stream(pimdl_ctx* ctx, void* hip_stream)
{
    if (!ctx) return PIMDL_ERR_INVALID;
    int rc = activate(ctx);
    if (rc) return rc;
    rc = hip_check(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize(old stream)");
    ctx->stream = hip_stream ? reinterpret_cast<hipStream_t>(hip_stream) : ctx->own_stream;
    return rc;
}

int pimdl_synchronize(pimdl_ctx* ctx)
{
    if (!ctx) return PIMDL_ERR_INVALID;
    int rc = activate(ctx);
    if (rc) return rc;
    return hip_check(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
}

int pimdl_amm_create(pimdl_ctx* ctx, const pimdl_amm_desc* desc, const float* centroids, const void* lut,
                     const float* scales, const float* bias, pimdl_amm** out)
{
    return pimdl_amm_create_with(ctx, desc, centroids, lut, scales, bias, nullptr, out);
}

int pimdl_amm_create_tuned(pimdl_ctx* ctx, const pimdl_amm_desc* desc, const float* centroids, const void* lut,
                           const float* scales, const float* bias, uint32_t col_block, pimdl_amm** out)
{
    pimdl_amm_tuning t;
    memset(&t, 0, sizeof(t));
    t.col_block = col_block;
    return pimdl_amm_create_with(ctx, desc, centroids, lut, scales, bias, &t, out);
}

int pimdl_amm_set_tuning(pimdl_amm* a, const pimdl_amm_tuning* t)
{
    if (!a) return PIMDL_ERR_INVALID;
    Ctx* ctx = a->ctx;
    if (!t) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_set_tuning: null argument");
    const uint32_t kind = a->g.gather_kind == 0 ? PIMDL_GATHER_ROWS : a->g.gather_kind == 1 ? PIMDL_GATHER_ONEHOT : PIMDL_GATHER_SPARSE;
    if ((t->col_block && t->col_block != a->g.col_block) || (t->gather_kernel && t->gather_kernel != kind))
        return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_set_tuning: col_block and gather_kernel fix the resident table; "
                                                 "create the operator with them (pimdl_amm_create_with)");
    std::string why;
    AmmGeom g = a->g;
    if (!apply_runtime_tuning(&g, *t, &why)) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_set_tuning: %s", why.c_str());
    a->g = g;
    return PIMDL_OK;
}

int pimdl_amm_get_tuning(const pimdl_amm* a, pimdl_amm_tuning* t)
{
    if (!a || !t) return PIMDL_ERR_INVALID;
    t->col_block = a->g.col_block;
    t->gather_kernel = a->g.gather_kind == 0 ? PIMDL_GATHER_ROWS : a->g.gather_kind == 1 ? PIMDL_GATHER_ONEHOT : PIMDL_GATHER_SPARSE;
    t->token_item = a->g.tune_token_item;
    t->cb_per_slice = a->g.tune_cb_per_slice;
    t->xcd_col_split = a->g.tune_xcd_col_split;
    t->search_kernel = a->g.tune_search;
    t->search_token_tile = a->g.tune_search_tile;
    return PIMDL_OK;
}

int pimdl_amm_create_with(pimdl_ctx* ctx, const pimdl_amm_desc* desc, const float* centroids, const void* lut,
                          const float* scales, const float* bias, const pimdl_amm_tuning* tuning, pimdl_amm** out)
{
    if (!ctx) return PIMDL_ERR_INVALID;
    if (!desc || !centroids || !lut || !out) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_create: null argument");
    *out = nullptr;
    int rc = activate(ctx);
    if (rc) return rc;
    const bool i8_in = desc->lut_dtype == PIMDL_LUT_I8;
    // One scale per group of codebooks: the table is kept as fp32 integers and gathered by the
    // fp32 kernel, which applies scale[g] at the end of each group.
    const bool grouped = i8_in && desc->scale_group != 0;
    pimdl_amm_desc plan = *desc;
    if (grouped) plan.lut_dtype = PIMDL_LUT_F32;
    AmmGeom g;
    memset(&g, 0, sizeof(g));
    std::string why;
    if (!plan_geometry(plan, ctx->prop.multiProcessorCount, &g, &why, tuning)) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_create: %s", why.c_str());
    if (i8_in && !scales) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_create: int8 LUT needs scales");
    if (grouped && desc->lut_bias != 0.0f)
        return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_create: scale_group > 0 has no zero point: lut_bias must be 0");
    if (grouped && desc->scale_group > (1u << 16))
        return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_create: scale_group=%u: a group's sum must stay below 2^24", desc->scale_group);
    const bool i8 = i8_in && !grouped;  // resident as int8

    pimdl_amm* a = new pimdl_amm();
    a->ctx = ctx;
    a->desc = *desc;
    a->g = g;
    a->d_centroids = nullptr;
    a->d_lut = nullptr;
    a->d_scales = nullptr;
    a->d_bias = nullptr;
    a->grouped = grouped;
    a->prescaled = grouped && desc->scale_group == 1;
    a->d_op_scales = nullptr;
    a->op_col_tiles = 0;
    a->op_idx_stride = 0;
    a->nscales = grouped ? (g.CB + desc->scale_group - 1) / desc->scale_group : i8 ? 1 : 0;
    a->h_scale0 = i8 ? scales[0] : 1.0f;

    const size_t cent_bytes = (size_t)g.CB * g.C * g.v * sizeof(float);
    const size_t elem = i8 ? 1 : 4;
    const uint32_t row_elems = g.col_block;
    a->lut_bytes = (size_t)g.M_pad * g.CB_pad * g.C_tile * elem;
    std::vector<unsigned char> tiled;
    try {
        tiled.assign(a->lut_bytes, 0);
    } catch (...) {
        delete a;
        return set_error(ctx, PIMDL_ERR_NOMEM, "pimdl_amm_create: host staging of %zu bytes failed", a->lut_bytes);
    }
    if (i8 && g.gather_kind != 0) retile_lut_onehot(reinterpret_cast<const int8_t*>(lut), reinterpret_cast<int8_t*>(tiled.data()), g);
    else if (i8) retile_lut(reinterpret_cast<const int8_t*>(lut), reinterpret_cast<int8_t*>(tiled.data()), g, row_elems);
    else if (grouped) {
        std::vector<float> wide;
        try {
            const int8_t* q = reinterpret_cast<const int8_t*>(lut);
            wide.assign(q, q + (size_t)g.CB * g.C * g.M);  // int8 -> float, exact
            if (a->prescaled) {
                // one scale per codebook: a group's sum is the entry itself, so scaling it here (one fp32
                // rounding) is what the kernel would do at every group boundary, and the adds that remain are
                // those of an fp32 table in the same order
                const size_t per_cb = (size_t)g.C * g.M;
                for (uint32_t cb = 0; cb < g.CB; ++cb) {
                    const float sc = scales[cb];
                    float* w = wide.data() + cb * per_cb;
                    for (size_t i = 0; i < per_cb; ++i) w[i] = w[i] * sc;
                }
            }
        } catch (...) {
            delete a;
            return set_error(ctx, PIMDL_ERR_NOMEM, "pimdl_amm_create: host staging of the widened table failed");
        }
        retile_lut(wide.data(), reinterpret_cast<float*>(tiled.data()), g, row_elems);
    } else retile_lut(reinterpret_cast<const float*>(lut), reinterpret_cast<float*>(tiled.data()), g, row_elems);

    rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&a->d_centroids), ccs_centroid_bytes(g)), "hipMalloc(centroids)");
    if (!rc) rc = hip_check(ctx, hipMalloc(&a->d_lut, a->lut_bytes), "hipMalloc(lut)");
    if (!rc) rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&a->d_bias), (size_t)g.M * sizeof(float)), "hipMalloc(bias)");
    if (!rc && a->nscales) rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&a->d_scales), sizeof(float) * a->nscales), "hipMalloc(scales)");
    if (!rc) rc = hip_check(ctx, hipMemcpy(a->d_centroids, centroids, cent_bytes, hipMemcpyHostToDevice), "H2D centroids");
    if (!rc) rc = launch_ccs_prep(ctx, g, a->d_centroids);
    if (!rc) rc = hip_check(ctx, hipMemcpy(a->d_lut, tiled.data(), a->lut_bytes, hipMemcpyHostToDevice), "H2D lut");
    if (!rc) {
        try {
            if (bias) a->h_bias.assign(bias, bias + g.M);
            else a->h_bias.assign(g.M, 0.0f);
        } catch (...) {
            rc = set_error(ctx, PIMDL_ERR_NOMEM, "pimdl_amm_create: out of host memory");
        }
    }
    if (!rc) rc = hip_check(ctx, hipMemcpy(a->d_bias, a->h_bias.data(), (size_t)g.M * sizeof(float), hipMemcpyHostToDevice), "H2D bias");
    if (!rc && a->nscales) rc = hip_check(ctx, hipMemcpy(a->d_scales, scales, sizeof(float) * a->nscales, hipMemcpyHostToDevice), "H2D scales");
    // the index scratch of the largest batch now, so that runs on device buffers never allocate
    if (!rc) rc = ensure(ctx, &ctx->d_idx, &ctx->idx_bytes, idx_buffer_bytes(g, desc->max_n), "hipMalloc(index scratch)");
    if (rc) {
        pimdl_amm_destroy(a);
        return rc;
    }
    *out = a;
    return PIMDL_OK;
}

int pimdl_amm_set_bias(pimdl_amm* a, const float* bias)
{
    if (!a) return PIMDL_ERR_INVALID;
    Ctx* ctx = a->ctx;
    int rc = activate(ctx);
    if (rc) return rc;
    const size_t bytes = (size_t)a->g.M * sizeof(float);
    // the device already holds these values: nothing to send, nothing to wait for
    if (a->h_bias.size() == a->g.M &&
        (bias ? memcmp(a->h_bias.data(), bias, bytes) == 0
              : std::all_of(a->h_bias.begin(), a->h_bias.end(), [](float f) { uint32_t b; memcpy(&b, &f, 4); return b == 0; })))
        return PIMDL_OK;
    // a copy and a wait cannot be recorded into a graph
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(ctx->stream, &cap) != hipSuccess) (void)hipGetLastError();
    if (cap != hipStreamCaptureStatusNone)
        return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_set_bias: the stream is being captured; change the bias outside the capture");
    try {
        if (bias) a->h_bias.assign(bias, bias + a->g.M);
        else a->h_bias.assign(a->g.M, 0.0f);
    } catch (...) {
        return set_error(ctx, PIMDL_ERR_NOMEM, "pimdl_amm_set_bias: out of host memory");
    }
    // ordered on the context's stream behind the launches that still read the old values
    rc = hip_check(ctx, hipMemcpyAsync(a->d_bias, a->h_bias.data(), bytes, hipMemcpyHostToDevice, ctx->stream), "H2D bias");
    if (rc) {
        a->h_bias.clear();
        return rc;
    }
    return hip_check(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
}

int pimdl_amm_destroy(pimdl_amm* a)
{
    if (!a) return PIMDL_OK;
    (void)hipSetDevice(a->ctx->device);
    (void)hipStreamSynchronize(a->ctx->stream);
    (void)hipFree(a->d_centroids);
    (void)hipFree(a->d_lut);
    (void)hipFree(a->d_scales);
    (void)hipFree(a->d_bias);
    delete a;
    return PIMDL_OK;
}

int pimdl_amm_group_create(pimdl_ctx* ctx, pimdl_amm* const* amms, uint32_t count, pimdl_amm_group** out)
{
    if (!ctx) return PIMDL_ERR_INVALID;
    if (!out) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_group_create: out is null");
    *out = nullptr;
    if (!amms || count < 2 || count > 16) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_group_create: 2..16 operators expected");
    int rc = activate(ctx);
    if (rc) return rc;
    const Amm* first = amms[0];
    if (!first) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_group_create: null operator");
    uint32_t max_n = first->desc.max_n;
    for (uint32_t i = 0; i < count; ++i) {
        const Amm* a = amms[i];
        if (!a) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_group_create: null operator");
        if (a->ctx != ctx) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_group_create: operator %u belongs to another context", i);
        if (a->g.K != first->g.K || a->g.v != first->g.v || a->g.C != first->g.C)
            return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_group_create: operator %u differs in input_feature_len, sub_vec_len or num_centroid", i);
        if (a->g.idx_tiled != first->g.idx_tiled || a->g.idx_bits != first->g.idx_bits)
            return set_error(ctx, PIMDL_ERR_UNSUPPORTED, "pimdl_amm_group_create: operator %u uses another index layout (LUT type differs)", i);
        max_n = a->desc.max_n < max_n ? a->desc.max_n : max_n;
    }
    if (first->g.CB != first->g.CB_pad)
        return set_error(ctx, PIMDL_ERR_UNSUPPORTED, "pimdl_amm_group_create: num_codebook=%u is not a multiple of 32", first->g.CB);
    AmmGeom g = first->g;
    g.K *= count;
    g.CB *= count;
    g.CB_pad *= count;
    g.idx_row_bytes *= count;
    if (!ccs_supports_shared_input(g, first->g.K))
        return set_error(ctx, PIMDL_ERR_UNSUPPORTED, "pimdl_amm_group_create: no shared-input search for sub_vec_len=%u, num_centroid=%u, input_feature_len=%u",
                         g.v, g.C, first->g.K);
    pimdl_amm_group* grp = new pimdl_amm_group();
    grp->ctx = ctx;
    grp->members.assign(amms, amms + count);
    grp->g = g;
    grp->d_centroids = nullptr;
    grp->x_cols = first->g.K;
    grp->max_n = max_n;
    grp->has_merged = false;
    rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&grp->d_centroids), ccs_centroid_bytes(g)), "hipMalloc(group centroids)");
    const size_t one = (size_t)first->g.CB * g.C * g.v;  // raw centroid floats of one member
    for (uint32_t i = 0; i < count && !rc; ++i)
        rc = hip_check(ctx, hipMemcpyAsync(grp->d_centroids + i * one, amms[i]->d_centroids, one * sizeof(float),
                                           hipMemcpyDeviceToDevice, ctx->stream), "D2D centroids");
    if (!rc) rc = launch_ccs_prep(ctx, g, grp->d_centroids);
    if (!rc) rc = ensure(ctx, &ctx->d_idx, &ctx->idx_bytes, idx_buffer_bytes(g, max_n), "hipMalloc(index scratch)");
    // one gather launch for all members?
    bool same = first->desc.lut_dtype == PIMDL_LUT_I8 && !first->grouped && first->g.gather_kind != 0 &&
                first->g.M % first->g.col_block == 0;
    const float lbt0 = first->desc.bias_mode == PIMDL_BIAS_TIMES_CB ? first->desc.lut_bias * (float)first->g.CB : first->desc.lut_bias;
    for (uint32_t i = 1; i < count && same; ++i) {
        const Amm* a = amms[i];
        const float lbt = a->desc.bias_mode == PIMDL_BIAS_TIMES_CB ? a->desc.lut_bias * (float)a->g.CB : a->desc.lut_bias;
        same = a->desc.lut_dtype == PIMDL_LUT_I8 && !a->grouped && a->g.gather_kind == first->g.gather_kind && a->g.M == first->g.M &&
               a->g.q == first->g.q && a->g.C_tile == first->g.C_tile && a->g.CB_pad == first->g.CB_pad &&
               a->lut_bytes == first->lut_bytes && a->desc.activation == first->desc.activation && lbt == lbt0;
    }
    if (!rc && same) {
        Amm& m = grp->merged;
        m = *first;  // geometry, epilogue constants; the pointers below are the group's own
        m.d_centroids = nullptr;
        m.d_scales = nullptr;
        m.d_lut = nullptr;
        m.d_bias = nullptr;
        m.d_op_scales = nullptr;
        m.g.M = m.g.M_pad = first->g.M * count;
        m.desc.output_feature_len = m.g.M;
        m.desc.max_n = max_n;
        m.g.idx_row_bytes = g.idx_row_bytes;
        m.op_col_tiles = first->g.M / first->g.col_block;
        m.op_idx_stride = first->g.idx_row_bytes * 64;  // tiled index rows: a byte range is a range of 256-byte blocks
        m.lut_bytes = first->lut_bytes * count;
        std::vector<float> sc(count);
        for (uint32_t i = 0; i < count; ++i) sc[i] = amms[i]->h_scale0;
        rc = hip_check(ctx, hipMalloc(&m.d_lut, m.lut_bytes), "hipMalloc(group lut)");
        if (!rc) rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&m.d_bias), (size_t)m.g.M * sizeof(float)), "hipMalloc(group bias)");
        if (!rc) rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&m.d_op_scales), count * sizeof(float)), "hipMalloc(group scales)");
        for (uint32_t i = 0; i < count && !rc; ++i) {
            rc = hip_check(ctx, hipMemcpyAsync(static_cast<char*>(m.d_lut) + (size_t)i * first->lut_bytes, amms[i]->d_lut,
                                               first->lut_bytes, hipMemcpyDeviceToDevice, ctx->stream), "D2D lut");
            if (!rc) rc = hip_check(ctx, hipMemcpyAsync(m.d_bias + (size_t)i * first->g.M, amms[i]->d_bias,
                                                        (size_t)first->g.M * sizeof(float), hipMemcpyDeviceToDevice, ctx->stream), "D2D bias");
        }
        if (!rc) rc = hip_check(ctx, hipMemcpy(m.d_op_scales, sc.data(), count * sizeof(float), hipMemcpyHostToDevice), "H2D group scales");
        grp->has_merged = !rc;
    }
    if (!rc) rc = hip_check(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    if (rc) {
        pimdl_amm_group_destroy(grp);
        return rc;
    }
    *out = grp;
    return PIMDL_OK;
}

int pimdl_amm_group_destroy(pimdl_amm_group* grp)
{
    if (!grp) return PIMDL_OK;
    (void)hipSetDevice(grp->ctx->device);
    (void)hipStreamSynchronize(grp->ctx->stream);
    (void)hipFree(grp->d_centroids);
    if (grp->merged.d_lut) (void)hipFree(grp->merged.d_lut);
    if (grp->merged.d_bias) (void)hipFree(grp->merged.d_bias);
    if (grp->merged.d_op_scales) (void)hipFree(grp->merged.d_op_scales);
    delete grp;
    return PIMDL_OK;
}

int pimdl_amm_group_fused_cols(const pimdl_amm_group* grp, uint32_t* cols)
{
    if (!grp || !cols) return PIMDL_ERR_INVALID;
    *cols = grp->has_merged ? grp->merged.g.M : 0;
    return PIMDL_OK;
}

int pimdl_amm_group_run_fused(pimdl_amm_group* grp, const float* in, uint32_t n, float* out)
{
    if (!grp) return PIMDL_ERR_INVALID;
    Ctx* ctx = grp->ctx;
    if (!grp->has_merged)
        return set_error(ctx, PIMDL_ERR_UNSUPPORTED, "pimdl_amm_group_run_fused: the members do not share one matrix-core gather shape");
    if (!in || !out) return set_error(ctx, PIMDL_ERR_INVALID, "null buffer");
    if (n > grp->max_n) return set_error(ctx, PIMDL_ERR_INVALID, "n=%u exceeds max_n=%u of this group", n, grp->max_n);
    int rc = activate(ctx);
    if (rc || n == 0) return rc;
    const float* d_in;
    float* d_out;
    bool out_host;
    if ((rc = stage_input(ctx, grp->members[0]->g, in, n, &d_in))) return rc;
    if ((rc = stage_output(ctx, grp->merged.g, out, n, &d_out, &out_host))) return rc;
    if ((rc = ensure(ctx, &ctx->d_idx, &ctx->idx_bytes, idx_buffer_bytes(grp->g, n), "hipMalloc(index scratch)"))) return rc;
    if ((rc = launch_ccs(ctx, grp->g, d_in, grp->d_centroids, ctx->d_idx, n, grp->x_cols))) return rc;
    if ((rc = launch_gather(ctx, grp->merged, ctx->d_idx, d_out, nullptr, n))) return rc;
    return finish_output(ctx, grp->merged.g, out, n, out_host);
}

int pimdl_amm_group_run(pimdl_amm_group* grp, const float* in, uint32_t n, float* const* outs)
{
    if (!grp) return PIMDL_ERR_INVALID;
    Ctx* ctx = grp->ctx;
    if (!in || !outs) return set_error(ctx, PIMDL_ERR_INVALID, "null buffer");
    for (size_t i = 0; i < grp->members.size(); ++i)
        if (!outs[i]) return set_error(ctx, PIMDL_ERR_INVALID, "null output %zu", i);
    if (n > grp->max_n) return set_error(ctx, PIMDL_ERR_INVALID, "n=%u exceeds max_n=%u of this group", n, grp->max_n);
    int rc = activate(ctx);
    if (rc || n == 0) return rc;
    const float* d_in;
    if ((rc = stage_input(ctx, grp->members[0]->g, in, n, &d_in))) return rc;
    if ((rc = ensure(ctx, &ctx->d_idx, &ctx->idx_bytes, idx_buffer_bytes(grp->g, n), "hipMalloc(index scratch)"))) return rc;
    if ((rc = launch_ccs(ctx, grp->g, d_in, grp->d_centroids, ctx->d_idx, n, grp->x_cols))) return rc;
    for (size_t i = 0; i < grp->members.size(); ++i) {
        // member i's index bytes are bytes i*rb .. (i+1)*rb-1 of every row of the common buffer
        Amm view = *grp->members[i];
        const size_t rb = view.g.idx_row_bytes;
        view.g.idx_row_bytes = grp->g.idx_row_bytes;
        const uint8_t* idx_i = ctx->d_idx + (grp->g.idx_tiled ? i * rb * 64 : i * rb);
        float* d_out;
        bool out_host;
        if ((rc = stage_output(ctx, view.g, outs[i], n, &d_out, &out_host))) return rc;
        if ((rc = launch_gather(ctx, view, idx_i, d_out, nullptr, n))) return rc;
        if ((rc = finish_output(ctx, view.g, outs[i], n, out_host))) return rc;
    }
    return PIMDL_OK;
}

int pimdl_amm_run(pimdl_amm* a, const float* in, uint32_t n, float* out)
{
    int rc = check_run_args(a, in, out, n);
    if (rc || n == 0) return rc;
    Ctx* ctx = a->ctx;
    if ((rc = ensure(ctx, &ctx->d_idx, &ctx->idx_bytes, idx_buffer_bytes(a->g, n), "hipMalloc(index scratch)"))) return rc;
    auto run_rows = [&](const float* d_in, float* d_out, uint32_t tokens) -> int {
        int r = launch_ccs(ctx, a->g, d_in, a->d_centroids, ctx->d_idx, tokens);
        return r ? r : launch_gather(ctx, *a, ctx->d_idx, d_out, nullptr, tokens);
    };
    const bool in_host = !is_device_ptr(in), out_host = !is_device_ptr(out);
    if (in_host || out_host) return run_piped(ctx, a->g.K, a->g.M, in, in_host, out, out_host, n, run_rows);
    return run_rows(in, out, n);
}

int pimdl_amm_run_noalloc(pimdl_amm* a, const float* in_dev, uint32_t n, float* out_dev)
{
    int rc = check_run_args(a, in_dev, out_dev, n);
    if (rc) return rc;
    Ctx* ctx = a->ctx;
    if (!is_device_ptr(in_dev) || !is_device_ptr(out_dev))
        return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_run_noalloc: in and out must be device pointers (staging host buffers would allocate)");
    const size_t need = idx_buffer_bytes(a->g, n);
    if (need > (size_t)PIMDL_NOALLOC_SCRATCH_BYTES)
        return set_error(ctx, PIMDL_ERR_INVALID,
                         "pimdl_amm_run_noalloc: n=%u tokens x %u index bytes per token = %zu bytes of packed indices exceed the "
                         "fixed scratch of %u bytes; use pimdl_amm_run or a smaller batch", n, a->g.idx_row_bytes, need,
                         (unsigned)PIMDL_NOALLOC_SCRATCH_BYTES);
    if (n == 0) return PIMDL_OK;
    // Nothing in the scratch has to start at zero: the search kernel writes every index byte the gather reads,
    // padded codebooks included, and index bytes of tokens past n only reach accumulators that are never stored.
    uint8_t* d_idx = ctx->d_static_scratch;  // the device address from hipGetSymbolAddress, never the array's name
    if ((rc = launch_ccs(ctx, a->g, in_dev, a->d_centroids, d_idx, n))) return rc;
    return launch_gather(ctx, *a, d_idx, out_dev, nullptr, n);
}

int pimdl_amm_run_debug(pimdl_amm* a, const float* in, uint32_t n, float* out, uint16_t* idx_out, int32_t* acc_out)
{
    int rc = check_run_args(a, in, out, n);
    if (rc || n == 0) return rc;
    Ctx* ctx = a->ctx;
    const AmmGeom& g = a->g;
    if (acc_out && (a->desc.lut_dtype != PIMDL_LUT_I8 || a->grouped))
        return set_error(ctx, PIMDL_ERR_INVALID, "acc_out is only defined for int8 LUTs with one scale (scale_group 0)");
    const float* d_in;
    float* d_out;
    bool out_host;
    if ((rc = stage_input(ctx, g, in, n, &d_in))) return rc;
    if ((rc = stage_output(ctx, g, out, n, &d_out, &out_host))) return rc;
    if ((rc = ensure(ctx, &ctx->d_idx, &ctx->idx_bytes, idx_buffer_bytes(g, n), "hipMalloc(index scratch)"))) return rc;
    if (acc_out && (rc = ensure(ctx, &ctx->d_acc, &ctx->acc_bytes, (size_t)n * g.M * 4, "hipMalloc(acc scratch)"))) return rc;
    if (idx_out && (rc = ensure(ctx, &ctx->d_idx16, &ctx->idx16_bytes, (size_t)n * g.CB * 2, "hipMalloc(idx16 scratch)"))) return rc;
    if ((rc = launch_ccs(ctx, g, d_in, a->d_centroids, ctx->d_idx, n))) return rc;
    if ((rc = launch_gather(ctx, *a, ctx->d_idx, d_out, acc_out ? ctx->d_acc : nullptr, n))) return rc;
    if (idx_out) {
        if ((rc = launch_unpack_idx(ctx, g, ctx->d_idx, ctx->d_idx16, n, n, g.CB))) return rc;
        if ((rc = hip_check(ctx, hipMemcpyAsync(idx_out, ctx->d_idx16, (size_t)n * g.CB * 2, hipMemcpyDeviceToHost, ctx->stream), "D2H idx"))) return rc;
    }
    if (acc_out &&
        (rc = hip_check(ctx, hipMemcpyAsync(acc_out, ctx->d_acc, (size_t)n * g.M * 4, hipMemcpyDeviceToHost, ctx->stream), "D2H acc")))
        return rc;
    if ((rc = finish_output(ctx, g, out, n, out_host))) return rc;
    return hip_check(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
}

int pimdl_amm_profile(pimdl_amm* a, const float* in_dev, uint32_t n, float* out_dev, uint32_t warmup, uint32_t iters,
                      pimdl_amm_timing* timing)
{
    int rc = check_run_args(a, in_dev, out_dev, n);
    if (rc) return rc;
    Ctx* ctx = a->ctx;
    if (!timing || !iters || !n) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_profile: bad arguments");
    if (!is_device_ptr(in_dev) || !is_device_ptr(out_dev))
        return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_profile: in/out must be device pointers");
    if ((rc = ensure(ctx, &ctx->d_idx, &ctx->idx_bytes, idx_buffer_bytes(a->g, n), "hipMalloc(index scratch)"))) return rc;
    for (uint32_t i = 0; i < warmup; ++i) {
        if ((rc = launch_ccs(ctx, a->g, in_dev, a->d_centroids, ctx->d_idx, n))) return rc;
        if ((rc = launch_gather(ctx, *a, ctx->d_idx, out_dev, nullptr, n))) return rc;
    }
    float ms[3] = {0, 0, 0};
    for (int phase = 0; phase < 3; ++phase) {
        if ((rc = hip_check(ctx, hipEventRecord(ctx->ev[0], ctx->stream), "hipEventRecord"))) return rc;
        for (uint32_t i = 0; i < iters; ++i) {
            if (phase != 1 && (rc = launch_ccs(ctx, a->g, in_dev, a->d_centroids, ctx->d_idx, n))) return rc;
            if (phase != 0 && (rc = launch_gather(ctx, *a, ctx->d_idx, out_dev, nullptr, n))) return rc;
        }
        if ((rc = hip_check(ctx, hipEventRecord(ctx->ev[1], ctx->stream), "hipEventRecord"))) return rc;
        if ((rc = hip_check(ctx, hipEventSynchronize(ctx->ev[1]), "hipEventSynchronize"))) return rc;
        if ((rc = hip_check(ctx, hipEventElapsedTime(&ms[phase], ctx->ev[0], ctx->ev[1]), "hipEventElapsedTime"))) return rc;
    }
    timing->ccs_ms = ms[0] / iters;
    timing->gather_ms = ms[1] / iters;
    timing->total_ms = ms[2] / iters;
    return PIMDL_OK;
}

// shared tail of the two index_calculation entry points
static int index_calc_common(Ctx* ctx, const AmmGeom& g, const float* in, const float* d_cent, uint32_t n,
                             uint16_t* idx_out, uint32_t n_stile_size, uint32_t cb_mtile_size)
{
    if (!n_stile_size) n_stile_size = n;
    if (!cb_mtile_size) cb_mtile_size = g.CB;
    if (n % n_stile_size || g.CB % cb_mtile_size)
        return set_error(ctx, PIMDL_ERR_INVALID, "n_stile_size must divide n and cb_mtile_size must divide num_codebook");
    int rc;
    const float* d_in;
    if ((rc = stage_input(ctx, g, in, n, &d_in))) return rc;
    if ((rc = ensure(ctx, &ctx->d_idx, &ctx->idx_bytes, idx_buffer_bytes(g, n), "hipMalloc(index scratch)"))) return rc;
    if ((rc = ensure(ctx, &ctx->d_idx16, &ctx->idx16_bytes, (size_t)n * g.CB * 2, "hipMalloc(idx16 scratch)"))) return rc;
    if ((rc = launch_ccs(ctx, g, d_in, d_cent, ctx->d_idx, n))) return rc;
    if ((rc = launch_unpack_idx(ctx, g, ctx->d_idx, ctx->d_idx16, n, n_stile_size, cb_mtile_size))) return rc;
    if ((rc = hip_check(ctx, hipMemcpyAsync(idx_out, ctx->d_idx16, (size_t)n * g.CB * 2, hipMemcpyDeviceToHost, ctx->stream), "D2H idx"))) return rc;
    return hip_check(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
}

int pimdl_amm_index_calculation(pimdl_amm* a, const float* in, uint32_t n, uint16_t* idx_out, uint32_t n_stile_size,
                                uint32_t cb_mtile_size)
{
    int rc = check_run_args(a, in, idx_out, n);
    if (rc || n == 0) return rc;
    return index_calc_common(a->ctx, a->g, in, a->d_centroids, n, idx_out, n_stile_size, cb_mtile_size);
}

int pimdl_index_calculation(pimdl_ctx* ctx, const float* in, const float* centroids, uint32_t n, uint32_t K,
                            uint32_t v, uint32_t C, uint16_t* idx_out, uint32_t n_stile_size, uint32_t cb_mtile_size)
{
    if (!ctx) return PIMDL_ERR_INVALID;
    if (!in || !centroids || !idx_out) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_index_calculation: null buffer");
    int rc = activate(ctx);
    if (rc || n == 0) return rc;
    pimdl_amm_desc d;
    memset(&d, 0, sizeof(d));
    d.max_n = n; d.input_feature_len = K; d.sub_vec_len = v; d.num_centroid = C; d.output_feature_len = 1;
    d.lut_dtype = PIMDL_LUT_I8;
    AmmGeom g;
    memset(&g, 0, sizeof(g));
    std::string why;
    if (!plan_geometry(d, ctx->prop.multiProcessorCount, &g, &why)) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_index_calculation: %s", why.c_str());
    const size_t cent_bytes = (size_t)g.CB * C * v * sizeof(float);
    if ((rc = ensure(ctx, &ctx->d_cent, &ctx->cent_bytes, ccs_centroid_bytes(g), "hipMalloc(centroid scratch)"))) return rc;
    if ((rc = hip_check(ctx, hipMemcpyAsync(ctx->d_cent, centroids, cent_bytes, hipMemcpyHostToDevice, ctx->stream), "H2D centroids"))) return rc;
    if ((rc = launch_ccs_prep(ctx, g, ctx->d_cent))) return rc;
    return index_calc_common(ctx, g, in, ctx->d_cent, n, idx_out, n_stile_size, cb_mtile_size);
}

static int resolve_tiling(Ctx* ctx, const AmmGeom& g, uint32_t n, const pimdl_tiling* t, pimdl_tiling* r, bool* out_identity)
{
    r->n_stile_size = (t && t->n_stile_size) ? t->n_stile_size : n;
    r->cb_mtile_size = (t && t->cb_mtile_size) ? t->cb_mtile_size : g.CB;
    r->feature_stile_size = (t && t->feature_stile_size) ? t->feature_stile_size : g.M;
    r->feature_mtile_size = (t && t->feature_mtile_size) ? t->feature_mtile_size : r->feature_stile_size;
    if (n % r->n_stile_size || g.CB % r->cb_mtile_size || g.M % r->feature_stile_size ||
        r->feature_stile_size % r->feature_mtile_size)
        return set_error(ctx, PIMDL_ERR_INVALID,
                         "tiling does not divide the shape (n=%u ns=%u, CB=%u cm=%u, M=%u fs=%u fm=%u)", n,
                         r->n_stile_size, g.CB, r->cb_mtile_size, g.M, r->feature_stile_size, r->feature_mtile_size);
    *out_identity = r->n_stile_size == n && r->feature_stile_size == g.M && r->feature_mtile_size == g.M;
    return PIMDL_OK;
}

// gather into `out` (host or device) in the requested output order
static int gather_to(Amm* a, uint32_t n, float* out, const pimdl_tiling& til, bool out_identity)
{
    Ctx* ctx = a->ctx;
    const AmmGeom& g = a->g;
    int rc;
    float* d_out;
    bool out_host;
    if ((rc = stage_output(ctx, g, out, n, &d_out, &out_host))) return rc;
    if (out_identity) {
        if ((rc = launch_gather(ctx, *a, ctx->d_idx, d_out, nullptr, n))) return rc;
    } else {
        if ((rc = ensure(ctx, &ctx->d_tmp, &ctx->tmp_bytes, (size_t)n * g.M * 4, "hipMalloc(row-major scratch)"))) return rc;
        if ((rc = launch_gather(ctx, *a, ctx->d_idx, ctx->d_tmp, nullptr, n))) return rc;
        if ((rc = launch_retile_output(ctx, ctx->d_tmp, d_out, n, g.M, til.n_stile_size, til.feature_stile_size,
                                       til.feature_mtile_size)))
            return rc;
    }
    return finish_output(ctx, g, out, n, out_host);
}

int pimdl_amm_run_tiled(pimdl_amm* a, const float* in, uint32_t n, float* out, const pimdl_tiling* tiling)
{
    int rc = check_run_args(a, in, out, n);
    if (rc || n == 0) return rc;
    Ctx* ctx = a->ctx;
    pimdl_tiling til;
    bool ident;
    if ((rc = resolve_tiling(ctx, a->g, n, tiling, &til, &ident))) return rc;
    if (ident) return pimdl_amm_run(a, in, n, out);  // row-major in and out (the search never sees cb_mtile_size)
    const float* d_in;
    if ((rc = stage_input(ctx, a->g, in, n, &d_in))) return rc;
    if ((rc = ensure(ctx, &ctx->d_idx, &ctx->idx_bytes, idx_buffer_bytes(a->g, n), "hipMalloc(index scratch)"))) return rc;
    if ((rc = launch_ccs(ctx, a->g, d_in, a->d_centroids, ctx->d_idx, n))) return rc;
    return gather_to(a, n, out, til, ident);
}

int pimdl_amm_run_breakdown(pimdl_amm* a, const float* in, uint32_t n, float* out, const pimdl_tiling* tiling,
                            pimdl_amm_breakdown* acc)
{
    int rc = check_run_args(a, in, out, n);
    if (rc) return rc;
    Ctx* ctx = a->ctx;
    if (!acc) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_amm_run_breakdown: null result pointer");
    if (n == 0) return PIMDL_OK;
    pimdl_tiling til;
    bool ident;
    if ((rc = resolve_tiling(ctx, a->g, n, tiling, &til, &ident))) return rc;
    auto now = [] { return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count(); };
    auto sync = [&] { return hip_check(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize"); };
    // one phase after the other, each waited for, as the reference's own breakdown does (dpu_sync between phases)
    if ((rc = sync())) return rc;
    const double t0 = now();
    const float* d_in;
    if ((rc = stage_input(ctx, a->g, in, n, &d_in))) return rc;
    if ((rc = ensure(ctx, &ctx->d_idx, &ctx->idx_bytes, idx_buffer_bytes(a->g, n), "hipMalloc(index scratch)"))) return rc;
    float* d_out;
    bool out_host;
    if ((rc = stage_output(ctx, a->g, out, n, &d_out, &out_host))) return rc;
    if (!ident && (rc = ensure(ctx, &ctx->d_tmp, &ctx->tmp_bytes, (size_t)n * a->g.M * 4, "hipMalloc(row-major scratch)"))) return rc;
    if ((rc = sync())) return rc;
    const double t1 = now();
    if ((rc = launch_ccs(ctx, a->g, d_in, a->d_centroids, ctx->d_idx, n))) return rc;
    if ((rc = sync())) return rc;
    const double t2 = now();
    if ((rc = launch_gather(ctx, *a, ctx->d_idx, ident ? d_out : ctx->d_tmp, nullptr, n))) return rc;
    if (!ident && (rc = launch_retile_output(ctx, ctx->d_tmp, d_out, n, a->g.M, til.n_stile_size, til.feature_stile_size,
                                             til.feature_mtile_size)))
        return rc;
    if ((rc = sync())) return rc;
    const double t3 = now();
    if ((rc = finish_output(ctx, a->g, out, n, out_host))) return rc;
    if ((rc = sync())) return rc;
    const double t4 = now();
    acc->h2d_s += t1 - t0;
    acc->search_s += t2 - t1;
    acc->gather_s += t3 - t2;
    acc->d2h_s += t4 - t3;
    return PIMDL_OK;
}

int pimdl_lut_gather_tiled(pimdl_amm* a, const uint16_t* idx, uint32_t n, float* out, const pimdl_tiling* tiling)
{
    int rc = check_run_args(a, idx, out, n);
    if (rc || n == 0) return rc;
    Ctx* ctx = a->ctx;
    const AmmGeom& g = a->g;
    pimdl_tiling til;
    bool ident;
    if ((rc = resolve_tiling(ctx, g, n, tiling, &til, &ident))) return rc;
    // Every entry must be a centroid id.  The kernels index LDS tables with it, and a buffer that pim_lut has
    // already rewritten in place (pim_lut_host.cpp:40-104 turns ids into table offsets) would otherwise be
    // gathered from rows of other codebooks without any error.
    {
        const size_t count = (size_t)n * g.CB;
        uint32_t worst = 0;
        for (size_t i = 0; i < count; ++i) worst = idx[i] > worst ? idx[i] : worst;
        if (worst >= g.C) {
            size_t i = 0;
            while (idx[i] < g.C) ++i;
            const size_t ns = til.n_stile_size, cm = til.cb_mtile_size;
            const size_t in_stile = i % (ns * g.CB), in_mtile = in_stile % (ns * cm);
            const size_t tok = i / (ns * g.CB) * ns + in_mtile / cm, cb = in_stile / (ns * cm) * cm + in_mtile % cm;
            return set_error(ctx, PIMDL_ERR_INVALID,
                             "index buffer entry %zu (token %zu, codebook %zu) is %u: not a centroid id below num_centroid = %u",
                             i, tok, cb, (unsigned)idx[i], g.C);
        }
    }
    if ((rc = ensure(ctx, &ctx->d_idx, &ctx->idx_bytes, idx_buffer_bytes(g, n), "hipMalloc(index scratch)"))) return rc;
    if ((rc = ensure(ctx, &ctx->d_idx16, &ctx->idx16_bytes, (size_t)n * g.CB * 2, "hipMalloc(idx16 scratch)"))) return rc;
    if ((rc = hip_check(ctx, hipMemcpyAsync(ctx->d_idx16, idx, (size_t)n * g.CB * 2, hipMemcpyHostToDevice, ctx->stream), "H2D idx"))) return rc;
    if ((rc = launch_pack_idx(ctx, g, ctx->d_idx16, ctx->d_idx, n, til.n_stile_size, til.cb_mtile_size))) return rc;
    return gather_to(a, n, out, til, ident);
}

int pimdl_lut_gather(pimdl_amm* a, const uint16_t* idx, uint32_t n, float* out)
{
    return pimdl_lut_gather_tiled(a, idx, n, out, nullptr);
}

int pimdl_lutgen(pimdl_ctx* ctx, const float* centroids, const float* weight, uint32_t CB, uint32_t C, uint32_t v,
                 uint32_t M, uint32_t lut_dtype, uint32_t scale_group, void* lut_out, float* scales_out)
{
    return pimdl_lutgen_mode(ctx, centroids, weight, CB, C, v, M, lut_dtype, scale_group, PIMDL_LUTGEN_MFMA, lut_out, scales_out);
}

int pimdl_lutgen_mode(pimdl_ctx* ctx, const float* centroids, const float* weight, uint32_t CB, uint32_t C, uint32_t v,
                      uint32_t M, uint32_t lut_dtype, uint32_t scale_group, uint32_t mode, void* lut_out, float* scales_out)
{
    if (!ctx) return PIMDL_ERR_INVALID;
    if (mode != PIMDL_LUTGEN_MFMA && mode != PIMDL_LUTGEN_ORDERED) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_lutgen: unknown mode");
    if (!centroids || !weight || !lut_out) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_lutgen: null argument");
    if (!CB || !C || !v || !M) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_lutgen: zero-sized dimension");
    if (lut_dtype != PIMDL_LUT_I8 && lut_dtype != PIMDL_LUT_F32) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_lutgen: unknown lut_dtype");
    if (lut_dtype == PIMDL_LUT_I8 && !scales_out) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_lutgen: scales_out is null");
    if (CB > 65535) return set_error(ctx, PIMDL_ERR_UNSUPPORTED, "pimdl_lutgen: more than 65535 codebooks");
    int rc = activate(ctx);
    if (rc) return rc;
    const size_t cent_bytes = (size_t)CB * C * v * 4, w_bytes = (size_t)CB * v * M * 4, lut_elems = (size_t)CB * C * M;
    const uint32_t ngroups = scale_group ? (CB + scale_group - 1) / scale_group : 1;
    float *d_cent = nullptr, *d_w = nullptr, *d_lut = nullptr, *d_scales = nullptr;
    int8_t* d_q = nullptr;
    rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&d_cent), cent_bytes), "hipMalloc(lutgen centroids)");
    if (!rc) rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&d_w), w_bytes), "hipMalloc(lutgen weight)");
    if (!rc) rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&d_lut), lut_elems * 4), "hipMalloc(lutgen lut)");
    if (!rc) rc = hip_check(ctx, hipMemcpyAsync(d_cent, centroids, cent_bytes, hipMemcpyHostToDevice, ctx->stream), "H2D centroids");
    if (!rc) rc = hip_check(ctx, hipMemcpyAsync(d_w, weight, w_bytes, hipMemcpyHostToDevice, ctx->stream), "H2D weight");
    if (!rc) rc = launch_lutgen_f32(ctx, d_cent, d_w, d_lut, CB, C, v, M, mode == PIMDL_LUTGEN_ORDERED);
    if (!rc && lut_dtype == PIMDL_LUT_F32) {
        rc = hip_check(ctx, hipMemcpyAsync(lut_out, d_lut, lut_elems * 4, hipMemcpyDeviceToHost, ctx->stream), "D2H lut");
    } else if (!rc) {
        rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&d_q), lut_elems), "hipMalloc(lutgen q)");
        if (!rc) rc = hip_check(ctx, hipMalloc(reinterpret_cast<void**>(&d_scales), sizeof(float) * ngroups), "hipMalloc(lutgen scales)");
        if (!rc) rc = launch_lut_quant(ctx, d_lut, d_q, d_scales, CB, C, M, scale_group);
        if (!rc) rc = hip_check(ctx, hipMemcpyAsync(lut_out, d_q, lut_elems, hipMemcpyDeviceToHost, ctx->stream), "D2H lut");
        if (!rc) rc = hip_check(ctx, hipMemcpyAsync(scales_out, d_scales, sizeof(float) * ngroups, hipMemcpyDeviceToHost, ctx->stream), "D2H scales");
    }
    if (!rc) rc = hip_check(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    else (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(d_cent);
    (void)hipFree(d_w);
    (void)hipFree(d_lut);
    (void)hipFree(d_q);
    (void)hipFree(d_scales);
    return rc;
}

int pimdl_get_device_info(pimdl_ctx* ctx, pimdl_device_info* info)
{
    if (!ctx || !info) return PIMDL_ERR_INVALID;
    memset(info, 0, sizeof(*info));
    strncpy(info->name, ctx->prop.name, sizeof(info->name) - 1);
    strncpy(info->arch, ctx->prop.gcnArchName, sizeof(info->arch) - 1);
    info->compute_units = ctx->prop.multiProcessorCount;
    info->clock_khz = ctx->prop.clockRate;
    info->lds_bytes_per_cu = (uint32_t)ctx->prop.maxSharedMemoryPerMultiProcessor;
    info->hbm_bytes = ctx->prop.totalGlobalMem;
    return PIMDL_OK;
}

int pimdl_amm_last_gather_kernel(const pimdl_amm* a, char* name, size_t len)
{
    if (!a || !name || len == 0) return PIMDL_ERR_INVALID;
    strncpy(name, a->last_gather, len - 1);
    name[len - 1] = 0;
    return PIMDL_OK;
}

int pimdl_amm_get_geometry(const pimdl_amm* a, pimdl_amm_geometry* out)
{
    if (!a || !out) return PIMDL_ERR_INVALID;
    const AmmGeom& g = a->g;
    out->num_codebook = g.CB;
    out->num_codebook_padded = g.CB_pad;
    out->idx_bits = g.idx_bits;
    out->idx_row_bytes = g.idx_row_bytes;
    out->col_block = g.col_block;
    out->row_pitch = g.row_pitch;
    // the gather launcher picks among instances of its kernel by the batch it is given: report the last launch's
    // shape once there has been one, the plan's defaults before
    const bool ran = a->last_threads != 0;
    out->cb_per_slice = ran ? a->last_cb_per_slice : g.cb_per_slice;
    out->lds_bytes = ran ? a->last_lds_bytes : g.gather_lds_bytes;
    out->tokens_per_wg = ran ? a->last_tokens_per_wg : g.tokens_per_wg;
    out->gather_threads = ran ? a->last_threads : g.gather_threads;
    out->ccs_tokens_per_wg = 64;
    out->ccs_cb_per_wg = g.ccs_cb_per_wg;
    out->ccs_threads = 256;
    out->ccs_lds_bytes = g.ccs_lds_bytes;
    return PIMDL_OK;
}

int pimdl_attention(pimdl_ctx* ctx, const float* q, const float* k, const float* v, float* out, uint32_t batch,
                    uint32_t seq, uint32_t heads, uint32_t head_dim, uint32_t in_stride, uint32_t out_stride, float scale)
{
    if (!ctx) return PIMDL_ERR_INVALID;
    if (!q || !k || !v || !out) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_attention: null buffer");
    if (head_dim != 64) return set_error(ctx, PIMDL_ERR_UNSUPPORTED, "pimdl_attention: head_dim=%u (only 64 is built)", head_dim);
    if (batch > 65535 || heads > 65535) return set_error(ctx, PIMDL_ERR_UNSUPPORTED, "pimdl_attention: batch and heads must be below 65536");
    if ((uint64_t)heads * 64 > in_stride || (uint64_t)heads * 64 > out_stride || in_stride % 4 || out_stride % 4)
        return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_attention: strides must hold heads*64 floats and be multiples of 4");
    if (!is_device_ptr(q) || !is_device_ptr(k) || !is_device_ptr(v) || !is_device_ptr(out))
        return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_attention: q, k, v and out must be device pointers");
    if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
         reinterpret_cast<uintptr_t>(out)) & 15)
        return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_attention: pointers must be 16-byte aligned");
    int rc = activate(ctx);
    if (rc) return rc;
    return launch_attention_hd64(ctx, q, k, v, out, batch, seq, heads, in_stride, out_stride, scale);
}

int pimdl_layer_norm(pimdl_ctx* ctx, const float* x, const float* weight, const float* bias, const float* residual,
                     float* out, uint32_t n, uint32_t d, float eps)
{
    if (!ctx) return PIMDL_ERR_INVALID;
    if (!x || !weight || !bias || !out) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_layer_norm: null buffer");
    if (d == 0) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_layer_norm: zero-sized row");
    int rc = activate(ctx);
    if (rc || n == 0) return rc;
    // every buffer may be a host or a device pointer; host buffers go through temporary device copies
    const size_t row_bytes = (size_t)d * sizeof(float), mat_bytes = (size_t)n * row_bytes;
    struct Tmp {
        void* p = nullptr;
        ~Tmp() { if (p) (void)hipFree(p); }
    } tx, tw, tb, tr, to;
    auto to_dev = [&](const float* h, size_t bytes, Tmp& t, const float** dptr) -> int {
        if (is_device_ptr(h)) {
            *dptr = h;
            return PIMDL_OK;
        }
        int r = hip_check(ctx, hipMalloc(&t.p, bytes), "hipMalloc(layer_norm staging)");
        if (!r) r = hip_check(ctx, hipMemcpyAsync(t.p, h, bytes, hipMemcpyHostToDevice, ctx->stream), "H2D layer_norm");
        *dptr = static_cast<const float*>(t.p);
        return r;
    };
    const float *dx, *dw, *db, *dr = nullptr;
    if ((rc = to_dev(x, mat_bytes, tx, &dx))) return rc;
    if ((rc = to_dev(weight, row_bytes, tw, &dw))) return rc;
    if ((rc = to_dev(bias, row_bytes, tb, &db))) return rc;
    if (residual && (rc = to_dev(residual, mat_bytes, tr, &dr))) return rc;
    const bool out_host = !is_device_ptr(out);
    float* dout = out;
    if (out_host) {
        if ((rc = hip_check(ctx, hipMalloc(&to.p, mat_bytes), "hipMalloc(layer_norm staging)"))) return rc;
        dout = static_cast<float*>(to.p);
    }
    if ((rc = launch_layer_norm(ctx, dx, dw, db, dr, dout, n, d, eps))) return rc;
    if (out_host) {
        if ((rc = hip_check(ctx, hipMemcpyAsync(out, dout, mat_bytes, hipMemcpyDeviceToHost, ctx->stream), "D2H layer_norm"))) return rc;
    }
    if (out_host || tx.p || tw.p || tb.p || tr.p)  // temporaries die at return
        return hip_check(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    return PIMDL_OK;
}

int pimdl_diag_bandwidth(pimdl_ctx* ctx, uint64_t bytes, float* copy_gbps, float* lds_gbps)
{
    if (!ctx) return PIMDL_ERR_INVALID;
    int rc = activate(ctx);
    if (rc) return rc;
    return launch_diag(ctx, bytes, copy_gbps, lds_gbps);
}

int pimdl_diag_host_copy(pimdl_ctx* ctx, uint64_t bytes, float* to_pinned_gbps, float* from_pinned_gbps, float* h2d_gbps,
                         float* d2h_gbps)
{
    if (!ctx) return PIMDL_ERR_INVALID;
    if (!bytes || !to_pinned_gbps || !from_pinned_gbps || !h2d_gbps || !d2h_gbps)
        return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_diag_host_copy: bad arguments");
    int rc = activate(ctx);
    if (rc) return rc;
    void *pinned = nullptr, *dev = nullptr;
    char* pageable = static_cast<char*>(malloc(bytes));
    if (!pageable) return set_error(ctx, PIMDL_ERR_NOMEM, "pimdl_diag_host_copy: out of host memory");
    memset(pageable, 1, bytes);
    rc = hip_check(ctx, hipHostMalloc(&pinned, bytes, hipHostMallocDefault), "hipHostMalloc(diag)");
    if (!rc) rc = hip_check(ctx, hipMalloc(&dev, bytes), "hipMalloc(diag)");
    auto now = [] { return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count(); };
    constexpr int REPS = 5;
    auto rate = [&](auto fn, float* out) {
        fn();
        const double t0 = now();
        for (int i = 0; i < REPS && !rc; ++i) fn();
        *out = (float)((double)bytes * REPS / (now() - t0) / 1e9);
    };
    if (!rc) {
        rate([&] { parallel_copy(pinned, pageable, bytes); }, to_pinned_gbps);
        rate([&] { parallel_copy(pageable, pinned, bytes); }, from_pinned_gbps);
        rate([&] {
            rc = hip_check(ctx, hipMemcpyAsync(dev, pinned, bytes, hipMemcpyHostToDevice, ctx->stream), "H2D diag");
            if (!rc) rc = hip_check(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
        }, h2d_gbps);
        rate([&] {
            rc = hip_check(ctx, hipMemcpyAsync(pinned, dev, bytes, hipMemcpyDeviceToHost, ctx->stream), "D2H diag");
            if (!rc) rc = hip_check(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
        }, d2h_gbps);
    }
    if (pinned) (void)hipHostFree(pinned);
    (void)hipFree(dev);
    free(pageable);
    return rc;
}

int pimdl_diag_mfma_error(pimdl_ctx* ctx, uint32_t trials, float* max_err_u)
{
    if (!ctx) return PIMDL_ERR_INVALID;
    if (!max_err_u) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_diag_mfma_error: null result pointer");
    int rc = activate(ctx);
    if (rc) return rc;
    return launch_diag_mfma_error(ctx, trials, false, max_err_u);
}

int pimdl_diag_mfma_error_crafted(pimdl_ctx* ctx, float* max_err_u)
{
    if (!ctx) return PIMDL_ERR_INVALID;
    if (!max_err_u) return set_error(ctx, PIMDL_ERR_INVALID, "pimdl_diag_mfma_error_crafted: null result pointer");
    int rc = activate(ctx);
    if (rc) return rc;
    return launch_diag_mfma_error(ctx, 0, true, max_err_u);
}

}  // extern "C"
