// The process-wide host thread pool (host_pool.h).  Plain host code.
#include "host_pool.h"

#include <immintrin.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include <condition_variable>
#include <mutex>
#include <thread>
#include <vector>

namespace pimdl {
namespace {

class Pool final : public HostPool {
public:
    explicit Pool(int width) : width_(width < 1 ? 1 : width)
    {
        for (int i = 1; i < width_; ++i) workers_.emplace_back([this] { loop(); });
    }
    ~Pool() override
    {
        {
            std::lock_guard<std::mutex> lock(mu_);
            stop_ = true;
        }
        wake_.notify_all();
        for (auto& t : workers_) t.join();
    }
    int width() const override { return width_; }

    void run(int pieces, const std::function<void(int)>& fn) override
    {
        if (pieces <= 0) return;
        if (pieces == 1 || width_ == 1) {
            for (int i = 0; i < pieces; ++i) fn(i);
            return;
        }
        std::lock_guard<std::mutex> turn(job_mu_);  // one job at a time
        uint64_t gen;
        {
            std::lock_guard<std::mutex> lock(mu_);
            fn_ = &fn;
            pieces_ = pieces;
            next_ = 0;
            left_ = pieces;
            gen = ++generation_;
        }
        wake_.notify_all();
        work(gen);  // the caller takes pieces too
        std::unique_lock<std::mutex> lock(mu_);
        done_.wait(lock, [this] { return left_ == 0; });
        fn_ = nullptr;
    }

private:
    // Takes pieces of job `gen` until none are left.  Pieces are handed out under the mutex (a job has at most
    // `width` of them), so a thread that is late for its job can never take a piece of the next one by mistake.
    void work(uint64_t gen)
    {
        for (;;) {
            int i;
            const std::function<void(int)>* fn;
            {
                std::lock_guard<std::mutex> lock(mu_);
                if (gen != generation_ || next_ >= pieces_) return;
                i = next_++;
                fn = fn_;
            }
            (*fn)(i);
            std::lock_guard<std::mutex> lock(mu_);
            if (--left_ == 0) done_.notify_all();
        }
    }
    void loop()
    {
        uint64_t seen = 0;
        for (;;) {
            {
                std::unique_lock<std::mutex> lock(mu_);
                wake_.wait(lock, [&] { return stop_ || generation_ != seen; });
                if (stop_) return;
                seen = generation_;
            }
            work(seen);
        }
    }

    const int width_;
    std::vector<std::thread> workers_;
    std::mutex mu_, job_mu_;
    std::condition_variable wake_, done_;
    const std::function<void(int)>* fn_ = nullptr;
    int pieces_ = 0, left_ = 0, next_ = 0;
    uint64_t generation_ = 0;
    bool stop_ = false;
};

int pool_width()
{
    int w = 8;
    if (const char* e = getenv("PIMDL_COPY_THREADS")) w = atoi(e);
    const int hw = (int)std::thread::hardware_concurrency();
    if (hw > 0 && w > hw) w = hw;
    if (w < 1) w = 1;
    if (w > 64) w = 64;
    return w;
}

}  // namespace

HostPool& host_pool()
{
    static Pool pool(pool_width());
    return pool;
}

// memcpy for buffers that are not read again soon (staging buffers, outputs): streaming stores, so the
// destination's lines are not fetched before they are overwritten (a third less memory traffic than a copy
// through the caches) and do not evict what the caller works on.
static void stream_copy(char* dst, const char* src, size_t bytes)
{
    const size_t head = (64 - (reinterpret_cast<uintptr_t>(dst) & 63)) & 63;
    if (bytes < 4096 || head > bytes) {
        memcpy(dst, src, bytes);
        return;
    }
    memcpy(dst, src, head);
    dst += head, src += head, bytes -= head;
    const size_t blocks = bytes / 64;
    for (size_t i = 0; i < blocks; ++i) {
        _mm_prefetch(src + 1024, _MM_HINT_NTA);
        const __m128i a = _mm_loadu_si128(reinterpret_cast<const __m128i*>(src));
        const __m128i b = _mm_loadu_si128(reinterpret_cast<const __m128i*>(src + 16));
        const __m128i c = _mm_loadu_si128(reinterpret_cast<const __m128i*>(src + 32));
        const __m128i d = _mm_loadu_si128(reinterpret_cast<const __m128i*>(src + 48));
        _mm_stream_si128(reinterpret_cast<__m128i*>(dst), a);
        _mm_stream_si128(reinterpret_cast<__m128i*>(dst + 16), b);
        _mm_stream_si128(reinterpret_cast<__m128i*>(dst + 32), c);
        _mm_stream_si128(reinterpret_cast<__m128i*>(dst + 48), d);
        src += 64, dst += 64;
    }
    _mm_sfence();
    memcpy(dst, src, bytes - blocks * 64);
}

__attribute__((target("avx2"))) static void stream_copy_avx2(char* dst, const char* src, size_t bytes)
{
    const size_t head = (64 - (reinterpret_cast<uintptr_t>(dst) & 63)) & 63;
    if (bytes < 4096 || head > bytes) {
        memcpy(dst, src, bytes);
        return;
    }
    memcpy(dst, src, head);
    dst += head, src += head, bytes -= head;
    const size_t blocks = bytes / 128;
    for (size_t i = 0; i < blocks; ++i) {
        _mm_prefetch(src + 2048, _MM_HINT_NTA);
        _mm_prefetch(src + 2048 + 64, _MM_HINT_NTA);
        const __m256i a = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(src));
        const __m256i b = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(src + 32));
        const __m256i c = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(src + 64));
        const __m256i d = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(src + 96));
        _mm256_stream_si256(reinterpret_cast<__m256i*>(dst), a);
        _mm256_stream_si256(reinterpret_cast<__m256i*>(dst + 32), b);
        _mm256_stream_si256(reinterpret_cast<__m256i*>(dst + 64), c);
        _mm256_stream_si256(reinterpret_cast<__m256i*>(dst + 96), d);
        src += 128, dst += 128;
    }
    _mm_sfence();
    memcpy(dst, src, bytes - blocks * 128);
}

// how a piece is copied: 0 memcpy, 1 streaming stores (SSE2), 2 streaming stores (AVX2 where the CPU has it)
static int copy_mode()
{
    static const int mode = [] {
        const char* e = getenv("PIMDL_COPY_MODE");
        int m = e ? atoi(e) : 1;
        if (m == 2 && !__builtin_cpu_supports("avx2")) m = 1;
        return m;
    }();
    return mode;
}

static void copy_piece(char* dst, const char* src, size_t bytes)
{
    switch (copy_mode()) {
        case 1: stream_copy(dst, src, bytes); break;
        case 2: stream_copy_avx2(dst, src, bytes); break;
        default: memcpy(dst, src, bytes);
    }
}

void parallel_copy(void* dst, const void* src, size_t bytes)
{
    constexpr size_t SMALL = 256 * 1024;  // below this a hand-over to other threads costs more than it saves
    HostPool& pool = host_pool();
    if (bytes <= SMALL || pool.width() == 1) {
        copy_piece(static_cast<char*>(dst), static_cast<const char*>(src), bytes);
        return;
    }
    size_t pieces = (bytes + SMALL - 1) / SMALL;
    if (pieces > (size_t)pool.width()) pieces = pool.width();
    const size_t per = ((bytes + pieces - 1) / pieces + 63) & ~(size_t)63;
    pool.run((int)pieces, [&](int i) {
        const size_t off = (size_t)i * per;
        if (off >= bytes) return;
        const size_t len = off + per <= bytes ? per : bytes - off;
        copy_piece(static_cast<char*>(dst) + off, static_cast<const char*>(src) + off, len);
    });
}

}  // namespace pimdl
