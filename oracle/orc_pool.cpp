// CPU oracle (test infrastructure only): a persistent row-chunked worker pool
// and the threaded GEMV used as the timed "restated cera AVX2 path" baseline.
// Threading model follows cera's decode RowPool (cera/src/backend/threadpool.rs:
// 1-80): long-lived workers, each handed a disjoint contiguous row range, no
// reduction between workers (cera/src/backend/cpu.rs:387-391).
#include "orc_common.h"

#include <atomic>
#include <condition_variable>
#include <functional>
#include <mutex>
#include <thread>
#include <vector>

namespace {
struct Pool {
    std::vector<std::thread> workers;
    std::mutex mu;
    std::condition_variable cv_start, cv_done;
    std::function<void(int)> job;
    uint64_t generation = 0;
    int pending = 0;
    bool stop = false;
    int n = 1;

    explicit Pool(int n_threads) : n(n_threads < 1 ? 1 : n_threads) {
        for (int t = 1; t < n; ++t) workers.emplace_back([this, t] { loop(t); });
    }
    ~Pool() {
        {
            std::lock_guard<std::mutex> lk(mu);
            stop = true;
            ++generation;
        }
        cv_start.notify_all();
        for (auto& w : workers) w.join();
    }
    void loop(int tid) {
        uint64_t seen = 0;
        for (;;) {
            std::function<void(int)> j;
            {
                std::unique_lock<std::mutex> lk(mu);
                cv_start.wait(lk, [&] { return generation != seen; });
                seen = generation;
                if (stop) return;
                j = job;
            }
            j(tid);
            {
                std::lock_guard<std::mutex> lk(mu);
                if (--pending == 0) cv_done.notify_one();
            }
        }
    }
    void run(const std::function<void(int)>& f) {
        if (n == 1) { f(0); return; }
        {
            std::lock_guard<std::mutex> lk(mu);
            job = f;
            pending = n - 1;
            ++generation;
        }
        cv_start.notify_all();
        f(0);
        std::unique_lock<std::mutex> lk(mu);
        cv_done.wait(lk, [&] { return pending == 0; });
    }
};
}  // namespace

void* orc_pool_create(int n_threads) { return new Pool(n_threads); }
void orc_pool_destroy(void* p) { delete static_cast<Pool*>(p); }
int orc_pool_threads(void* p) { return static_cast<Pool*>(p)->n; }
void orc_pool_run(void* p, void (*fn)(int, int, void*), void* arg) {
    Pool* pool = static_cast<Pool*>(p);
    int n = pool->n;
    pool->run([=](int tid) { fn(tid, n, arg); });
}

int orc_gemv_mt(void* pool, uint32_t dtype, const void* wv, const float* x, float* y, uint64_t m,
                uint64_t k) {
    Pool* p = static_cast<Pool*>(pool);
    uint64_t rb = orc_row_bytes(dtype, k);
    if (rb == 0) return -1;
    bool int8 = dtype == ORC_Q4_0 || dtype == ORC_Q8_0 || dtype == ORC_Q4_1 || dtype == ORC_Q4_K ||
                dtype == ORC_Q6_K;
    if (!int8) return orc_gemv(dtype, wv, x, y, m, k, 0);
    std::vector<float> xs(k / 32);
    std::vector<int8_t> xq(k);
    orc_quantize_q8_0(x, k, xs.data(), xq.data());  // once per call, as cpu.rs:787-790
    int variant = orc_have_avx2() ? 1 : 0;
    const uint8_t* w = static_cast<const uint8_t*>(wv);
    int nt = p->n;
    std::atomic<int> rc{0};
    p->run([&](int tid) {
        uint64_t r0 = m * uint64_t(tid) / uint64_t(nt), r1 = m * uint64_t(tid + 1) / uint64_t(nt);
        if (r1 > r0) {
            int e = orc_gemm_preq(dtype, w + r0 * rb, xs.data(), xq.data(), y + r0, r1 - r0, 1, k, variant);
            if (e) rc = e;
        }
    });
    return rc;
}
