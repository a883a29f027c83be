// Host <-> device staging for the BLAS entry points that take host pointers.
//
// The caller's matrices live in pageable memory.  Handing them to
// hipMemcpyAsync directly makes the runtime bounce them through its own small
// pinned buffer on one thread; here a few helper threads copy column ranges
// into a ring of pinned buffers while the DMA engine drains the previous ones,
// and results come back the same way in the other direction.  (The reference
// has no counterpart: its operands never leave host memory.  The ring plays
// the part of its static pack-buffer pool, ulmblas/auxiliary/memorypool.tcc.)
#pragma once

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <mutex>
#include <thread>
#include <vector>

namespace ulmgpu {

// A small fork-join pool: run(n, fn) calls fn(u) for u in [0, n) on the pool's
// threads and the calling thread, and returns when all units are done.
class CopyPool {
public:
    explicit CopyPool(int nthreads)
    {
        for (int i = 0; i + 1 < nthreads; ++i) workers_.emplace_back([this] { loop(); });
    }
    ~CopyPool()
    {
        {
            std::lock_guard<std::mutex> l(mu_);
            stop_ = true;
        }
        cv_.notify_all();
        for (auto &t : workers_) t.join();
    }
    int size() const { return (int)workers_.size() + 1; }

    void run(int units, const std::function<void(int)> &fn)
    {
        if (units <= 0) return;
        if (units == 1 || workers_.empty()) {
            for (int u = 0; u < units; ++u) fn(u);
            return;
        }
        {
            std::lock_guard<std::mutex> l(mu_);
            fn_ = &fn;
            units_ = units;
            next_.store(0);
            pending_ = (int)workers_.size();
            ++generation_;
        }
        cv_.notify_all();
        work();
        std::unique_lock<std::mutex> l(mu_);
        done_cv_.wait(l, [this] { return pending_ == 0; });
        fn_ = nullptr;
    }

private:
    void work()
    {
        for (;;) {
            const int u = next_.fetch_add(1);
            if (u >= units_) break;
            (*fn_)(u);
        }
    }
    void loop()
    {
        unsigned long seen = 0;
        for (;;) {
            {
                std::unique_lock<std::mutex> l(mu_);
                cv_.wait(l, [&] { return stop_ || generation_ != seen; });
                if (stop_) return;
                seen = generation_;
            }
            work();
            {
                std::lock_guard<std::mutex> l(mu_);
                if (--pending_ == 0) done_cv_.notify_one();
            }
        }
    }

    std::vector<std::thread> workers_;
    std::mutex mu_;
    std::condition_variable cv_, done_cv_;
    const std::function<void(int)> *fn_ = nullptr;
    int units_ = 0, pending_ = 0;
    std::atomic<int> next_{0};
    unsigned long generation_ = 0;
    bool stop_ = false;
};

// Copy a rows x cols window (bytes_per_row = rows * element size) between a
// strided matrix and a compact buffer, columns spread over the pool.
inline void copy_window_host(CopyPool &pool, char *dst, size_t dst_pitch, const char *src, size_t src_pitch,
                             size_t row_bytes, size_t cols)
{
    if (row_bytes == 0 || cols == 0) return;
    if (dst_pitch == row_bytes && src_pitch == row_bytes) {
        const size_t total = row_bytes * cols;
        const size_t unit = (size_t)1 << 20;
        const int units = (int)((total + unit - 1) / unit);
        pool.run(units, [&](int u) {
            const size_t off = (size_t)u * unit;
            memcpy(dst + off, src + off, std::min(unit, total - off));
        });
        return;
    }
    const size_t cols_per_unit = std::max<size_t>(1, ((size_t)1 << 20) / row_bytes);
    const int units = (int)((cols + cols_per_unit - 1) / cols_per_unit);
    pool.run(units, [&](int u) {
        const size_t c0 = (size_t)u * cols_per_unit, c1 = std::min(cols, c0 + cols_per_unit);
        for (size_t c = c0; c < c1; ++c) memcpy(dst + c * dst_pitch, src + c * src_pitch, row_bytes);
    });
}

// A ring of pinned buffers with one event each: a buffer is reusable once the
// DMA that last read (or wrote) it has completed.
class PinnedRing {
public:
    static constexpr size_t kChunkBytes = (size_t)32 << 20;

    bool init(int count)
    {
        if (!slots_.empty()) return true;
        for (int i = 0; i < count; ++i) {
            Slot s;
            if (hipHostMalloc(&s.ptr, kChunkBytes, hipHostMallocDefault) != hipSuccess) return fail();
            if (hipEventCreateWithFlags(&s.done, hipEventDisableTiming) != hipSuccess) {
                (void)hipHostFree(s.ptr);
                return fail();
            }
            slots_.push_back(s);
        }
        return true;
    }
    void release()
    {
        for (auto &s : slots_) {
            (void)hipEventDestroy(s.done);
            (void)hipHostFree(s.ptr);
        }
        slots_.clear();
        next_ = 0;
    }
    int count() const { return (int)slots_.size(); }
    // next buffer in ring order, after waiting for its previous use to finish
    hipError_t acquire(int &index)
    {
        index = next_;
        next_ = (next_ + 1) % (int)slots_.size();
        if (slots_[index].busy) {
            hipError_t e = hipEventSynchronize(slots_[index].done);
            if (e != hipSuccess) return e;
            slots_[index].busy = false;
        }
        return hipSuccess;
    }
    char *ptr(int i) { return static_cast<char *>(slots_[i].ptr); }
    hipEvent_t event(int i) { return slots_[i].done; }
    // mark buffer i as in use until everything enqueued on `stream` so far is done
    hipError_t mark(int i, hipStream_t stream)
    {
        slots_[i].busy = true;
        return hipEventRecord(slots_[i].done, stream);
    }
    hipError_t wait(int i)
    {
        if (!slots_[i].busy) return hipSuccess;
        hipError_t e = hipEventSynchronize(slots_[i].done);
        if (e == hipSuccess) slots_[i].busy = false;
        return e;
    }

private:
    struct Slot {
        void *ptr = nullptr;
        hipEvent_t done = nullptr;
        bool busy = false;
    };
    bool fail()
    {
        release();
        return false;
    }
    std::vector<Slot> slots_;
    int next_ = 0;
};

inline int staging_threads()
{
    if (const char *e = getenv("ULMBLAS_GPU_COPY_THREADS")) {
        const int v = atoi(e);
        if (v >= 1 && v <= 64) return v;
    }
    const unsigned hw = std::thread::hardware_concurrency();
    return (int)std::max(1u, std::min(8u, hw ? hw : 1u));
}

}  // namespace ulmgpu
