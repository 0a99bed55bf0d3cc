// A few host threads that copy memory: the streamed pipeline uses them to move host arrays that
// are not pinned (ordinary CPU tensors) into pinned bounce buffers while earlier chunks are on the
// host link.  Plain C++ threads; nothing here touches the GPU runtime.
#pragma once

#include <algorithm>
#include <condition_variable>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <deque>
#include <mutex>
#include <thread>
#include <vector>

namespace rt {

class CopyPool {
public:
    // The copies submitted under one group are waited for together.
    struct Group {
        size_t left = 0;  // guarded by the pool's mutex
    };

    explicit CopyPool(unsigned n_threads) {
        for (unsigned i = 0; i < n_threads; ++i) workers_.emplace_back([this] { run(); });
    }
    CopyPool(const CopyPool&) = delete;
    CopyPool& operator=(const CopyPool&) = delete;
    ~CopyPool() {
        {
            std::lock_guard<std::mutex> lk(mu_);
            stop_ = true;
        }
        work_cv_.notify_all();
        for (auto& t : workers_) t.join();
    }

    // Queues dst[0, bytes) = src[0, bytes) in slices that the workers share.
    void submit(Group* g, void* dst, const void* src, size_t bytes) {
        if (bytes == 0) return;
        constexpr size_t kSlice = 2u << 20;
        {
            std::lock_guard<std::mutex> lk(mu_);
            for (size_t off = 0; off < bytes; off += kSlice) {
                jobs_.push_back(Job{g, (uint8_t*)dst + off, (const uint8_t*)src + off, std::min(kSlice, bytes - off)});
                ++g->left;
            }
        }
        work_cv_.notify_all();
    }

    // Returns when every copy submitted under g has been made.
    void wait(Group* g) {
        std::unique_lock<std::mutex> lk(mu_);
        done_cv_.wait(lk, [g] { return g->left == 0; });
    }

private:
    struct Job {
        Group* group;
        uint8_t* dst;
        const uint8_t* src;
        size_t bytes;
    };

    void run() {
        std::unique_lock<std::mutex> lk(mu_);
        for (;;) {
            work_cv_.wait(lk, [this] { return stop_ || !jobs_.empty(); });
            if (jobs_.empty()) return;  // stop_ with nothing left to do
            const Job j = jobs_.front();
            jobs_.pop_front();
            lk.unlock();
            memcpy(j.dst, j.src, j.bytes);
            lk.lock();
            if (--j.group->left == 0) done_cv_.notify_all();
        }
    }

    std::mutex mu_;
    std::condition_variable work_cv_, done_cv_;
    std::deque<Job> jobs_;
    std::vector<std::thread> workers_;
    bool stop_ = false;
};

}  // namespace rt
