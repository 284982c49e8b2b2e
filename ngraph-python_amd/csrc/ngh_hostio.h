// Host <-> device copies of large buffers through pinned staging memory.
//
// The reference moves tensors with pycuda's GPUArray.set / .get on whatever NumPy array the
// caller holds (ngraph/transformers/gputransform.py:710-744, 807-871).  Such arrays are pageable,
// and a copy engine cannot read pageable memory: the runtime stages it itself, on one thread
// (measured here: 30 GB/s in, 10 GB/s out into a freshly allocated array, most of the latter
// spent taking the array's page faults one by one).  This file does the staging in the open:
// a ring of pinned buffers allocated once per context (hipHostMalloc: registering memory that
// already exists is refused on this platform), a few host threads that copy between the
// caller's array and a ring slot in parallel -- which also spreads the page faults of a fresh
// destination -- and the copy engine working on one slot while the threads fill or drain the
// next.  Everything here is host code.
#pragma once
#include <hip/hip_runtime.h>
#include <sys/mman.h>

#include <atomic>
#include <condition_variable>
#include <cstdint>
#include <cstring>
#include <mutex>
#include <thread>
#include <vector>

namespace ngh {

// A fixed crew of threads that copies one block of memory at a time, each thread a share.
class CopyCrew {
  public:
    explicit CopyCrew(int n) {
        for (int i = 0; i < n; ++i) threads_.emplace_back([this, i] { work(i); });
    }
    ~CopyCrew() {
        {
            std::lock_guard<std::mutex> lock(m_);
            stop_ = true;
            ++job_;
        }
        wake_.notify_all();
        for (auto& t : threads_) t.join();
    }
    int size() const { return (int)threads_.size(); }
    // dst[0, n) = src[0, n); returns when every share is done
    void copy(void* dst, const void* src, size_t n) {
        {
            std::lock_guard<std::mutex> lock(m_);
            dst_ = (char*)dst;
            src_ = (const char*)src;
            n_ = n;
            left_ = (int)threads_.size();
            ++job_;
        }
        wake_.notify_all();
        std::unique_lock<std::mutex> lock(m_);
        done_.wait(lock, [this] { return left_ == 0; });
    }

  private:
    void work(int me) {
        unsigned long long seen = 0;
        for (;;) {
            char* dst;
            const char* src;
            size_t n;
            {
                std::unique_lock<std::mutex> lock(m_);
                wake_.wait(lock, [&] { return job_ != seen; });
                seen = job_;
                if (stop_) return;
                dst = dst_; src = src_; n = n_;
            }
            // shares in whole pages, so that two threads never fault on the same page
            const size_t parts = threads_.size(), page = 4096;
            const size_t share = ((n + parts - 1) / parts + page - 1) / page * page;
            const size_t lo = std::min(n, share * me), hi = std::min(n, lo + share);
            if (hi > lo) memcpy(dst + lo, src + lo, hi - lo);
            {
                std::lock_guard<std::mutex> lock(m_);
                if (--left_ == 0) done_.notify_all();
            }
        }
    }
    std::vector<std::thread> threads_;
    std::mutex m_;
    std::condition_variable wake_, done_;
    char* dst_ = nullptr;
    const char* src_ = nullptr;
    size_t n_ = 0;
    int left_ = 0;
    unsigned long long job_ = 0;
    bool stop_ = false;
};

// The ring and the crew of one context.
struct HostStaging {
    static constexpr int kSlots = 4;
    size_t      slot_bytes = 0;
    char*       slot[kSlots] = {nullptr, nullptr, nullptr, nullptr};
    hipEvent_t  done[kSlots] = {nullptr, nullptr, nullptr, nullptr};
    CopyCrew*   crew = nullptr;

    hipError_t ensure(size_t bytes_per_slot, int threads) {
        if (slot[0]) return hipSuccess;
        for (int i = 0; i < kSlots; ++i) {
            hipError_t e = hipHostMalloc((void**)&slot[i], bytes_per_slot, hipHostMallocDefault);
            if (e == hipSuccess) e = hipEventCreateWithFlags(&done[i], hipEventDisableTiming);
            if (e != hipSuccess) { release(); return e; }
        }
        slot_bytes = bytes_per_slot;
        crew = new CopyCrew(threads);
        return hipSuccess;
    }
    void release() {
        delete crew;
        crew = nullptr;
        for (int i = 0; i < kSlots; ++i) {
            if (done[i]) (void)hipEventDestroy(done[i]);
            if (slot[i]) (void)hipHostFree(slot[i]);
            done[i] = nullptr;
            slot[i] = nullptr;
        }
        slot_bytes = 0;
    }

    // host -> device: the crew fills slot i while the copy engine empties slot i - 1
    hipError_t to_device(void* dev, const void* host, size_t bytes, hipStream_t stream) {
        size_t off = 0;
        for (int i = 0; off < bytes; ++i) {
            const int s = i % kSlots;
            const size_t n = std::min(slot_bytes, bytes - off);
            if (i >= kSlots) {
                hipError_t e = hipEventSynchronize(done[s]);       // the copy that last read this slot
                if (e != hipSuccess) return e;
            }
            crew->copy(slot[s], (const char*)host + off, n);
            hipError_t e = hipMemcpyAsync((char*)dev + off, slot[s], n, hipMemcpyHostToDevice, stream);
            if (e == hipSuccess) e = hipEventRecord(done[s], stream);
            if (e != hipSuccess) return e;
            off += n;
        }
        return hipStreamSynchronize(stream);
    }

    // device -> host: the copy engine fills the slots ahead, the crew drains them in order
    hipError_t to_host(void* host, const void* dev, size_t bytes, hipStream_t stream) {
        // A destination that has never been touched takes a page fault per 4 KiB, which is most of
        // what such a copy costs; asking for huge pages (a hint, and only where the system
        // offers them on request) turns 512 of them into one.
        {
            const uintptr_t huge = 2u << 20;
            const uintptr_t lo = ((uintptr_t)host + huge - 1) / huge * huge, hi = ((uintptr_t)host + bytes) / huge * huge;
            if (hi > lo) (void)madvise((void*)lo, hi - lo, MADV_HUGEPAGE);
        }
        const size_t chunks = (bytes + slot_bytes - 1) / slot_bytes;
        auto issue = [&](size_t c) {
            const size_t off = c * slot_bytes, n = std::min(slot_bytes, bytes - off);
            hipError_t e = hipMemcpyAsync(slot[c % kSlots], (const char*)dev + off, n, hipMemcpyDeviceToHost, stream);
            if (e == hipSuccess) e = hipEventRecord(done[c % kSlots], stream);
            return e;
        };
        for (size_t c = 0; c < chunks && c < (size_t)kSlots; ++c) {
            hipError_t e = issue(c);
            if (e != hipSuccess) return e;
        }
        for (size_t c = 0; c < chunks; ++c) {
            const size_t off = c * slot_bytes, n = std::min(slot_bytes, bytes - off);
            hipError_t e = hipEventSynchronize(done[c % kSlots]);
            if (e != hipSuccess) return e;
            crew->copy((char*)host + off, slot[c % kSlots], n);
            if (c + kSlots < chunks) {
                e = issue(c + kSlots);
                if (e != hipSuccess) return e;
            }
        }
        return hipStreamSynchronize(stream);
    }
};

}  // namespace ngh
