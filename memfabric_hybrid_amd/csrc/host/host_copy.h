// CPU-side copies between caller memory and the pinned staging ring.
//
// One core moves about 33 GB/s with memcpy, the host link about 55 GB/s, so a copy that is staged
// by the calling thread alone is bound by that core (reference counterpart: the staging copies of
// HostDataOpSDMA::CopyLH2GD / CopyGD2LH, src/hybm/csrc/data_operation/host/hybm_data_op_sdma.cpp:
// 111-221, which run on the calling thread).  Here helper threads take equal shares of every large
// set of pieces.
#ifndef MF_HOST_COPY_H
#define MF_HOST_COPY_H

#include <atomic>
#include <condition_variable>
#include <cstddef>
#include <cstdint>
#include <mutex>

namespace mf {

class HostCopyHelper {
public:
    // The one helper pool of the process.  Never destroyed: its threads sleep until the process
    // ends and touch nothing but this object.
    static HostCopyHelper &Instance();

    struct Task {
        void *dst;
        const void *src;
        size_t len;
    };

    // memcpy(dst, src, len).  kSplitMin bytes and more are shared with the helper threads when no
    // other caller is using them; the call returns when every byte has been copied.
    void Copy(void *dst, const void *src, size_t len)
    {
        const Task one{dst, src, len};
        CopySet(&one, 1);
    }

    // The same for a set of pieces that do not overlap one another: the bytes of the set are cut
    // into equal shares (inside a piece if need be), one for the caller and one per helper.
    void CopySet(const Task *tasks, size_t count);

    static constexpr size_t kSplitMin = 512u << 10;
    static constexpr uint32_t kWorkers = 2;

    uint64_t SharedCopies() const   // sets the helpers took part in (for tests)
    {
        return shared_.load(std::memory_order_relaxed);
    }

private:
    HostCopyHelper() = default;

    // A place in a set: byte `offset` of piece `piece`; piece == count is the end of the set.
    struct Cut {
        size_t piece = 0;
        size_t offset = 0;
    };
    // A share of a set: everything from `begin` up to, not including, `end`.
    struct Share {
        const Task *tasks = nullptr;
        size_t count = 0;
        Cut begin;
        Cut end;
    };
    struct Worker {
        Share share;                       // written by the caller before seq moves, read by the worker after it saw the move
        std::atomic<uint64_t> seq{0};      // shares posted
        std::atomic<uint64_t> done{0};     // shares finished
        std::atomic<bool> sleeping{false};
        std::mutex m;
        std::condition_variable cv;
    };
    static void Run(const Share &share);
    void Loop(Worker *worker);

    std::mutex owner_;                 // one caller at a time hands work to the helpers
    uint32_t started_ = 0;             // workers running; guarded by owner_
    bool unavailable_ = false;         // a thread could not be started: no further attempts
    Worker workers_[kWorkers];
    std::atomic<uint64_t> shared_{0};
};

}  // namespace mf

#endif  // MF_HOST_COPY_H
