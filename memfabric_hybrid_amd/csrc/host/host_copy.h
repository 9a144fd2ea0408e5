// CPU-side copies between caller memory and the pinned staging ring.
//
// One core moves about 33 GB/s with memcpy, the host link about 55 GB/s, so a copy that is staged
// by the calling thread alone is bound by that core (reference counterpart: the staging copies of
// HostDataOpSDMA::CopyLH2GD / CopyGD2LH, src/hybm/csrc/data_operation/host/hybm_data_op_sdma.cpp:
// 111-221, which run on the calling thread).  Here a second thread takes the upper half of every
// large piece.
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
    // The one helper of the process.  Never destroyed: its thread sleeps until the process ends and
    // touches nothing but this object.
    static HostCopyHelper &Instance();

    struct Task {
        void *dst;
        const void *src;
        size_t len;
    };

    // memcpy(dst, src, len).  Pieces of kSplitMin bytes and more are shared with the helper thread
    // when no other caller is using it; the call returns when every byte has been copied.
    void Copy(void *dst, const void *src, size_t len)
    {
        const Task one{dst, src, len};
        CopySet(&one, 1);
    }

    // The same for a set of pieces that do not overlap one another: the set is cut at half of its
    // bytes (inside a piece if need be), the helper takes the upper part.
    void CopySet(const Task *tasks, size_t count);

    static constexpr size_t kSplitMin = 512u << 10;

    uint64_t SharedCopies() const   // pieces the helper took part in (for tests)
    {
        return shared_.load(std::memory_order_relaxed);
    }

private:
    HostCopyHelper() = default;
    void Loop();

    std::mutex owner_;                 // one caller at a time hands work to the helper
    bool started_ = false;             // guarded by owner_
    bool unavailable_ = false;         // the thread could not be started: callers copy alone

    // the helper's share: written by the caller before seq_ moves, read by the helper after it saw the move
    const Task *tasks_ = nullptr;      // pieces [first_, count_), the first one from byte skip_ on
    size_t first_ = 0;
    size_t count_ = 0;
    size_t skip_ = 0;
    std::atomic<uint64_t> seq_{0};     // tasks posted
    std::atomic<uint64_t> done_{0};    // tasks finished
    std::atomic<bool> sleeping_{false};
    std::mutex m_;
    std::condition_variable cv_;
    std::atomic<uint64_t> shared_{0};
};

}  // namespace mf

#endif  // MF_HOST_COPY_H
