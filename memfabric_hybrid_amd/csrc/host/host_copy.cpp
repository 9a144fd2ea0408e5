#include "host_copy.h"

#include <cstring>
#include <thread>

namespace mf {
namespace {

inline void CpuRelax()
{
#if defined(__x86_64__) || defined(__i386__)
    __builtin_ia32_pause();
#else
    std::this_thread::yield();
#endif
}

constexpr int kSpinRounds = 2000;   // about 100 us of polling between the pieces of one transfer

}  // namespace

HostCopyHelper &HostCopyHelper::Instance()
{
    static HostCopyHelper *helper = new HostCopyHelper();
    return *helper;
}

void HostCopyHelper::Run(const Share &share)
{
    for (size_t i = share.begin.piece; i < share.count && i <= share.end.piece; ++i) {
        const size_t from = i == share.begin.piece ? share.begin.offset : 0;
        const size_t to = i == share.end.piece ? share.end.offset : share.tasks[i].len;
        if (to > from) {
            std::memcpy(static_cast<uint8_t *>(share.tasks[i].dst) + from, static_cast<const uint8_t *>(share.tasks[i].src) + from,
                        to - from);
        }
    }
}

void HostCopyHelper::Loop(Worker *worker)
{
    uint64_t seen = 0;
    for (;;) {
        bool posted = false;
        for (int i = 0; i < kSpinRounds; ++i) {
            if (worker->seq.load(std::memory_order_acquire) != seen) {
                posted = true;
                break;
            }
            CpuRelax();
        }
        if (!posted) {
            std::unique_lock<std::mutex> lock(worker->m);
            worker->sleeping.store(true, std::memory_order_seq_cst);
            worker->cv.wait(lock, [&] { return worker->seq.load(std::memory_order_seq_cst) != seen; });
            worker->sleeping.store(false, std::memory_order_seq_cst);
        }
        seen = worker->seq.load(std::memory_order_acquire);   // one share is outstanding at most: the caller waits for it
        Run(worker->share);
        worker->done.store(seen, std::memory_order_release);
    }
}

void HostCopyHelper::CopySet(const Task *tasks, size_t count)
{
    size_t total = 0;
    for (size_t i = 0; i < count; ++i) {
        total += tasks[i].len;
    }
    auto alone = [&]() {
        for (size_t i = 0; i < count; ++i) {
            std::memcpy(tasks[i].dst, tasks[i].src, tasks[i].len);
        }
    };
    if (total < kSplitMin || !owner_.try_lock()) {
        alone();
        return;
    }
    std::lock_guard<std::mutex> owner(owner_, std::adopt_lock);
    while (started_ < kWorkers && !unavailable_) {
        try {
            std::thread(&HostCopyHelper::Loop, this, &workers_[started_]).detach();
            ++started_;
        } catch (...) {
            unavailable_ = true;
        }
    }
    if (started_ == 0) {
        alone();
        return;
    }
    // Equal shares by bytes; a cut inside a piece is moved down to a multiple of 4096 so that every
    // share stays page-aligned relative to the piece.  Share 0 is the caller's.
    const uint32_t parts = started_ + 1;
    Cut cuts[kWorkers + 2];
    cuts[parts] = Cut{count, 0};
    size_t piece = 0;
    size_t before = 0;      // bytes of the pieces in front of `piece`
    for (uint32_t p = 1; p < parts; ++p) {
        const size_t at = total / parts * p;
        while (piece < count && before + tasks[piece].len <= at) {
            before += tasks[piece].len;
            ++piece;
        }
        cuts[p] = piece < count ? Cut{piece, (at - before) & ~static_cast<size_t>(4095)} : Cut{count, 0};
    }
    Share shares[kWorkers + 1];
    for (uint32_t p = 0; p < parts; ++p) {
        shares[p] = Share{tasks, count, cuts[p], cuts[p + 1]};
    }
    uint64_t tickets[kWorkers];
    for (uint32_t w = 0; w < started_; ++w) {
        Worker &worker = workers_[w];
        worker.share = shares[w + 1];
        tickets[w] = worker.seq.fetch_add(1, std::memory_order_seq_cst) + 1;
        if (worker.sleeping.load(std::memory_order_seq_cst)) {
            std::lock_guard<std::mutex> lock(worker.m);
            worker.cv.notify_one();
        }
    }
    Run(shares[0]);
    for (uint32_t w = 0; w < started_; ++w) {
        for (int spins = 0; workers_[w].done.load(std::memory_order_acquire) != tickets[w]; ++spins) {
            if (spins < kSpinRounds) {
                CpuRelax();
            } else {
                std::this_thread::yield();   // the helper has not been scheduled: do not hold the core it may need
            }
        }
    }
    shared_.fetch_add(1, std::memory_order_relaxed);
}

}  // namespace mf
