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

void HostCopyHelper::Loop()
{
    uint64_t seen = 0;
    for (;;) {
        bool posted = false;
        for (int i = 0; i < kSpinRounds; ++i) {
            if (seq_.load(std::memory_order_acquire) != seen) {
                posted = true;
                break;
            }
            CpuRelax();
        }
        if (!posted) {
            std::unique_lock<std::mutex> lock(m_);
            sleeping_.store(true, std::memory_order_seq_cst);
            cv_.wait(lock, [&] { return seq_.load(std::memory_order_seq_cst) != seen; });
            sleeping_.store(false, std::memory_order_seq_cst);
        }
        seen = seq_.load(std::memory_order_acquire);   // one task is outstanding at most: the caller waits for it
        size_t skip = skip_;
        for (size_t i = first_; i < count_; ++i) {
            std::memcpy(static_cast<uint8_t *>(tasks_[i].dst) + skip, static_cast<const uint8_t *>(tasks_[i].src) + skip,
                        tasks_[i].len - skip);
            skip = 0;
        }
        done_.store(seen, std::memory_order_release);
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
    if (!started_ && !unavailable_) {
        try {
            std::thread(&HostCopyHelper::Loop, this).detach();
            started_ = true;
        } catch (...) {
            unavailable_ = true;
        }
    }
    if (!started_) {
        alone();
        return;
    }
    // the cut: piece `cut`, byte `within` (a multiple of 4096 so that both sides stay page-aligned
    // relative to the piece)
    const size_t half = total / 2;
    size_t cut = 0;
    size_t before = 0;
    while (cut < count && before + tasks[cut].len <= half) {
        before += tasks[cut].len;
        ++cut;
    }
    const size_t within = (half - before) & ~static_cast<size_t>(4095);   // half < total, so cut < count here
    tasks_ = tasks;
    first_ = cut;
    count_ = count;
    skip_ = within;
    const uint64_t ticket = seq_.fetch_add(1, std::memory_order_seq_cst) + 1;
    if (sleeping_.load(std::memory_order_seq_cst)) {
        std::lock_guard<std::mutex> lock(m_);
        cv_.notify_one();
    }
    for (size_t i = 0; i < cut; ++i) {
        std::memcpy(tasks[i].dst, tasks[i].src, tasks[i].len);
    }
    std::memcpy(tasks[cut].dst, tasks[cut].src, within);
    for (int spins = 0; done_.load(std::memory_order_acquire) != ticket; ++spins) {
        if (spins < kSpinRounds) {
            CpuRelax();
        } else {
            std::this_thread::yield();   // the helper has not been scheduled: do not hold the core it may need
        }
    }
    shared_.fetch_add(1, std::memory_order_relaxed);
}

}  // namespace mf
