#include "xcopy_engine.h"

#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <thread>

#include "../../../include/mf_xcopy_types.h"
#include "../rt/mf_rt.h"
#include "mf_log.h"

namespace mf {
namespace {

constexpr uint32_t kSlots = 8;                // table staging slots per thread
constexpr uint32_t kGuardEvery = 4;           // one event is recorded per this many table launches
constexpr uint64_t kInlinePiece = 1ull << 30; // cut for segments the 32-bit inline length cannot hold

std::atomic<uint64_t> g_launches{0};

// One descriptor table in flight: the host fills `host`; the table kernel reads it there, or a copy
// kernel moves it to `dev` first.  The slot may be rewritten once an event recorded behind its
// kernels has fired.  Recording an event costs the stream about 3 us, as much as the launch gap
// it sits in, so one event guards kGuardEvery consecutive launches: a slot is Queued until that
// event is recorded and Guarded (by the slot that owns the event) afterwards.
struct StagingSlot {
    enum State : uint8_t { kFree, kQueued, kGuarded };
    void *host = nullptr;
    void *dev = nullptr;
    uint64_t capacity = 0;      // of host
    uint64_t devCapacity = 0;
    void *event = nullptr;
    State state = kFree;
    StagingSlot *guard = nullptr;
};

// GPU resources of one calling thread: its stream, its staging slots, its bounce area.  They are
// owned by the engine, not by the thread: a thread holds a lease, and when the thread ends the
// lease goes back to the idle list without any GPU call (thread-exit destructors run when the
// runtime, or a tool hooked into it, may already have torn down its own per-thread state).  The
// next new thread takes an idle lease over; Stop() releases all of them.
struct ThreadLease {
    uint32_t ordinal = 0;           // position in creation order
    void *stream = nullptr;
    StagingSlot slots[kSlots];
    uint32_t cursor = 0;
    uint32_t queued = 0;            // slots in state kQueued; their kernels all run on queuedStream
    void *queuedStream = nullptr;
    StagingSlot *lastQueued = nullptr;
    bool adopted = false;           // taken over from a thread that ended: its queued kernels ran on streams unknown here
    uint64_t *doneWord = nullptr;   // pinned; a one-lane launch stores doneSeq there behind a blocking copy
    uint32_t doneSeq = 0;
    uint64_t pendingBytes = 0;      // bytes of the copies queued on `stream` since the thread last waited for it
    void *bounce = nullptr;
    uint64_t bounceBytes = 0;
    void *bounceEvents[XcopyEngine::kBounceEvents] = {};
    // unordered batches handed to the submit threads: fanDirty bit w = submitter w holds batches of this thread that the
    // thread's stream has not been made to wait for, the last of them under ticket fanTicket[w]
    void *fanEvent[XcopyEngine::kFanStreams] = {};
    uint64_t fanTicket[XcopyEngine::kFanStreams] = {};
    uint32_t fanDirty = 0;
    uint32_t fanCursor = 0;

    void Destroy()   // GPU calls: only from Stop(), on a thread that is alive and bound
    {
        bool busy = false;
        for (auto &slot : slots) {
            busy = busy || slot.state != StagingSlot::kFree;
        }
        if (busy) {
            (void)mfrt_device_sync();   // kernels that read the slots may run on streams of the callers
        }
        queued = 0;
        queuedStream = nullptr;
        lastQueued = nullptr;
        for (auto &slot : slots) {
            if (slot.event != nullptr) {
                (void)mfrt_event_destroy(slot.event);
            }

            if (slot.host != nullptr) {
                (void)mfrt_free_host(slot.host);
            }
            if (slot.dev != nullptr) {
                (void)mfrt_free_device(slot.dev);
            }
            slot = StagingSlot{};
        }
        if (stream != nullptr) {
            (void)mfrt_stream_sync(stream);
            (void)mfrt_stream_destroy(stream);
            stream = nullptr;
        }

        if (bounce != nullptr) {
            (void)mfrt_free_host(bounce);
            bounce = nullptr;
            bounceBytes = 0;
        }
        if (doneWord != nullptr) {
            (void)mfrt_free_host(doneWord);
            doneWord = nullptr;
        }
        for (uint32_t i = 0; i < XcopyEngine::kFanStreams; ++i) {
            if (fanEvent[i] != nullptr) {
                (void)mfrt_event_destroy(fanEvent[i]);
                fanEvent[i] = nullptr;
            }
        }
        fanDirty = 0;
        for (void *&event : bounceEvents) {
            if (event != nullptr) {
                (void)mfrt_event_destroy(event);
                event = nullptr;
            }
        }
    }
};

// The streams of the engine, made at Start() and dealt out in an order in which consecutive takers sit on different
// hardware queues.  The runtime spreads the streams of a process over a few hardware queues (four here), not
// evenly (of the first eight streams after the thread's own, the second and third shared a queue in every process
// measured), and launches on streams that share a queue run one after the other: four submit threads whose streams
// sat on two queues measured 4.3 us per 9 MB batch, on four queues 3.6 us.  So the deck asks
// (mfrt_streams_share_queue, 50 us per pair, all streams idle) which of its streams share, and deals one stream of
// every queue before the second of any.  Streams beyond the deck are made on demand and not classified.
struct StreamDeck {
    std::mutex lock;
    std::vector<void *> order;          // untaken streams, the next one last
    std::vector<uint32_t> classes;      // hardware queue of the deck's streams in the order they are dealt, for reports

    void Build(uint32_t count)
    {
        std::lock_guard<std::mutex> guard(lock);
        DestroyLocked();
        std::vector<void *> made;
        std::vector<uint32_t> queueOf;
        std::vector<void *> firstOfQueue;
        bool known = true;
        for (uint32_t i = 0; i < count; ++i) {
            void *stream = mfrt_stream_create();
            if (stream == nullptr) {
                break;
            }
            uint32_t q = static_cast<uint32_t>(firstOfQueue.size());   // a queue of its own unless it shares one
            for (uint32_t c = 0; known && c < firstOfQueue.size(); ++c) {
                const int shared = mfrt_streams_share_queue(firstOfQueue[c], stream);
                if (shared < 0) {
                    known = false;      // no answer: from here on the streams keep the order they were made in
                    q = static_cast<uint32_t>(firstOfQueue.size());
                } else if (shared == 1) {
                    q = c;
                    break;
                }
            }
            if (q == firstOfQueue.size()) {
                firstOfQueue.push_back(stream);
            }
            made.push_back(stream);
            queueOf.push_back(q);
        }
        // round by round: the first untaken stream of every queue, queues in the order they appeared
        std::vector<bool> dealt(made.size(), false);
        std::vector<void *> sequence;
        const uint32_t queues = static_cast<uint32_t>(firstOfQueue.size());
        while (sequence.size() < made.size()) {
            for (uint32_t q = 0; q < queues; ++q) {
                for (size_t i = 0; i < made.size(); ++i) {
                    if (!dealt[i] && queueOf[i] == q) {
                        dealt[i] = true;
                        sequence.push_back(made[i]);
                        classes.push_back(q);
                        break;
                    }
                }
            }
        }
        order.assign(sequence.rbegin(), sequence.rend());
    }

    void *Take()
    {
        {
            std::lock_guard<std::mutex> guard(lock);
            if (!order.empty()) {
                void *stream = order.back();
                order.pop_back();
                return stream;
            }
        }
        return mfrt_stream_create();
    }

    void DestroyLocked()
    {
        for (void *stream : order) {
            (void)mfrt_stream_destroy(stream);
        }
        order.clear();
        classes.clear();
    }

    void Destroy()
    {
        std::lock_guard<std::mutex> guard(lock);
        DestroyLocked();
    }
};

StreamDeck &Deck()
{
    static StreamDeck *deck = new StreamDeck();   // never destroyed, as the lease pool
    return *deck;
}

std::atomic<uint32_t> g_leasesOut{0};   // leases held by live threads: more than one means launches of several streams may overlap

struct LeasePool {
    std::mutex lock;
    std::vector<std::unique_ptr<ThreadLease>> all;
    std::vector<ThreadLease *> idle;
    uint64_t epoch = 1;   // bumped by Stop(): leases handed out before are gone

    ThreadLease *Take(uint64_t &epochOut)
    {
        std::lock_guard<std::mutex> guard(lock);
        epochOut = epoch;
        if (!idle.empty()) {
            // The oldest idle lease, not the one handed back last: the runtime spreads streams over its
            // few hardware queues in creation order, and two streams on one hardware queue do not overlap
            // (two submitting threads whose streams share a queue measured 4.9 us per 9 MB batch, the same
            // as one thread; on different queues 4.1 us).  N threads alive at a time then hold the N
            // oldest streams, which sit on different queues as far as there are queues.
            size_t best = 0;
            for (size_t i = 1; i < idle.size(); ++i) {
                if (idle[i]->ordinal < idle[best]->ordinal) {
                    best = i;
                }
            }
            ThreadLease *lease = idle[best];
            idle.erase(idle.begin() + static_cast<std::ptrdiff_t>(best));
            lease->adopted = true;
            g_leasesOut.store(static_cast<uint32_t>(all.size() - idle.size()), std::memory_order_relaxed);
            return lease;
        }
        all.emplace_back(new ThreadLease());
        all.back()->ordinal = static_cast<uint32_t>(all.size() - 1);
        g_leasesOut.store(static_cast<uint32_t>(all.size() - idle.size()), std::memory_order_relaxed);
        return all.back().get();
    }
    void GiveBack(ThreadLease *lease, uint64_t leaseEpoch)
    {
        std::lock_guard<std::mutex> guard(lock);
        if (leaseEpoch == epoch) {
            idle.push_back(lease);
            g_leasesOut.store(static_cast<uint32_t>(all.size() - idle.size()), std::memory_order_relaxed);
        }
    }
    void DestroyAll()
    {
        std::lock_guard<std::mutex> guard(lock);
        for (auto &lease : all) {
            lease->Destroy();
        }
        all.clear();
        idle.clear();
        g_leasesOut.store(0, std::memory_order_relaxed);
        ++epoch;
    }
    uint64_t Epoch()
    {
        std::lock_guard<std::mutex> guard(lock);
        return epoch;
    }
};

LeasePool &Leases()
{
    static LeasePool *pool = new LeasePool();   // never destroyed: threads may end after static destructors ran
    return *pool;
}

std::atomic<uint64_t> g_leaseEpoch{1};   // copy of the pool's epoch that can be read without the lock

struct ThreadCtx {
    ThreadLease *lease = nullptr;
    uint64_t epoch = 0;
    SegList segs;
    ~ThreadCtx()
    {
        if (lease != nullptr) {
            Leases().GiveBack(lease, epoch);
            lease = nullptr;
        }
    }
    ThreadLease &Lease()
    {
        if (lease == nullptr || epoch != g_leaseEpoch.load(std::memory_order_acquire)) {
            lease = Leases().Take(epoch);
        }
        return *lease;
    }
    bool HasLiveLease() const
    {
        return lease != nullptr && epoch == g_leaseEpoch.load(std::memory_order_acquire);
    }
};

thread_local ThreadCtx t_ctx;

// Copies queued on the calling thread's own stream are added up, so that its next wait knows whether polling pays.
void NotePending(void *stream, uint64_t bytes)
{
    if (t_ctx.HasLiveLease() && stream == t_ctx.lease->stream) {
        uint64_t &pending = t_ctx.lease->pendingBytes;
        pending = pending + bytes < pending ? ~0ull : pending + bytes;
    }
}

// Submit threads.  One thread that launches on several streams in turn gains nothing (the launches cost it more
// than they cost on one stream: 4.6 to 5.1 us per 9 MB batch on two to four streams against 4.5 us), while several
// threads with a stream each do overlap on the GPU (eight threads: 3.9 us).  So a caller that declares its batches
// unordered can have them launched by up to kFanStreams threads of the library's, each with a stream of its own
// (six of them: 3.87 us per batch with the caller's thread spending 1.2 us on each): the caller plans the batch and puts the
// plan into a submitter's queue (a bounded queue of sequence-numbered cells, any number of producers, one consumer),
// the submitter launches it.  A ticket per queue tells the caller how far the submitter has got.
struct FanJob {
    InlinePlan plan;
    int route;
    uint32_t grid;
    uint32_t hold;
};

struct Submitter {
    static constexpr uint32_t kCells = 64;
    struct Cell {
        std::atomic<uint64_t> seq;
        FanJob job;
    };
    Cell cells[kCells];
    std::atomic<uint64_t> head{0};          // tickets handed to producers
    std::atomic<uint64_t> launched{0};      // jobs the thread has launched (in ticket order)
    std::atomic<int> error{0};              // first launch error, sticky until a caller has seen it
    std::atomic<bool> stop{false};
    std::atomic<bool> asleep{false};
    std::atomic<bool> ready{false};         // Run() has made its stream (or failed to)
    std::mutex lock;
    std::condition_variable wake;
    void *stream = nullptr;
    std::thread thread;

    Submitter()
    {
        for (uint32_t i = 0; i < kCells; ++i) {
            cells[i].seq.store(i, std::memory_order_relaxed);
        }
    }

    // Producer: returns the job's ticket.  Waits while the queue is full.
    uint64_t Push(const InlinePlan &plan, int route, uint32_t grid, uint32_t hold)
    {
        const uint64_t ticket = head.fetch_add(1, std::memory_order_relaxed);
        Cell &cell = cells[ticket % kCells];
        while (cell.seq.load(std::memory_order_acquire) != ticket) {
            std::this_thread::yield();      // kCells jobs ahead: the submitter is behind, or asleep and about to be woken
            Wake();
        }
        cell.job.plan = plan;
        cell.job.route = route;
        cell.job.grid = grid;
        cell.job.hold = hold;
        cell.seq.store(ticket + 1, std::memory_order_seq_cst);   // before the look at `asleep`: the submitter does both in the other order
        Wake();
        return ticket;
    }

    void Wake()
    {
        if (asleep.load(std::memory_order_seq_cst)) {
            std::lock_guard<std::mutex> guard(lock);
            wake.notify_one();
        }
    }

    void Run()
    {
        if (mfrt_bind_thread() != 0) {
            error.store(-1, std::memory_order_relaxed);
        }
        stream = Deck().Take();
        ready.store(true, std::memory_order_release);
        if (stream == nullptr) {
            return;
        }
        uint64_t next = 0;
        uint32_t idle = 0;
        while (!stop.load(std::memory_order_acquire)) {
            Cell &cell = cells[next % kCells];
            if (cell.seq.load(std::memory_order_acquire) == next + 1) {
                // a copy of its own first: the cell's lines come from the producer's core, and fetching them inside the launch
                // call would keep whatever the runtime holds locked there for as long
                const FanJob job = cell.job;
                const int err = mfk_xcopy_inline(&job.plan, job.route, job.grid, nullptr, 0, stream, 0, job.hold);
                if (err != 0) {
                    int none = 0;
                    (void)error.compare_exchange_strong(none, err, std::memory_order_relaxed);
                }
                cell.seq.store(next + kCells, std::memory_order_release);
                ++next;
                launched.store(next, std::memory_order_release);
                idle = 0;
                continue;
            }
            if (++idle < 20000) {           // some tens of microseconds of polling before the thread gives up its core
                continue;
            }
            std::unique_lock<std::mutex> guard(lock);
            asleep.store(true, std::memory_order_seq_cst);
            if (cell.seq.load(std::memory_order_seq_cst) != next + 1 && !stop.load(std::memory_order_acquire)) {
                // the bound is a net under the handshake, not part of it (by the system clock: the wait on the steady
                // clock is a call the thread sanitizer of this toolchain does not know, and it then misreads the mutex)
                wake.wait_until(guard, std::chrono::system_clock::now() + std::chrono::milliseconds(50));
            }
            asleep.store(false, std::memory_order_release);
            idle = 0;
        }
    }
};

struct SubmitPool {
    std::mutex lock;
    Submitter *submitters[XcopyEngine::kFanStreams] = {};
    std::atomic<uint32_t> alive{0};

    // Submitter w, started on first use; NULL when its stream or thread cannot be had.
    Submitter *Get(uint32_t w)
    {
        if (w < alive.load(std::memory_order_acquire)) {
            return submitters[w];
        }
        std::lock_guard<std::mutex> guard(lock);
        while (alive.load(std::memory_order_relaxed) <= w) {
            const uint32_t at = alive.load(std::memory_order_relaxed);
            Submitter *raw = new Submitter();
            raw->thread = std::thread([raw] { raw->Run(); });
            while (!raw->ready.load(std::memory_order_acquire)) {
                std::this_thread::yield();
            }
            if (raw->stream == nullptr) {
                raw->thread.join();
                delete raw;
                return nullptr;
            }
            submitters[at] = raw;
            alive.store(at + 1, std::memory_order_release);
        }
        return submitters[w];
    }

    // Submitter w if it runs.
    Submitter *Peek(uint32_t w)
    {
        return w < alive.load(std::memory_order_acquire) ? submitters[w] : nullptr;
    }

    // From Stop(): the threads end, their streams are drained and destroyed.
    void Shutdown()
    {
        std::lock_guard<std::mutex> guard(lock);
        const uint32_t count = alive.load(std::memory_order_relaxed);
        for (uint32_t w = 0; w < count; ++w) {
            Submitter *sub = submitters[w];
            sub->stop.store(true, std::memory_order_release);
            {
                std::lock_guard<std::mutex> inner(sub->lock);
                sub->wake.notify_one();
            }
            sub->thread.join();
            (void)mfrt_stream_sync(sub->stream);
            (void)mfrt_stream_destroy(sub->stream);
            delete sub;
            submitters[w] = nullptr;
        }
        alive.store(0, std::memory_order_release);
    }
};

SubmitPool &Submitters()
{
    static SubmitPool *pool = new SubmitPool();   // never destroyed: see Leases()
    return *pool;
}

// Makes `stream` (the lease's own) wait for the unordered batches the lease has handed to the submit threads: first until
// each has been launched, then, by an event on the submitter's stream, until it has run.
int JoinFan(ThreadLease &lease, void *stream)
{
    int failed = 0;
    for (uint32_t w = 0; lease.fanDirty != 0 && w < XcopyEngine::kFanStreams; ++w) {
        if ((lease.fanDirty & (1u << w)) == 0) {
            continue;
        }
        lease.fanDirty &= ~(1u << w);
        Submitter *sub = Submitters().Peek(w);
        if (sub == nullptr) {
            continue;   // stopped in the meantime: Stop() has drained it
        }
        while (sub->launched.load(std::memory_order_acquire) <= lease.fanTicket[w]) {
            sub->Wake();
            std::this_thread::yield();
        }
        const int err = sub->error.exchange(0, std::memory_order_relaxed);
        failed = failed != 0 ? failed : err;
        if (lease.fanEvent[w] == nullptr) {
            lease.fanEvent[w] = mfrt_event_create();
        }
        const bool joined = lease.fanEvent[w] != nullptr && mfrt_event_record(lease.fanEvent[w], sub->stream) == 0 &&
                            mfrt_stream_wait_event(stream, lease.fanEvent[w]) == 0;
        if (!joined) {
            const int syncErr = mfrt_stream_sync(sub->stream);
            if (syncErr != 0) {
                MF_FAIL(BM_ERROR, "unordered copies could not be awaited: " << mfrt_error_string(syncErr));
            }
        }
    }
    if (failed != 0) {
        MF_FAIL(BM_ERROR, "an unordered copy failed to launch: " << mfrt_error_string(failed));
    }
    return BM_OK;
}

uint64_t RoundUp(uint64_t v, uint64_t to)
{
    return (v + to - 1) / to * to;
}

// Records the event that guards every queued slot.  If the record fails the stream is drained instead.
int SealQueued(ThreadLease &ctx)
{
    if (ctx.queued == 0) {
        return BM_OK;
    }
    StagingSlot *owner = ctx.lastQueued;
    const bool recorded = owner != nullptr && owner->event != nullptr && mfrt_event_record(owner->event, ctx.queuedStream) == 0;
    if (!recorded && mfrt_stream_sync(ctx.queuedStream) != 0) {
        const int err = mfrt_device_sync();
        if (err != 0) {
            MF_FAIL(BM_ERROR, "staging slots could not be released: " << mfrt_error_string(err));
        }
    }
    for (auto &slot : ctx.slots) {
        if (slot.state == StagingSlot::kQueued) {
            slot.state = recorded ? StagingSlot::kGuarded : StagingSlot::kFree;
            slot.guard = recorded ? owner : nullptr;
        }
    }
    ctx.queued = 0;
    ctx.lastQueued = nullptr;
    return BM_OK;
}

// The kernels just launched on `stream` read `slot`.  Only launches on the lease's own stream wait
// for a shared event: a caller's stream may be gone by the time the next launch comes.
int MarkQueued(ThreadLease &ctx, StagingSlot *slot, void *stream, bool sealNow)
{
    sealNow = sealNow || stream != ctx.stream;
    slot->state = StagingSlot::kQueued;
    slot->guard = nullptr;
    ctx.queuedStream = stream;
    ctx.lastQueued = slot;
    ++ctx.queued;
    return sealNow || ctx.queued >= kGuardEvery ? SealQueued(ctx) : BM_OK;
}

// The next slot of the ring, free to be rewritten, with at least `bytes` of pinned host memory.
int AcquireSlot(ThreadLease &ctx, uint64_t bytes, void *stream, StagingSlot *&out)
{
    if (ctx.adopted) {
        // The thread that filled these slots is gone, and with it the knowledge which streams its
        // last launches went to: wait for the whole device once.
        bool busy = false;
        for (auto &slot : ctx.slots) {
            busy = busy || slot.state != StagingSlot::kFree;
        }
        if (busy) {
            const int err = mfrt_device_sync();
            if (err != 0) {
                MF_FAIL(BM_ERROR, "device wait failed: " << mfrt_error_string(err));
            }
            for (auto &slot : ctx.slots) {
                slot.state = StagingSlot::kFree;
                slot.guard = nullptr;
            }
        }
        ctx.queued = 0;
        ctx.lastQueued = nullptr;
        ctx.adopted = false;
    }
    StagingSlot &slot = ctx.slots[ctx.cursor];
    ctx.cursor = (ctx.cursor + 1) % kSlots;
    if (ctx.queued != 0 && (slot.state == StagingSlot::kQueued || ctx.queuedStream != stream)) {
        // one event guards launches of one stream only; and a slot about to be reused needs its guard now
        const int ret = SealQueued(ctx);
        if (ret != BM_OK) {
            return ret;
        }
    }
    if (slot.state == StagingSlot::kGuarded) {
        StagingSlot *guard = slot.guard;
        const int err = mfrt_event_sync(guard->event);
        if (err != 0) {
            MF_FAIL(BM_ERROR, "staging slot wait failed: " << mfrt_error_string(err));
        }
        for (auto &other : ctx.slots) {   // everything that event guarded is free now
            if (other.state == StagingSlot::kGuarded && other.guard == guard) {
                other.state = StagingSlot::kFree;
                other.guard = nullptr;
            }
        }
    }
    if (slot.capacity < bytes) {
        if (slot.host != nullptr) {
            (void)mfrt_free_host(slot.host);
            slot.host = nullptr;
        }
        const uint64_t cap = RoundUp(bytes < 65536 ? 65536 : bytes, 65536);
        slot.host = mfrt_alloc_host(cap);
        if (slot.host == nullptr) {
            slot.capacity = 0;
            MF_FAIL(BM_MALLOC_FAILED, "descriptor staging allocation of " << cap << " bytes failed");
        }
        slot.capacity = cap;
    }
    if (slot.event == nullptr) {
        slot.event = mfrt_event_create();
        if (slot.event == nullptr) {
            MF_FAIL(BM_ERROR, "event creation failed");
        }
    }
    out = &slot;
    return BM_OK;
}

// Device half of a slot, for the forms that need the table or the prefix in HBM.
int EnsureDevice(StagingSlot &slot, uint64_t bytes)
{
    if (slot.devCapacity >= bytes) {
        return BM_OK;
    }
    if (slot.dev != nullptr) {
        (void)mfrt_free_device(slot.dev);
        slot.dev = nullptr;
        slot.devCapacity = 0;
    }
    const uint64_t cap = RoundUp(bytes < 65536 ? 65536 : bytes, 65536);
    slot.dev = mfrt_alloc_device(cap);
    if (slot.dev == nullptr) {
        MF_FAIL(BM_MALLOC_FAILED, "descriptor staging allocation of " << cap << " bytes in HBM failed");
    }
    slot.devCapacity = cap;
    return BM_OK;
}

uint32_t GridFor(uint64_t nchunk, uint32_t cuCount, int route, const XcopyTuning &tuning)
{
    // HBM routes: one workgroup per chunk unless a cap is set.  Measured on 128 MiB ... 4 GiB copies:
    // letting the hardware dispatcher hand out the chunks one by one sustains 6.0-6.2 TB/s, a
    // grid capped at 16 workgroups per CU that strides over the chunks 5.3-5.7 TB/s (its static
    // assignment leaves a tail).  Link routes: one workgroup per CU, more only adds contention.
    const bool link = route == MFRT_ROUTE_TO_HOST || route == MFRT_ROUTE_FROM_HOST;
    const uint32_t perCu = link ? (tuning.wgPerCuLink == 0 ? 1 : tuning.wgPerCuLink) : tuning.wgPerCu;
    const uint64_t limit = (1ull << 24) - 1;   // grid size in lanes must stay below 2^32 with up to 256 lanes per workgroup
    uint64_t cap = perCu == 0 ? limit : static_cast<uint64_t>(cuCount == 0 ? 256 : cuCount) * perCu;
    if (cap > limit) {
        cap = limit;
    }
    uint64_t grid = nchunk < cap ? nchunk : cap;
    return grid == 0 ? 1u : static_cast<uint32_t>(grid);
}

// Grid of a table launch whose chunk count only the GPU knows: workgroups walk the chunks with the grid as their
// stride, surplus workgroups leave at once.  Eight workgroups per segment (pages of 32 KiB have eight chunks)
// between 32 and 4096 per CU: measured on 262 144 pages of 32 KiB, 256 / 512 / 1024 / 2048 / 4096 per CU take
// 3.27 / 3.21 / 3.15 / 3.09 / 3.06 ms (one workgroup per chunk, which needs the count: 3.05 ms), while on 4096 pages
// 512 per CU cost 14 us in workgroups that find nothing to do (69 against 55 us).
uint32_t DeviceTableGrid(uint32_t nseg, uint32_t cuCount, int route, const XcopyTuning &tuning)
{
    const uint64_t cus = cuCount == 0 ? 256 : cuCount;
    uint64_t want = tuning.deviceTableWgPerCu != 0 ? cus * tuning.deviceTableWgPerCu : 8ull * nseg;
    if (tuning.deviceTableWgPerCu == 0) {
        want = want < 32 * cus ? 32 * cus : (want > 4096 * cus ? 4096 * cus : want);
    }
    return GridFor(want, cuCount, route, tuning);
}

}  // namespace

void NormalizeSegments(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n, uint64_t pieceLimit,
                       SegList &out)
{
    out.Clear();
    uint64_t curSrc = 0;
    uint64_t curDst = 0;
    uint64_t curLen = 0;
    auto flush = [&]() {
        while (curLen > 0) {
            uint64_t piece = (pieceLimit != 0 && curLen > pieceLimit) ? pieceLimit : curLen;
            out.src.push_back(curSrc);
            out.dst.push_back(curDst);
            out.len.push_back(piece);
            out.totalBytes += piece;
            curSrc += piece;
            curDst += piece;
            curLen -= piece;
        }
    };
    for (uint32_t i = 0; i < n; ++i) {
        if (len[i] == 0) {
            continue;
        }
        if (curLen > 0 && curSrc + curLen == src[i] && curDst + curLen == dst[i]) {
            curLen += len[i];
            continue;
        }
        flush();
        curSrc = src[i];
        curDst = dst[i];
        curLen = len[i];
    }
    flush();
}

uint32_t ChooseUnits(uint64_t totalBytes, uint32_t cuCount, int route, const XcopyTuning &tuning)
{
    (void)cuCount;
    if (tuning.unitsOverride != 0) {
        return static_cast<uint32_t>(RoundUp(tuning.unitsOverride, 64));
    }
    // Measured on MI355X (256 CUs).  HBM routes: 4 KiB chunks, which the launcher gives to single-wave
    // workgroups, one workgroup per chunk: the fastest shape from a 1 MiB copy (3.4 us against 4.5 us
    // with four-wave workgroups on 16 KiB chunks) over the 9 MB KV batch (4.8 against 5.5 us) to a
    // 1 GiB copy (6.4 against 6.25 TB/s).  4 KiB also divides the usual power-of-two block sizes, so
    // no workgroup runs a ragged tile.
    if (route == MFRT_ROUTE_TO_HOST || route == MFRT_ROUTE_FROM_HOST) {
        // The host link, not the GPU, is the bound: one four-wave workgroup per CU with small chunks
        // keeps the link busy without flooding it (measured: 56 GB/s out, 55 GB/s in on a Gen5 x16 link).
        if (totalBytes > (256ull << 20)) {
            return 4 * kXcopyThreads;
        }
        return route == MFRT_ROUTE_TO_HOST ? kXcopyThreads : 2 * kXcopyThreads;
    }
    (void)totalBytes;
    return tuning.minUnits;
}

bool BuildInlinePlan(const SegList &segs, uint32_t units, InlinePlan &plan)
{
    const uint32_t n = segs.Size();
    if (n > kInlineSegs) {
        return false;
    }
    uint64_t run = 0;
    for (uint32_t i = 0; i < n; ++i) {
        if (segs.len[i] > 0xFFFFFFFFull) {
            return false;
        }
        plan.src[i] = segs.src[i];
        plan.dst[i] = segs.dst[i];
        plan.len[i] = static_cast<uint32_t>(segs.len[i]);
        plan.first[i] = static_cast<uint32_t>(run);
        run += SegmentChunks(segs.dst[i], segs.len[i], units);
        if (run >= kNoChunk) {
            return false;
        }
    }
    for (uint32_t i = n; i < kInlineSegs; ++i) {
        plan.src[i] = 0;
        plan.dst[i] = 0;
        plan.len[i] = 0;
        plan.first[i] = kNoChunk;
    }
    plan.nchunk = static_cast<uint32_t>(run);
    plan.units = units;
    return true;
}

// Normalisation and inline planning in one pass over the caller's arrays, for the common case
// of a batch that ends up with at most kInlineSegs segments below 4 GiB each.  Returns false
// (plan contents undefined) when the batch needs the general path.
bool BuildInlineDirect(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n, uint32_t units,
                       InlinePlan &plan)
{
    const bool pow2 = (units & (units - 1)) == 0;
    const uint32_t shift = pow2 ? static_cast<uint32_t>(__builtin_ctz(units)) : 0;
    // The usual batch (blocks scattered over a pool) has nothing to merge, nothing empty and nothing of 4 GiB: one pass
    // without branches says so, and the plan is then filled by a straight-line loop (the general loop below merges as it
    // goes and tests every step).
    if (n != 0 && n <= kInlineSegs && pow2) {
        uint64_t special = (len[n - 1] == 0 ? 1u : 0u) | (len[n - 1] >> 32);
        for (uint32_t i = 0; i + 1 < n; ++i) {
            const uint64_t l = len[i];
            special |= (l == 0 ? 1u : 0u) | (l >> 32) |
                       ((src[i] + l == src[i + 1] ? 1u : 0u) & (dst[i] + l == dst[i + 1] ? 1u : 0u));
        }
        if (special == 0) {
            uint32_t run32 = 0;
            for (uint32_t i = 0; i < n; ++i) {
                const uint64_t l = len[i];
                uint64_t head = (0 - dst[i]) & (kUnitBytes - 1);
                head = head > l ? l : head;
                const uint64_t chunks = ((l - head) / kUnitBytes + units - 1) >> shift;
                plan.src[i] = src[i];
                plan.dst[i] = dst[i];
                plan.len[i] = static_cast<uint32_t>(l);
                plan.first[i] = run32;
                run32 += static_cast<uint32_t>(chunks == 0 ? 1 : chunks);      // n * 2^32 / 4096 chunks at most: no overflow
            }
            for (uint32_t i = n; i < kInlineSegs; ++i) {
                plan.src[i] = 0;
                plan.dst[i] = 0;
                plan.len[i] = 0;
                plan.first[i] = kNoChunk;
            }
            plan.nchunk = run32;
            plan.units = units;
            return run32 < kNoChunk;
        }
    }
    uint32_t used = 0;
    uint64_t run = 0;
    uint64_t curSrc = 0;
    uint64_t curDst = 0;
    uint64_t curLen = 0;
    auto flush = [&]() -> bool {
        if (curLen == 0) {
            return true;
        }
        if (used == kInlineSegs || curLen > 0xFFFFFFFFull) {
            return false;
        }
        uint64_t head = (0 - curDst) & (kUnitBytes - 1);
        if (head > curLen) {
            head = curLen;
        }
        const uint64_t body = (curLen - head) / kUnitBytes;
        uint64_t chunks = pow2 ? (body + units - 1) >> shift : (body + units - 1) / units;
        if (chunks == 0) {
            chunks = 1;
        }
        plan.src[used] = curSrc;
        plan.dst[used] = curDst;
        plan.len[used] = static_cast<uint32_t>(curLen);
        plan.first[used] = static_cast<uint32_t>(run);
        run += chunks;
        ++used;
        return true;
    };
    for (uint32_t i = 0; i < n; ++i) {
        const uint64_t l = len[i];
        if (l == 0) {
            continue;
        }
        if (curLen > 0 && curSrc + curLen == src[i] && curDst + curLen == dst[i]) {
            curLen += l;
            continue;
        }
        if (!flush()) {
            return false;
        }
        curSrc = src[i];
        curDst = dst[i];
        curLen = l;
    }
    if (!flush() || run >= kNoChunk) {
        return false;
    }
    for (uint32_t i = used; i < kInlineSegs; ++i) {
        plan.src[i] = 0;
        plan.dst[i] = 0;
        plan.len[i] = 0;
        plan.first[i] = kNoChunk;
    }
    plan.nchunk = static_cast<uint32_t>(run);
    plan.units = units;
    return true;
}

uint64_t BuildTablePlan(const SegList &segs, uint32_t units, uint64_t *triples, uint32_t *first)
{
    const uint32_t n = segs.Size();
    uint64_t run = 0;
    for (uint32_t i = 0; i < n; ++i) {
        triples[3 * i] = segs.src[i];
        triples[3 * i + 1] = segs.dst[i];
        triples[3 * i + 2] = segs.len[i];
        first[i] = static_cast<uint32_t>(run);
        run += SegmentChunks(segs.dst[i], segs.len[i], units);
    }
    first[n] = static_cast<uint32_t>(run);
    return run;
}

// Normalisation (empty segments dropped, neighbours that continue each other merged) and table
// planning in one pass over the caller's arrays, straight into the staging slot: a 4096-segment
// batch costs the host about as long as the GPU needs to copy it, so nothing is built twice.
// triples: room for 3 * n words, first: room for n + 1.  Returns the chunk count, count = segments.
uint64_t BuildTableDirect(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n, uint32_t units,
                          uint64_t *triples, uint32_t *first, uint32_t &count, ChunkPattern *pattern)
{
    const bool pow2 = (units & (units - 1)) == 0;
    const uint32_t shift = pow2 ? static_cast<uint32_t>(__builtin_ctz(units)) : 0;
    uint32_t used = 0;
    uint64_t run = 0;
    uint64_t recent[kMaxPeriod] = {};   // chunk counts of the last kMaxPeriod segments, by index modulo kMaxPeriod
    uint64_t leading[kMaxPeriod] = {};  // and of the first ones
    uint32_t alive = 0x1FEu;            // bit p: the counts so far repeat with period p (1 .. kMaxPeriod)
    uint64_t curSrc = 0;
    uint64_t curDst = 0;
    uint64_t curLen = 0;
    auto flush = [&]() {
        if (curLen == 0) {
            return;
        }
        uint64_t head = (0 - curDst) & (kUnitBytes - 1);
        if (head > curLen) {
            head = curLen;
        }
        const uint64_t body = (curLen - head) / kUnitBytes;
        uint64_t chunks = pow2 ? (body + units - 1) >> shift : (body + units - 1) / units;
        if (chunks == 0) {
            chunks = 1;
        }
        triples[3 * used] = curSrc;
        triples[3 * used + 1] = curDst;
        triples[3 * used + 2] = curLen;
        first[used] = static_cast<uint32_t>(run < kNoChunk ? run : kNoChunk);
        if (alive != 0) {
            for (uint32_t p = 1; p <= kMaxPeriod; ++p) {
                if (used >= p && recent[(used - p) % kMaxPeriod] != chunks) {
                    alive &= ~(1u << p);
                }
            }
            recent[used % kMaxPeriod] = chunks;
            if (used < kMaxPeriod) {
                leading[used] = chunks;
            }
        }
        run += chunks;
        ++used;
    };
    for (uint32_t i = 0; i < n; ++i) {
        const uint64_t l = len[i];
        if (l == 0) {
            continue;
        }
        if (curLen > 0 && curSrc + curLen == src[i] && curDst + curLen == dst[i]) {
            curLen += l;
            continue;
        }
        flush();
        curSrc = src[i];
        curDst = dst[i];
        curLen = l;
    }
    flush();
    first[used] = static_cast<uint32_t>(run < kNoChunk ? run : kNoChunk);
    count = used;
    if (pattern != nullptr) {
        *pattern = ChunkPattern{};
        if (used != 0 && alive != 0 && run < kNoChunk) {
            const uint32_t period = static_cast<uint32_t>(__builtin_ctz(alive));
            uint32_t sum = 0;
            for (uint32_t i = 0; i < period; ++i) {
                pattern->start[i] = sum;
                sum += static_cast<uint32_t>(leading[i]);   // the shortest period never exceeds the segment count
            }
            pattern->start[period] = sum;
            pattern->period = period;
            pattern->chunksPerPeriod = sum;
        }
    }
    return run;
}

void ChooseCalibration(const float *batchMicros, const float *copyMicros, uint32_t defaultWindowMBps, uint32_t defaultAlignedMBps,
                       uint32_t defaultLongMBps, XcopyCalibration &out)
{
    out = XcopyCalibration{};
    out.windowMBps = defaultWindowMBps;
    out.windowAlignedMBps = defaultAlignedMBps;
    out.windowLongMBps = defaultLongMBps;
    for (int i = 0; i < 4; ++i) {
        out.batchMicros[i] = batchMicros[i];
    }
    for (int i = 0; i < 4; ++i) {
        out.copyMicros[i] = copyMicros[i];
    }
    const bool batchMeasured = batchMicros[0] > 0 && batchMicros[1] > 0 && batchMicros[2] > 0 && batchMicros[3] > 0;
    if (batchMeasured) {
        // the rule's own wait unless a neighbour is clearly better (2 %: less is noise between rounds and between boxes)
        int best = 2;
        for (int v : {1, 3}) {
            if (batchMicros[v] < batchMicros[best] * 0.98f) {
                best = v;
            }
        }
        out.holdDeltaNanos = (best - 2) * kCalibrateHoldStepNanos;
        out.holdEnabled = batchMicros[best] <= batchMicros[0] * (1.0f - kCalibrateMinGain);
        out.ran = true;
    }
    const bool copyMeasured = copyMicros[0] > 0 && copyMicros[1] > 0 && copyMicros[2] > 0;
    if (copyMeasured) {
        const bool slowerWins = copyMicros[2] < copyMicros[1] * 0.99f;
        const float windowed = slowerWins ? copyMicros[2] : copyMicros[1];
        const uint32_t rate = slowerWins ? static_cast<uint32_t>(static_cast<uint64_t>(defaultWindowMBps) * kCalibrateSlowerWindowPercent / 100)
                                         : defaultWindowMBps;
        out.windowMBps = windowed <= copyMicros[0] * (1.0f - kCalibrateMinWindowGain) ? rate : 0u;
        // the higher rate of aligned segments only where an aligned copy held it here: 2 % better than the rate just chosen
        // (the rate between the two, for shorter segments on cache lines, goes with it: a GPU that holds the highest holds that one)
        const bool higherHolds = out.windowMBps != 0 && copyMicros[3] > 0 && copyMicros[3] < windowed * 0.98f;
        out.windowLongMBps = higherHolds ? defaultLongMBps : out.windowMBps;
        out.windowAlignedMBps = higherHolds ? defaultAlignedMBps : out.windowMBps;
        out.ran = true;
    }
}

int XcopyEngine::Calibrate()
{
    if (!Started()) {
        return BM_NOT_INITIALIZED;
    }
    void *stream = ThreadStream();
    if (stream == nullptr) {
        return BM_ERROR;
    }
    const uint32_t rule = HoldNanosFor(2196, 2196, kXcopyThreads, false);
    const uint32_t holds[3] = {rule - kCalibrateHoldStepNanos, rule, rule + kCalibrateHoldStepNanos};
    const uint32_t defaultRate = XcopyTuning{}.windowMBps;
    const uint32_t defaultLong = XcopyTuning{}.windowLongMBps;
    const uint32_t rates[3] = {defaultRate, static_cast<uint32_t>(static_cast<uint64_t>(defaultRate) * kCalibrateSlowerWindowPercent / 100),
                               defaultLong};
    float us[8] = {};
    const int err = mfk_xcopy_calibrate(stream, holds, rates, us);
    if (err != 0) {
        calibration_ = XcopyCalibration{};
        MF_ERROR("calibration run failed (" << mfrt_error_string(err) << "): the fitted defaults stay");
        return BM_ERROR;
    }
    ChooseCalibration(us, us + 4, defaultRate, XcopyTuning{}.windowAlignedMBps, defaultLong, calibration_);
    if (calibration_.ran) {
        tuning_.holdDeltaNanos = calibration_.holdDeltaNanos;
        tuning_.holdCalibratedOff = !calibration_.holdEnabled;
        if (windowsAvailable_) {
            tuning_.windowMBps = calibration_.windowMBps;
            tuning_.windowAlignedMBps = calibration_.windowAlignedMBps;
            tuning_.windowLongMBps = calibration_.windowLongMBps;
            windowRateCalibrated_ = true;
        }
    }
    return BM_OK;
}

XcopyEngine &XcopyEngine::Instance()
{
    static XcopyEngine engine;
    return engine;
}

int XcopyEngine::Start(int device)
{
    int err = mfrt_init(device);
    if (err != 0) {
        MF_FAIL(BM_ERROR, "GPU runtime start on device " << device << " failed: " << mfrt_error_string(err));
    }
#ifndef MF_RT_HIDDEN
    err = mfk_xcopy_static_setup();   // the device is current on this thread: mfrt_init has just selected it
    if (err != 0) {
        // only the entry point that allocates nothing needs it, and that one reports the missing set-up itself
        MF_ERROR("address of the static descriptor scratch not available: " << mfrt_error_string(err));
    }
#endif
    windowsAvailable_ = mfk_xcopy_windows_available() != 0;
    Deck().Build(kDeckStreams);   // before the first stream is handed out: the calling thread's own is the deck's first
    tuning_.holdDeltaNanos = 0;
    tuning_.holdCalibratedOff = false;
    if (windowRateCalibrated_) {   // what an earlier start of this process chose does not outlive it
        tuning_.windowMBps = XcopyTuning{}.windowMBps;
        tuning_.windowAlignedMBps = XcopyTuning{}.windowAlignedMBps;
        tuning_.windowLongMBps = XcopyTuning{}.windowLongMBps;
        windowRateCalibrated_ = false;
    }
    calibration_ = XcopyCalibration{};
    started_.store(true, std::memory_order_release);
    {
        // every copy kernel once, then the timing rules checked against this GPU
        void *stream = ThreadStream();
        if (stream == nullptr || mfk_xcopy_prelaunch(stream) != 0) {
            MF_ERROR("the copy kernels could not be launched once at start");
        }
        const char *env = std::getenv("MF_HIP_CALIBRATE");
        if (stream != nullptr && !(env != nullptr && env[0] == '0')) {
            (void)Calibrate();
        }
        if (stream != nullptr) {
            (void)mfrt_stream_sync(stream);
        }
    }
    started_.store(true, std::memory_order_release);
    return BM_OK;
}

void XcopyEngine::Stop()
{
    if (!started_.load(std::memory_order_acquire)) {
        return;
    }
    (void)mfrt_bind_thread();
    Submitters().Shutdown();
    (void)mfrt_device_sync();
    Leases().DestroyAll();   // every thread's stream and staging memory, not only the caller's
    Deck().Destroy();
    g_leaseEpoch.store(Leases().Epoch(), std::memory_order_release);
    started_.store(false, std::memory_order_release);
    mfrt_shutdown();
}

uint32_t XcopyEngine::StreamQueues(uint32_t *queues, uint32_t capacity) const
{
    StreamDeck &deck = Deck();
    std::lock_guard<std::mutex> guard(deck.lock);
    const uint32_t count = static_cast<uint32_t>(deck.classes.size());
    for (uint32_t i = 0; i < count && i < capacity; ++i) {
        queues[i] = deck.classes[i];
    }
    return count;
}

bool XcopyEngine::Started() const
{
    return started_.load(std::memory_order_acquire);
}

void *XcopyEngine::ThreadStream()
{
    ThreadLease &lease = t_ctx.Lease();
    if (lease.stream == nullptr) {
        if (mfrt_bind_thread() != 0) {
            return nullptr;
        }
        lease.stream = Deck().Take();
    }
    if (lease.fanDirty != 0 && lease.stream != nullptr && JoinFan(lease, lease.stream) != BM_OK) {
        return nullptr;
    }
    return lease.stream;
}

void *XcopyEngine::ThreadBounce(uint64_t bytes)
{
    ThreadLease &lease = t_ctx.Lease();
    if (lease.bounceBytes < bytes) {
        if (mfrt_bind_thread() != 0) {
            return nullptr;
        }
        if (lease.bounce != nullptr) {
            (void)mfrt_free_host(lease.bounce);
            lease.bounce = nullptr;
            lease.bounceBytes = 0;
        }
        lease.bounce = mfrt_alloc_host(bytes);
        lease.bounceBytes = lease.bounce != nullptr ? bytes : 0;
    }
    return lease.bounce;
}

void *XcopyEngine::ThreadBounceEvent(uint32_t index)
{
    if (index >= kBounceEvents) {
        return nullptr;
    }
    ThreadLease &lease = t_ctx.Lease();
    if (lease.bounceEvents[index] == nullptr && mfrt_bind_thread() == 0) {
        lease.bounceEvents[index] = mfrt_event_create();
    }
    return lease.bounceEvents[index];
}

int XcopyEngine::DrainThread()
{
    if (!Started()) {
        return BM_NOT_INITIALIZED;
    }
    if (!t_ctx.HasLiveLease() || t_ctx.lease->stream == nullptr) {
        return BM_OK;
    }
    // a short queue is awaited like a blocking call: by polling (20 KV batches and a wait: 3 us sooner than the stream wait)
    return WaitStream(t_ctx.lease->stream, t_ctx.lease->pendingBytes);
}

// A blocking call is a launch and a wait.  hipStreamSynchronize first has to put a marker with a
// completion signal behind the kernel and then takes 7 us to see it fire, whatever the wait policy
// of the device (measured: 16.1 us per blocking 9 MB batch with the default policy and with
// hipDeviceScheduleSpin alike; an event recorded behind the launch and polled or waited for:
// 15.5 us; hipStreamWriteValue64 polled: 13.1 us; the kernel launched with a stop event of its own
// and that event polled: 13.3 us).  A one-lane launch that stores a sequence number
// into pinned memory, polled by the caller, is the shortest way round: 11.8 us.  It starts after
// the copy kernel has ended, so it carries the same guarantee as the stream wait: the copy's
// end-of-kernel release has made its stores visible to the device, and stores to host memory were
// issued, in order, before the word's.
int XcopyEngine::WaitStream(void *stream, uint64_t bytes)
{
    if (t_ctx.HasLiveLease() && stream == t_ctx.lease->stream) {
        const uint64_t queued = t_ctx.lease->pendingBytes;
        bytes = queued > bytes ? queued : bytes;     // what else the thread has queued there is waited for as well
        t_ctx.lease->pendingBytes = 0;
        if (t_ctx.lease->fanDirty != 0) {            // and the unordered batches on its side streams
            const int ret = JoinFan(*t_ctx.lease, stream);
            if (ret != BM_OK) {
                return ret;
            }
        }
    }
    if (bytes != 0 && bytes <= kSpinBytes) {
        ThreadLease &lease = t_ctx.Lease();
        if (lease.doneWord == nullptr) {
            lease.doneWord = static_cast<uint64_t *>(mfrt_alloc_host(64));
            if (lease.doneWord != nullptr) {
                *lease.doneWord = 0;
                lease.doneSeq = 0;
            }
        }
        if (lease.doneWord != nullptr) {
            const uint32_t seq = ++lease.doneSeq == 0 ? ++lease.doneSeq : lease.doneSeq;   // 0 is the initial contents
            if (mfk_xcopy_signal(lease.doneWord, seq, stream) == 0) {   // not counted by LaunchCount(): it moves no data
                const auto start = std::chrono::steady_clock::now();
                for (uint32_t polls = 1;; ++polls) {
                    if (__atomic_load_n(lease.doneWord, __ATOMIC_ACQUIRE) == seq) {
                        return BM_OK;
                    }
                    if ((polls & 63u) == 0 &&
                        std::chrono::steady_clock::now() - start > std::chrono::microseconds(kSpinMicros)) {
                        break;   // longer than expected (or the GPU is busy with other work): sleep on the stream instead
                    }
                }
            }
        }
    }
    const int err = mfrt_stream_sync(stream);
    if (err != 0) {
        MF_FAIL(BM_ERROR, "copy failed on the GPU: " << mfrt_error_string(err));
    }
    return BM_OK;
}

void XcopyEngine::NoteQueued(void *stream, uint64_t bytes)
{
    NotePending(stream, bytes);
}

void XcopyEngine::QuiesceSubmitters()
{
    for (uint32_t w = 0; w < kFanStreams; ++w) {
        Submitter *sub = Submitters().Peek(w);
        if (sub == nullptr) {
            break;
        }
        const uint64_t handed = sub->head.load(std::memory_order_acquire);
        while (sub->launched.load(std::memory_order_acquire) < handed) {
            sub->Wake();
            std::this_thread::yield();
        }
    }
}

uint64_t XcopyEngine::LaunchCount() const
{
    return g_launches.load();
}

// How long the waves of a launch keep their data before they store (0: not at all): the tuning knob over
// HoldNanosFor's rule, for HBM routes and ordered launches only.
uint32_t XcopyEngine::HoldFor(const InlinePlan &plan, uint32_t grid, int route, bool unordered) const
{
    if (route != MFRT_ROUTE_HBM || unordered || tuning_.holdNanos == 0) {
        return 0;
    }
    // With launches of another thread's stream on the chip at the same time not every wave of a large launch is
    // resident at once, and the wait costs instead of gaining (two submitting threads, 24 MiB copies: 8.2 us per
    // copy without, 9.0 us with; 21 MB batches 7.9 / 8.2 us; 16 MB and below: the same or better with the wait).
    if ((plan.nchunk > kHoldSharedMaxChunks || plan.units == kDeepUnits) && g_leasesOut.load(std::memory_order_relaxed) > 1) {
        return 0;
    }
    const uint32_t rule = HoldNanosFor(plan.nchunk, grid, plan.units, plan.first[1] == kNoChunk && plan.units != kDeepUnits);
    if (rule == 0 || tuning_.holdNanos > 0) {
        return rule != 0 ? static_cast<uint32_t>(tuning_.holdNanos) : 0;
    }
    if (tuning_.holdCalibratedOff) {
        return 0;
    }
    const int64_t with = static_cast<int64_t>(rule) + tuning_.holdDeltaNanos;
    return with > 0 ? static_cast<uint32_t>(with) : 0;
}

// Hold of a table launch.  Under a pattern (pinned) its waves fetch their descriptors across the host link and issue
// their loads that much later than those of a launch whose descriptors are kernel arguments; without one they find them
// through the group map in device memory, two dependent loads.
uint32_t XcopyEngine::HoldForTable(uint32_t nchunk, uint32_t grid, uint32_t units, int route, bool unordered, bool pinned) const
{
    if (route != MFRT_ROUTE_HBM || unordered || tuning_.holdNanos == 0) {
        return 0;
    }
    if ((nchunk > kHoldSharedMaxChunks || units == kDeepUnits) && g_leasesOut.load(std::memory_order_relaxed) > 1) {
        return 0;
    }
    const uint32_t rule = HoldNanosFor(nchunk, grid, units, false);
    if (rule == 0) {
        return 0;
    }
    if (tuning_.holdNanos > 0) {
        return static_cast<uint32_t>(tuning_.holdNanos);
    }
    if (tuning_.holdCalibratedOff) {
        return 0;
    }
    // The 16 KiB form wants its wait another 800 ns longer than the link round trip explains (sixteen loads per lane take
    // longer to leave than four): K and V blocks of 3 / 4 / 5 / 6 requests, 27 to 54 MB, with 1600 / 2000 / 2400 / 2800 ns on
    // top of the rule: 13.3 / 12.7 / 13.0 / 13.4 us, 17.2 / 16.5 / 16.1 / 16.4, 20.3 / 19.8 / 19.1 / 19.3, 24.3 / 23.8 / 23.5 / 23.5;
    // two requests on 4 KiB chunks 9.3 / 9.7 / 10.1 / 10.5 (and 9.3 with 1200).
    // Ragged tables, whose descriptors were uploaded: 36 / 40 / 58 MB on 16 KiB chunks 18.4 / 20.0 / 26.2 us with 500 ns on top
    // of the rule (19.0 / 20.5 / 27.0 with none, 18.7 / 20.4 / 26.0 with 1000) against 20.5 / 22.6 / 28.7 us not held; 12 / 13 /
    // 20 / 19 MB on 4 KiB chunks 10.9 / 11.6 / 13.8 / 13.9 us with 800 ns against 11.3 / 12.3 / 14.8 / 14.7 (6 MB: 9.3 either way).
    const int32_t extra = pinned ? tuning_.holdPinnedExtraNanos + (units == kDeepUnits ? kHoldPinnedDeepExtraNanos : 0)
                                 : (units == kDeepUnits ? kHoldLookupDeepExtraNanos : kHoldLookupExtraNanos);
    const int64_t with = static_cast<int64_t>(rule) + extra + tuning_.holdDeltaNanos;
    return with > 0 ? static_cast<uint32_t>(with) : 0;
}

bool XcopyEngine::DeepHoldApplies(uint64_t bytes, uint32_t n, int route, bool unordered) const
{
    return route == MFRT_ROUTE_HBM && !unordered && tuning_.holdNanos != 0 && tuning_.unitsOverride == 0 && tuning_.deepHold &&
           bytes > kDeepMinBytes && bytes <= kDeepMaxBytes && n != 0 && bytes / n >= kDeepMinSegmentBytes &&
           g_leasesOut.load(std::memory_order_relaxed) <= 1;
}

bool XcopyEngine::WindowsApply(uint64_t bytes, int route, uint64_t minBytes) const
{
    // Two such launches at a time would each cut their periods for the whole chip's rate, so a second thread with a
    // stream of its own switches the form off, as it does for the largest held launches.
    return route == MFRT_ROUTE_HBM && bytes >= minBytes && tuning_.windowMBps != 0 && tuning_.unitsOverride == 0 &&
           windowsAvailable_ && g_leasesOut.load(std::memory_order_relaxed) <= 1;
}

bool XcopyEngine::SingleSubmitter() const
{
    return g_leasesOut.load(std::memory_order_relaxed) <= 1;
}

int XcopyEngine::Submit(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n, int route,
                        void *stream, void *mask, uint32_t maskValue, bool unordered)
{
    return SubmitOne(src, dst, len, n, route, stream, mask, maskValue, unordered, true);
}

// A batch of up to kInlineSegs segments that moves twice kWindowPieceBytes and more, submitted as consecutive runs of
// kWindowPieceBytes to twice that, one windowed launch each.  Runs end at segment ends where the segments are short and
// inside a segment, at a multiple of 1 MiB from its start, where one is long.
int XcopyEngine::SubmitInPieces(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n, uint64_t total, int route,
                                void *stream, void *mask, uint32_t maskValue)
{
    const uint64_t pieces = total / kWindowPieceBytes;
    const uint64_t target = (total + pieces - 1) / pieces;
    constexpr uint64_t kCutUnit = 1ull << 20;
    std::vector<uint64_t> ps;
    std::vector<uint64_t> pd;
    std::vector<uint64_t> pl;
    uint64_t inPiece = 0;
    uint64_t left = total;
    auto flush = [&](bool last) -> int {
        if (ps.empty()) {
            return BM_OK;
        }
        const int ret = SubmitOne(ps.data(), pd.data(), pl.data(), static_cast<uint32_t>(ps.size()), route, stream, last ? mask : nullptr,
                                  maskValue, false, false);
        ps.clear();
        pd.clear();
        pl.clear();
        inPiece = 0;
        return ret;
    };
    for (uint32_t i = 0; i < n; ++i) {
        uint64_t at = 0;
        while (at < len[i]) {
            uint64_t take = len[i] - at;
            const uint64_t room = target > inPiece ? target - inPiece : 0;
            // what is left behind this piece must still make a launch of its own, else it stays with this one
            if (take > room && left - room >= kWindowPieceBytes) {
                const uint64_t cut = room / kCutUnit * kCutUnit;
                if (take >= 16 * kCutUnit && cut != 0 && take - cut >= kCutUnit) {
                    take = cut;
                } else if (inPiece != 0 && room < take / 2) {
                    const int ret = flush(false);      // the segment starts the next piece whole
                    if (ret != BM_OK) {
                        return ret;
                    }
                    continue;
                }
            }
            ps.push_back(src[i] + at);
            pd.push_back(dst[i] + at);
            pl.push_back(take);
            at += take;
            inPiece += take;
            left -= take;
            if (inPiece >= target && left >= kWindowPieceBytes) {
                const int ret = flush(false);
                if (ret != BM_OK) {
                    return ret;
                }
            }
        }
    }
    return flush(true);
}

// maySlice: a table of long segments may be cut into launches of kInlineSegs segments; a slice is submitted
// with false, so that one that cannot take the kernel-argument form (a segment of 4 GiB and more is cut into
// pieces, which can carry it past kInlineSegs rows) goes to the table form instead of being sliced again.
int XcopyEngine::SubmitOne(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n, int route,
                           void *stream, void *mask, uint32_t maskValue, bool unordered, bool maySlice)
{
    if (!Started()) {
        MF_FAIL(BM_NOT_INITIALIZED, "xcopy engine not started");
    }
    if (mfrt_bind_thread() != 0) {
        MF_FAIL(BM_ERROR, "cannot make the GPU current on this thread");
    }
    ThreadCtx &ctx = t_ctx;
    const uint32_t cu = mfrt_cu_count();
    InlinePlan plan;
    if (stream == nullptr) {
        // An unordered batch that can travel in the kernel arguments is handed to one of the submit threads in turn, where
        // the caller asked for them: launched there in order on the submitter's stream, beside whatever the others launch.
        const uint32_t fanCount = tuning_.unorderedStreams < kFanStreams ? tuning_.unorderedStreams : kFanStreams;
        if (unordered && fanCount >= 2 && n <= kInlineSegs && mask == nullptr && route == MFRT_ROUTE_HBM) {
            uint64_t total = 0;
            for (uint32_t i = 0; i < n; ++i) {
                total += len[i];
            }
            const uint32_t fanUnits = ChooseUnits(total, cu, route, tuning_);
            if (total <= kFanMaxBytes && BuildInlineDirect(src, dst, len, n, fanUnits, plan)) {
                ThreadLease &lease = ctx.Lease();
                if (lease.stream == nullptr && ThreadStream() == nullptr) {
                    MF_FAIL(BM_ERROR, "cannot create the thread's stream");
                }
                const uint32_t w = lease.fanCursor % fanCount;
                Submitter *sub = Submitters().Get(w);
                if (sub != nullptr) {
                    lease.fanCursor = w + 1;
                    if (plan.nchunk != 0) {
                        const uint32_t grid = GridFor(plan.nchunk, cu, route, tuning_);
                        const uint32_t hold = tuning_.holdOnSideStreams ? HoldFor(plan, grid, route, false) : 0;
                        lease.fanTicket[w] = sub->Push(plan, route, grid, hold);
                        lease.fanDirty |= 1u << w;
                        g_launches.fetch_add(1, std::memory_order_relaxed);
                        NotePending(lease.stream, total);   // the thread's next wait covers the submitters' streams
                    }
                    return BM_OK;
                }
            }
        }
        stream = ThreadStream();
        if (stream == nullptr) {
            MF_FAIL(BM_ERROR, "cannot create the thread's stream");
        }
    }
    bool inlined = false;
    uint32_t units = 0;
    bool oversized = false;      // a run the 32-bit length of the inline table cannot hold is possible
    bool windowed = false;
    uint32_t windowRate = tuning_.windowMBps;
    uint64_t queuedBytes = 0;
    if (n <= 4 * kInlineSegs) {  // small enough that a failed attempt costs next to nothing
        uint64_t total = 0;
        uint64_t addressBits = 0;      // low bits any source or destination address has set
        uint64_t apartBits = 0;        // low bits in which a source differs from its destination
        for (uint32_t i = 0; i < n; ++i) {
            total += len[i];
            addressBits |= src[i] | dst[i];
            apartBits |= src[i] ^ dst[i];
        }
        queuedBytes = total;
        oversized = total > 0xFFFFFFFFull;
        units = ChooseUnits(total, cu, route, tuning_);
        // Large HBM copies of one submitter: 16 KiB chunks for the kernel that alternates between read and write windows.
        // Not where a source and its destination differ modulo 16: the kernels align their 128-bit units on the destination,
        // the loads then straddle units, cost twice the issue slots, and the waves keep no schedule at any rate that pays
        // (100 segments of 10 MB: 5.35 TB/s in windows cut for 6.8, 5.26 for 7.4, 5.51 to 5.56 without windows).
        const bool aligned = (addressBits & (kWindowAlignBytes - 1)) == 0;
        windowed = !unordered && (apartBits & (kUnitBytes - 1)) == 0 && WindowsApply(total, route, kWindowMinBytes);
        // Segments that all start on cache lines, in source and destination, hold a higher rate.  Back to back at 6.8 / 7.1 /
        // 7.4 TB/s, the same in four processes: 2 GiB in one segment 6.65 / 6.95 / 7.02 to 7.27, 32 x 16 MiB 6.65 / 6.95 / 7.05 to
        // 7.26, 128 x 9 MiB 6.65 / 6.95 / 6.76 to 7.32.  The reshard's launches of 128 segments of 0.4 to 17 MB from eight
        // places hold 7.1 in every process (6.87 to 7.00) and 7.4 only in some (7.0 to 7.2 in one, 5.8 to 6.1 in three others):
        // long segments take the highest rate, other aligned ones the one between.  Where segments start between cache lines
        // every wave's kilobyte straddles a line it shares with its neighbour; such launches hold 6.8 (6.24 to 6.27 against 5.65
        // to 5.80 TB/s without windows) and fall apart at 7.4 (5.36 to 5.48).
        const bool longSegments = windowed && total / n >= kWindowLongSegmentBytes;
        if (longSegments && maySlice && total >= 2 * kWindowPieceBytes) {
            // A windowed launch that loses its schedule runs the rest of its bytes at the rate without windows, and the longer
            // it runs the likelier that is: launches of kWindowPieceBytes to twice that, each with a schedule of its own, hold
            // a target the whole copy in one launch does not (2 GiB at 7.4 TB/s: 7.1 TB/s on average in four launches,
            // 6.6 to 6.8 in one).  Only long segments are worth it: 896 segments of some 10 MB in launches of 64 or 96
            // segments (600 to 900 MB) were no faster than in launches of 128.
            return SubmitInPieces(src, dst, len, n, total, route, stream, mask, maskValue);
        }
        windowRate = tuning_.windowMBps;
        if (aligned && longSegments && tuning_.windowLongMBps != 0) {
            windowRate = tuning_.windowLongMBps;
        } else if (aligned && tuning_.windowAlignedMBps != 0) {
            windowRate = tuning_.windowAlignedMBps;
        }
        if (windowed) {
            units = mfk_xcopy_window_units();
        }
        const bool deep = !windowed && DeepHoldApplies(total, n, route, unordered);
        inlined = BuildInlineDirect(src, dst, len, n, deep ? kDeepUnits : units, plan);
        if (inlined && deep && HoldNanosFor(plan.nchunk, plan.nchunk, kDeepUnits, false) == 0) {
            inlined = BuildInlineDirect(src, dst, len, n, units, plan);   // ragged enough to exceed the waves that hold: the usual chunks
        }
    }
    if (!inlined && oversized) {
        // a run of 4 GiB and more may have made the one-pass attempt give up: the general inline path cuts it into pieces
        NormalizeSegments(src, dst, len, n, kInlinePiece, ctx.segs);
        units = windowed ? mfk_xcopy_window_units() : ChooseUnits(ctx.segs.totalBytes, cu, route, tuning_);
        inlined = BuildInlinePlan(ctx.segs, units, plan);
    }
    if (inlined && windowed) {
        int err = mfk_xcopy_windowed(&plan, windowRate, mask, maskValue, stream);
        if (err != 0) {
            MF_FAIL(BM_ERROR, "xcopy launch failed: " << mfrt_error_string(err));
        }
        g_launches.fetch_add(1, std::memory_order_relaxed);
        NotePending(stream, queuedBytes);
        return BM_OK;
    }
    if (inlined) {
        const uint32_t grid = GridFor(plan.nchunk, cu, route, tuning_);
        // a completion word is stored by a launch of its own behind the copy, which an unordered copy would not hold back
        int err = mfk_xcopy_inline(&plan, route, grid, mask, maskValue, stream, unordered && mask == nullptr ? 1 : 0,
                                   HoldFor(plan, grid, route, unordered));
        if (err != 0) {
            MF_FAIL(BM_ERROR, "xcopy launch failed: " << mfrt_error_string(err));
        }
        g_launches.fetch_add(1, std::memory_order_relaxed);
        NotePending(stream, queuedBytes);
        return BM_OK;
    }

    // Table form: {triples, prefix} are built in a pinned slot; the general form moves them to HBM
    // with a copy launch and searches them there.  The slot is sized for n segments; merging can only make the table shorter.
    bool deepTable = false;
    {
        uint64_t total = 0;
        uint64_t longest = 0;
        uint64_t addressBits = 0;
        for (uint32_t i = 0; i < n; ++i) {
            total += len[i];
            longest = len[i] > longest ? len[i] : longest;
            addressBits |= src[i] | dst[i];
        }
        queuedBytes = total;
        // A table of long segments between HBM addresses is cut into launches of kInlineSegs segments, each of which
        // then takes the form with read and write windows: the few extra launches cost microseconds, the windows
        // gain 8 % (896 segments, 8.5 GB: 2.55 ms in seven launches against 2.78 ms in one).  Segments on cache lines
        // are worth it from 1 MiB each, 128 MiB a launch (1024 x 1 MiB 327 against 361 us, 1024 x 2 MiB 658 against
        // 753 to 772 us, 512 x 3 MiB 458 against 588 us; 1024 x 512 KiB, 64 MiB a launch, the same either way).  The table form
        // itself was measured under windows three times, with the prefix search it once had, with the division and
        // group map it has now, and with full periods at rates from 6.0 to 7.1 TB/s, and is left without them: 262 144
        // pages of 32 KiB at random places lose 7 to 12 % (3.23 to 3.45 against 3.04 ms; the third time 2.93 to 3.38
        // against 2.89 to 3.06), 4096 pages take 58 to 60 instead of 46.5 to 49 us, 16 384 ragged segments lose 3 %, and
        // the 896 long segments in one windowed table launch are no faster than in seven launches of the kernel-argument form.
        if (maySlice && n > kInlineSegs && route == MFRT_ROUTE_HBM && !unordered && tuning_.windowMBps != 0 && windowsAvailable_ &&
            tuning_.unitsOverride == 0 &&
            total / n >= ((addressBits & (kWindowAlignBytes - 1)) == 0 && tuning_.windowAlignedMBps != 0 ? kWindowSliceMinAlignedSegmentBytes
                                                                                                         : kWindowSliceMinSegmentBytes) &&
            g_leasesOut.load(std::memory_order_relaxed) <= 1) {
            for (uint32_t at = 0; at < n; at += kInlineSegs) {
                const uint32_t m = n - at < kInlineSegs ? n - at : kInlineSegs;
                const bool last = at + m == n;
                const int ret = SubmitOne(src + at, dst + at, len + at, m, route, stream, last ? mask : nullptr, maskValue, false,
                                          true);
                if (ret != BM_OK) {
                    return ret;
                }
            }
            return BM_OK;
        }
        units = ChooseUnits(total, cu, route, tuning_);
        deepTable = DeepHoldApplies(total, n, route, unordered);
        // Many short segments: a chunk size that holds the longest of them gives every segment exactly
        // one chunk, which is the equal-count form below (no prefix, no search, no upload): 16 384
        // segments of 2-14 KB take 62 us instead of 74 us.
        if (tuning_.unitsOverride == 0 && longest != 0 && !deepTable) {
            for (uint32_t u = units; u <= 4 * kXcopyThreads; u *= 2) {
                if (longest <= static_cast<uint64_t>(u) * kUnitBytes - kUnitBytes) {
                    units = u;
                    break;
                }
            }
        }
    }
    // Slot layout: triples | prefix | group map.  The map's size follows from the chunk count, which is bounded
    // here by one chunk per segment plus one per full chunk of payload.
    const uint64_t tripleBytes = 24ull * n;
    const uint64_t prefixBytes = RoundUp(4ull * (n + 1), 8);
    const uint64_t chunkBound = static_cast<uint64_t>(n) + queuedBytes / (static_cast<uint64_t>(units) * kUnitBytes);
    const uint32_t groupCapacity = static_cast<uint32_t>(
        std::min<uint64_t>(GroupCapacityFor(n), (chunkBound >> kGroupShiftMin) + 2));
    const uint64_t slotBytes = RoundUp(tripleBytes + prefixBytes + 4ull * groupCapacity, kUnitBytes);
    StagingSlot *slot = nullptr;
    ThreadLease &lease = ctx.Lease();
    int ret = AcquireSlot(lease, slotBytes, stream, slot);
    if (ret != BM_OK) {
        return ret;
    }
    uint64_t *triples = static_cast<uint64_t *>(slot->host);
    uint32_t *first = reinterpret_cast<uint32_t *>(static_cast<uint8_t *>(slot->host) + tripleBytes);
    uint32_t count = 0;
    ChunkPattern pattern;
    uint64_t nchunk = 0;
    if (deepTable) {
        nchunk = BuildTableDirect(src, dst, len, n, kDeepUnits, triples, first, count, &pattern);
        if (HoldNanosFor(static_cast<uint32_t>(nchunk < kNoChunk ? nchunk : 0), static_cast<uint32_t>(nchunk), kDeepUnits, false) != 0) {
            units = kDeepUnits;
        } else {
            deepTable = false;   // ragged enough to exceed the waves that hold: the usual chunks
        }
    }
    if (!deepTable) {
        nchunk = BuildTableDirect(src, dst, len, n, units, triples, first, count, &pattern);
    }
    if (nchunk >= kNoChunk) {
        MF_FAIL(BM_INVALID_PARAM, "batch too large for one launch: " << nchunk << " chunks");
    }
    if (count == 0) {   // nothing but empty segments
        InlinePlan empty;
        SegList none;
        (void)BuildInlinePlan(none, kXcopyThreads, empty);
        int err = mfk_xcopy_inline(&empty, route, 1, mask, maskValue, stream, 0, 0);
        return err == 0 ? BM_OK : BM_ERROR;
    }

    const uint32_t grid = GridFor(nchunk, cu, route, tuning_);
    TablePlan table{};
    table.nseg = count;
    table.nchunk = static_cast<uint32_t>(nchunk);
    table.units = units;
    int err = 0;
    // Chunk counts that repeat (pages of one size, K and V blocks in turn): a workgroup finds its descriptor by
    // a division and a few comparisons, so the only thing it needs from the table is that one descriptor, which it
    // can read straight out of the pinned slot.  No upload launch, nothing serial in front of the copy (a 4096-page
    // gather on an idle stream: 50 us instead of 55); the 64 bytes per workgroup that cross the host link stay
    // below 2 % of the payload rate.  (Uploading the table by a launch of its own that carries no barrier, so that
    // it runs beside the caller's earlier copies, was measured for these batches too: the extra launch costs the
    // stream 2 us whether it overlaps or not, more than the fetch from HBM saves: 36 MB of K and V blocks 20.5
    // against 18.4 us per call.)
    if (pattern.period != 0) {
        const uint32_t hold = HoldForTable(static_cast<uint32_t>(nchunk), grid, units, route, unordered, true);
        table.triples = triples;
        table.pattern = pattern;
        err = mfk_xcopy_table(&table, route, grid, mask, maskValue, stream, hold);
        g_launches.fetch_add(1, std::memory_order_relaxed);
    } else {
        // Ragged segments: prefix and group map go to HBM with the triples (with them in host memory every
        // step of the lookup is a link round trip: 16 384 ragged segments 135 us against 74).  The upload is
        // launched without a barrier: the slot's device half is free (AcquireSlot has waited for its last
        // reader), so it may run while the caller's earlier copies still do; the table launch behind it waits
        // for both.
        uint32_t *group = reinterpret_cast<uint32_t *>(static_cast<uint8_t *>(slot->host) + tripleBytes + prefixBytes);
        table.groupShift = BuildGroupMap(first, count, group, groupCapacity);
        const uint64_t usedBytes =
            RoundUp(tripleBytes + prefixBytes + 4ull * (GroupCount(nchunk, table.groupShift) + 1), kUnitBytes);
        ret = EnsureDevice(*slot, slotBytes);
        if (ret != BM_OK) {
            return ret;
        }
        const uint64_t hostAddr = reinterpret_cast<uint64_t>(slot->host);
        const uint64_t devAddr = reinterpret_cast<uint64_t>(slot->dev);
        InlinePlan stagePlan;
        if (!BuildInlineDirect(&hostAddr, &devAddr, &usedBytes, 1, kXcopyThreads, stagePlan)) {
            MF_FAIL(BM_INVALID_PARAM, "descriptor table of " << usedBytes << " bytes is too large");
        }
        err = mfk_xcopy_inline(&stagePlan, MFRT_ROUTE_FROM_HOST, stagePlan.nchunk, nullptr, 0, stream,
                               tuning_.stageUnordered ? 1 : 0, 0);
        if (err != 0) {
            MF_FAIL(BM_ERROR, "descriptor staging launch failed: " << mfrt_error_string(err));
        }
        const uint8_t *devBase = static_cast<const uint8_t *>(slot->dev);
        table.triples = reinterpret_cast<const uint64_t *>(devBase);
        table.first = reinterpret_cast<const uint32_t *>(devBase + tripleBytes);
        table.group = reinterpret_cast<const uint32_t *>(devBase + tripleBytes + prefixBytes);
        err = mfk_xcopy_table(&table, route, grid, mask, maskValue, stream,
                              HoldForTable(static_cast<uint32_t>(nchunk), grid, units, route, unordered, false));
        g_launches.fetch_add(2, std::memory_order_relaxed);
    }
    if (err != 0) {
        // an earlier launch may still be reading the slot: keep it reserved until the stream has passed this point
        (void)MarkQueued(lease, slot, stream, true);
        MF_FAIL(BM_ERROR, "xcopy table launch failed: " << mfrt_error_string(err));
    }
    NotePending(stream, queuedBytes);
    return MarkQueued(lease, slot, stream, false);
}

int XcopyEngine::SubmitDeviceTable(const void *triples, uint32_t n, int route, void *stream, void *mask,
                                   uint32_t maskValue)
{
    if (!Started()) {
        MF_FAIL(BM_NOT_INITIALIZED, "xcopy engine not started");
    }
    if (mfrt_bind_thread() != 0) {
        MF_FAIL(BM_ERROR, "cannot make the GPU current on this thread");
    }
    if (stream == nullptr) {
        stream = ThreadStream();
        if (stream == nullptr) {
            MF_FAIL(BM_ERROR, "cannot create the thread's stream");
        }
    }
    if (n == 0) {
        InlinePlan empty;
        SegList none;
        (void)BuildInlinePlan(none, kXcopyThreads, empty);
        int err = mfk_xcopy_inline(&empty, route, 1, mask, maskValue, stream, 0, 0);
        return err == 0 ? BM_OK : BM_ERROR;
    }
    // Prefix, group map and pattern are computed on the GPU; their slot is only ever touched by kernels of this stream.
    ThreadCtx &ctx = t_ctx;
    StagingSlot *slot = nullptr;
    const uint32_t groupCapacity = GroupCapacityFor(n);
    const uint64_t scratchBytes = RoundUp(4ull * mfk_xcopy_plan_scratch_words(n, groupCapacity), kUnitBytes);
    ThreadLease &lease = ctx.Lease();
    int ret = AcquireSlot(lease, 0, stream, slot);
    if (ret == BM_OK) {
        ret = EnsureDevice(*slot, scratchBytes);
    }
    if (ret != BM_OK) {
        return ret;
    }
    const uint32_t cu = mfrt_cu_count();
    const uint32_t units = ChooseUnits(0, cu, route, tuning_);   // sizes are only known on the GPU
    TablePlan table;
    int err = mfk_xcopy_plan(triples, n, units, slot->dev, groupCapacity, &table, stream);
    if (err != 0) {
        MF_FAIL(BM_ERROR, "xcopy plan launch failed: " << mfrt_error_string(err));
    }
    const uint32_t grid = DeviceTableGrid(n, cu, route, tuning_);
    err = mfk_xcopy_table(&table, route, grid, mask, maskValue, stream, 0);
    if (err != 0) {
        (void)MarkQueued(lease, slot, stream, true);   // the plan launch writes the slot
        MF_FAIL(BM_ERROR, "xcopy table launch failed: " << mfrt_error_string(err));
    }
    g_launches.fetch_add(2, std::memory_order_relaxed);
    NotePending(stream, ~0ull);   // sizes unknown here: the next wait sleeps on the stream
    return MarkQueued(lease, slot, stream, false);
}

#ifndef MF_RT_HIDDEN
int XcopyEngine::SubmitDeviceTableStatic(const void *triples, uint32_t n, int route, void *stream)
{
    if (!Started()) {
        MF_FAIL(BM_NOT_INITIALIZED, "xcopy engine not started");
    }
    if (n > MFK_STATIC_TABLE_SEGMENTS) {
        MF_FAIL(BM_INVALID_PARAM, "table of " << n << " segments exceeds the " << MFK_STATIC_TABLE_SEGMENTS
                << " the statically allocated scratch holds; split the table or use mf_xcopy_device_table");
    }
    if (n == 0) {
        return BM_OK;
    }
    if (mfrt_bind_thread() != 0) {
        MF_FAIL(BM_ERROR, "cannot make the GPU current on this thread");
    }
    const uint32_t cu = mfrt_cu_count();
    const uint32_t units = ChooseUnits(0, cu, route, tuning_);   // sizes are only known on the GPU
    const uint32_t grid = DeviceTableGrid(n, cu, route, tuning_);
    const int err = mfk_xcopy_table_static(triples, n, units, route, grid, stream);
    if (err != 0) {
        MF_FAIL(BM_ERROR, "static-scratch table launch failed (" << err << ")");
    }
    g_launches.fetch_add(2, std::memory_order_relaxed);
    NotePending(stream, ~0ull);
    return BM_OK;
}
#endif

}  // namespace mf
