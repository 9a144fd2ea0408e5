// Host planner and submission engine of the xcopy kernels (plain C++, no HIP
// types).  It turns a caller's segment list into one fused kernel launch on a
// stream: the job HostDataOpSDMA::BatchCopyG2G / BatchCopyExtend do with one
// SDMA descriptor per segment or a 32-block plugin launch
// (src/hybm/csrc/data_operation/host/hybm_data_op_sdma.cpp:504-595).
#ifndef MF_XCOPY_ENGINE_H
#define MF_XCOPY_ENGINE_H

#include <stdint.h>

#include <atomic>
#include <vector>

#include "../kernels/xcopy_plan.h"

namespace mf {

// Segment list after normalisation: empty segments dropped, neighbours that
// continue each other on both sides merged (the reference merges the same
// way before building descriptors, hybm_data_op_sdma.cpp:571-574).
struct SegList {
    std::vector<uint64_t> src;
    std::vector<uint64_t> dst;
    std::vector<uint64_t> len;
    uint64_t totalBytes = 0;
    void Clear()
    {
        src.clear();
        dst.clear();
        len.clear();
        totalBytes = 0;
    }
    uint32_t Size() const
    {
        return static_cast<uint32_t>(src.size());
    }
};

// pieceLimit: segments longer than this are cut into pieces of at most that
// many bytes (the inline plan stores 32-bit lengths); 0 = never cut.
void NormalizeSegments(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n, uint64_t pieceLimit,
                       SegList &out);

struct XcopyTuning {
    uint32_t unitsOverride = 0;  // 16-byte units per chunk, 0 = choose from batch size
    uint32_t wgPerCu = 0;        // HBM routes: grid cap in workgroups per CU, 0 = one workgroup per chunk
    uint32_t wgPerCuLink = 1;    // routes bound by the host link: workgroups per CU
    uint32_t minUnits = kXcopyThreads;   // 4 KiB: the chunk of HBM routes
    int32_t holdNanos = -1;      // stores held back in inline launches: -1 = HoldNanosFor's rule (+ holdDeltaNanos), 0 = never, else that long
    int32_t holdDeltaNanos = 0;  // added to the rule's wait: what the calibration at start found best on this GPU
    bool holdCalibratedOff = false;   // the calibration found no gain in holding stores on this GPU
    uint32_t unorderedStreams = 0;   // unordered batches are launched by this many submit threads of the library's, a stream each (0, 1: by the caller on its own stream)
    bool holdOnSideStreams = false;  // launches of the submit threads overlap on purpose: their stores are not held
    bool deepHold = true;        // batches of 24 to 64 MiB hold the stores of 16 KiB per wave
    int32_t holdPinnedExtraNanos = 1600;   // added to the rule for table launches, whose descriptors come from pinned host memory: a link round trip before the loads
    bool stageUnordered = true;  // the upload of a ragged table's descriptors is launched without a barrier
    uint32_t deviceTableWgPerCu = 0;   // grid of a device-resident table in workgroups per CU, 0 = eight per segment between 32 and 4096 per CU
    uint32_t windowMBps = 6800000;   // HBM copies of kWindowRectMinBytes and more alternate between read and write windows cut for this rate; 0 = never
    uint32_t windowAlignedMBps = 7100000;   // the same for launches of segments that all start at multiples of kWindowAlignBytes in source and destination, which hold more; 0 = the rate above
    uint32_t windowLongMBps = 7400000;      // and for those of them whose segments are kWindowLongSegmentBytes and longer on average, which hold more still; 0 = the rate above
};

// From this total on a batch of up to 128 segments between HBM addresses is copied in read and write windows.
// Segments on cache lines, paced for windowAlignedMBps, gain from where the held stores of 16 KiB per wave end:
// back to back, 32 segments, windows against none: 66 MiB 6.37 against 5.71 TB/s, 80 MiB 6.57 against 5.76, 130 MiB
// 6.94 against 6.14, 256 MiB 7.14 against 6.37, 600 MiB 7.20 against 6.31 (at 64 MiB and below the held stores are
// as fast).  A launch on its own gains less and less steadily below 128 MiB (80 MiB: 32.4 against 31.9 us), hence
// the limit.  Segments between cache lines, paced for windowMBps, gain 5 to 7 % from there on (136 MB 43.7 against
// 46.8 us, 272 MB 85 against 91.5, 407 MB 129.5 against 137).  Rectangles do not below 512 MiB (136 MB 45 against
// 47 us, but 407 MB 141 against 136): they keep the limit they were measured at.
constexpr uint64_t kWindowMinBytes = 128ull << 20;
constexpr uint64_t kWindowRectMinBytes = 512ull << 20;
constexpr uint64_t kWindowPieceBytes = 512ull << 20;          // launches into which long segments are cut
constexpr uint64_t kWindowLongSegmentBytes = 64ull << 20;     // launches whose segments average this much go out in pieces of kWindowPieceBytes and more
constexpr int32_t kHoldLookupExtraNanos = 800;                // on top of the rule where a table launch finds its descriptors through the group map
constexpr int32_t kHoldLookupDeepExtraNanos = 500;            // the same on 16 KiB chunks
constexpr int32_t kHoldPinnedDeepExtraNanos = 800;            // on top of holdPinnedExtraNanos where a table launch works on 16 KiB chunks
constexpr uint64_t kWindowAlignBytes = 128;                   // a cache line: segments that start on one are read and written in whole lines by every wave
constexpr uint64_t kWindowSliceMinSegmentBytes = 4ull << 20;   // tables of segments this long on average are cut into windowed launches
constexpr uint64_t kWindowSliceMinAlignedSegmentBytes = 1ull << 20;   // the same for segments on cache lines: kInlineSegs of them reach kWindowMinBytes

// What Start() measured on the GPU it runs on and chose from it (XcopyEngine::Calibrate).
struct XcopyCalibration {
    bool ran = false;               // false: skipped (MF_HIP_CALIBRATE=0), failed, or not run yet: the fitted defaults apply
    bool holdEnabled = true;        // the held stores beat the launch that stores at once by kCalibrateMinGain
    int32_t holdDeltaNanos = 0;     // added to every wait HoldNanosFor gives
    uint32_t windowMBps = 0;        // rate the read and write windows are cut for; 0: the form lost against the plain kernel
    uint32_t windowAlignedMBps = 0;    // rate for launches of segments on cache-line boundaries
    uint32_t windowLongMBps = 0;       // rate for launches of long segments on cache-line boundaries; both the higher ones where a long copy held the highest, else the rate above
    float batchMicros[4] = {};      // 2196-chunk batch: not held, rule - step, rule, rule + step
    float copyMicros[4] = {};       // 512 MiB copy: no windows, default rate, reduced rate, the rate of long segments on cache lines
};
constexpr int32_t kCalibrateHoldStepNanos = 200;
constexpr float kCalibrateMinGain = 0.03f;          // held stores that do not gain this much over the plain launch are switched off
constexpr float kCalibrateMinWindowGain = 0.005f;   // windows stay unless they lose: on the 512 MiB that is measured they gain least (2 to 5 %, 8 % on 1 GiB)
constexpr uint32_t kCalibrateSlowerWindowPercent = 94;   // the second window rate tried, in percent of the default
// The choice, from the measured times alone (microseconds; a time of 0 means "not measured" and leaves the default).
void ChooseCalibration(const float *batchMicros, const float *copyMicros, uint32_t defaultWindowMBps, uint32_t defaultAlignedMBps, uint32_t defaultLongMBps,
                       XcopyCalibration &out);

uint32_t ChooseUnits(uint64_t totalBytes, uint32_t cuCount, int route, const XcopyTuning &tuning);

// Returns false when the list does not fit the inline form.
bool BuildInlinePlan(const SegList &segs, uint32_t units, InlinePlan &plan);

// The same result as NormalizeSegments + BuildInlinePlan in one pass over the caller's arrays;
// false when the batch does not fit the inline form (more than kInlineSegs merged segments, or
// one of 4 GiB and more, which the general path cuts into pieces).
bool BuildInlineDirect(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n, uint32_t units,
                       InlinePlan &plan);

// triples: 3 * segs.Size() words, first: segs.Size() + 1 words.  Returns total chunks.
uint64_t BuildTablePlan(const SegList &segs, uint32_t units, uint64_t *triples, uint32_t *first);

// The same result as NormalizeSegments (no piece limit) + BuildTablePlan in one pass over the
// caller's arrays.  triples: room for 3 * n words, first: room for n + 1; count = segments written.
// pattern (optional) receives the shortest period (up to kMaxPeriod) with which the chunk counts
// of the segments repeat, period 0 when there is none.
uint64_t BuildTableDirect(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n, uint32_t units,
                          uint64_t *triples, uint32_t *first, uint32_t &count, ChunkPattern *pattern = nullptr);

class XcopyEngine {
public:
    static XcopyEngine &Instance();

    int Start(int device);          // BM_* code
    void Stop();
    bool Started() const;

    XcopyTuning &Tuning()
    {
        return tuning_;
    }
    const XcopyCalibration &Calibration() const
    {
        return calibration_;
    }
    // Measures, on the calling thread's stream, the 2196-chunk batch with its stores not held and held for the rule's wait
    // and kCalibrateHoldStepNanos either side of it, and a 512 MiB copy without windows and at two window rates; keeps
    // the best wait (or none) and the best rate (or none) for the process.  About 15 ms and 1 GiB of HBM for its duration.
    // Start() runs it unless the environment says MF_HIP_CALIBRATE=0.
    int Calibrate();

    // Whether an ordered launch that moves `bytes` on `route` takes the form with read and write windows.
    bool WindowsApply(uint64_t bytes, int route, uint64_t minBytes = kWindowRectMinBytes) const;
    // Hardware queue (numbered in order of appearance) of each of the streams made at Start(), in the order they are handed out; returns their number.
    uint32_t StreamQueues(uint32_t *queues, uint32_t capacity) const;
    // No second thread holds a stream of the library: kernels that pace themselves for the whole chip may be used.
    bool SingleSubmitter() const;

    // The calling thread's own stream (created on first use).  Unordered batches that were handed to the submit
    // threads are joined first: work queued on the returned stream afterwards waits for them.
    void *ThreadStream();
    static constexpr uint32_t kFanStreams = 8;   // most submit threads for unordered batches (9 MB batches: 2 / 3 / 4 / 6 / 8 threads 4.3 / 3.8 / 3.6 / 3.8 / 3.6-4.0 us per batch)
    static constexpr uint32_t kDeckStreams = 8;   // streams made at Start() and dealt out so that consecutive takers sit on different hardware queues
    static constexpr uint64_t kFanMaxBytes = 64ull << 20;   // larger batches gain nothing from a second queue
    // Pinned, device-mapped staging memory of the calling thread, at least `bytes` long; it lives
    // until Stop().  NULL when it cannot be allocated.
    void *ThreadBounce(uint64_t bytes);
    // One of the calling thread's events for slots of that staging memory (index < kBounceEvents).
    static constexpr uint32_t kBounceEvents = 16;
    void *ThreadBounceEvent(uint32_t index);
    // Wait for everything this thread enqueued on its own stream.
    int DrainThread();
    // Wait for everything queued on `stream` so far: what a blocking copy does after its launch.
    // Work expected to be short (`bytes` moved, 0 = unknown) is awaited by polling a word in pinned
    // memory that a one-lane launch behind the copy stores, for at most kSpinMicros; anything else,
    // and a poll that runs out of time, waits on the stream.
    static constexpr uint64_t kSpinBytes = 256ull << 20;
    static constexpr uint32_t kSpinMicros = 200;
    int WaitStream(void *stream, uint64_t bytes);
    // Work that another part of the library has queued on `stream`: if it is the calling thread's own stream, the next
    // DrainThread() takes `bytes` into account when it chooses between polling and sleeping (~0: sleep).
    void NoteQueued(void *stream, uint64_t bytes);

    // Enqueue one batch.  Addresses must be device-accessible.  stream may be
    // NULL (thread stream).  mask/maskValue: plugin completion word or NULL.
    // Returns 0 or a negative BM_* code; never waits for the copy itself.
    // unordered: the caller vouches that the batch is independent of everything still in flight on
    // `stream`; a batch that fits the kernel-argument form is then launched without a barrier.
    int Submit(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n, int route, void *stream,
               void *mask, uint32_t maskValue, bool unordered = false);

    // Same for a triple table that lives in device memory the host cannot read.
    int SubmitDeviceTable(const void *triples, uint32_t n, int route, void *stream, void *mask, uint32_t maskValue);

    // The same, with the chunk prefix in the statically allocated device scratch: allocates nothing
    // (no stream either: `stream` is used as given, NULL being the null stream), at most
    // MFK_STATIC_TABLE_SEGMENTS segments, calls on one GPU must not overlap.
    int SubmitDeviceTableStatic(const void *triples, uint32_t n, int route, void *stream);

    // Returns once every batch handed to the submit threads so far has been launched (a device wait then covers it).
    void QuiesceSubmitters();

    uint64_t LaunchCount() const;

private:
    XcopyEngine() = default;

    uint32_t HoldFor(const InlinePlan &plan, uint32_t grid, int route, bool unordered) const;
    uint32_t HoldForTable(uint32_t nchunk, uint32_t grid, uint32_t units, int route, bool unordered, bool pinned) const;
    // Whether a batch of `bytes` in n segments is planned in chunks of kDeepUnits units, to hold the stores of 16 KiB per wave.
    bool DeepHoldApplies(uint64_t bytes, uint32_t n, int route, bool unordered) const;
    int SubmitInPieces(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n, uint64_t total, int route,
                       void *stream, void *mask, uint32_t maskValue);
    int SubmitOne(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n, int route, void *stream,
                  void *mask, uint32_t maskValue, bool unordered, bool maySlice);

    XcopyTuning tuning_;
    XcopyCalibration calibration_;
    bool windowRateCalibrated_ = false;  // tuning_.windowMBps holds what Calibrate() chose, not a caller's setting
    bool windowsAvailable_ = false;      // set by Start(): the device's constant-rate clock is known
    std::atomic<bool> started_{false};   // read by every calling thread, flipped by Start / Stop
};

}  // namespace mf

#endif  // MF_XCOPY_ENGINE_H
