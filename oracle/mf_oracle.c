/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of the reference's algorithms on
 * the xcopy path, used as the checker by tests/, by __graft_entry__.smoke()
 * and as the timed "cpu_baseline" leg of bench.py.  Nothing in the product
 * (memfabric_hybrid_amd/, include/) may link, load or call this file.
 *
 * Every function cites the reference code it restates (paths relative to the
 * reference tree).  How each one is pinned:
 *   orc_batch_copy / orc_copy        closed form (memcpy); also checked against the reference's own
 *                                    DlHybridApi::Memcpy built into oracle/_ref
 *   orc_lcg_fill / orc_lcg_mismatch  the reference's data pattern, known answers in tests/golden
 *   orc_direct_map / orc_infer_table / orc_check_map
 *                                    literal tables; the reference has no test for them
 *                                    ("parity unpinned" by reference tests) - cross-checked
 *                                    against an independent arithmetic derivation and, for
 *                                    orc_infer_table, against the reference's HybmVaManager in oracle/_ref
 *   orc_va_*                         known answers of test/ut/testcase/hybm/hybm_va_manager_test.cpp
 *                                    and the reference's HybmVaManager in oracle/_ref
 *   orc_gva_* / orc_mask48           closed-form integer arithmetic, brute-forced in tests
 *   orc_coalesce                     invariant: byte result unchanged
 *   orc_trans_*                      transfer front-end arithmetic; the reference's tests need two
 *                                    processes and a config store and hold no vectors for it
 *                                    ("parity unpinned" by reference tests) - pinned by closed forms
 *                                    (page hull is the minimal aligned cover), a brute-force
 *                                    page-bitmap union, and a linear-scan lookup
 *   orc_ref_kernel_*                 partition formulas of the AscendC kernel; pinned by coverage
 *                                    properties (no reference test exists)
 *   orc_moe_*                        NO reference implementation exists ("parity unpinned" by the
 *                                    reference): pinned by invariants and a torch argsort/index_add
 *                                    cross-check in tests
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------
 * Copies.  HostDataOpRDMA::BatchCopyLH2LH
 * (src/hybm/csrc/data_operation/host/hybm_data_op_host_rdma.cpp:697-709) calls,
 * per segment and in segment order, DlHybridApi::Memcpy whose host branch is
 * std::copy_n over chars with the guards kind == HOST_TO_HOST and
 * count <= destMax (src/hybm/csrc/under_api/dl_hybrid_api.h:157-168).
 * Returns 0 or -2 (BM_INVALID_PARAM) like that branch.
 * ---------------------------------------------------------------------- */
int32_t orc_copy(void *dst, uint64_t dstMax, const void *src, uint64_t count)
{
    if (count > dstMax) {
        return -2;
    }
    const char *s = (const char *)src;
    char *d = (char *)dst;
    for (uint64_t i = 0; i < count; ++i) { /* std::copy_n: forward, element by element */
        d[i] = s[i];
    }
    return 0;
}

int32_t orc_batch_copy(void *const *dsts, void *const *srcs, const uint64_t *counts, uint32_t batchSize)
{
    for (uint32_t i = 0; i < batchSize; ++i) {
        int32_t ret = orc_copy(dsts[i], counts[i], srcs[i], counts[i]);
        if (ret != 0) {
            return ret;
        }
    }
    return 0;
}

/* The same loop with libc memcpy: what an optimising build of the loop above
 * turns into; this is the variant the CPU baseline times. */
int32_t orc_batch_copy_fast(void *const *dsts, void *const *srcs, const uint64_t *counts, uint32_t batchSize)
{
    for (uint32_t i = 0; i < batchSize; ++i) {
        memcpy(dsts[i], srcs[i], counts[i]);
    }
    return 0;
}

/* Strided 2-D copy, the closed form the reshard workload reduces to. */
void orc_copy_2d(void *dst, uint64_t dpitch, const void *src, uint64_t spitch, uint64_t width, uint64_t height)
{
    for (uint64_t r = 0; r < height; ++r) {
        memcpy((char *)dst + r * dpitch, (const char *)src + r * spitch, width);
    }
}

/* ------------------------------------------------------------------------
 * Data pattern of the reference's benchmark and examples: GenerateData /
 * CheckData, example/bm/BmBenchmark/band_width_calculator.cpp:25-27,47-79
 * (identical in example/bm/BmCpp/main.cpp:47-49,59-90).
 * ---------------------------------------------------------------------- */
void orc_lcg_fill(void *ptr, int32_t rank, uint32_t len)
{
    if (ptr == NULL) {
        return;
    }
    int32_t *arr = (int32_t *)ptr;
    const int32_t mod = INT16_MAX;
    int32_t base = rank;
    for (uint32_t i = 0; i < len / sizeof(int); i++) {
        base = (base * 23 + 17) % mod;
        if ((i + rank) % 3 == 0) {
            arr[i] = -base;
        } else {
            arr[i] = base;
        }
    }
}

int64_t orc_lcg_mismatch(const void *base, const void *ptr, uint32_t len)
{
    int64_t wrong = 0;
    if (base == NULL || ptr == NULL) {
        return wrong;
    }
    const int32_t *a = (const int32_t *)base;
    const int32_t *b = (const int32_t *)ptr;
    for (uint32_t i = 0; i < len / sizeof(int); i++) {
        if (a[i] != b[i]) {
            wrong++;
        }
    }
    return wrong;
}

/* ------------------------------------------------------------------------
 * Direction tables, restated literally.
 * ---------------------------------------------------------------------- */
enum {
    LH2GH = 0, LH2GD = 1, LD2GH = 2, LD2GD = 3, GH2GH = 4, GH2GD = 5, GH2LH = 6, GH2LD = 7,
    GD2GH = 8, GD2GD = 9, GD2LH = 10, GD2LD = 11, DIR_AUTO = 12, DIR_BUTT = 13
};

/* directMap[src smem type][dst smem type], smem types LOCAL_DEVICE=0,
 * LOCAL_HOST=1, DEVICE=2, HOST=3, BUTT=4
 * (src/smem/csrc/smem_bm/smem_bm_entry.cpp:256-267). */
static const int32_t kDirectMap[5][5] = {
    {DIR_BUTT, DIR_BUTT, LD2GD, LD2GH, DIR_BUTT},
    {DIR_BUTT, DIR_BUTT, LH2GD, LH2GH, DIR_BUTT},
    {GD2LD, GD2LH, GD2GD, GD2GH, DIR_BUTT},
    {GH2LD, GH2LH, GH2GD, GH2GH, DIR_BUTT},
    {DIR_BUTT, DIR_BUTT, DIR_BUTT, DIR_BUTT, DIR_BUTT},
};

int32_t orc_direct_map(int32_t srcType, int32_t dstType)
{
    if (srcType < 0 || srcType > 4 || dstType < 0 || dstType > 4) {
        return DIR_BUTT;
    }
    return kDirectMap[srcType][dstType];
}

/* SmemBmEntry::TransToHybmDirection (smem_bm_entry.cpp:279-310): the pool
 * classification of each side is overridden by the copy type, then the table
 * decides.  Copy types: L2G 0, G2L 1, G2H 2, H2G 3, L2GH 4, GH2L 5, GH2H 6,
 * H2GH 7, G2G 8. */
int32_t orc_trans_direction(int32_t copyType, int32_t srcPoolType, int32_t dstPoolType)
{
    int32_t s = srcPoolType;
    int32_t d = dstPoolType;
    switch (copyType) {
        case 0: s = 0; break;
        case 1: d = 0; break;
        case 2: d = 1; break;
        case 3: s = 1; break;
        case 7: s = 1; break;
        case 6: d = 1; break;
        case 8:
        default: break;
    }
    return orc_direct_map(s, d);
}

/* COPY_DIRECTION_TABLE[src category][dst category], categories GLOBAL_DEVICE=0,
 * GLOBAL_HOST=1, LOCAL_DEVICE=2, LOCAL_HOST=3 (src/hybm/csrc/mm/hybm_va_manager.h:244-261). */
static const int32_t kInferTable[4][4] = {
    {GD2GD, GD2GH, GD2LD, GD2LH},
    {GH2GD, GH2GH, GH2LD, GH2LH},
    {LD2GD, LD2GH, DIR_BUTT, DIR_BUTT},
    {LH2GD, LH2GH, DIR_BUTT, DIR_BUTT},
};

int32_t orc_infer_table(int32_t srcCategory, int32_t dstCategory)
{
    if (srcCategory < 0 || srcCategory > 3 || dstCategory < 0 || dstCategory > 3) {
        return DIR_BUTT;
    }
    return kInferTable[srcCategory][dstCategory];
}

/* g_checkMap[direction] = {direction, check source, check destination}
 * (src/hybm/csrc/hybm_data_op_entry.cpp:24-30).  which: 1 = source, 2 = destination. */
static const uint32_t kCheckMap[12][3] = {
    {LH2GH, 0, 1}, {LH2GD, 0, 1}, {LD2GH, 0, 1}, {LD2GD, 0, 1}, {GH2GH, 1, 1}, {GH2GD, 1, 1},
    {GH2LH, 1, 0}, {GH2LD, 1, 0}, {GD2GH, 1, 1}, {GD2GD, 1, 1}, {GD2LH, 1, 0}, {GD2LD, 1, 0},
};

int32_t orc_check_map(int32_t direction, int32_t which)
{
    if (direction < 0 || direction > 11 || which < 1 || which > 2) {
        return 0;
    }
    return (int32_t)kCheckMap[direction][which];
}

/* ------------------------------------------------------------------------
 * Pool window arithmetic.
 * ---------------------------------------------------------------------- */
/* Valid48BitsAddress, src/hybm/csrc/common/hybm_define.h:77-80 */
uint64_t orc_mask48(uint64_t address)
{
    return address & 0xffffffffffffULL;
}

/* SmemBmEntry::AddrInHostGva / AddrInDeviceGva (smem_bm_entry.cpp:421-455) and
 * MemSegment::MemoryInRange (hybm_conn_based_segment.cpp:247-258): reject when
 * the window is absent, when addr + size lies past the end, when addr lies
 * before the base; in that order. */
int32_t orc_gva_contains(uint64_t base, uint64_t perRank, uint64_t rankCount, uint64_t addr, uint64_t size)
{
    if (base == 0) {
        return 0;
    }
    uint64_t total = perRank * rankCount;
    if (addr + size > base + total) {
        return 0;
    }
    if (addr < base) {
        return 0;
    }
    return 1;
}

/* SmemBmEntry::GetRankIdByGva (smem_bm_entry.cpp:337-347): probe of one byte,
 * divisor is the *VASpace of the window, UINT32_MAX when outside. */
uint32_t orc_gva_rank(uint64_t base, uint64_t perRank, uint64_t rankCount, uint64_t vaSpace, uint64_t addr)
{
    if (orc_gva_contains(base, perRank, rankCount, addr, 1) && vaSpace != 0) {
        return (uint32_t)((addr - base) / vaSpace);
    }
    return UINT32_MAX;
}

/* smem_bm_ptr_by_mem_type (src/smem/csrc/smem_bm/smem_bm.cpp:305-316) */
uint64_t orc_gva_ptr_of_rank(uint64_t base, uint64_t perRank, uint32_t rank)
{
    return base + perRank * rank;
}

/* DataOperator::GetRankIdByGva (src/hybm/csrc/data_operation/hybm_data_operator.h:78-90)
 * for one memory type. */
uint32_t orc_operator_rank(uint64_t gva, uint64_t base, uint64_t localSpace, uint64_t rankCount)
{
    if (gva >= base && gva < base + rankCount * localSpace) {
        return (uint32_t)((gva - base) / localSpace);
    }
    return UINT32_MAX;
}

/* ------------------------------------------------------------------------
 * Address registry (HybmVaManager, src/hybm/csrc/mm/hybm_va_manager.cpp:34-256)
 * restated over a flat array: small, obviously correct, O(n) per query.
 * mem types: DEVICE = 1, HOST = 2, BUTT = 3.
 * ---------------------------------------------------------------------- */
#define ORC_VA_MAX 1024
typedef struct {
    uint64_t gva, size, lva;
    int32_t memType;
    uint32_t localRank, importedRank;
    int used;
} orc_va_entry;
typedef struct {
    uint64_t start, size;
    int32_t memType;
    int used;
} orc_rsv_entry;
static orc_va_entry g_va[ORC_VA_MAX];
static orc_rsv_entry g_rsv[ORC_VA_MAX];

void orc_va_clear(void)
{
    memset(g_va, 0, sizeof(g_va));
    memset(g_rsv, 0, sizeof(g_rsv));
}

static uint32_t va_rank(const orc_va_entry *e)
{
    return e->importedRank != UINT32_MAX ? e->importedRank : e->localRank;
}

/* AddVaInfo (.cpp:34-66): gva 0 is an error, size 0 is accepted and ignored,
 * overlap is judged among ranges of the same memory type only, re-adding an
 * identical range (same gva, size, rank) is fine. */
int32_t orc_va_add(uint64_t gva, uint64_t size, int32_t memType, uint64_t lva, uint32_t localRank,
                   uint32_t importedRank)
{
    if (gva == 0) {
        return -1;
    }
    if (size == 0) {
        return 0;
    }
    if (memType >= 3) {
        return -1;
    }
    uint64_t end = gva + size;
    uint32_t rank = importedRank != UINT32_MAX ? importedRank : localRank;
    int freeSlot = -1;
    for (int i = 0; i < ORC_VA_MAX; ++i) {
        if (!g_va[i].used) {
            if (freeSlot < 0) {
                freeSlot = i;
            }
            continue;
        }
        if (g_va[i].memType != memType) {
            continue;
        }
        uint64_t og = g_va[i].gva;
        uint64_t oe = og + g_va[i].size;
        if ((gva >= og && gva < oe) || (gva <= og && end > og)) {
            if (og == gva && g_va[i].size == size && va_rank(&g_va[i]) == rank) {
                return 0;
            }
            return -1;
        }
    }
    if (freeSlot < 0) {
        return -1;
    }
    g_va[freeSlot].gva = gva;
    g_va[freeSlot].size = size;
    g_va[freeSlot].lva = lva;
    g_va[freeSlot].memType = memType;
    g_va[freeSlot].localRank = localRank;
    g_va[freeSlot].importedRank = importedRank;
    g_va[freeSlot].used = 1;
    return 0;
}

static orc_va_entry *va_by_gva(uint64_t a)
{
    for (int i = 0; i < ORC_VA_MAX; ++i) {
        if (g_va[i].used && a >= g_va[i].gva && a < g_va[i].gva + g_va[i].size) {
            return &g_va[i];
        }
    }
    return NULL;
}

static orc_va_entry *va_by_lva(uint64_t a)
{
    for (int i = 0; i < ORC_VA_MAX; ++i) {
        if (g_va[i].used && g_va[i].lva != 0 && a >= g_va[i].lva && a < g_va[i].lva + g_va[i].size) {
            return &g_va[i];
        }
    }
    return NULL;
}

/* GetGvaByLva / GetLvaByGva (.cpp:127-168): 0 when unknown, offset preserved. */
uint64_t orc_va_gva_of_lva(uint64_t lva)
{
    if (lva == 0) {
        return 0;
    }
    orc_va_entry *e = va_by_lva(lva);
    return e ? e->gva + (lva - e->lva) : 0;
}

uint64_t orc_va_lva_of_gva(uint64_t gva)
{
    if (gva == 0) {
        return 0;
    }
    orc_va_entry *e = va_by_gva(gva);
    return e ? e->lva + (gva - e->gva) : 0;
}

/* IsGva (.cpp:170-185) */
int32_t orc_va_is_gva(uint64_t va)
{
    return (va != 0 && va_by_gva(va) != NULL) ? 1 : 0;
}

/* IsValidAddr (.cpp:256-261) */
int32_t orc_va_is_known(uint64_t va)
{
    return (orc_va_is_gva(va) || orc_va_gva_of_lva(va) != 0) ? 1 : 0;
}

/* GetMemType (.cpp:187-220): pool range, then local mapping, then reservation,
 * else BUTT; a zero address answers DEVICE.  (In the local-mapping branch the
 * reference reads the type through the iterator of the first lookup; with
 * lva == gva, which is how local slices are registered, both name the same
 * entry.  The restatement returns the matched entry's type.) */
int32_t orc_va_mem_type(uint64_t va)
{
    if (va == 0) {
        return 1;
    }
    orc_va_entry *e = va_by_gva(va);
    if (e) {
        return e->memType;
    }
    e = va_by_lva(va);
    if (e) {
        return e->memType;
    }
    for (int i = 0; i < ORC_VA_MAX; ++i) {
        if (g_rsv[i].used && va >= g_rsv[i].start && va < g_rsv[i].start + g_rsv[i].size) {
            return g_rsv[i].memType;
        }
    }
    return 3;
}

/* GetRank (.cpp:238-254): -1 when not found. */
int64_t orc_va_rank(uint64_t gva)
{
    if (gva == 0) {
        return -1;
    }
    orc_va_entry *e = va_by_gva(gva);
    return e ? (int64_t)va_rank(e) : -1;
}

/* RemoveOneVaInfo (.cpp:93-125): only the first address of a range (or the
 * local address that maps to it) removes the range. */
void orc_va_remove(uint64_t va)
{
    uint64_t gva = va;
    if (!orc_va_is_gva(va)) {
        gva = orc_va_gva_of_lva(va);
    }
    if (gva == 0) {
        return;
    }
    for (int i = 0; i < ORC_VA_MAX; ++i) {
        if (g_va[i].used && g_va[i].gva == gva) {
            g_va[i].used = 0;
            return;
        }
    }
}

/* AllocReserveGva / FindFreeSpace (.cpp:263-292,361-409): first fit inside
 * [0x2800_0000_0000, 0xA800_0000_0000) (hybm_define.h:56-57). */
uint64_t orc_va_reserve(uint64_t size, int32_t memType)
{
    const uint64_t start = 0x280000000000ULL;
    const uint64_t end = 0xA80000000000ULL;
    if (size == 0 || size > end - start) {
        return 0;
    }
    uint64_t current = start;
    for (;;) { /* repeatedly take the lowest reservation at or after `current` */
        int best = -1;
        for (int i = 0; i < ORC_VA_MAX; ++i) {
            if (g_rsv[i].used && g_rsv[i].start + g_rsv[i].size > current &&
                (best < 0 || g_rsv[i].start < g_rsv[best].start)) {
                best = i;
            }
        }
        if (best < 0) {
            break;
        }
        if (g_rsv[best].start > current && g_rsv[best].start - current >= size) {
            break;
        }
        current = g_rsv[best].start + g_rsv[best].size;
    }
    if (end - current < size) {
        return 0;
    }
    for (int i = 0; i < ORC_VA_MAX; ++i) {
        if (!g_rsv[i].used) {
            g_rsv[i].start = current;
            g_rsv[i].size = size;
            g_rsv[i].memType = memType;
            g_rsv[i].used = 1;
            return current;
        }
    }
    return 0;
}

void orc_va_unreserve(uint64_t start)
{
    for (int i = 0; i < ORC_VA_MAX; ++i) {
        if (g_rsv[i].used && g_rsv[i].start == start) {
            g_rsv[i].used = 0;
        }
    }
}

/* ClassifyAddress + InferCopyDirection (.cpp:222-236): pool type first, then
 * the fixed device VA window [0x1000_0000_0000, +0x800_0000_0000)
 * (hybm_define.h:33-34), else local host. */
int32_t orc_va_classify(uint64_t va)
{
    int32_t t = orc_va_mem_type(va);
    if (t == 1) {
        return 0;
    }
    if (t == 2) {
        return 1;
    }
    if (va >= 0x100000000000ULL && va < 0x100000000000ULL + 0x80000000000ULL) {
        return 2;
    }
    return 3;
}

int32_t orc_va_infer_direction(uint64_t srcVa, uint64_t dstVa)
{
    return orc_infer_table(orc_va_classify(srcVa), orc_va_classify(dstVa));
}

/* ------------------------------------------------------------------------
 * Adjacent-segment merge of HostDataOpSDMA::BatchCopyG2G
 * (src/hybm/csrc/data_operation/host/hybm_data_op_sdma.cpp:565-584): a segment
 * that continues the running one on both sides extends it.  Writes merged
 * triples to out[3*k..], returns how many.  (Like the reference, a zero-length
 * first segment still produces a descriptor.)
 * ---------------------------------------------------------------------- */
uint32_t orc_coalesce(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n, uint64_t *out)
{
    uint64_t s = 0, d = 0, l = 0;
    uint32_t k = 0;
    for (uint32_t i = 0; i < n; ++i) {
        if (l > 0 && s + l == src[i] && d + l == dst[i]) {
            l += len[i];
            continue;
        }
        if (l > 0) {
            out[3 * k] = s; out[3 * k + 1] = d; out[3 * k + 2] = l; ++k;
        }
        s = src[i]; d = dst[i]; l = len[i];
    }
    if (n > 0) {
        out[3 * k] = s; out[3 * k + 1] = d; out[3 * k + 2] = l; ++k;
    }
    return k;
}

/* ------------------------------------------------------------------------
 * Transfer front-end arithmetic (src/smem/csrc/smem_trans/smem_trans_entry.cpp).
 * ---------------------------------------------------------------------- */
/* SmemTransEntry::AlignMemory (:604-615): widen [*addr, *addr + *size) to whole 2 MiB pages. */
void orc_trans_align(uint64_t *addr, uint64_t *size)
{
    const uint64_t page = 2ull * 1024 * 1024;
    const uint64_t mask = ~(page - 1);
    const uint64_t aligned = *addr & mask;
    *size += *addr - aligned;
    *size = (*size + page - 1) & mask;
    *addr = aligned;
}

static int orc_pair_less(const void *a, const void *b)
{
    const uint64_t *x = (const uint64_t *)a, *y = (const uint64_t *)b;
    if (x[0] != y[0]) {
        return x[0] < y[0] ? -1 : 1;
    }
    return x[1] < y[1] ? -1 : (x[1] > y[1] ? 1 : 0);
}

/* SmemTransEntry::CombineMemories (:617-640): sort the (start, size) pairs, then fold every pair
 * that starts inside or right at the end of the running one into it.  pairs[2*n] is sorted in
 * place; merged pairs go to out[2*k..]; returns k.  n must be at least 1. */
uint32_t orc_trans_combine(uint64_t *pairs, uint32_t n, uint64_t *out)
{
    qsort(pairs, n, 2 * sizeof(uint64_t), orc_pair_less);
    uint64_t curStart = pairs[0], curSize = pairs[1];
    uint32_t k = 0;
    for (uint32_t i = 1; i < n; ++i) {
        const uint64_t start = pairs[2 * i], size = pairs[2 * i + 1];
        if (curStart + curSize >= start) {
            const uint64_t diff = start - curStart;
            if (diff > UINT64_MAX - size) {
                out[2 * k] = curStart; out[2 * k + 1] = curSize; ++k;
                curStart = start; curSize = size;
                continue;
            }
            curSize = curSize > diff + size ? curSize : diff + size;
        } else {
            out[2 * k] = curStart; out[2 * k + 1] = curSize; ++k;
            curStart = start; curSize = size;
        }
    }
    out[2 * k] = curStart; out[2 * k + 1] = curSize; ++k;
    return k;
}

/* Remote-address translation of SmemTransEntry::BatchSyncTransfer (:337-356).  The slice map is
 * ordered by start address, descending (smem_trans_entry.h:123-124), so lower_bound(remote) is the
 * slice with the greatest start <= remote.  slices[3*n] = {start, size, mapped}.  Returns the
 * mapped address, or 0 where the reference returns SM_INVALID_PARAM. */
uint64_t orc_trans_translate(const uint64_t *slices, uint32_t n, uint64_t remote, uint64_t size)
{
    int64_t best = -1;
    for (uint32_t i = 0; i < n; ++i) {
        if (slices[3 * i] <= remote && (best < 0 || slices[3 * i] > slices[3 * best])) {
            best = i;
        }
    }
    if (best < 0) {
        return 0;
    }
    const uint64_t start = slices[3 * best], len = slices[3 * best + 1], mapped = slices[3 * best + 2];
    if (remote + size > start + len) {
        return 0;
    }
    return mapped + (remote - start);
}

/* ------------------------------------------------------------------------
 * Work partition of the reference's device kernels
 * (src/hybm/csrc/copy_extend/hybm_copy_kernel.cpp:68-78,97-111), kept to
 * document and test what the HIP kernels deliberately do differently.
 * ---------------------------------------------------------------------- */
/* hybm_copy_kernel: byte range [*begin, *end) of block idx out of num. */
void orc_ref_kernel_single_range(uint64_t len, uint32_t idx, uint32_t num, uint64_t *begin, uint64_t *end)
{
    uint64_t offset = ((len + 128 - 1U) / 128 + num - 1U) / num * 128;
    uint64_t size = offset * (idx + 1) < len ? offset * (idx + 1) : len;
    offset = offset * idx;
    *begin = offset;
    *end = size; /* the kernel copies size - offset bytes; for offset > len that difference wraps */
}

/* hybm_batch_copy_kernel: segment index range [*begin, *end) of block idx. */
void orc_ref_kernel_batch_range(uint32_t count, uint32_t idx, uint32_t num, uint32_t *begin, uint32_t *end)
{
    uint32_t per = (count + num - 1) / num;
    uint32_t start = per * idx;
    uint32_t stop = start + per < count ? start + per : count;
    *begin = start;
    *end = stop;
}

/* ------------------------------------------------------------------------
 * MoE local dispatch / combine.  The reference has no implementation; this is
 * the specification the HIP kernels are held to.
 *
 * dispatch: tokens x[T][H] (16-bit elements, moved as opaque words),
 * topk[T][K] expert ids in [0, E).  Entry i = t*K + k goes to row
 * offsets[e] + (number of entries j < i with topk[j] == e): a stable counting
 * sort of the flat (t, k) order by expert.
 * ---------------------------------------------------------------------- */
int32_t orc_moe_dispatch(const uint16_t *x, const int32_t *topk, uint32_t T, uint32_t H, uint32_t K, uint32_t E,
                         uint16_t *out, int32_t *counts, int32_t *offsets, int32_t *rowOf, int32_t *srcOf)
{
    for (uint32_t e = 0; e < E; ++e) {
        counts[e] = 0;
    }
    for (uint64_t i = 0; i < (uint64_t)T * K; ++i) {
        if (topk[i] < 0 || (uint32_t)topk[i] >= E) {
            return -2;
        }
        counts[topk[i]]++;
    }
    int32_t run = 0;
    for (uint32_t e = 0; e < E; ++e) {
        offsets[e] = run;
        run += counts[e];
    }
    int32_t *cursor = (int32_t *)malloc(sizeof(int32_t) * E);
    if (cursor == NULL) {
        return -3;
    }
    memcpy(cursor, offsets, sizeof(int32_t) * E);
    for (uint64_t i = 0; i < (uint64_t)T * K; ++i) {
        int32_t row = cursor[topk[i]]++;
        if (rowOf != NULL) {
            rowOf[i] = row;
        }
        if (srcOf != NULL) {
            srcOf[row] = (int32_t)i;
        }
        if (out != NULL && x != NULL) {
            memcpy(out + (uint64_t)row * H, x + (i / K) * H, (uint64_t)H * 2);
        }
    }
    free(cursor);
    return 0;
}

static float bf16_to_f32(uint16_t v)
{
    uint32_t w = (uint32_t)v << 16;
    float f;
    memcpy(&f, &w, 4);
    return f;
}

/* round to nearest even; NaN stays NaN (quiet) */
static uint16_t f32_to_bf16_rne(float f)
{
    uint32_t w;
    memcpy(&w, &f, 4);
    if ((w & 0x7fffffffu) > 0x7f800000u) {
        return (uint16_t)((w >> 16) | 0x0040u);
    }
    uint32_t bias = 0x7fffu + ((w >> 16) & 1u);
    return (uint16_t)((w + bias) >> 16);
}

/* combine: y[t][h] = bf16_rne( fma(w[t][K-1], v_{K-1}, ... fma(w[t][0], v_0, 0)) ),
 * v_k = float(rows[rowOf[t*K+k]][h]): fp32 accumulation in slot order with one
 * rounding per step (fmaf), a single final rounding to bf16.  A slot whose
 * rowOf is negative (an expert id that dispatch flagged as out of range) is
 * skipped: no row is read for it and the chain goes on with the next slot. */
void orc_moe_combine(const uint16_t *rows, const int32_t *rowOf, const float *w, uint32_t T, uint32_t H, uint32_t K,
                     uint16_t *y)
{
    for (uint32_t t = 0; t < T; ++t) {
        for (uint32_t h = 0; h < H; ++h) {
            float acc = 0.0f;
            for (uint32_t k = 0; k < K; ++k) {
                if (rowOf[(uint64_t)t * K + k] < 0) {
                    continue;
                }
                float v = bf16_to_f32(rows[(uint64_t)rowOf[(uint64_t)t * K + k] * H + h]);
                acc = fmaf(w[(uint64_t)t * K + k], v, acc);
            }
            y[(uint64_t)t * H + h] = f32_to_bf16_rne(acc);
        }
    }
}

/* Router used to synthesise inputs: top-K of logits[T][E] by value, ties to
 * the lower expert id, weights = softmax over the K selected logits (fp32,
 * max-subtracted, exp via expf, divided by the running sum). */
void orc_moe_route(const float *logits, uint32_t T, uint32_t E, uint32_t K, int32_t *topk, float *weights)
{
    for (uint32_t t = 0; t < T; ++t) {
        const float *row = logits + (uint64_t)t * E;
        for (uint32_t k = 0; k < K; ++k) {
            int32_t best = -1;
            for (uint32_t e = 0; e < E; ++e) {
                int taken = 0;
                for (uint32_t j = 0; j < k; ++j) {
                    if (topk[(uint64_t)t * K + j] == (int32_t)e) {
                        taken = 1;
                    }
                }
                if (!taken && (best < 0 || row[e] > row[best])) {
                    best = (int32_t)e;
                }
            }
            topk[(uint64_t)t * K + k] = best;
        }
        float mx = row[topk[(uint64_t)t * K]];
        float sum = 0.0f;
        for (uint32_t k = 0; k < K; ++k) {
            float ex = expf(row[topk[(uint64_t)t * K + k]] - mx);
            weights[(uint64_t)t * K + k] = ex;
            sum += ex;
        }
        for (uint32_t k = 0; k < K; ++k) {
            weights[(uint64_t)t * K + k] /= sum;
        }
    }
}

/* ------------------------------------------------------------------------
 * Deterministic input bytes: splitmix64 stream, 8 bytes per step.
 * ---------------------------------------------------------------------- */
void orc_fill_random(void *ptr, uint64_t bytes, uint64_t seed)
{
    uint8_t *p = (uint8_t *)ptr;
    uint64_t state = seed;
    uint64_t i = 0;
    while (i < bytes) {
        state += 0x9E3779B97F4A7C15ULL;
        uint64_t z = state;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
        z = z ^ (z >> 31);
        uint64_t take = bytes - i < 8 ? bytes - i : 8;
        memcpy(p + i, &z, take);
        i += take;
    }
}
