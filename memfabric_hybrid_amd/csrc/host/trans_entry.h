// Named transfer objects: one-sided batch read / write between objects that
// know each other by "ip:port" names.  Counterpart of SmemTransEntry
// (src/smem/csrc/smem_trans/smem_trans_entry.{h,cpp}) for objects that live in
// one process on one GPU: the slice map, its lookup and the range checks are
// the reference's; the config store and the watch threads that fill the map
// there are replaced by TransDirectory, which hands a newly registered slice
// to every interested object before the registration call returns.
#ifndef MF_TRANS_ENTRY_H
#define MF_TRANS_ENTRY_H

#include <array>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <shared_mutex>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include "../../../include/mf_xcopy_api.h"

namespace mf {

constexpr uint64_t kTransHostMax = 128ull << 30;   // largest smem_trans_malloc (smem_trans_entry.cpp:33,186)

// Name of a transfer object in binary form: address family, 16 address bytes, port.
using WorkerKey = std::array<uint8_t, 20>;
struct WorkerKeyHash {
    size_t operator()(const WorkerKey &k) const;
};

// "a.b.c.d:port" (port above 1024, address not 0.0.0.0) or "[v6]:port"
// (smem_trans_entry.cpp:374-397, src/smem/csrc/net/smem_net_common.cpp:67-96).
bool ParseWorkerName(const std::string &name, WorkerKey &key);

// Sorted union of (start, size) ranges: ranges that overlap or touch become one
// (smem_trans_entry.cpp:617-640).  The input must not be empty.
std::vector<std::pair<uint64_t, uint64_t>> CombineRanges(std::vector<std::pair<uint64_t, uint64_t>> input);

// What an object knows about one contiguous run of a peer's registered memory.  The reference
// widens every registration to whole 2 MiB pages (smem_trans_entry.cpp:604-615) because its
// driver pins pages; nothing is pinned here, and a copy that strays outside the bytes that were
// really registered would fault the GPU, so runs are kept exact and a transfer must lie inside one.
struct PeerSlice {
    uint64_t mapped;     // where the run is addressable from here
    uint64_t size;
    hybm_mem_type type;  // HBM or pinned host memory
};

// Runs of one peer by the peer's own start address, descending, so that lower_bound(a) is the
// run with the greatest start <= a (smem_trans_entry.h:123-124).
using PeerSliceMap = std::map<uint64_t, PeerSlice, std::greater<uint64_t>>;

// Translate one peer address; 0 or SM_INVALID_PARAM (smem_trans_entry.cpp:337-356).
int TranslatePeerAddress(const PeerSliceMap &slices, uint64_t remote, uint64_t size, uint64_t &mapped,
                         hybm_mem_type &type);

class TransEntry;

// In-process stand-in for the config store: who exists, which role, which slices.
class TransDirectory {
public:
    static TransDirectory &Instance();
    int Join(TransEntry *entry);        // SM_DUPLICATED_OBJECT when the name is taken
    void Leave(TransEntry *entry);
    void Publish(TransEntry *owner, uint64_t base, const PeerSlice &slice);
    void Withdraw(TransEntry *owner, uint64_t base);
    std::shared_ptr<TransEntry> FindByHandle(const void *handle);
    void Adopt(std::shared_ptr<TransEntry> entry);
    std::shared_ptr<TransEntry> Release(const void *handle);
    uint16_t NextEntityId();

private:
    struct Published {
        uint64_t base;
        PeerSlice slice;
    };
    static bool Interested(const TransEntry &watcher, const TransEntry &owner);
    std::mutex lock_;
    std::unordered_map<WorkerKey, TransEntry *, WorkerKeyHash> members_;
    std::unordered_map<TransEntry *, std::vector<Published>> published_;
    std::shared_mutex handleLock_;   // handle lookups are on the transfer path, kept off lock_
    std::unordered_map<const void *, std::shared_ptr<TransEntry>> handles_;
    uint16_t nextEntityId_ = 0;
};

class TransEntry {
public:
    TransEntry(std::string name, const smem_trans_config_t &config);
    ~TransEntry();

    int Initialize();
    void UnInitialize();

    int RegisterLocalMemory(const void *address, uint64_t size, uint32_t flags);
    int RegisterLocalMemories(const std::vector<std::pair<const void *, size_t>> &memories, uint32_t flags);
    int DeregisterLocalMemory(const void *address);
    void *MallocHost(uint64_t size);
    int FreeHost(void *address);

    // opcode: SMEMB_COPY_L2G = write to the peer, SMEMB_COPY_G2L = read from it.
    int BatchTransfer(void *localAddrs[], const char *remoteName, void *remoteAddrs[], const size_t dataSizes[],
                      uint32_t batchSize, smem_bm_copy_type opcode, void *stream, uint32_t flags);

    const WorkerKey &Key() const
    {
        return key_;
    }
    smem_trans_role_t Role() const
    {
        return config_.role;
    }
    const std::string &Name() const
    {
        return name_;
    }

    // Called by the directory.
    void ImportSlice(const WorkerKey &owner, uint64_t base, const PeerSlice &slice);
    void DropSlice(const WorkerKey &owner, uint64_t base);

private:
    int RegisterOne(uint64_t base, uint64_t size);

    std::string name_;
    smem_trans_config_t config_;
    WorkerKey key_{};
    hybm_entity_t entity_ = nullptr;
    bool joined_ = false;

    std::mutex localLock_;
    struct LocalReg {
        hybm_mem_slice_t slice;
        uint64_t size;
        bool allocated;   // from smem_trans_malloc: the entity owns the memory
    };
    std::map<uint64_t, LocalReg> local_;   // by start address

    std::shared_mutex peerLock_;
    std::unordered_map<WorkerKey, PeerSliceMap, WorkerKeyHash> peers_;
};

}  // namespace mf

#endif  // MF_TRANS_ENTRY_H
