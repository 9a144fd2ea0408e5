// Address arithmetic of the pooled ("global") virtual address space.
//
// One window per memory type; rank r owns [base + r*stride, base + (r+1)*stride).
// Restates, as pure functions on integers,
//   SmemBmEntry::AddrInHostGva / AddrInDeviceGva / GetRankIdByGva
//       (src/smem/csrc/smem_bm/smem_bm_entry.cpp:337-347,421-455)
//   smem_bm_ptr_by_mem_type        (src/smem/csrc/smem_bm/smem_bm.cpp:290-317)
//   MemSegment::MemoryInRange / GetRankIdByAddr
//       (src/hybm/csrc/mm/hybm_conn_based_segment.cpp:247-270,
//        src/hybm/csrc/mm/hybm_dev_legacy_segment.cpp:446-457,485-496)
//   Valid48BitsAddress             (src/hybm/csrc/common/hybm_define.h:77-92)
#ifndef MF_GVA_LAYOUT_H
#define MF_GVA_LAYOUT_H

#include <stdint.h>

namespace mf {

constexpr uint64_t kAddressMask48 = 0xffffffffffffULL;
constexpr uint32_t kNoRank = 0xFFFFFFFFu;

inline uint64_t Mask48(uint64_t address)
{
    return address & kAddressMask48;
}

struct GvaWindow {
    uint64_t base = 0;       // 0 = this memory type is not part of the pool
    uint64_t stride = 0;     // bytes of address space per rank (max{HBM,DRAM}Size)
    uint64_t rankCount = 0;
    uint64_t rankSpace = 0;  // divisor of the rank lookup ({device,host}VASpace at the smem layer)

    uint64_t Span() const
    {
        return stride * rankCount;
    }

    // The reference rejects only addr + size > end, so a range that ends exactly
    // at the end of the window is inside and a zero-size probe at `end` is too.
    bool Contains(uint64_t addr, uint64_t size) const
    {
        if (base == 0 || addr + size < addr) {   // a range that wraps round the address space is never inside
            return false;
        }
        if (addr + size > base + Span()) {
            return false;
        }
        return addr >= base;
    }

    uint32_t RankBySpace(uint64_t addr) const
    {
        if (!Contains(addr, 1) || rankSpace == 0) {
            return kNoRank;
        }
        return static_cast<uint32_t>((addr - base) / rankSpace);
    }

    uint32_t RankByStride(uint64_t addr, uint64_t size, uint32_t otherwise, bool &inside) const
    {
        inside = Contains(addr, size) && stride != 0;
        return inside ? static_cast<uint32_t>((addr - base) / stride) : otherwise;
    }

    uint64_t PtrOfRank(uint32_t rank) const
    {
        return base + stride * rank;
    }
};

}  // namespace mf

#endif  // MF_GVA_LAYOUT_H
