// Device memory arena: a best-fit free list over large blocks obtained from a raw allocator (hipMalloc on the device,
// malloc in the CPU tests). It plays the role of the reference's buffer managers behind Device::Realloc/Free
// (src/ppl/nn/utils/compact_buffer_manager.cc, stack_buffer_manager.cc:31-86, engines/llm_cuda/buffered_device.cc:25-56):
// allocations are aligned, `BufferDesc::desc` carries the usable size, freed ranges are coalesced and reused, and the
// blocks go back to the raw allocator only when the arena dies (so Realloc/Free never call hipMalloc/hipFree in steady state).
#ifndef PPLNN_LLM_HIP_ARENA_H_
#define PPLNN_LLM_HIP_ARENA_H_

#include <map>
#include <mutex>

#include "core.h"

namespace ppl { namespace nn { namespace utils {

class ArenaBufferManager final {
public:
    typedef std::function<void*(uint64_t)> RawAlloc;
    typedef std::function<void(void*)> RawFree;
    // How a request picks among the free pieces: the smallest that fits (MM_BEST_FIT, the reference's
    // bestfit_buffered_device.cc) or the one at the lowest address (MM_COMPACT, buffered_device.cc over the compact
    // manager: the heap stays packed towards its start). kPlain keeps nothing: every request is a raw allocation
    // that goes back to the raw allocator when it is freed (MM_PLAIN, plain_device.cc).
    enum Policy { kBestFit, kCompact, kPlain };
    ArenaBufferManager(const RawAlloc& a, const RawFree& f, uint64_t alignment, uint64_t block_bytes,
                       Policy policy = kBestFit)
        : raw_alloc_(a), raw_free_(f), alignment_(alignment), block_bytes_(block_bytes), policy_(policy) {}
    ~ArenaBufferManager() {
        for (auto& b : blocks_) raw_free_(b.first);
    }
    RetCode Alloc(uint64_t bytes, BufferDesc* buffer) {
        std::lock_guard<std::mutex> guard(lock_);
        const uint64_t need = Align(bytes ? bytes : 1);
        auto best = free_by_addr_.end();
        for (auto it = free_by_addr_.begin(); it != free_by_addr_.end(); ++it) {
            if (it->second < need) continue;
            if (policy_ == kCompact) { // the map is ordered by address: the first that fits is the lowest
                best = it;
                break;
            }
            if (best == free_by_addr_.end() || it->second < best->second) best = it;
        }
        if (best == free_by_addr_.end()) {
            const uint64_t block = (policy_ == kPlain || need > block_bytes_) ? need : block_bytes_;
            void* p = raw_alloc_(block);
            if (!p) {
                LOG(ERROR) << "arena: raw allocation of " << block << " bytes failed";
                return ppl::common::RC_OUT_OF_MEMORY;
            }
            blocks_[(char*)p] = block;
            buffered_bytes_ += block;
            best = free_by_addr_.emplace((char*)p, block).first;
        }
        char* addr = best->first;
        const uint64_t size = best->second;
        free_by_addr_.erase(best);
        if (size > need) free_by_addr_[addr + need] = size - need;
        used_[addr] = need;
        buffer->addr = addr;
        buffer->desc = need;
        return ppl::common::RC_SUCCESS;
    }
    void Free(BufferDesc* buffer) {
        std::lock_guard<std::mutex> guard(lock_);
        auto it = used_.find((char*)buffer->addr);
        if (it == used_.end()) return; // not ours (e.g. a borrowed pointer): nothing to do
        char* addr = it->first;
        uint64_t size = it->second;
        used_.erase(it);
        if (policy_ == kPlain) { // the piece is a raw block of its own
            blocks_.erase(addr);
            buffered_bytes_ -= size;
            raw_free_(addr);
            buffer->addr = nullptr;
            buffer->desc = 0;
            return;
        }
        // coalesce with the neighbours, but never across raw blocks
        auto next = free_by_addr_.lower_bound(addr);
        if (next != free_by_addr_.end() && addr + size == next->first && !IsBlockStart(next->first)) {
            size += next->second;
            next = free_by_addr_.erase(next);
        }
        if (next != free_by_addr_.begin()) {
            auto prev = std::prev(next);
            if (prev->first + prev->second == addr && !IsBlockStart(addr)) {
                prev->second += size;
                buffer->addr = nullptr;
                buffer->desc = 0;
                return;
            }
        }
        free_by_addr_[addr] = size;
        buffer->addr = nullptr;
        buffer->desc = 0;
    }
    uint64_t GetBufferedBytes() const { return buffered_bytes_; } // bytes held from the raw allocator
    uint64_t GetUsedBytes() const {
        uint64_t n = 0;
        for (auto& u : used_) n += u.second;
        return n;
    }

private:
    uint64_t Align(uint64_t n) const { return (n + alignment_ - 1) / alignment_ * alignment_; }
    bool IsBlockStart(char* p) const { return blocks_.find(p) != blocks_.end(); }
    RawAlloc raw_alloc_;
    RawFree raw_free_;
    uint64_t alignment_, block_bytes_;
    Policy policy_;
    std::map<char*, uint64_t> blocks_, free_by_addr_, used_;
    uint64_t buffered_bytes_ = 0;
    std::mutex lock_;
};

}}} // namespace ppl::nn::utils

#endif
