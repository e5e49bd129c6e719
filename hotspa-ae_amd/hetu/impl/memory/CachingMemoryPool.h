// Stream-aware caching allocator behind device NDArrays (the job of
// hetu/impl/memory/CUDACachingMemoryPool.{cuh,cu} in the reference, redone for
// one 288 GB HBM3E device):
//   * requests are rounded to 256 B; requests under 1 MiB are carved out of 2 MiB
//     segments, larger ones get a segment of their own size rounded to 2 MiB;
//   * free blocks are kept per stream (best fit by size, then address); a block
//     freed on the stream it was allocated for is reusable there at once, because
//     the stream orders the old work before the new;
//   * a block that other streams touched (MarkDataSpaceUsedByStream) parks behind
//     one event per such stream and returns to its list when those have passed;
//   * a stream with nothing cached may take another stream's free block: an event
//     recorded on the owner stream is waited for by the taking stream, which costs
//     no host synchronisation and no new segment;
//   * a cached block is split when it is at most `max_split_size`, otherwise it is
//     handed out whole if the waste stays under `max_internal_fragment_size`
//     (HETU_MAX_SPLIT_SIZE_MB, default 200; HETU_MAX_INTERNAL_FRAGMENT_SIZE_MB,
//     default 20 -- the reference's knobs and defaults,
//     CUDACachingMemoryPool.cu:1236-1277);
//   * when the device refuses a segment, parked blocks are collected, every fully
//     free segment is returned to the device and the request is tried once more.
// The device is reached through a small backend interface so the caching logic
// itself can be exercised on the host.
#pragma once

#include <map>
#include <set>
#include <unordered_map>

#include "hetu/core/memory_pool.h"

namespace hetu {
namespace impl {

// What the pool needs from a device runtime.
class PoolBackend {
 public:
  virtual ~PoolBackend() = default;
  virtual void* RawAlloc(size_t bytes) = 0;              // nullptr when the device is out of memory
  virtual void RawFree(void* ptr) = 0;
  virtual void* EventRecord(const Stream& stream) = 0;   // an event recorded at the tail of `stream`
  virtual bool EventDone(void* event) = 0;
  virtual void EventSync(void* event) = 0;
  virtual void EventRelease(void* event) = 0;
  virtual void StreamWaitEvent(const Stream& stream, void* event) = 0;
  virtual void StreamSync(const Stream& stream) = 0;
  virtual void DeviceSync() = 0;
};

struct PoolStats {
  size_t allocated{0}, peak_allocated{0};   // bytes handed out (rounded sizes)
  size_t reserved{0}, peak_reserved{0};     // bytes held from the device
  size_t alloc_cnt{0}, free_cnt{0}, mark_cnt{0};
  size_t segment_allocs{0}, segment_frees{0};
  size_t cache_hits{0}, cross_stream_takes{0}, parked{0}, splits{0}, merges{0}, retries_after_oom{0};
};

class CachingMemoryPool : public MemoryPool {
 public:
  static constexpr size_t kAlignment = 256;
  static constexpr size_t kSmallRequest = 1u << 20;
  static constexpr size_t kSegmentRoundUp = 2u << 20;

  CachingMemoryPool(Device device, std::string name, std::unique_ptr<PoolBackend> backend, size_t max_split_size,
                    size_t max_internal_fragment_size);
  ~CachingMemoryPool() override;

  DataPtr AllocDataSpace(size_t num_bytes, const Stream& stream = Stream()) override;
  DataPtr BorrowDataSpace(void* ptr, size_t num_bytes, DataPtrDeleter deleter,
                          const Stream& stream = Stream()) override;
  void FreeDataSpace(DataPtr data_ptr) override;
  void EmptyCache() override;
  void MarkDataSpaceUsedByStream(DataPtr data_ptr, const Stream& stream) override;
  void MarkDataSpacesUsedByStream(DataPtrList& data_ptrs, const Stream& stream) override;
  std::future<void> WaitDataSpace(DataPtr data_ptr, bool async = true) override;
  void PrintSummary() override;
  PoolStats stats();
  static size_t RoundRequest(size_t bytes) { return (bytes + kAlignment - 1) / kAlignment * kAlignment; }

 private:
  struct Block {
    uint8_t* ptr{nullptr};
    size_t size{0};
    Block* prev{nullptr};   // neighbours inside the segment, by address
    Block* next{nullptr};
    bool in_use{false};
    PackedStreamId owner{0};              // stream whose order protects the contents
    std::vector<PackedStreamId> used_by;  // other streams with work queued on it
    DataPtrId id{0};
  };
  struct BlockLess {
    bool operator()(const Block* a, const Block* b) const {
      return a->size != b->size ? a->size < b->size : a->ptr < b->ptr;
    }
  };
  using FreeList = std::set<Block*, BlockLess>;
  struct Parked {
    Block* block;
    std::vector<void*> events;
  };
  struct Borrowed {
    DataPtr ptr;
    DataPtrDeleter deleter;
    std::vector<PackedStreamId> used_by;
  };

  Stream normalize(const Stream& stream) const;
  Block* take_from(FreeList& list, size_t bytes);
  Block* split(Block* block, size_t bytes);
  Block* new_segment(size_t bytes, PackedStreamId owner);
  void release(Block* block);                 // to its owner's free list, merging neighbours
  void collect_parked(bool wait);
  size_t release_free_segments();
  DataPtr hand_out(Block* block, bool fresh);

  std::unique_ptr<PoolBackend> _backend;
  const size_t _max_split_size;
  const size_t _max_internal_fragment_size;
  std::map<PackedStreamId, FreeList> _free;
  std::unordered_map<DataPtrId, Block*> _live;
  std::unordered_map<DataPtrId, Borrowed> _borrowed;
  std::vector<Parked> _parked;
  PoolStats _stats;
};

// HETU_MAX_SPLIT_SIZE_MB / HETU_MAX_INTERNAL_FRAGMENT_SIZE_MB in bytes; a value
// that does not parse as a positive integer is reported and the default used.
size_t ParsePoolKnobMB(const char* env_name, size_t default_mb);

} // namespace impl
} // namespace hetu
