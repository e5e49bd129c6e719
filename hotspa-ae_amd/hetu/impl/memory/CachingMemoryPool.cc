#include "hetu/impl/memory/CachingMemoryPool.h"

#include <algorithm>
#include <cstdlib>

#include "hetu/common/logging.h"

namespace hetu {
namespace impl {

size_t ParsePoolKnobMB(const char* env_name, size_t default_mb) {
  size_t mb = default_mb;
  if (const char* s = std::getenv(env_name)) {
    char* end = nullptr;
    long long v = std::strtoll(s, &end, 10);
    if (end == s || *end != '\0' || v <= 0) {
      HT_LOG_WARN << "Invalid " << env_name << ": \"" << s << "\", please provide a positive integer; using "
                  << default_mb << " MiB";
    } else {
      mb = size_t(v);
    }
  }
  return mb << 20;
}

CachingMemoryPool::CachingMemoryPool(Device device, std::string name, std::unique_ptr<PoolBackend> backend,
                                     size_t max_split_size, size_t max_internal_fragment_size)
: MemoryPool(device, std::move(name)),
  _backend(std::move(backend)),
  _max_split_size(max_split_size),
  _max_internal_fragment_size(max_internal_fragment_size) {}

CachingMemoryPool::~CachingMemoryPool() {
  // Pools live until the process ends (the registry never destroys them); a pool a
  // test built by hand gives its segments back here.
  try {
    std::lock_guard<std::mutex> lock(_mtx);
    collect_parked(true);
    release_free_segments();
  } catch (...) {}
}

Stream CachingMemoryPool::normalize(const Stream& stream) const {
  // an undefined stream means the device's blocking stream
  return stream.is_defined() ? stream : Stream(_device, kBlockingStream);
}

CachingMemoryPool::Block* CachingMemoryPool::take_from(FreeList& list, size_t bytes) {
  Block key;
  key.size = bytes;
  key.ptr = nullptr;
  auto it = list.lower_bound(&key);
  if (it == list.end()) return nullptr;
  Block* b = *it;
  const size_t waste = b->size - bytes;
  if (b->size > _max_split_size && waste > _max_internal_fragment_size) return nullptr;
  list.erase(it);
  if (b->size <= _max_split_size && waste >= kAlignment) b = split(b, bytes);
  return b;
}

// Keeps the first `bytes` of `block`; the tail becomes a free block of the same owner.
CachingMemoryPool::Block* CachingMemoryPool::split(Block* block, size_t bytes) {
  Block* tail = new Block();
  tail->ptr = block->ptr + bytes;
  tail->size = block->size - bytes;
  tail->prev = block;
  tail->next = block->next;
  tail->owner = block->owner;
  if (block->next) block->next->prev = tail;
  block->next = tail;
  block->size = bytes;
  _free[tail->owner].insert(tail);
  _stats.splits++;
  return block;
}

CachingMemoryPool::Block* CachingMemoryPool::new_segment(size_t bytes, PackedStreamId owner) {
  const size_t seg = bytes < kSmallRequest ? kSegmentRoundUp : (bytes + kSegmentRoundUp - 1) / kSegmentRoundUp * kSegmentRoundUp;
  void* p = _backend->RawAlloc(seg);
  if (p == nullptr) {
    // give the device back what is cached and try once more
    collect_parked(true);
    release_free_segments();
    _stats.retries_after_oom++;
    p = _backend->RawAlloc(seg);
    if (p == nullptr) return nullptr;
  }
  _stats.segment_allocs++;
  _stats.reserved += seg;
  _stats.peak_reserved = std::max(_stats.peak_reserved, _stats.reserved);
  Block* b = new Block();
  b->ptr = static_cast<uint8_t*>(p);
  b->size = seg;
  b->owner = owner;
  if (seg - bytes >= kAlignment && (seg <= _max_split_size || bytes < kSmallRequest)) b = split(b, bytes);
  return b;
}

void CachingMemoryPool::release(Block* block) {
  block->in_use = false;
  block->used_by.clear();
  block->id = 0;
  // merge with free neighbours of the same owner: contents of both halves are then
  // ordered by the same stream
  auto try_merge = [&](Block* left, Block* right) -> Block* {
    if (!left || !right || left->in_use || right->in_use || left->owner != right->owner) return nullptr;
    auto& list = _free[left->owner];
    list.erase(left);
    list.erase(right);
    left->size += right->size;
    left->next = right->next;
    if (right->next) right->next->prev = left;
    delete right;
    _stats.merges++;
    return left;
  };
  // a parked neighbour is neither in use nor in a list; only merge with listed ones
  auto listed = [&](Block* b) { return b && !b->in_use && _free[b->owner].count(b) > 0; };
  if (listed(block->next)) {
    if (Block* m = try_merge(block, block->next)) block = m;
  }
  if (listed(block->prev)) {
    if (Block* m = try_merge(block->prev, block)) block = m;
  }
  _free[block->owner].insert(block);
}

void CachingMemoryPool::collect_parked(bool wait) {
  for (size_t i = 0; i < _parked.size();) {
    auto& p = _parked[i];
    for (size_t e = 0; e < p.events.size();) {
      if (wait) _backend->EventSync(p.events[e]);
      if (wait || _backend->EventDone(p.events[e])) {
        _backend->EventRelease(p.events[e]);
        p.events[e] = p.events.back();
        p.events.pop_back();
      } else {
        ++e;
      }
    }
    if (p.events.empty()) {
      Block* b = p.block;
      _parked[i] = std::move(_parked.back());
      _parked.pop_back();
      release(b);
    } else {
      ++i;
    }
  }
}

size_t CachingMemoryPool::release_free_segments() {
  // Work still queued on a cached block must finish before the device gets it
  // back.  Once the device is idle the stream a free block belonged to no longer
  // matters, so neighbours of different owners can be joined as well: that is
  // what lets a segment whose pieces wandered between streams become whole again.
  _backend->DeviceSync();
  std::vector<Block*> blocks;
  for (auto& kv : _free) blocks.insert(blocks.end(), kv.second.begin(), kv.second.end());
  std::set<Block*> listed(blocks.begin(), blocks.end());
  for (Block* b : blocks) {
    if (!listed.count(b)) continue;   // already absorbed by its left neighbour
    bool grew = false;
    while (b->next && listed.count(b->next)) {
      Block* n = b->next;
      if (!grew) {
        _free[b->owner].erase(b);
        grew = true;
      }
      _free[n->owner].erase(n);
      listed.erase(n);
      b->size += n->size;
      b->next = n->next;
      if (n->next) n->next->prev = b;
      delete n;
      _stats.merges++;
    }
    if (grew) _free[b->owner].insert(b);
  }
  size_t freed = 0;
  for (auto& kv : _free) {
    auto& list = kv.second;
    for (auto it = list.begin(); it != list.end();) {
      Block* b = *it;
      if (b->prev == nullptr && b->next == nullptr) {
        _backend->RawFree(b->ptr);
        _stats.segment_frees++;
        _stats.reserved -= b->size;
        freed += b->size;
        it = list.erase(it);
        delete b;
      } else {
        ++it;
      }
    }
  }
  return freed;
}

DataPtr CachingMemoryPool::hand_out(Block* block, bool fresh) {
  block->in_use = true;
  block->id = next_id();
  block->used_by.clear();
  _live[block->id] = block;
  _stats.alloc_cnt++;
  _stats.allocated += block->size;
  _stats.peak_allocated = std::max(_stats.peak_allocated, _stats.allocated);
  return DataPtr(block->ptr, block->size, _device, block->id, fresh);
}

DataPtr CachingMemoryPool::AllocDataSpace(size_t num_bytes, const Stream& stream_in) {
  if (num_bytes == 0) return DataPtr(nullptr, 0, _device, 0);
  const Stream stream = normalize(stream_in);
  const PackedStreamId sid = stream.pack();
  const size_t bytes = RoundRequest(num_bytes);
  std::lock_guard<std::mutex> lock(_mtx);
  if (!_parked.empty()) collect_parked(false);

  if (Block* b = take_from(_free[sid], bytes)) {
    _stats.cache_hits++;
    return hand_out(b, false);
  }
  // another stream's cached block, ordered behind that stream's queued work
  for (auto& kv : _free) {
    if (kv.first == sid || kv.second.empty()) continue;
    if (Block* b = take_from(kv.second, bytes)) {
      const Stream owner = Stream::unpack(b->owner);
      void* ev = _backend->EventRecord(owner);
      _backend->StreamWaitEvent(stream, ev);
      _backend->EventRelease(ev);
      b->owner = sid;
      _stats.cross_stream_takes++;
      return hand_out(b, false);
    }
  }
  Block* b = new_segment(bytes, sid);
  if (b == nullptr) {
    HT_RUNTIME_ERROR << name() << ": out of memory on " << _device << " while allocating " << bytes
                     << " bytes (allocated " << (_stats.allocated >> 20) << " MiB, reserved "
                     << (_stats.reserved >> 20)
                     << " MiB); if the reserved memory is fragmented, set HETU_MAX_SPLIT_SIZE_MB smaller";
  }
  return hand_out(b, true);
}

DataPtr CachingMemoryPool::BorrowDataSpace(void* ptr, size_t num_bytes, DataPtrDeleter deleter, const Stream&) {
  HT_VALUE_ERROR_IF(ptr == nullptr && num_bytes > 0) << "Borrowing a null pointer";
  std::lock_guard<std::mutex> lock(_mtx);
  DataPtr dp(ptr, num_bytes, _device, next_id());
  _borrowed[dp.id] = Borrowed{dp, std::move(deleter), {}};
  return dp;
}

void CachingMemoryPool::FreeDataSpace(DataPtr data_ptr) {
  if (data_ptr.ptr == nullptr && data_ptr.size == 0 && data_ptr.id == 0) return;
  std::unique_lock<std::mutex> lock(_mtx);
  auto bit = _borrowed.find(data_ptr.id);
  if (bit != _borrowed.end()) {
    Borrowed br = std::move(bit->second);
    _borrowed.erase(bit);
    lock.unlock();
    // the lender may reuse the memory as soon as the deleter runs
    for (auto s : br.used_by) _backend->StreamSync(Stream::unpack(s));
    if (br.deleter) br.deleter(br.ptr);
    return;
  }
  auto it = _live.find(data_ptr.id);
  HT_VALUE_ERROR_IF(it == _live.end()) << name() << ": cannot find " << data_ptr << " (freed twice?)";
  Block* b = it->second;
  _live.erase(it);
  _stats.free_cnt++;
  _stats.allocated -= b->size;
  if (b->used_by.empty()) {
    release(b);
    return;
  }
  Parked p;
  p.block = b;
  b->in_use = false;
  for (auto s : b->used_by) p.events.push_back(_backend->EventRecord(Stream::unpack(s)));
  _parked.push_back(std::move(p));
  _stats.parked++;
}

void CachingMemoryPool::MarkDataSpaceUsedByStream(DataPtr data_ptr, const Stream& stream) {
  if (data_ptr.ptr == nullptr || !stream.is_defined()) return;
  const PackedStreamId sid = stream.pack();
  std::lock_guard<std::mutex> lock(_mtx);
  std::vector<PackedStreamId>* used = nullptr;
  auto it = _live.find(data_ptr.id);
  if (it != _live.end()) {
    if (it->second->owner == sid) return;
    used = &it->second->used_by;
  } else {
    auto bit = _borrowed.find(data_ptr.id);
    HT_VALUE_ERROR_IF(bit == _borrowed.end()) << name() << ": cannot find " << data_ptr;
    used = &bit->second.used_by;
  }
  if (std::find(used->begin(), used->end(), sid) == used->end()) {
    used->push_back(sid);
    _stats.mark_cnt++;
  }
}

void CachingMemoryPool::MarkDataSpacesUsedByStream(DataPtrList& data_ptrs, const Stream& stream) {
  for (auto& p : data_ptrs) MarkDataSpaceUsedByStream(p, stream);
}

std::future<void> CachingMemoryPool::WaitDataSpace(DataPtr data_ptr, bool async) {
  std::vector<PackedStreamId> streams;
  {
    std::lock_guard<std::mutex> lock(_mtx);
    auto it = _live.find(data_ptr.id);
    if (it != _live.end()) {
      streams = it->second->used_by;
      streams.push_back(it->second->owner);
    } else {
      auto bit = _borrowed.find(data_ptr.id);
      if (bit != _borrowed.end()) streams = bit->second.used_by;
    }
  }
  auto wait = [this, streams]() {
    for (auto s : streams) _backend->StreamSync(Stream::unpack(s));
  };
  if (async) return std::async(std::launch::async, wait);
  wait();
  std::promise<void> done;
  done.set_value();
  return done.get_future();
}

void CachingMemoryPool::EmptyCache() {
  std::lock_guard<std::mutex> lock(_mtx);
  collect_parked(true);
  release_free_segments();
}

PoolStats CachingMemoryPool::stats() {
  std::lock_guard<std::mutex> lock(_mtx);
  return _stats;
}

void CachingMemoryPool::PrintSummary() {
  PoolStats s = stats();
  const double mib = 1024.0 * 1024.0;
  HT_LOG_INFO << name() << ": allocated = " << s.allocated / mib << " MiB, peak_allocated = "
              << s.peak_allocated / mib << " MiB, reserved = " << s.reserved / mib << " MiB, peak_reserved = "
              << s.peak_reserved / mib << " MiB, alloc_cnt = " << s.alloc_cnt << ", free_cnt = " << s.free_cnt
              << ", mark_cnt = " << s.mark_cnt << ", segments = " << s.segment_allocs - s.segment_frees
              << ", cache_hits = " << s.cache_hits << ", cross_stream_takes = " << s.cross_stream_takes
              << ", parked = " << s.parked;
}

} // namespace impl
} // namespace hetu
