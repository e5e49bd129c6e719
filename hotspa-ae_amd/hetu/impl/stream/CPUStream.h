// Host streams and events behind hetu::Stream / hetu::Event for Device(kCPU)
// (hetu/impl/stream/CPUStream.{h,cc}:15-48 and hetu/utils/task_queue.h:15-133 of
// the reference): a host stream is a queue of tasks that one worker thread, created
// with the stream's first task, runs in the order they were enqueued.  Stream index
// 0 (the blocking stream) has no queue: its tasks run at once in the calling thread.
//
// Two things are stricter here than in the reference.  A task that throws does not
// vanish with its future: the stream keeps the first such failure and the next
// Sync() on it rethrows it.  And a task that is enqueued from the stream's own
// worker (a host kernel calling another on its stream) runs at once, inside the
// running task, instead of waiting behind it.
#pragma once

#include <chrono>
#include <functional>
#include <future>
#include <memory>
#include <string>

#include "hetu/core/stream.h"

namespace hetu {
namespace impl {

class CPUStream final {
 public:
  explicit CPUStream(const Stream& stream);

  // f runs after every task enqueued on this stream before it.  The future becomes ready when f has run and
  // carries what f threw, if anything.
  std::future<void> EnqueueTask(std::function<void()> f, const std::string& name = "");

  // Returns when every task enqueued before the call has run; rethrows the first failure among them (once).
  void Sync();

  StreamIndex stream_id() const noexcept { return _stream_id; }

  // Tasks enqueued on this stream so far / of those, how many have run (for tests and diagnostics).
  uint64_t num_enqueued_tasks() const;
  uint64_t num_completed_tasks() const;

 private:
  StreamIndex _stream_id;
};

inline CPUStream GetCPUStream(StreamIndex stream_id) { return CPUStream(Stream(Device(kCPU), stream_id)); }
inline CPUStream GetCPUComputingStream() { return GetCPUStream(kComputingStream); }

void SynchronizeAllCPUStreams();

// True while any host stream still has a task to run (one relaxed load: cheap enough to ask after every call).
bool AnyCPUStreamBusy();

// Threads a host kernel's OpenMP team takes, whichever thread runs it (0 = the runtime's default).  The value
// lives in this library rather than in the OpenMP runtime's per-thread setting, which a stream's worker thread
// would not see.
void SetHostKernelThreads(int threads);
int HostKernelThreads();

class CPUEvent final : public Event {
 public:
  explicit CPUEvent(bool enable_timing = true);
  bool IsRecorded() override { return _recorded; }
  // a task on `stream` that stamps the time: the event has happened when the stream gets there
  void Record(const Stream& stream) override;
  void Sync() override;
  // a task on `stream` that waits for the event: what is enqueued on it afterwards runs after the event
  void Block(const Stream& stream) override;
  int64_t TimeSince(const Event& event) const override;   // ns from `event` to this one

 private:
  struct State {
    std::shared_future<void> reached;
    std::chrono::time_point<std::chrono::steady_clock> at;
  };
  // shared with the tasks, so that an event may be destroyed while a stream still has to get to it
  std::shared_ptr<State> _state;
  bool _recorded{false};
};

} // namespace impl
} // namespace hetu
