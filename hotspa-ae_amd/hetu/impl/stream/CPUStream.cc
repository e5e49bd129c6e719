#include "hetu/impl/stream/CPUStream.h"

#include <atomic>
#include <condition_variable>
#include <deque>
#include <mutex>
#include <thread>

#include "hetu/common/except.h"

namespace hetu {
namespace impl {

namespace {

// as many tasks may wait on one stream before EnqueueTask holds its caller back (task_queue.h:21 of the reference)
constexpr size_t kMaxPendingTasks = 10240;

struct Task {
  std::function<void()> run;
  std::promise<void> done;
  std::string name;
};

// One host stream: its tasks, the thread that runs them, and what Sync() waits on.
struct Lane {
  std::mutex mtx;
  std::condition_variable wake;       // a task has arrived
  std::condition_variable progress;   // a task has run, or has been taken off a full queue
  std::deque<Task> tasks;
  uint64_t enqueued = 0;
  uint64_t completed = 0;
  std::exception_ptr failure;         // the first task that threw since the last Sync()
  std::string failed_task;
};

// The lanes live until the process ends and their workers are never joined: a worker that waits for a task when
// the process exits is simply ended with it, and nothing has to be torn down in an order that static destructors
// could get wrong.
struct Lanes {
  std::mutex create;
  std::atomic<Lane*> lane[HT_NUM_STREAMS_PER_DEVICE];
  Lanes() {
    for (auto& l : lane) l.store(nullptr, std::memory_order_relaxed);
  }
};

Lanes& lanes() {
  static Lanes* l = new Lanes();
  return *l;
}

std::atomic<int64_t> g_pending{0};
std::atomic<int> g_host_kernel_threads{0};

// index of the stream whose worker the current thread is, -1 for every other thread
thread_local StreamIndex tl_worker_of = -1;

void RunLane(Lane* lane, StreamIndex index) {
  tl_worker_of = index;
  for (;;) {
    Task task;
    {
      std::unique_lock<std::mutex> lock(lane->mtx);
      lane->wake.wait(lock, [lane] { return !lane->tasks.empty(); });
      task = std::move(lane->tasks.front());
      lane->tasks.pop_front();
    }
    lane->progress.notify_all();   // room in the queue again
    std::exception_ptr thrown;
    try {
      task.run();
    } catch (...) {
      thrown = std::current_exception();
    }
    task.run = nullptr;   // what the task held (arrays, events) goes before anyone is told that it has run
    {
      std::lock_guard<std::mutex> lock(lane->mtx);
      lane->completed++;
      if (thrown && !lane->failure) {
        lane->failure = thrown;
        lane->failed_task = task.name;
      }
    }
    if (thrown) task.done.set_exception(thrown);
    else task.done.set_value();
    g_pending.fetch_sub(1, std::memory_order_release);
    lane->progress.notify_all();
  }
}

Lane* FindLane(StreamIndex index) { return lanes().lane[index].load(std::memory_order_acquire); }

Lane* LaneOf(StreamIndex index) {
  Lane* lane = FindLane(index);
  if (lane != nullptr) return lane;
  auto& all = lanes();
  std::lock_guard<std::mutex> lock(all.create);
  lane = all.lane[index].load(std::memory_order_acquire);
  if (lane == nullptr) {
    lane = new Lane();
    std::thread(RunLane, lane, index).detach();
    all.lane[index].store(lane, std::memory_order_release);
  }
  return lane;
}

} // namespace

CPUStream::CPUStream(const Stream& stream) : _stream_id(stream.stream_index()) {
  HT_ASSERT(stream.device().is_cpu()) << "Initializing CPU stream for non-host device: " << stream.device();
  HT_ASSERT(_stream_id >= kBlockingStream && _stream_id < HT_NUM_STREAMS_PER_DEVICE)
    << "Invalid device stream id: " << _stream_id;
}

std::future<void> CPUStream::EnqueueTask(std::function<void()> f, const std::string& name) {
  if (_stream_id == kBlockingStream || tl_worker_of == _stream_id) {
    f();   // in the calling thread; what it throws goes to the caller
    std::promise<void> done;
    done.set_value();
    return done.get_future();
  }
  Lane* lane = LaneOf(_stream_id);
  Task task;
  task.run = std::move(f);
  task.name = name;
  std::future<void> future = task.done.get_future();
  {
    std::unique_lock<std::mutex> lock(lane->mtx);
    lane->progress.wait(lock, [lane] { return lane->tasks.size() < kMaxPendingTasks; });
    lane->tasks.push_back(std::move(task));
    lane->enqueued++;
    g_pending.fetch_add(1, std::memory_order_relaxed);
  }
  lane->wake.notify_one();
  return future;
}

void CPUStream::Sync() {
  if (_stream_id == kBlockingStream) return;
  // from the stream's own worker: everything enqueued before the running task has run already
  if (tl_worker_of == _stream_id) return;
  Lane* lane = FindLane(_stream_id);
  if (lane == nullptr) return;
  std::exception_ptr failure;
  std::string failed_task;
  {
    std::unique_lock<std::mutex> lock(lane->mtx);
    const uint64_t target = lane->enqueued;
    lane->progress.wait(lock, [lane, target] { return lane->completed >= target; });
    failure = lane->failure;
    lane->failure = nullptr;
    failed_task.swap(lane->failed_task);
  }
  if (failure) std::rethrow_exception(failure);
}

uint64_t CPUStream::num_enqueued_tasks() const {
  Lane* lane = _stream_id == kBlockingStream ? nullptr : FindLane(_stream_id);
  if (lane == nullptr) return 0;
  std::lock_guard<std::mutex> lock(lane->mtx);
  return lane->enqueued;
}

uint64_t CPUStream::num_completed_tasks() const {
  Lane* lane = _stream_id == kBlockingStream ? nullptr : FindLane(_stream_id);
  if (lane == nullptr) return 0;
  std::lock_guard<std::mutex> lock(lane->mtx);
  return lane->completed;
}

void SynchronizeAllCPUStreams() {
  // every stream is waited for even if an earlier one reports a failure; the first failure is the one rethrown
  std::exception_ptr first;
  for (StreamIndex i = 0; i < HT_NUM_STREAMS_PER_DEVICE; ++i) {
    try {
      GetCPUStream(i).Sync();
    } catch (...) {
      if (!first) first = std::current_exception();
    }
  }
  if (first) std::rethrow_exception(first);
}

bool AnyCPUStreamBusy() { return g_pending.load(std::memory_order_acquire) > 0; }

void SetHostKernelThreads(int threads) { g_host_kernel_threads.store(threads > 0 ? threads : 0, std::memory_order_relaxed); }
int HostKernelThreads() { return g_host_kernel_threads.load(std::memory_order_relaxed); }

CPUEvent::CPUEvent(bool enable_timing) : Event(Device(kCPU), enable_timing) {}

void CPUEvent::Record(const Stream& stream) {
  auto state = std::make_shared<State>();
  const bool timing = enable_timing();
  // the task owns the state until it has run, so the stamp is written whatever happens to this object meanwhile
  std::future<void> reached = CPUStream(stream).EnqueueTask(
    [state, timing]() {
      if (timing) state->at = std::chrono::steady_clock::now();
    },
    "Event_Record");
  state->reached = reached.share();
  _state = std::move(state);
  _recorded = true;
}

void CPUEvent::Sync() {
  HT_ASSERT(_recorded) << "Event has not been recorded";
  _state->reached.wait();
}

void CPUEvent::Block(const Stream& stream) {
  HT_ASSERT(_recorded) << "Event has not been recorded";
  auto state = _state;
  CPUStream(stream).EnqueueTask([state]() { state->reached.wait(); }, "Event_Block");
}

int64_t CPUEvent::TimeSince(const Event& event) const {
  const auto* other = dynamic_cast<const CPUEvent*>(&event);
  HT_VALUE_ERROR_IF(other == nullptr) << "TimeSince needs another host event";
  HT_VALUE_ERROR_IF(!enable_timing() || !other->enable_timing()) << "Cannot measure time when timing is disabled";
  HT_ASSERT(_recorded == other->_recorded) << "Only one of Start/Stop event has been recorded!";
  if (!_recorded) return 0;
  _state->reached.wait();
  other->_state->reached.wait();
  return std::chrono::duration_cast<std::chrono::nanoseconds>(_state->at - other->_state->at).count();
}

} // namespace impl
} // namespace hetu
