// Host-side checks of the C++ operator layer that need no GPU: dtypes, devices,
// streams, axis parsing, exceptions, the host pool, NDArray views, the device
// switch, and the caching pool's policy driven through a scripted backend.
// Prints one line per check; exit status is the number of failed checks.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <atomic>
#include <functional>
#include <future>
#include <set>
#include <string>
#include <thread>
#include <vector>

#include "hetu/core/ndarray.h"
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/memory/CachingMemoryPool.h"
#include "hetu/impl/random/CPURandomState.h"
#include "hetu/impl/stream/CPUStream.h"
#include "hetu/impl/utils/dispatch.h"

using namespace hetu;
using hetu::impl::CachingMemoryPool;
using hetu::impl::PoolBackend;

static int g_failed = 0, g_run = 0;

#define CHECK(cond)                                                                    \
  do {                                                                                 \
    if (!(cond)) {                                                                     \
      std::printf("    CHECK FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);          \
      throw std::runtime_error("check failed");                                        \
    }                                                                                  \
  } while (0)

template <typename E, typename F>
static bool throws(F&& f, const char* needle = nullptr) {
  try {
    f();
  } catch (const E& e) {
    return needle == nullptr || std::string(e.what()).find(needle) != std::string::npos;
  } catch (...) {
    return false;
  }
  return false;
}

static void run(const char* name, const std::function<void()>& body) {
  ++g_run;
  try {
    body();
    std::printf("[ OK ] %s\n", name);
  } catch (const std::exception& e) {
    ++g_failed;
    std::printf("[FAIL] %s: %s\n", name, e.what());
  }
  std::fflush(stdout);
}

// ---- scripted device: addresses are never dereferenced ----
struct FakeDevice : PoolBackend {
  size_t capacity;
  size_t in_use = 0;
  uintptr_t next_addr = uintptr_t(1) << 32;
  std::map<void*, size_t> live;
  struct Ev { Stream stream; bool done; };
  std::vector<Ev*> events;
  std::vector<std::pair<PackedStreamId, PackedStreamId>> waits;   // (waiting stream, recorded-on stream)
  int device_syncs = 0, stream_syncs = 0;
  bool auto_complete = false;

  explicit FakeDevice(size_t cap) : capacity(cap) {}
  ~FakeDevice() override { for (auto* e : events) delete e; }
  void* RawAlloc(size_t bytes) override {
    if (in_use + bytes > capacity) return nullptr;
    void* p = reinterpret_cast<void*>(next_addr);
    next_addr += (bytes + (size_t(2) << 20) - 1) / (size_t(2) << 20) * (size_t(2) << 20) + (size_t(2) << 20);
    live[p] = bytes;
    in_use += bytes;
    return p;
  }
  void RawFree(void* ptr) override {
    auto it = live.find(ptr);
    if (it == live.end()) throw std::runtime_error("RawFree of unknown pointer");
    in_use -= it->second;
    live.erase(it);
  }
  void* EventRecord(const Stream& s) override {
    auto* e = new Ev{s, auto_complete};
    events.push_back(e);
    return e;
  }
  bool EventDone(void* e) override { return static_cast<Ev*>(e)->done; }
  void EventSync(void* e) override { static_cast<Ev*>(e)->done = true; }
  void EventRelease(void*) override {}
  void StreamWaitEvent(const Stream& s, void* e) override {
    waits.emplace_back(s.pack(), static_cast<Ev*>(e)->stream.pack());
  }
  void StreamSync(const Stream&) override { ++stream_syncs; }
  void DeviceSync() override { ++device_syncs; }
  void complete_all() { for (auto* e : events) e->done = true; }
};

static const size_t MiB = size_t(1) << 20;

struct PoolFixture {
  FakeDevice* dev;
  std::unique_ptr<CachingMemoryPool> pool;
  Stream s1{Device(kCUDA, 0), 1}, s2{Device(kCUDA, 0), 2}, s3{Device(kCUDA, 0), 3};
  explicit PoolFixture(size_t capacity = 4096 * MiB, size_t max_split = 200 * MiB, size_t max_frag = 20 * MiB) {
    dev = new FakeDevice(capacity);
    pool.reset(new CachingMemoryPool(Device(kCUDA, 0), "TestPool", std::unique_ptr<PoolBackend>(dev), max_split,
                                     max_frag));
  }
};

int main() {
  run("dtype sizes and names", [] {
    CHECK(DataType2Size(kFloat32) == 4 && DataType2Size(kBFloat16) == 2 && DataType2Size(kFloat16) == 2);
    CHECK(DataType2Size(kFloat64) == 8 && DataType2Size(kInt64) == 8 && DataType2Size(kUInt8) == 1);
    CHECK(int(kFloat16) == 5 && int(kFloat32) == 6 && int(kFloat64) == 7 && int(kBFloat16) == 8 && int(kInt64) == 4);
    CHECK(DataType2Str(kBFloat16) == "bfloat16");
  });

  run("seed source: unseeded follows the clock, seeded replays a 64-bit Mersenne Twister", [] {
    using hetu::impl::GenNextRandomSeed;
    using hetu::impl::SetCPURandomSeed;
    CHECK(GenNextRandomSeed() != 0);
    SetCPURandomSeed(0);                                     // ignored
    SetCPURandomSeed(5489);                                  // the generator's own default seed
    CHECK(GenNextRandomSeed() == 14514284786278117030ull);   // its documented first output
    uint64_t v = 0;
    for (int i = 1; i < 10000; ++i) v = GenNextRandomSeed();
    CHECK(v == 9981545732273789042ull);                      // and its 10000th (the C++ standard's check value)
    SetCPURandomSeed(5489);
    CHECK(GenNextRandomSeed() == 14514284786278117030ull);
  });

  run("bfloat16 rounds to nearest even and keeps NaN", [] {
    CHECK(bfloat16(1.0f).val == 0x3F80);
    // 1 + 2^-8 is the midpoint between 1 and the next bf16: ties go to even (1.0)
    CHECK(bfloat16(1.0f + 0.00390625f).val == 0x3F80);
    // 1 + 3*2^-8 is the midpoint between 0x3F81 and 0x3F82: even is 0x3F82
    CHECK(bfloat16(1.0f + 3 * 0.00390625f).val == 0x3F82);
    CHECK(bfloat16(std::nanf("")).val == 0x7FC0);
    CHECK(float(bfloat16(-2.5f)) == -2.5f);
    CHECK(std::isinf(float(bfloat16(3.4e38f))));
  });

  run("float16 round trip of every finite half", [] {
    for (uint32_t h = 0; h < 65536; ++h) {
      float16 a;
      a.val = uint16_t(h);
      const bool nan = ((h & 0x7C00) == 0x7C00) && (h & 0x3FF);
      if (nan) { CHECK(std::isnan(float(a))); continue; }
      CHECK(float16(float(a)).val == h);
    }
    CHECK(float16(65520.f).val == 0x7C00 && float16(65519.f).val == 0x7BFF);
    CHECK(float16(1.0f + 0.00048828125f).val == 0x3C00);   // tie -> even
  });

  run("device and stream handles", [] {
    Device d(kCUDA, 3), c(kCPU, 5);
    CHECK(d.is_cuda() && d.index() == 3 && c.is_cpu() && c.index() == 0);
    CHECK(throws<assertion_error>([] { Device(kCUDA, 16); }));
    for (int dev = 0; dev < 16; ++dev)
      for (int id = 0; id < HT_NUM_STREAMS_PER_DEVICE; ++id) {
        Stream s(Device(kCUDA, DeviceIndex(dev)), id);
        CHECK(Stream::unpack(s.pack()) == s);
      }
    CHECK(Stream::unpack(Stream(Device(kCPU), 0).pack()) == Stream(Device(kCPU), 0));
    CHECK(throws<assertion_error>([] { Stream(Device(kCUDA, 0), 16); }));
    CHECK(throws<assertion_error>([] { Stream(Device(kCUDA, 0), -1); }));
    CHECK(!Stream().is_defined() && Stream(Device(kCUDA, 0)).is_blocking());
    CHECK(kBlockingStream == 0 && kComputingStream == 1 && NDArray::DEFAULT_STREAM == kComputingStream);
  });

  run("exceptions carry kind and message", [] {
    CHECK(throws<assertion_error>([] { HT_ASSERT(1 == 2) << "custom text " << 42; }, "custom text 42"));
    CHECK(throws<not_implemented>([] { HT_NOT_IMPLEMENTED << "nope"; }, "nope"));
    CHECK(throws<value_error>([] { HT_VALUE_ERROR_IF(true) << "bad value"; }, "bad value"));
    CHECK(throws<runtime_error>([] { HT_RUNTIME_ERROR << "rt"; }, "rt"));
    CHECK(throws<hetu_exception>([] { HT_ASSERT_EQ(1, 2) << "eq"; }));
    bool ran = false;
    HT_ASSERT(true) << "never evaluated";
    HT_VALUE_ERROR_IF(false) << "never";
    ran = true;
    CHECK(ran);
  });

  run("axis parsing and reduced shapes", [] {
    CHECK(NDArrayMeta::ParseAxis(-1, 3) == 2 && NDArrayMeta::ParseAxis(0, 3) == 0);
    CHECK(throws<assertion_error>([] { NDArrayMeta::ParseAxis(3, 3); }));
    CHECK(throws<assertion_error>([] { NDArrayMeta::ParseAxis(-4, 3); }));
    CHECK((NDArrayMeta::ParseAxes({}, 3) == HTAxes{0, 1, 2}));
    CHECK((NDArrayMeta::ParseAxes({-1, 0, 2, 0}, 3) == HTAxes{0, 2}));
    CHECK((NDArrayMeta::Reduce({4, 5, 6}, {1}, false) == HTShape{4, 6}));
    CHECK((NDArrayMeta::Reduce({4, 5, 6}, {1}, true) == HTShape{4, 1, 6}));
    CHECK((NDArrayMeta::Reduce({4, 5, 6}, {}, false) == HTShape{1}));
    CHECK((NDArrayMeta::Reduce({4, 5, 6}, {0, -1}, false) == HTShape{5}));
    CHECK((NDArrayMeta::Reduce({4, 5, 6}, {}, true) == HTShape{1, 1, 1}));
  });

  run("meta strides and contiguity", [] {
    NDArrayMeta m({2, 3, 4}, kFloat32, Device(kCPU));
    CHECK((m.stride == HTStride{12, 4, 1}) && m.is_contiguous() && m.numel() == 24);
    m.set_stride({1, 2, 6});
    CHECK(!m.is_contiguous());
    CHECK(throws<assertion_error>([&] { m.set_stride({1, 2}); }));
    NDArrayMeta one({1, 1}, kFloat32, Device(kCPU), {7, 9});
    CHECK(one.is_contiguous());
  });

  run("dtype switch macros", [] {
    size_t size = 0;
    HT_DISPATCH_FLOATING_TYPES(kBFloat16, spec_t, "probe", [&]() { size = sizeof(spec_t); });
    CHECK(size == 2);
    HT_DISPATCH_INTEGER_AND_FLOATING_TYPES(kInt64, spec_t, "probe", [&]() { size = sizeof(spec_t); });
    CHECK(size == 8);
    CHECK(throws<not_implemented>(
      [&] { HT_DISPATCH_FLOATING_TYPES(kInt32, spec_t, "probe", [&]() { size = sizeof(spec_t); }); }, "probe"));
  });

  run("host pool: allocate, borrow, free", [] {
    auto pool = GetMemoryPool(Device(kCPU));
    DataPtr a = pool->AllocDataSpace(100);
    CHECK(a.ptr != nullptr && a.size >= 100 && (reinterpret_cast<uintptr_t>(a.ptr) % 64) == 0);
    std::memset(a.ptr, 0xAB, 100);
    pool->FreeDataSpace(a);
    CHECK(throws<value_error>([&] { pool->FreeDataSpace(a); }));
    DataPtr z = pool->AllocDataSpace(0);
    CHECK(z.ptr == nullptr && z.size == 0);
    pool->FreeDataSpace(z);
    int deleted = 0;
    float mine[4] = {1, 2, 3, 4};
    DataPtr b = pool->BorrowDataSpace(mine, sizeof(mine), [&](DataPtr) { ++deleted; });
    CHECK(b.ptr == mine);
    pool->FreeDataSpace(b);
    CHECK(deleted == 1 && mine[2] == 3.f);
  });

  run("host NDArray: views, permute, slice, contiguous", [] {
    NDArray a = NDArray::empty({2, 3, 4}, Device(kCPU), kFloat32);
    float* p = a->data_ptr<float>();
    for (int i = 0; i < 24; ++i) p[i] = float(i);
    NDArray v = NDArray::view(a, {6, -1});
    CHECK((v->shape() == HTShape{6, 4}) && v->data_ptr<float>() == p);
    CHECK(throws<value_error>([&] { NDArray::view(a, {5, -1}); }));
    NDArray t = NDArray::permute(a, {2, 0, 1});
    CHECK((t->shape() == HTShape{4, 2, 3}) && (t->stride() == HTStride{1, 12, 4}) && !t->is_contiguous());
    NDArray tc = NDArray::contiguous(t);   // on the host computing stream: a task, waited for before reading
    SynchronizeAllStreams(Device(kCPU));
    CHECK(tc->is_contiguous() && tc->data_ptr<float>() != p);
    // tc[k][i][j] = a[i][j][k]
    for (int k = 0; k < 4; ++k)
      for (int i = 0; i < 2; ++i)
        for (int j = 0; j < 3; ++j) CHECK(tc->data_ptr<float>()[(k * 2 + i) * 3 + j] == float((i * 3 + j) * 4 + k));
    NDArray s = NDArray::slice(a, {1, 1, 0}, {1, 2, 4});
    CHECK(s->storage_offset() == 16 && s->data_ptr<float>()[0] == 16.f);
    CHECK(throws<value_error>([&] { NDArray::slice(a, {1, 2, 0}, {1, 2, 4}); }));
    CHECK(throws<value_error>([&] { NDArray::permute(a, {0, 0, 1}); }));
    NDArray z = NDArray::zeros({5}, Device(kCPU), kInt64);
    for (int i = 0; i < 5; ++i) CHECK(z->data_ptr<int64_t>()[i] == 0);
    NDArray e = NDArray::empty({0, 7}, Device(kCPU), kFloat32);
    CHECK(e->numel() == 0 && e->is_contiguous());
    // a view that reaches past its storage (96 B, held in 128) is refused
    CHECK(throws<assertion_error>([&] { NDArray::as_strided(a, {2, 3, 4}, {12, 4, 1}, 9); }));
  });

  run("device switch: host arrays run the host twins, accelerator-only kernels refuse them", [] {
    NDArray a = NDArray::zeros({4, 8}, Device(kCPU), kFloat32);
    NDArray g = NDArray::zeros({8}, Device(kCPU), kFloat32);
    for (int i = 0; i < 32; ++i) a->data_ptr<float>()[i] = float(i % 8);
    for (int i = 0; i < 8; ++i) g->data_ptr<float>()[i] = 1.f;
    NDArray sm = NDArray::softmax(a, 1);
    Stream(Device(kCPU), kComputingStream).Sync();
    for (int r = 0; r < 4; ++r) {
      float s = 0.f;
      for (int c = 0; c < 8; ++c) s += sm->data_ptr<float>()[r * 8 + c];
      CHECK(std::fabs(s - 1.f) < 1e-6f);
    }
    NDArray cs = NDArray::sum(a, {0});
    Stream(Device(kCPU), kComputingStream).Sync();
    for (int c = 0; c < 8; ++c) CHECK(cs->data_ptr<float>()[c] == 4.f * float(c));
    NDArrayList ln = NDArray::layernorm(a, g, NDArray::zeros({8}, Device(kCPU), kFloat32), {8});
    Stream(Device(kCPU), kComputingStream).Sync();
    CHECK(std::fabs(ln[1]->data_ptr<float>()[0] - 3.5f) < 1e-6f);     // mean of 0..7
    CHECK(std::fabs(ln[2]->data_ptr<float>()[0] - 5.25f) < 1e-5f);    // variance of 0..7
    // the fused variant exists for the accelerator only: the switch itself refuses
    CHECK(throws<not_implemented>([&] { NDArray::fused_layernorm(a, g, g, {8}); }, "cpu"));
    NDArray lab = NDArray::zeros({4}, Device(kCPU), kInt64);
    lab->data_ptr<int64_t>()[1] = -1;   // ignored
    NDArray loss = NDArray::sceloss(a, lab, int64_t(-1), kNONE);
    Stream(Device(kCPU), kComputingStream).Sync();
    CHECK(loss->data_ptr<float>()[1] == 0.f && loss->data_ptr<float>()[0] > 7.f);
    // an accelerator kernel handed host arrays fails its device assertion
    NDArray out = NDArray::empty_like(a);
    CHECK(throws<assertion_error>([&] { hetu::impl::SoftmaxCuda(a, out, 1, Stream(Device(kCUDA, 0), 1)); }));
    CHECK(throws<assertion_error>(
      [&] { hetu::impl::ReduceCuda(a, out, {0}, kSUM, Stream(Device(kCUDA, 0), 1)); }));
  });

  run("host streams: a worker per stream, order within a stream, events across streams, failures at Sync", [] {
    using hetu::impl::CPUEvent;
    using hetu::impl::CPUStream;
    using hetu::impl::GetCPUStream;
    const Device cpu(kCPU);
    // the blocking stream runs in the calling thread, before EnqueueTask returns, and throws to the caller
    std::thread::id ran_on;
    GetCPUStream(kBlockingStream).EnqueueTask([&] { ran_on = std::this_thread::get_id(); });
    CHECK(ran_on == std::this_thread::get_id());
    CHECK(throws<value_error>([] { GetCPUStream(kBlockingStream).EnqueueTask([] { HT_VALUE_ERROR << "now"; }); }, "now"));
    // any other stream has its own thread and keeps the order of its tasks
    std::vector<int> order;
    std::thread::id worker3, worker4;
    std::promise<void> gate;
    std::shared_future<void> open = gate.get_future().share();
    CPUStream s3 = GetCPUStream(3), s4 = GetCPUStream(4);
    const uint64_t before = s3.num_enqueued_tasks();
    s3.EnqueueTask([&, open] { open.wait(); worker3 = std::this_thread::get_id(); order.push_back(1); }, "first");
    for (int i = 2; i <= 50; ++i) s3.EnqueueTask([&order, i] { order.push_back(i); });
    CHECK(s3.num_enqueued_tasks() == before + 50 && s3.num_completed_tasks() == before);   // nothing ran: the call returned
    CHECK(hetu::impl::AnyCPUStreamBusy());
    s4.EnqueueTask([&] { worker4 = std::this_thread::get_id(); });
    s4.Sync();                         // stream 4 does not wait for stream 3
    CHECK(order.empty());
    gate.set_value();
    Stream(cpu, 3).Sync();             // through the device-independent handle
    CHECK(order.size() == 50);
    for (int i = 0; i < 50; ++i) CHECK(order[size_t(i)] == i + 1);
    CHECK(worker3 != std::this_thread::get_id() && worker4 != std::this_thread::get_id() && worker3 != worker4);
    CHECK(s3.num_completed_tasks() == before + 50);
    // a task enqueued from the stream's own worker runs inside the running task, not behind it
    std::vector<int> nested;
    s3.EnqueueTask([&] {
      nested.push_back(1);
      GetCPUStream(3).EnqueueTask([&] { nested.push_back(2); });
      GetCPUStream(3).Sync();          // from the worker: nothing to wait for
      nested.push_back(3);
    });
    s3.Sync();
    CHECK((nested == std::vector<int>{1, 2, 3}));
    // events: stream 4 waits for a point of stream 3
    std::promise<void> gate2;
    std::shared_future<void> open2 = gate2.get_future().share();
    std::atomic<int> stage{0};
    CPUEvent start, reached;
    CHECK(!reached.IsRecorded());
    CHECK(throws<assertion_error>([&] { reached.Sync(); }));
    start.Record(Stream(cpu, 3));
    s3.EnqueueTask([&, open2] { open2.wait(); stage = 1; });
    reached.Record(Stream(cpu, 3));
    reached.Block(Stream(cpu, 4));
    int seen_by_4 = -1;
    s4.EnqueueTask([&] { seen_by_4 = stage.load(); });
    CHECK(seen_by_4 == -1);
    gate2.set_value();
    reached.Sync();
    s4.Sync();
    CHECK(seen_by_4 == 1);
    CHECK(reached.TimeSince(start) >= 0);
    {   // an event may go away while its stream still has to reach it
      std::promise<void> gate3;
      std::shared_future<void> open3 = gate3.get_future().share();
      s3.EnqueueTask([open3] { open3.wait(); });
      { CPUEvent gone; gone.Record(Stream(cpu, 3)); }
      gate3.set_value();
      s3.Sync();
    }
    // a task that throws: its future carries the failure, and the next Sync on the stream reports the first one, once
    std::future<void> failed = s3.EnqueueTask([] { HT_VALUE_ERROR << "task one"; }, "one");
    s3.EnqueueTask([] { HT_RUNTIME_ERROR << "task two"; }, "two");
    int after = 0;
    s3.EnqueueTask([&] { after = 7; });
    CHECK(throws<value_error>([&] { s3.Sync(); }, "task one"));
    CHECK(after == 7);                 // the stream went on
    CHECK(throws<value_error>([&] { failed.get(); }, "task one"));
    s3.Sync();                         // reported once
    s3.EnqueueTask([] { HT_VALUE_ERROR << "again"; });
    CHECK(throws<value_error>([] { SynchronizeAllStreams(Device(kCPU)); }, "again"));
    CHECK(!hetu::impl::AnyCPUStreamBusy());
    CHECK(throws<assertion_error>([] { CPUStream(Stream(Device(kCUDA, 0), 1)); }));
  });

  run("host twins on a stream: argument checks at the call, the work in stream order, results after Sync", [] {
    const Device cpu(kCPU);
    const Stream st(cpu, 5);
    const int64_t rows = 64, cols = 96;
    NDArray x = NDArray::empty({rows, cols}, cpu, kFloat32);
    for (int64_t i = 0; i < rows * cols; ++i) x->data_ptr<float>()[i] = float((i * 37) % 101) * 0.05f - 2.f;
    // the same chain on the blocking stream (in this thread) and on stream 5 behind a gate
    auto chain = [&](const Stream& s, NDArray& y, NDArray& e, NDArray& sum) {
      hetu::impl::SoftmaxCpu(x, y, 1, s);
      hetu::impl::ExpCpu(y, e, s);                           // reads what the task before it writes
      hetu::impl::ReduceCpu(e, sum, {1}, kSUM, s);
    };
    NDArray y0 = NDArray::empty_like(x), e0 = NDArray::empty_like(x), s0 = NDArray::empty({rows}, cpu, kFloat32);
    chain(Stream(cpu, kBlockingStream), y0, e0, s0);
    NDArray y1 = NDArray::zeros({rows, cols}, cpu, kFloat32), e1 = NDArray::zeros({rows, cols}, cpu, kFloat32);
    NDArray s1 = NDArray::zeros({rows}, cpu, kFloat32);
    std::promise<void> gate;
    std::shared_future<void> open = gate.get_future().share();
    hetu::impl::CPUStream(st).EnqueueTask([open] { open.wait(); });
    chain(st, y1, e1, s1);
    CHECK(s1->data_ptr<float>()[0] == 0.f && y1->data_ptr<float>()[0] == 0.f);   // nothing has run yet
    // a bad argument is refused at the call, in this thread, while the stream is still held
    NDArray wrong = NDArray::empty({rows, cols + 1}, cpu, kFloat32);
    CHECK(throws<assertion_error>([&] { hetu::impl::SoftmaxCpu(x, wrong, 1, st); }));
    CHECK(throws<not_implemented>([&] {
      NDArray xi = NDArray::zeros({4, 4}, cpu, kInt32), yi = NDArray::zeros({4, 4}, cpu, kInt32);
      hetu::impl::SoftmaxCpu(xi, yi, 1, st);
    }));
    gate.set_value();
    st.Sync();
    CHECK(std::memcmp(y0->raw_data_ptr(), y1->raw_data_ptr(), size_t(rows * cols) * 4) == 0);
    CHECK(std::memcmp(e0->raw_data_ptr(), e1->raw_data_ptr(), size_t(rows * cols) * 4) == 0);
    CHECK(std::memcmp(s0->raw_data_ptr(), s1->raw_data_ptr(), size_t(rows) * 4) == 0);
    // a strided input is gathered inside the task, after the task that fills it
    NDArray base = NDArray::zeros({cols, rows}, cpu, kFloat32);
    NDArray xt = NDArray::permute(base, {1, 0});             // [rows, cols] view, not dense
    std::promise<void> gate2;
    std::shared_future<void> open2 = gate2.get_future().share();
    hetu::impl::CPUStream(st).EnqueueTask([open2, base, x, rows, cols] {
      open2.wait();
      for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) base->data_ptr<float>()[c * rows + r] = x->data_ptr<float>()[r * cols + c];
    });
    NDArray y2 = NDArray::empty_like(x);
    hetu::impl::SoftmaxCpu(xt, y2, 1, st);
    gate2.set_value();
    st.Sync();
    CHECK(std::memcmp(y0->raw_data_ptr(), y2->raw_data_ptr(), size_t(rows * cols) * 4) == 0);
    // the team size set through the library reaches the stream's worker
    hetu::impl::SetHostKernelThreads(1);
    NDArray big = NDArray::zeros({512, 512}, cpu, kFloat32), bigy = NDArray::empty({512, 512}, cpu, kFloat32);
    hetu::impl::SoftmaxCpu(big, bigy, 1, st);
    st.Sync();
    CHECK(std::fabs(bigy->data_ptr<float>()[0] - 1.f / 512.f) < 1e-7f);
    hetu::impl::SetHostKernelThreads(0);
    CHECK(hetu::impl::HostKernelThreads() == 0);
  });

  run("host twins of the neighbours: broadcasting arithmetic, broadcasts, norms, losses, batch norm", [] {
    const Device cpu(kCPU);
    const Stream st(cpu, 0);
    // [3, 1, 5] op [4, 1] -> [3, 4, 5], one operand read through a transposed view
    NDArray a = NDArray::empty({3, 1, 5}, cpu, kFloat32), b = NDArray::empty({1, 4}, cpu, kFloat32);
    for (int i = 0; i < 15; ++i) a->data_ptr<float>()[i] = float(i + 1);
    for (int i = 0; i < 4; ++i) b->data_ptr<float>()[i] = float(2 * i + 1);
    NDArray bt = NDArray::permute(b, {1, 0});   // [4, 1], strides {1, 4}
    NDArray out = NDArray::empty({3, 4, 5}, cpu, kFloat32);
    hetu::impl::SubElewiseCpu(a, bt, out, st);
    hetu::impl::DivElewiseCpu(out, bt, out, st);   // in place
    for (int i = 0; i < 3; ++i)
      for (int j = 0; j < 4; ++j)
        for (int k = 0; k < 5; ++k)
          CHECK(out->data_ptr<float>()[(i * 4 + j) * 5 + k] == (float(i * 5 + k + 1) - float(2 * j + 1)) / float(2 * j + 1));
    CHECK(throws<assertion_error>([&] { hetu::impl::AddElewiseCpu(a, NDArray::empty({3}, cpu, kFloat32), out, st); }));
    // integers wrap, a zero divisor gives zero
    NDArray i8 = NDArray::empty({4}, cpu, kInt8), j8 = NDArray::empty({4}, cpu, kInt8), o8 = NDArray::empty({4}, cpu, kInt8);
    const int8_t xs[4] = {127, -128, 100, 7}, ys[4] = {1, -1, 0, -2};
    for (int i = 0; i < 4; ++i) { i8->data_ptr<int8_t>()[i] = xs[i]; j8->data_ptr<int8_t>()[i] = ys[i]; }
    hetu::impl::AddElewiseCpu(i8, j8, o8, st);
    CHECK(o8->data_ptr<int8_t>()[0] == -128 && o8->data_ptr<int8_t>()[1] == 127);
    hetu::impl::DivElewiseCpu(i8, j8, o8, st);
    CHECK(o8->data_ptr<int8_t>()[1] == -128 && o8->data_ptr<int8_t>()[2] == 0 && o8->data_ptr<int8_t>()[3] == -3);
    hetu::impl::OppositeCpu(i8, o8, st);
    CHECK(o8->data_ptr<int8_t>()[0] == -127 && o8->data_ptr<int8_t>()[1] == -128);
    CHECK(throws<not_implemented>([&] { hetu::impl::ExpCpu(i8, o8, st); }));
    // constants: value - x, and a zero divisor is refused
    NDArray c = NDArray::empty({3, 1, 5}, cpu, kFloat32);
    hetu::impl::SubConstCpu(a, 20.0, c, st);
    CHECK(c->data_ptr<float>()[14] == 5.f);
    CHECK(throws<assertion_error>([&] { hetu::impl::DivConstCpu(a, 0.0, c, st); }, "Divided by 0"));
    // broadcast [5] -> [2, 5, 3] with the input's dimension in the middle, times a constant
    NDArray v = NDArray::empty({5}, cpu, kFloat32);
    for (int i = 0; i < 5; ++i) v->data_ptr<float>()[i] = float(i);
    NDArray wide = NDArray::empty({2, 5, 3}, cpu, kFloat32);
    hetu::impl::BroadcastShapeMulCpu(v, 0.5, wide, {0, 2}, st);
    for (int i = 0; i < 30; ++i) CHECK(wide->data_ptr<float>()[i] == 0.5f * float((i / 3) % 5));
    CHECK(throws<assertion_error>([&] { hetu::impl::BroadcastShapeCpu(v, wide, {0, 0}, st); }, "twice"));
    // 3-4-5: the 2-norm over the middle dimension, its gradient, and a zero norm
    NDArray x = NDArray::zeros({2, 2, 3}, cpu, kFloat32);
    x->data_ptr<float>()[0] = 3.f; x->data_ptr<float>()[3] = -4.f;   // column (0, :, 0) = (3, -4)
    NDArray n = NDArray::empty({2, 3}, cpu, kFloat32), g = NDArray::empty({2, 3}, cpu, kFloat32);
    for (int i = 0; i < 6; ++i) g->data_ptr<float>()[i] = 10.f;
    hetu::impl::NormCpu(x, n, 1, 2, st);
    CHECK(n->data_ptr<float>()[0] == 5.f && n->data_ptr<float>()[1] == 0.f);
    NDArray dx = NDArray::empty({2, 2, 3}, cpu, kFloat32);
    hetu::impl::NormGradientCpu(x, n, g, dx, 1, 2, st);
    CHECK(dx->data_ptr<float>()[0] == 6.f && dx->data_ptr<float>()[3] == -8.f && dx->data_ptr<float>()[1] == 0.f);
    hetu::impl::NormCpu(x, n, -2, 1, st);
    CHECK(n->data_ptr<float>()[0] == 7.f);
    CHECK(throws<value_error>([&] { hetu::impl::NormCpu(x, n, 1, 0, st); }));
    // negative log likelihood: picks, and labels outside the classes
    NDArray pred = NDArray::empty({3, 4}, cpu, kFloat32), lab = NDArray::empty({3}, cpu, kInt64);
    for (int i = 0; i < 12; ++i) pred->data_ptr<float>()[i] = float(i);
    lab->data_ptr<int64_t>()[0] = 2; lab->data_ptr<int64_t>()[1] = -1; lab->data_ptr<int64_t>()[2] = 4;
    NDArray loss = NDArray::empty({3}, cpu, kFloat32);
    hetu::impl::NLLLossCpu(pred, lab, loss, st);
    CHECK(loss->data_ptr<float>()[0] == -2.f && loss->data_ptr<float>()[1] == 0.f && loss->data_ptr<float>()[2] == 0.f);
    NDArray dp = NDArray::empty({3, 4}, cpu, kFloat32);
    hetu::impl::NLLLossGradientCpu(pred, lab, loss, dp, st);
    CHECK(dp->data_ptr<float>()[2] == 8.f && dp->data_ptr<float>()[0] == 0.f && dp->data_ptr<float>()[6] == 0.f);
    // one-hot dense labels give the sparse loss
    NDArray oh = NDArray::zeros({3, 4}, cpu, kFloat32), dl = NDArray::empty({3}, cpu, kFloat32);
    NDArray sl = NDArray::empty({3}, cpu, kFloat32), cls = NDArray::empty({3}, cpu, kInt64);
    for (int r = 0; r < 3; ++r) { oh->data_ptr<float>()[r * 4 + r] = 1.f; cls->data_ptr<int64_t>()[r] = r; }
    hetu::impl::SoftmaxCrossEntropyCpu(pred, oh, dl, st);
    hetu::impl::SoftmaxCrossEntropySparseCpu(pred, cls, sl, -100, st);
    for (int r = 0; r < 3; ++r) CHECK(std::fabs(dl->data_ptr<float>()[r] - sl->data_ptr<float>()[r]) < 1e-6f);
    // batch norm of [2, 2, 3]: channel means, inverse deviations, running statistics; then its gradient sums
    NDArray bx = NDArray::empty({2, 2, 3}, cpu, kFloat32), by = NDArray::empty({2, 2, 3}, cpu, kFloat32);
    for (int i = 0; i < 12; ++i) bx->data_ptr<float>()[i] = float(i);
    NDArray sc = NDArray::empty({2}, cpu, kFloat32), bi = NDArray::zeros({2}, cpu, kFloat32);
    NDArray rm = NDArray::zeros({2}, cpu, kFloat32), rv = NDArray::zeros({2}, cpu, kFloat32);
    NDArray sm = NDArray::empty({2}, cpu, kFloat32), sv = NDArray::empty({2}, cpu, kFloat32);
    sc->data_ptr<float>()[0] = sc->data_ptr<float>()[1] = 1.f;
    hetu::impl::BatchNormCpu(bx, sc, bi, by, 0.5, 0.0, rm, rv, sm, sv, st);
    // channel 0 holds {0, 1, 2, 6, 7, 8}: mean 4, biased variance 58 / 6, unbiased 58 / 5
    CHECK(sm->data_ptr<float>()[0] == 4.f && sm->data_ptr<float>()[1] == 7.f);
    CHECK(std::fabs(sv->data_ptr<float>()[0] - 1.f / std::sqrt(58.f / 6.f)) < 1e-6f);
    CHECK(rm->data_ptr<float>()[0] == 2.f && std::fabs(rv->data_ptr<float>()[0] - 5.8f) < 1e-6f);
    float ysum = 0.f;
    for (int i = 0; i < 12; ++i) ysum += by->data_ptr<float>()[i];
    CHECK(std::fabs(ysum) < 1e-5f);
    NDArray bdx = NDArray::empty({2, 2, 3}, cpu, kFloat32), ds = NDArray::empty({2}, cpu, kFloat32),
            dbias = NDArray::empty({2}, cpu, kFloat32);
    hetu::impl::BatchNormGradientCpu(by, bx, sc, bdx, ds, dbias, 0.0, sm, sv, st);   // dy = y: dscale = count, dbias = 0
    CHECK(std::fabs(ds->data_ptr<float>()[0] - 6.f) < 1e-5f && std::fabs(dbias->data_ptr<float>()[1]) < 1e-5f);
    for (int i = 0; i < 12; ++i) CHECK(std::fabs(bdx->data_ptr<float>()[i]) < 1e-5f);   // y lies in the null space
    CHECK(throws<assertion_error>(
      [&] { hetu::impl::BatchNormCpu(bx, NDArray::empty({3}, cpu, kFloat32), bi, by, 0.5, 0.0, rm, rv, sm, sv, st); }));
    // instance norm = per-plane standardisation
    NDArray ix = NDArray::empty({1, 2, 2, 3}, cpu, kFloat32), iy = NDArray::empty({1, 2, 2, 3}, cpu, kFloat32);
    for (int i = 0; i < 12; ++i) ix->data_ptr<float>()[i] = float(i * i);
    NDArray im = NDArray::empty({1, 2, 1, 1}, cpu, kFloat32), iv = NDArray::empty({1, 2, 1, 1}, cpu, kFloat32);
    hetu::impl::InstanceNormCpu(ix, im, iv, iy, 0.f, st);
    float m0 = 0.f, q0 = 0.f;
    for (int i = 0; i < 6; ++i) { m0 += iy->data_ptr<float>()[i]; q0 += iy->data_ptr<float>()[i] * iy->data_ptr<float>()[i]; }
    CHECK(std::fabs(m0) < 1e-5f && std::fabs(q0 - 6.f) < 1e-4f);
    CHECK(std::fabs(im->data_ptr<float>()[0] - 55.f / 6.f) < 1e-5f);
  });

  // ------------------------------------------------------------------ pool policy
  run("pool: rounding, carving small requests from one segment", [] {
    PoolFixture f;
    CHECK(CachingMemoryPool::RoundRequest(1) == 256 && CachingMemoryPool::RoundRequest(256) == 256 &&
          CachingMemoryPool::RoundRequest(257) == 512);
    DataPtr a = f.pool->AllocDataSpace(1000, f.s1), b = f.pool->AllocDataSpace(1000, f.s1);
    CHECK(a.size == 1024 && b.size == 1024 && a.is_new_malloc && !b.is_new_malloc);
    CHECK(static_cast<uint8_t*>(b.ptr) == static_cast<uint8_t*>(a.ptr) + 1024);
    auto s = f.pool->stats();
    CHECK(s.segment_allocs == 1 && s.reserved == 2 * MiB && s.allocated == 2048 && s.alloc_cnt == 2);
    DataPtr z = f.pool->AllocDataSpace(0, f.s1);
    CHECK(z.ptr == nullptr && z.size == 0);
    f.pool->FreeDataSpace(z);
    f.pool->FreeDataSpace(a);
    f.pool->FreeDataSpace(b);
    CHECK(throws<value_error>([&] { f.pool->FreeDataSpace(b); }, "freed twice"));
  });

  run("pool: same-stream reuse needs no event, neighbours merge back", [] {
    PoolFixture f;
    DataPtr a = f.pool->AllocDataSpace(4096, f.s1);
    void* first = a.ptr;
    f.pool->FreeDataSpace(a);
    DataPtr b = f.pool->AllocDataSpace(4096, f.s1);
    CHECK(b.ptr == first && f.dev->events.empty() && f.pool->stats().cache_hits == 1);
    DataPtr c = f.pool->AllocDataSpace(8192, f.s1);
    f.pool->FreeDataSpace(b);
    f.pool->FreeDataSpace(c);
    // everything merged: the whole 2 MiB segment can be handed out again
    DataPtr whole = f.pool->AllocDataSpace(2 * MiB, f.s1);
    CHECK(whole.ptr == first && f.pool->stats().segment_allocs == 1 && f.pool->stats().merges >= 2);
    f.pool->FreeDataSpace(whole);
  });

  run("pool: another stream takes a cached block behind an event", [] {
    PoolFixture f;
    DataPtr a = f.pool->AllocDataSpace(3 * MiB, f.s1);
    void* first = a.ptr;
    f.pool->FreeDataSpace(a);
    DataPtr b = f.pool->AllocDataSpace(3 * MiB, f.s2);
    CHECK(b.ptr == first && f.pool->stats().cross_stream_takes == 1 && f.pool->stats().segment_allocs == 1);
    CHECK(f.dev->waits.size() == 1 && f.dev->waits[0].first == f.s2.pack() && f.dev->waits[0].second == f.s1.pack());
    // now owned by s2: freeing and reusing on s2 needs nothing more
    f.pool->FreeDataSpace(b);
    DataPtr c = f.pool->AllocDataSpace(3 * MiB, f.s2);
    CHECK(c.ptr == first && f.dev->waits.size() == 1);
    f.pool->FreeDataSpace(c);
  });

  run("pool: a block other streams used is parked until their events pass", [] {
    PoolFixture f;
    DataPtr a = f.pool->AllocDataSpace(4 * MiB, f.s1);
    void* first = a.ptr;
    f.pool->MarkDataSpaceUsedByStream(a, f.s1);   // the owner itself: nothing to record
    CHECK(f.pool->stats().mark_cnt == 0);
    f.pool->MarkDataSpaceUsedByStream(a, f.s2);
    f.pool->MarkDataSpaceUsedByStream(a, f.s2);
    f.pool->MarkDataSpaceUsedByStream(a, f.s3);
    CHECK(f.pool->stats().mark_cnt == 2);
    f.pool->FreeDataSpace(a);
    CHECK(f.pool->stats().parked == 1 && f.dev->events.size() == 2);
    DataPtr b = f.pool->AllocDataSpace(4 * MiB, f.s1);
    CHECK(b.ptr != first && f.pool->stats().segment_allocs == 2);   // still parked
    f.dev->events[0]->done = true;
    DataPtr c = f.pool->AllocDataSpace(4 * MiB, f.s1);
    CHECK(c.ptr != first);                                           // one event still pending
    f.dev->events[1]->done = true;
    DataPtr d = f.pool->AllocDataSpace(4 * MiB, f.s1);
    CHECK(d.ptr == first);
    f.pool->FreeDataSpace(b);
    f.pool->FreeDataSpace(c);
    f.pool->FreeDataSpace(d);
  });

  run("pool: large blocks are not split, bounded waste", [] {
    PoolFixture f;
    DataPtr big = f.pool->AllocDataSpace(300 * MiB, f.s1);
    void* first = big.ptr;
    f.pool->FreeDataSpace(big);
    DataPtr small = f.pool->AllocDataSpace(100 * MiB, f.s1);     // would waste 200 MiB: new segment
    CHECK(small.ptr != first);
    DataPtr close = f.pool->AllocDataSpace(290 * MiB, f.s1);     // wastes 10 MiB <= 20 MiB: whole block
    CHECK(close.ptr == first && close.size == 300 * MiB);
    f.pool->FreeDataSpace(small);
    // 100 MiB <= max split: it is split for a 10 MiB request
    DataPtr part = f.pool->AllocDataSpace(10 * MiB, f.s1);
    CHECK(part.ptr == small.ptr && part.size == 10 * MiB);
    f.pool->FreeDataSpace(part);
    f.pool->FreeDataSpace(close);
  });

  run("pool: out of memory releases the cache and retries, then reports", [] {
    PoolFixture f(/*capacity=*/64 * MiB);
    DataPtr a = f.pool->AllocDataSpace(40 * MiB, f.s1);
    f.pool->FreeDataSpace(a);
    // cached 40 MiB on s1 does not fit a 50 MiB request; the device has 24 MiB left
    DataPtr b = f.pool->AllocDataSpace(50 * MiB, f.s1);
    CHECK(b.ptr != nullptr && f.pool->stats().retries_after_oom == 1 && f.pool->stats().segment_frees == 1);
    CHECK(f.dev->device_syncs >= 1 && f.dev->in_use == 50 * MiB);
    CHECK(throws<runtime_error>([&] { f.pool->AllocDataSpace(32 * MiB, f.s1); }, "out of memory"));
    f.pool->FreeDataSpace(b);
    f.pool->EmptyCache();
    CHECK(f.pool->stats().reserved == 0 && f.dev->in_use == 0 && f.dev->live.empty());
  });

  run("pool: EmptyCache waits for parked blocks and keeps live ones", [] {
    PoolFixture f;
    DataPtr keep = f.pool->AllocDataSpace(5 * MiB, f.s1);
    DataPtr gone = f.pool->AllocDataSpace(5 * MiB, f.s1);
    f.pool->MarkDataSpaceUsedByStream(gone, f.s2);
    f.pool->FreeDataSpace(gone);
    f.pool->EmptyCache();
    auto s = f.pool->stats();
    CHECK(s.reserved == 6 * MiB && s.allocated == 5 * MiB && f.dev->live.size() == 1);
    f.pool->FreeDataSpace(keep);
  });

  run("pool: borrowed memory runs its deleter once, after marked streams drain", [] {
    PoolFixture f;
    int deleted = 0;
    char mine[64];
    DataPtr b = f.pool->BorrowDataSpace(mine, sizeof(mine), [&](DataPtr) { ++deleted; });
    f.pool->MarkDataSpaceUsedByStream(b, f.s2);
    f.pool->FreeDataSpace(b);
    CHECK(deleted == 1 && f.dev->stream_syncs == 1 && f.pool->stats().reserved == 0);
    CHECK(throws<value_error>([&] { f.pool->BorrowDataSpace(nullptr, 8, nullptr); }));
  });

  run("pool: WaitDataSpace drains owner and user streams", [] {
    PoolFixture f;
    DataPtr a = f.pool->AllocDataSpace(1 * MiB, f.s1);
    f.pool->MarkDataSpaceUsedByStream(a, f.s3);
    f.pool->WaitDataSpace(a, false).get();
    CHECK(f.dev->stream_syncs == 2);
    f.pool->WaitDataSpace(a, true).get();
    CHECK(f.dev->stream_syncs == 4);
    f.pool->FreeDataSpace(a);
  });

  run("pool: randomized alloc/free never overlaps live blocks", [] {
    PoolFixture f(/*capacity=*/512 * MiB, /*max_split=*/16 * MiB, /*max_frag=*/2 * MiB);
    f.dev->auto_complete = true;
    struct Live { DataPtr p; };
    std::vector<Live> live;
    uint64_t rng = 0x9E3779B97F4A7C15ull;
    auto next = [&] { rng ^= rng << 13; rng ^= rng >> 7; rng ^= rng << 17; return rng; };
    const Stream streams[3] = {f.s1, f.s2, f.s3};
    for (int step = 0; step < 4000; ++step) {
      const bool do_alloc = live.empty() || (next() % 100 < 55 && live.size() < 64);
      if (do_alloc) {
        const size_t cls = next() % 3;
        const size_t bytes = cls == 0 ? 1 + next() % 4096 : cls == 1 ? 1 + next() % (3 * MiB) : 1 + next() % (24 * MiB);
        DataPtr p;
        try {
          p = f.pool->AllocDataSpace(bytes, streams[next() % 3]);
        } catch (const runtime_error&) {
          continue;   // scripted device full: allowed
        }
        CHECK(p.size >= bytes && reinterpret_cast<uintptr_t>(p.ptr) % 256 == 0);
        for (auto& l : live) {
          auto* a0 = static_cast<uint8_t*>(l.p.ptr);
          auto* b0 = static_cast<uint8_t*>(p.ptr);
          CHECK(a0 + l.p.size <= b0 || b0 + p.size <= a0);
        }
        if (next() % 4 == 0) f.pool->MarkDataSpaceUsedByStream(p, streams[next() % 3]);
        live.push_back({p});
      } else {
        const size_t i = next() % live.size();
        f.pool->FreeDataSpace(live[i].p);
        live[i] = live.back();
        live.pop_back();
      }
    }
    size_t sum = 0;
    for (auto& l : live) sum += l.p.size;
    CHECK(f.pool->stats().allocated == sum && f.pool->stats().reserved >= sum);
    for (auto& l : live) f.pool->FreeDataSpace(l.p);
    f.pool->EmptyCache();
    CHECK(f.pool->stats().allocated == 0 && f.pool->stats().reserved == 0 && f.dev->live.empty());
  });

  run("pool knobs from the environment", [] {
    setenv("HETU_TEST_KNOB_MB", "64", 1);
    CHECK(hetu::impl::ParsePoolKnobMB("HETU_TEST_KNOB_MB", 200) == 64 * MiB);
    setenv("HETU_TEST_KNOB_MB", "sixty", 1);
    CHECK(hetu::impl::ParsePoolKnobMB("HETU_TEST_KNOB_MB", 200) == 200 * MiB);
    setenv("HETU_TEST_KNOB_MB", "-3", 1);
    CHECK(hetu::impl::ParsePoolKnobMB("HETU_TEST_KNOB_MB", 20) == 20 * MiB);
    unsetenv("HETU_TEST_KNOB_MB");
    CHECK(hetu::impl::ParsePoolKnobMB("HETU_TEST_KNOB_MB", 20) == 20 * MiB);
  });

  std::printf("%d checks, %d failed\n", g_run, g_failed);
  return g_failed;
}
