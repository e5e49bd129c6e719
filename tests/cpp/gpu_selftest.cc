// The C++ operator layer used natively on a GPU, the way a C++ caller would: host arrays go to the
// device through NDArray::cuda, operators run on the layer's streams with memory from its pool, results
// come back through NDArray::cpu and are compared with plain double-precision loops written here.
// Prints one line per check; exit status is the number of failed checks.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <limits>
#include <random>
#include <vector>

#include "hetu/core/ndarray.h"
#include "hetu/graph/ops/gradient_compute.h"
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/memory/CachingMemoryPool.h"
#include "hetu/impl/stream/HIPStream.h"

using namespace hetu;

static int g_failed = 0, g_run = 0;

#define CHECK(cond)                                                                    \
  do {                                                                                 \
    if (!(cond)) {                                                                     \
      std::printf("    CHECK FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);          \
      throw std::runtime_error("check failed");                                        \
    }                                                                                  \
  } while (0)

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

template <typename E, typename F>
static bool throws(F&& f) {
  try { f(); } catch (const E&) { return true; } catch (...) { return false; }
  return false;
}

static NDArray host_f32(const HTShape& shape, const std::vector<float>& v) {
  NDArray a = NDArray::empty(shape, Device(kCPU), kFloat32);
  std::memcpy(a->raw_data_ptr(), v.data(), v.size() * sizeof(float));
  return a;
}

static std::vector<float> fetch_f32(const NDArray& dev) {
  NDArray h = NDArray::cpu(dev);
  std::vector<float> v(h->numel());
  std::memcpy(v.data(), h->raw_data_ptr(), v.size() * sizeof(float));
  return v;
}

static double max_rel(const std::vector<float>& got, const std::vector<double>& want) {
  double rms = 0;
  for (double w : want) rms += w * w;
  rms = std::sqrt(rms / std::max<size_t>(1, want.size()));
  double worst = 0;
  for (size_t i = 0; i < want.size(); ++i)
    worst = std::max(worst, std::fabs(got[i] - want[i]) / (std::fabs(want[i]) + rms + 1e-30));
  return worst;
}

int main() {
  const Device gpu(kCUDA, 0);
  std::mt19937 rng(1234);
  std::normal_distribution<float> normal(0.f, 1.f);
  const int64_t rows = 37, cols = 1000;
  std::vector<float> x(rows * cols), gamma(cols), beta(cols);
  for (auto& v : x) v = normal(rng) * 2.f;
  for (auto& v : gamma) v = 1.f + 0.2f * normal(rng);
  for (auto& v : beta) v = 0.1f * normal(rng);

  run("host <-> device copies, zeros, views", [&] {
    NDArray d = NDArray::cuda(host_f32({rows, cols}, x));
    CHECK(d->is_cuda() && d->is_contiguous());
    CHECK(fetch_f32(d) == x);
    NDArray z = NDArray::zeros({5, 7}, gpu, kFloat32);
    for (float v : fetch_f32(z)) CHECK(v == 0.f);
    NDArray t = NDArray::contiguous(NDArray::permute(d, {1, 0}));     // device transpose
    std::vector<float> tt = fetch_f32(t);
    for (int64_t r = 0; r < rows; r += 9)
      for (int64_t c = 0; c < cols; c += 111) CHECK(tt[c * rows + r] == x[r * cols + c]);
    NDArray s = NDArray::contiguous(NDArray::slice(d, {3, 10}, {4, 20}));
    std::vector<float> ss = fetch_f32(s);
    CHECK(ss.size() == 80 && ss[0] == x[3 * cols + 10] && ss[79] == x[6 * cols + 29]);
  });

  run("softmax and its gradient", [&] {
    NDArray d = NDArray::cuda(host_f32({rows, cols}, x));
    NDArray y = NDArray::softmax(d, -1);
    std::vector<double> want(rows * cols);
    for (int64_t r = 0; r < rows; ++r) {
      double m = -1e300, s = 0;
      for (int64_t c = 0; c < cols; ++c) m = std::max<double>(m, x[r * cols + c]);
      for (int64_t c = 0; c < cols; ++c) s += std::exp(x[r * cols + c] - m);
      for (int64_t c = 0; c < cols; ++c) want[r * cols + c] = std::exp(x[r * cols + c] - m) / s;
    }
    std::vector<float> got = fetch_f32(y);
    CHECK(max_rel(got, want) < 1e-5);
    NDArray dx = NDArray::empty_like(d);
    Stream stream(gpu, NDArray::DEFAULT_STREAM);
    hetu::impl::SoftmaxGradientCuda(y, d, dx, 1, stream);     // dy := x
    std::vector<double> wdx(rows * cols);
    for (int64_t r = 0; r < rows; ++r) {
      double dot = 0;
      for (int64_t c = 0; c < cols; ++c) dot += double(got[r * cols + c]) * x[r * cols + c];
      for (int64_t c = 0; c < cols; ++c) wdx[r * cols + c] = double(got[r * cols + c]) * (x[r * cols + c] - dot);
    }
    CHECK(max_rel(fetch_f32(dx), wdx) < 1e-5);
  });

  run("layernorm (variance in the data type) and fused layernorm (float32 rstd)", [&] {
    NDArray d = NDArray::cuda(host_f32({rows, cols}, x));
    NDArray g = NDArray::cuda(host_f32({cols}, gamma)), b = NDArray::cuda(host_f32({cols}, beta));
    std::vector<double> want(rows * cols), wvar(rows), wrstd(rows);
    for (int64_t r = 0; r < rows; ++r) {
      double mean = 0, var = 0;
      for (int64_t c = 0; c < cols; ++c) mean += x[r * cols + c];
      mean /= cols;
      for (int64_t c = 0; c < cols; ++c) var += (x[r * cols + c] - mean) * (x[r * cols + c] - mean);
      var /= cols;
      wvar[r] = var;
      wrstd[r] = 1.0 / std::sqrt(var + 1e-5);
      for (int64_t c = 0; c < cols; ++c)
        want[r * cols + c] = (x[r * cols + c] - mean) * wrstd[r] * gamma[c] + beta[c];
    }
    NDArrayList out = NDArray::layernorm(d, g, b, {cols}, 1e-5);
    CHECK(out.size() == 3 && (out[1]->shape() == HTShape{rows, 1}) && out[2]->dtype() == kFloat32);
    CHECK(max_rel(fetch_f32(out[0]), want) < 1e-5);
    CHECK(max_rel(fetch_f32(out[2]), wvar) < 1e-5);
    NDArrayList fused = NDArray::fused_layernorm(d, g, b, {cols}, 1e-5);
    CHECK(max_rel(fetch_f32(fused[0]), want) < 1e-5);
    CHECK(max_rel(fetch_f32(fused[2]), wrstd) < 1e-5);
  });

  run("cross-entropy: mean over all rows, ignored rows contribute 0", [&] {
    NDArray d = NDArray::cuda(host_f32({rows, cols}, x));
    NDArray lab = NDArray::empty({rows}, Device(kCPU), kInt64);
    double total = 0;
    for (int64_t r = 0; r < rows; ++r) {
      const int64_t l = (r % 5 == 0) ? -100 : (r * 131) % cols;
      lab->data_ptr<int64_t>()[r] = l;
      if (l < 0) continue;
      double m = -1e300, s = 0;
      for (int64_t c = 0; c < cols; ++c) m = std::max<double>(m, x[r * cols + c]);
      for (int64_t c = 0; c < cols; ++c) s += std::exp(x[r * cols + c] - m);
      total += std::log(s) + m - x[r * cols + l];
    }
    NDArray loss = NDArray::sceloss(d, NDArray::cuda(lab), int64_t(-100), kMEAN);
    CHECK((loss->shape() == HTShape{1}));
    std::vector<float> got = fetch_f32(loss);
    CHECK(std::fabs(got[0] - total / rows) < 1e-5 * std::fabs(total / rows));
    NDArray per_row = NDArray::sceloss(d, NDArray::cuda(lab), int64_t(-100), kNONE);
    std::vector<float> pr = fetch_f32(per_row);
    for (int64_t r = 0; r < rows; r += 5) CHECK(pr[r] == 0.f);
  });

  run("vocabulary-parallel cross-entropy over two column shards, written as the loss op writes it", [&] {
    // the steps of VocabParallelCrossEntropyOpImpl::DoCompute (VocabParallelCrossEntropyLoss.cc:51-108 of the
    // reference); what it all-reduces across devices is combined here from the two shards this device holds
    NDArray d = NDArray::cuda(host_f32({rows, cols}, x));
    NDArray lab = NDArray::empty({rows}, Device(kCPU), kInt64);
    std::vector<double> want(rows, 0.0);
    for (int64_t r = 0; r < rows; ++r) {
      const int64_t l = (r % 7 == 0) ? -100 : (r * 131) % cols;
      lab->data_ptr<int64_t>()[r] = l;
      if (l < 0) continue;
      double m = -1e300, sum = 0;
      for (int64_t c = 0; c < cols; ++c) m = std::max<double>(m, x[r * cols + c]);
      for (int64_t c = 0; c < cols; ++c) sum += std::exp(x[r * cols + c] - m);
      want[r] = std::log(sum) + m - x[r * cols + l];
    }
    NDArray labels = NDArray::cuda(lab);
    const int64_t half = cols / 2;
    NDArray shard[2] = {NDArray::slice(d, {0, 0}, {rows, half}), NDArray::slice(d, {0, half}, {rows, half})};
    NDArray part_max[2], shifted[2], exps[2], part_sum[2], picked[2];
    for (int k = 0; k < 2; ++k) part_max[k] = NDArray::reduce(shard[k], kMAX, {-1}, true);
    std::vector<float> m0 = fetch_f32(part_max[0]), m1 = fetch_f32(part_max[1]), mm(rows);
    for (int64_t r = 0; r < rows; ++r) mm[r] = std::max(m0[r], m1[r]);
    NDArray row_max = NDArray::cuda(host_f32({rows, 1}, mm));             // all-reduce(max)
    for (int k = 0; k < 2; ++k) {
      shifted[k] = NDArray::sub(shard[k], row_max);                       // logits - max, [rows, half] - [rows, 1]
      exps[k] = NDArray::exp(shifted[k]);
      part_sum[k] = NDArray::reduce(exps[k], kSUM, {-1}, true);
    }
    NDArray row_sum = NDArray::add(part_sum[0], part_sum[1]);             // all-reduce(sum)
    NDArray softmax0 = NDArray::div(exps[0], row_sum, NDArray::DEFAULT_STREAM, exps[0]);   // in place
    CHECK(softmax0->raw_data_ptr() == exps[0]->raw_data_ptr());
    NDArray lse = NDArray::log(row_sum);
    Stream stream(gpu, NDArray::DEFAULT_STREAM);
    for (int k = 0; k < 2; ++k) {
      picked[k] = NDArray::empty({rows, 1}, gpu, kFloat32);
      hetu::impl::VocabParallelCrossEntropyCuda(shifted[k], labels, k * half, (k + 1) * half, -100, picked[k], lse,
                                                stream);
    }
    NDArray picked_all = NDArray::add(picked[0], picked[1]);              // all-reduce(sum)
    NDArray loss = NDArray::sub(lse, picked_all, NDArray::DEFAULT_STREAM, lse);              // in place
    CHECK((loss->shape() == HTShape{rows, 1}));
    CHECK(max_rel(fetch_f32(loss), want) < 1e-5);
    // softmax of shard 0 sums, with shard 1's, to one in every row
    std::vector<float> s0 = fetch_f32(NDArray::reduce(softmax0, kSUM, {-1}, false));
    std::vector<float> s1 = fetch_f32(NDArray::reduce(NDArray::div(exps[1], row_sum), kSUM, {-1}, false));
    for (int64_t r = 0; r < rows; ++r) CHECK(std::fabs(s0[r] + s1[r] - 1.0) < 1e-5);
    // gradient of shard 0: (softmax - onehot) * grad, ignored rows through a zero loss gradient
    std::vector<float> gl(rows);
    for (int64_t r = 0; r < rows; ++r) gl[r] = (r % 7 == 0) ? 0.f : 1.f / rows;
    NDArray grad = NDArray::empty({rows, half}, gpu, kFloat32);
    std::vector<float> sm = fetch_f32(softmax0);
    hetu::impl::VocabParallelCrossEntropyGradientCuda(softmax0, labels, 0, half, -100,
                                                      NDArray::cuda(host_f32({rows, 1}, gl)), grad, stream);
    std::vector<float> got = fetch_f32(grad);
    std::vector<double> wantg(rows * half);
    for (int64_t r = 0; r < rows; ++r) {
      const int64_t l = lab->data_ptr<int64_t>()[r];
      for (int64_t c = 0; c < half; ++c) wantg[r * half + c] = (double(sm[r * half + c]) - (c == l ? 1.0 : 0.0)) * gl[r];
    }
    CHECK(max_rel(got, wantg) < 1e-5);
    CHECK(throws<assertion_error>([&] { NDArray::add(shard[0], NDArray::slice(d, {0, 0}, {rows, half - 1})); }));
  });

  run("gradient of the mean cross-entropy: the loss op's two steps and the single kernel agree", [&] {
    NDArray d = NDArray::cuda(host_f32({rows, cols}, x));
    NDArray lab = NDArray::empty({rows}, Device(kCPU), kInt64);
    for (int64_t r = 0; r < rows; ++r) lab->data_ptr<int64_t>()[r] = (r % 5 == 0) ? -100 : (r * 131) % cols;
    NDArray labels = NDArray::cuda(lab);
    NDArray grad_output = NDArray::cuda(host_f32({1}, std::vector<float>{1.5f}));
    NDArray none;
    NDArray two_step = hetu::graph::SCESGradCompute(d, labels, grad_output, -100, kMEAN, NDArray::DEFAULT_STREAM,
                                                    none, /*fused=*/false);
    NDArray fused = hetu::graph::SCESGradCompute(d, labels, grad_output, -100, kMEAN, NDArray::DEFAULT_STREAM, none,
                                                 /*fused=*/true);
    std::vector<float> a = fetch_f32(two_step), b = fetch_f32(fused);
    CHECK(a == b);
    const float per_row = 1.5f * (1.0f / float(rows));
    std::vector<double> want(rows * cols);
    for (int64_t r = 0; r < rows; ++r) {
      const int64_t l = lab->data_ptr<int64_t>()[r];
      double m = -1e300, sum = 0;
      for (int64_t c = 0; c < cols; ++c) m = std::max<double>(m, x[r * cols + c]);
      for (int64_t c = 0; c < cols; ++c) sum += std::exp(x[r * cols + c] - m);
      for (int64_t c = 0; c < cols; ++c)
        want[r * cols + c] = l < 0 ? 0.0 : (std::exp(x[r * cols + c] - m) / sum - (c == l ? 1.0 : 0.0)) * per_row;
    }
    CHECK(max_rel(b, want) < 1e-5);
    // gradient of a mean over the columns: every element of a row gets grad[r] / cols
    std::vector<float> gr(rows);
    for (int64_t r = 0; r < rows; ++r) gr[r] = float(r + 1);
    NDArray back = hetu::graph::ReduceGradientCompute(NDArray::cuda(host_f32({rows}, gr)), {rows, cols}, kMEAN, {-1},
                                                      {false}, NDArray::DEFAULT_STREAM, none);
    std::vector<float> got = fetch_f32(back);
    for (int64_t r = 0; r < rows; ++r)
      for (int64_t c = 0; c < cols; c += 97) CHECK(std::fabs(got[r * cols + c] - gr[r] / cols) <= 1e-6 * gr[r] / cols);
    CHECK(throws<assertion_error>([&] {
      NDArray out = NDArray::empty({rows, cols}, gpu, kFloat32);
      hetu::impl::BroadcastShapeCuda(NDArray::cuda(host_f32({rows - 1}, std::vector<float>(rows - 1, 0.f))), out,
                                     {1}, Stream(gpu, NDArray::DEFAULT_STREAM));
    }));
  });

  run("reductions: sum / mean / max with keepdims, all dims", [&] {
    NDArray d = NDArray::cuda(host_f32({rows, cols}, x));
    NDArray s0 = NDArray::sum(d, {0});
    CHECK((s0->shape() == HTShape{cols}));
    std::vector<double> want(cols, 0.0);
    for (int64_t r = 0; r < rows; ++r)
      for (int64_t c = 0; c < cols; ++c) want[c] += x[r * cols + c];
    CHECK(max_rel(fetch_f32(s0), want) < 1e-5);
    NDArray m1 = NDArray::mean(d, {-1}, true);
    CHECK((m1->shape() == HTShape{rows, 1}));
    NDArray mx = NDArray::max(d);
    CHECK((mx->shape() == HTShape{1}));
    float top = -std::numeric_limits<float>::infinity();
    for (float v : x) top = std::max(top, v);
    CHECK(fetch_f32(mx)[0] == top);
  });

  run("events measure device time; streams synchronise", [&] {
    Stream s1(gpu, 1), s2(gpu, 2);
    hetu::impl::HIPEvent a(gpu), b(gpu);
    NDArray big = NDArray::empty({1 << 26}, gpu, kFloat32, 1);
    a.Record(s1);
    NDArray r = NDArray::sum(big, {0}, false, 1);
    b.Record(s1);
    b.Block(s2);                 // stream 2 waits for stream 1 without the host
    b.Sync();
    const int64_t ns = b.TimeSince(a);
    CHECK(ns > 1000 && ns < 100000000);
    s1.Sync();
    s2.Sync();
    SynchronizeAllStreams();
    CHECK(b.Query());
  });

  run("scratch goes back to the pool and is reused", [&] {
    auto pool = std::dynamic_pointer_cast<hetu::impl::CachingMemoryPool>(GetMemoryPool(gpu));
    CHECK(pool != nullptr);
    SynchronizeAllStreams();
    const auto before = pool->stats();
    {
      NDArray d = NDArray::cuda(host_f32({rows, cols}, x));
      for (int i = 0; i < 4; ++i) NDArray s = NDArray::sum(d, {0});
      Stream(gpu, NDArray::DEFAULT_STREAM).Sync();
    }
    const auto after = pool->stats();
    CHECK(after.allocated == before.allocated);
    CHECK(after.cache_hits > before.cache_hits);
    pool->EmptyCache();
    CHECK(pool->stats().reserved == pool->stats().allocated);
  });

  run("errors are exceptions of the right kind", [&] {
    NDArray d = NDArray::cuda(host_f32({rows, cols}, x));
    NDArray i32 = NDArray::zeros({rows, cols}, gpu, kInt32);
    CHECK(throws<not_implemented>([&] { NDArray::softmax(i32, -1); }));
    CHECK(throws<assertion_error>([&] { NDArray::softmax(d, 2); }));
    NDArray g = NDArray::cuda(host_f32({cols}, gamma));
    NDArray wrong = NDArray::zeros({cols + 1}, gpu, kFloat32);
    CHECK(throws<assertion_error>([&] { NDArray::layernorm(d, wrong, g, {cols}); }));
    CHECK(throws<not_implemented>([&] { NDArray::reduce(d, kNONE); }));
  });

  std::printf("%d checks, %d failed\n", g_run, g_failed);
  return g_failed;
}
