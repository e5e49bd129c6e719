// VocabParallelCrossEntropyCuda / VocabParallelCrossEntropyGradientCuda:
// arguments and meaning of hetu/impl/kernel/VocabParallelCrossEntropyLoss.cu:38-64
// and :94-119 of the reference.  The logits / softmax are this device's column
// shard [rows, vocab_end - vocab_start]; labels are global class numbers.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"

namespace hetu {
namespace impl {

void VocabParallelCrossEntropyCuda(const NDArray& vocab_parallel_logits, const NDArray& labels,
                                   const int64_t vocab_start_index, const int64_t vocab_end_index,
                                   const int64_t ignored_index, NDArray& predicted_logits_partial,
                                   NDArray& log_sum_exp_logits, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(vocab_parallel_logits);
  HT_ASSERT_SAME_DEVICE(vocab_parallel_logits, labels);
  HT_ASSERT_SAME_DEVICE(vocab_parallel_logits, predicted_logits_partial);
  HT_ASSERT_SAME_DEVICE(vocab_parallel_logits, log_sum_exp_logits);
  HT_ASSERT(vocab_parallel_logits->ndim() == 2) << "Logits must be [rows, vocab shard], got "
                                                << vocab_parallel_logits->shape();
  const int64_t rows = vocab_parallel_logits->shape(0), cols = vocab_parallel_logits->shape(1);
  HT_ASSERT(labels->dtype() == kInt64) << "Labels must be int64, got " << labels->dtype();
  HT_ASSERT(int64_t(labels->numel()) == rows) << "One label per row expected, got " << labels->shape();
  HT_ASSERT(int64_t(predicted_logits_partial->numel()) == rows && int64_t(log_sum_exp_logits->numel()) == rows)
    << "Per-row outputs expected, got " << predicted_logits_partial->shape() << " and "
    << log_sum_exp_logits->shape();
  HT_ASSERT_SAME_DTYPE(vocab_parallel_logits, predicted_logits_partial);
  HT_ASSERT_SAME_DTYPE(vocab_parallel_logits, log_sum_exp_logits);
  HT_ASSERT_CONTIGUOUS(predicted_logits_partial);
  HT_ASSERT_CONTIGUOUS(log_sum_exp_logits);
  HT_ASSERT(vocab_end_index - vocab_start_index == cols)
    << "The shard [" << vocab_start_index << ", " << vocab_end_index << ") does not match " << cols << " columns";
  if (rows == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray x = Dense(vocab_parallel_logits, stream), l = Dense(labels, stream);
  HK_CALL(hk_vocab_parallel_ce_gather(int(x->dtype()), x->raw_data_ptr(), l->data_ptr<int64_t>(), rows, cols,
                                      vocab_start_index, vocab_end_index, ignored_index,
                                      predicted_logits_partial->raw_data_ptr(), log_sum_exp_logits->raw_data_ptr(),
                                      hip_stream));
  NDArray::MarkUsedBy({x, l, predicted_logits_partial, log_sum_exp_logits}, stream);
}

void VocabParallelCrossEntropyGradientCuda(const NDArray& softmax, const NDArray& labels,
                                           const int64_t vocab_start_index, const int64_t vocab_end_index,
                                           const int64_t ignored_index, const NDArray& grad_loss, NDArray& output,
                                           const Stream& stream) {
  (void) vocab_end_index;   // the kernel of the reference does not read these two either (:69-92):
  (void) ignored_index;     // the caller zeroes grad_loss of ignored rows
  HT_ASSERT_CUDA_DEVICE(softmax);
  HT_ASSERT_SAME_DEVICE(softmax, labels);
  HT_ASSERT_SAME_DEVICE(softmax, grad_loss);
  HT_ASSERT_SAME_DEVICE(softmax, output);
  HT_ASSERT(softmax->ndim() == 2) << "Softmax must be [rows, vocab shard], got " << softmax->shape();
  const int64_t rows = softmax->shape(0), cols = softmax->shape(1);
  HT_ASSERT(labels->dtype() == kInt64) << "Labels must be int64, got " << labels->dtype();
  HT_ASSERT(int64_t(labels->numel()) == rows) << "One label per row expected, got " << labels->shape();
  HT_ASSERT(int64_t(grad_loss->numel()) == rows) << "One loss gradient per row expected, got " << grad_loss->shape();
  HT_ASSERT_SAME_SHAPE(softmax, output);
  HT_ASSERT_SAME_DTYPE(softmax, output);
  HT_ASSERT_SAME_DTYPE(softmax, grad_loss);
  HT_ASSERT_CONTIGUOUS(output);
  if (rows == 0 || cols == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray s = Dense(softmax, stream), l = Dense(labels, stream), g = Dense(grad_loss, stream);
  HK_CALL(hk_vocab_parallel_ce_bwd(int(s->dtype()), s->raw_data_ptr(), l->data_ptr<int64_t>(), g->raw_data_ptr(),
                                   output->raw_data_ptr(), rows, cols, vocab_start_index, hip_stream));
  NDArray::MarkUsedBy({s, l, g, output}, stream);
}

} // namespace impl
} // namespace hetu
