// extern "C" face of the operator layer (declared in hetu_ops_c.h).
#ifdef _OPENMP
#include <omp.h>
#endif
#include "hetu_ops_c.h"

#include <atomic>
#include <cstring>
#include <string>

#include "hetu/graph/ops/gradient_compute.h"
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/random/CPURandomState.h"
#include "hetu/impl/memory/CachingMemoryPool.h"
#include "hetu/impl/stream/CPUStream.h"
#include "hetu/impl/stream/HIPStream.h"

using namespace hetu;

namespace {

thread_local std::string g_error;

// Host arrays are borrowed from the caller, so by default a call on them has finished when it returns: whatever it
// put on a host stream is waited for.  ht_set_host_async(1) leaves the waiting to the caller (ht_host_stream_sync).
std::atomic<bool> g_host_async{false};

struct HostDrain {
  // on the way out of a failed call: nothing may still be reading the caller's buffers
  ~HostDrain() {
    if (armed && !g_host_async.load(std::memory_order_relaxed) && hetu::impl::AnyCPUStreamBusy()) {
      try {
        hetu::impl::SynchronizeAllCPUStreams();
      } catch (...) {
      }
    }
  }
  bool armed = true;
};

template <typename F>
int guarded(F&& fn) {
  try {
    HostDrain drain;
    fn();
    if (!g_host_async.load(std::memory_order_relaxed) && hetu::impl::AnyCPUStreamBusy())
      hetu::impl::SynchronizeAllCPUStreams();   // a host kernel that failed on its stream fails the call
    drain.armed = false;
    g_error.clear();
    return HT_OK;
  } catch (const hetu::not_implemented& e) {
    g_error = e.what();
    return HT_ERR_NOT_IMPLEMENTED;
  } catch (const hetu::assertion_error& e) {
    g_error = e.what();
    return HT_ERR_ASSERTION;
  } catch (const hetu::value_error& e) {
    g_error = e.what();
    return HT_ERR_VALUE;
  } catch (const hetu::bad_alloc& e) {
    g_error = e.what();
    return HT_ERR_BAD_ALLOC;
  } catch (const hetu::hetu_exception& e) {
    g_error = e.what();
    return HT_ERR_RUNTIME;
  } catch (const std::exception& e) {
    g_error = e.what();
    return HT_ERR_OTHER;
  }
}

Device device_of(const HtArray* a) {
  return a->device_type == HT_DEVICE_ACCEL ? Device(kCUDA, DeviceIndex(a->device_index)) : Device(kCPU);
}

NDArray wrap(const HtArray* a) {
  if (a == nullptr) return NDArray();
  HT_VALUE_ERROR_IF(a->ndim < 0 || a->ndim > HT_C_MAX_NDIM) << "array rank " << a->ndim << " out of range";
  HTShape shape(a->shape, a->shape + a->ndim);
  HTStride stride(a->stride, a->stride + a->ndim);
  return NDArray::borrow(a->data, shape, device_of(a), static_cast<DataType>(a->dtype), stride);
}

Stream stream_of(const HtArray* a, int stream_index) {
  return Stream(device_of(a), StreamIndex(stream_index));
}

// dense device-to-device copy of an operator result into caller memory
void copy_out(const NDArray& result, HtArray* out, const Stream& stream) {
  NDArray dst = wrap(out);
  HT_ASSERT(dst->is_contiguous()) << "result buffers must be dense";
  HT_ASSERT(dst->numel() == result->numel() && dst->dtype() == result->dtype())
    << "result " << result->meta() << " does not fit the buffer " << dst->meta();
  if (result->numel() == 0) return;
  NDArray src = NDArray::contiguous(result, stream.stream_index());
  if (stream.device().is_cpu()) {   // host result: a plain copy, on the stream that still has to produce it
    hetu::impl::CPUStream(stream).EnqueueTask(
      [src, dst]() {
        std::memcpy(dst->raw_data_ptr(), src->raw_data_ptr(), src->numel() * DataType2Size(src->dtype()));
      },
      "CopyOut");
    return;
  }
  hetu::impl::HIPStream hs(stream);
  hetu::hip::DeviceGuard guard(hs.device_id());
  HK_CALL(hk_memcpy_d2d(dst->raw_data_ptr(), src->raw_data_ptr(), src->numel() * DataType2Size(src->dtype()), hs));
  NDArray::MarkUsedBy({src, dst}, stream);
  stream.Sync();   // the caller owns dst and may read it right away
}

hetu::impl::CachingMemoryPool& caching_pool(int device_index) {
  auto pool = GetMemoryPool(Device(kCUDA, DeviceIndex(device_index)));
  auto* cp = dynamic_cast<hetu::impl::CachingMemoryPool*>(pool.get());
  HT_ASSERT(cp != nullptr) << "device pool is not the caching pool";
  return *cp;
}

} // namespace

extern "C" {

const char* ht_last_error(void) { return g_error.c_str(); }

int ht_layer_norm(const HtArray* in, const HtArray* scale, const HtArray* bias, HtArray* mean, HtArray* var,
                  HtArray* out, int64_t reduce_dims, float eps, int stream_index) {
  return guarded([&] {
    NDArray m = wrap(mean), v = wrap(var), o = wrap(out);
    const Stream st = stream_of(in, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_layer_norm", hetu::impl::LayerNorm, wrap(in), wrap(scale),
                                    wrap(bias), m, v, o, reduce_dims, eps, st);
  });
}

int ht_layer_norm_gradient(const HtArray* out_grads, const HtArray* in, const HtArray* scale, HtArray* grad_in,
                           HtArray* grad_scale, HtArray* grad_bias, const HtArray* mean, const HtArray* var,
                           int64_t reduce_dims, float eps, int stream_index) {
  return guarded([&] {
    NDArray gi = wrap(grad_in), gs = wrap(grad_scale), gb = wrap(grad_bias);
    const Stream st = stream_of(in, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_layer_norm_gradient", hetu::impl::LayerNormGradient,
                                    wrap(out_grads), wrap(in), wrap(scale), gi, gs, gb, wrap(mean), wrap(var),
                                    reduce_dims, eps, st);
  });
}

int ht_fused_layer_norm(const HtArray* in, const HtArray* scale, const HtArray* bias, HtArray* mean,
                        HtArray* invvar, HtArray* out, int64_t reduce_dims, float eps, int stream_index) {
  return guarded([&] {
    NDArray m = wrap(mean), v = wrap(invvar), o = wrap(out);
    hetu::impl::FusedLayerNormCuda(wrap(in), wrap(scale), wrap(bias), m, v, o, reduce_dims, eps,
                                   stream_of(in, stream_index));
  });
}

int ht_fused_layer_norm_gradient(const HtArray* out_grads, const HtArray* x_or_y, const HtArray* scale,
                                 const HtArray* bias, HtArray* grad_in, HtArray* grad_scale, HtArray* grad_bias,
                                 const HtArray* mean, const HtArray* invvar, int64_t reduce_dims, float eps,
                                 int inplace, int stream_index) {
  return guarded([&] {
    NDArray gi = wrap(grad_in), gs = wrap(grad_scale), gb = wrap(grad_bias);
    hetu::impl::FusedLayerNormGradientCuda(wrap(out_grads), wrap(x_or_y), wrap(scale), wrap(bias), gi, gs, gb,
                                           wrap(mean), wrap(invvar), reduce_dims, eps, inplace != 0,
                                           stream_of(x_or_y, stream_index));
  });
}

int ht_dropout_add_ln_fwd(const HtArray* x0, const HtArray* residual, const HtArray* gamma, const HtArray* beta,
                          const HtArray* rowscale, const HtArray* colscale, const HtArray* x0_subset,
                          const HtArray* z_subset, HtArray* z, HtArray* x, HtArray* dmask, HtArray* mu,
                          HtArray* rsigma, float dropout_p, float epsilon, float rowscale_const, int64_t z_numrows,
                          int residual_in_fp32, int is_rms_norm, int stream_index) {
  return guarded([&] {
    NDArray zz = wrap(z), xx = wrap(x), dm = wrap(dmask), m = wrap(mu), r = wrap(rsigma);
    hetu::impl::DropoutAddLnFwdCuda(wrap(x0), wrap(residual), wrap(gamma), wrap(beta), wrap(rowscale),
                                    wrap(colscale), wrap(x0_subset), wrap(z_subset), zz, xx, dm, m, r, dropout_p,
                                    epsilon, rowscale_const, z_numrows, residual_in_fp32 != 0, is_rms_norm != 0,
                                    stream_of(x0, stream_index));
  });
}

int ht_dropout_add_ln_bwd(const HtArray* dz, const HtArray* dx, const HtArray* x, const HtArray* x0,
                          const HtArray* dmask, const HtArray* mu, const HtArray* rsigma, const HtArray* gamma,
                          const HtArray* rowscale, const HtArray* colscale, const HtArray* x0_subset,
                          const HtArray* z_subset, HtArray* dx0, HtArray* dresidual, HtArray* dgamma,
                          HtArray* dbeta, HtArray* dcolscale, float dropout_p, float rowscale_const,
                          int64_t x0_numrows, int has_residual, int is_rms_norm, int stream_index) {
  return guarded([&] {
    NDArray d0 = wrap(dx0), dr = wrap(dresidual), dg = wrap(dgamma), db = wrap(dbeta), dc = wrap(dcolscale);
    NDArray p1, p2, p3;
    hetu::impl::DropoutAddLnBwdCuda(wrap(dz), wrap(dx), wrap(x), wrap(x0), wrap(dmask), wrap(mu), wrap(rsigma),
                                    wrap(gamma), wrap(rowscale), wrap(colscale), wrap(x0_subset), wrap(z_subset),
                                    d0, dr, dg, db, p1, p2, dc, p3, dropout_p, rowscale_const, x0_numrows,
                                    has_residual != 0, is_rms_norm != 0, stream_of(dz, stream_index));
  });
}

int ht_dropout_add_ln_parallel_residual_fwd(const HtArray* x0, const HtArray* x1, const HtArray* residual,
                                            const HtArray* gamma0, const HtArray* beta0, const HtArray* gamma1,
                                            const HtArray* beta1, HtArray* z0, HtArray* z1, HtArray* x,
                                            HtArray* dmask0, HtArray* dmask1, HtArray* mu, HtArray* rsigma,
                                            float dropout_p, float epsilon, int residual_in_fp32, int is_rms_norm,
                                            int stream_index) {
  return guarded([&] {
    NDArray a0 = wrap(z0), a1 = wrap(z1), xx = wrap(x), m0 = wrap(dmask0), m1 = wrap(dmask1), m = wrap(mu),
            r = wrap(rsigma);
    hetu::impl::DropoutAddLnParallelResidualFwdCuda(wrap(x0), wrap(x1), wrap(residual), wrap(gamma0), wrap(beta0),
                                                    wrap(gamma1), wrap(beta1), a0, a1, xx, m0, m1, m, r, dropout_p,
                                                    epsilon, residual_in_fp32 != 0, is_rms_norm != 0,
                                                    stream_of(x0, stream_index));
  });
}

int ht_dropout_add_ln_parallel_residual_bwd(const HtArray* dz0, const HtArray* dz1, const HtArray* dx,
                                            const HtArray* x, const HtArray* dmask0, const HtArray* dmask1,
                                            const HtArray* mu, const HtArray* rsigma, const HtArray* gamma0,
                                            const HtArray* gamma1, HtArray* dx0, HtArray* dx1, HtArray* dresidual,
                                            HtArray* dgamma0, HtArray* dbeta0, HtArray* dgamma1, HtArray* dbeta1,
                                            float dropout_p, int has_x1, int has_residual, int is_rms_norm,
                                            int stream_index) {
  return guarded([&] {
    NDArray d0 = wrap(dx0), d1 = wrap(dx1), dr = wrap(dresidual), g0 = wrap(dgamma0), b0 = wrap(dbeta0),
            g1 = wrap(dgamma1), b1 = wrap(dbeta1), p1, p2, p3, p4;
    hetu::impl::DropoutAddLnParallelResidualBwdCuda(wrap(dz0), wrap(dz1), wrap(dx), wrap(x), wrap(dmask0),
                                                    wrap(dmask1), wrap(mu), wrap(rsigma), wrap(gamma0), wrap(gamma1),
                                                    d0, d1, dr, g0, b0, g1, b1, p1, p2, p3, p4, dropout_p,
                                                    has_x1 != 0, has_residual != 0, is_rms_norm != 0,
                                                    stream_of(dz0, stream_index));
  });
}

int ht_set_random_seed(uint64_t seed) {
  return guarded([&] { hetu::impl::SetCPURandomSeed(seed); });
}

int ht_instance_norm(const HtArray* in, HtArray* mean, HtArray* var, HtArray* out, float eps, int stream_index) {
  return guarded([&] {
    NDArray m = wrap(mean), v = wrap(var), o = wrap(out);
    const Stream st = stream_of(in, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_instance_norm", hetu::impl::InstanceNorm, wrap(in), m, v, o,
                                    eps, st);
  });
}

int ht_instance_norm_gradient(const HtArray* out_grads, const HtArray* in, HtArray* grad_in, const HtArray* mean,
                              const HtArray* var, float eps, int stream_index) {
  return guarded([&] {
    NDArray g = wrap(grad_in);
    const Stream st = stream_of(in, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_instance_norm_gradient", hetu::impl::InstanceNormGradient,
                                    wrap(out_grads), wrap(in), g, wrap(mean), wrap(var), eps, st);
  });
}

int ht_softmax(const HtArray* in, HtArray* out, int64_t dim, int stream_index) {
  return guarded([&] {
    NDArray o = wrap(out);
    const Stream st = stream_of(in, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_softmax", hetu::impl::Softmax, wrap(in), o, dim, st);
  });
}

int ht_softmax_gradient(const HtArray* y, const HtArray* dy, HtArray* dx, int64_t dim, int stream_index) {
  return guarded([&] {
    NDArray o = wrap(dx);
    const Stream st = stream_of(y, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_softmax_gradient", hetu::impl::SoftmaxGradient, wrap(y),
                                    wrap(dy), o, dim, st);
  });
}

int ht_softmax_cross_entropy(const HtArray* pred, const HtArray* label, HtArray* loss, int stream_index) {
  return guarded([&] {
    NDArray o = wrap(loss);
    const Stream st = stream_of(pred, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_softmax_cross_entropy", hetu::impl::SoftmaxCrossEntropy,
                                    wrap(pred), wrap(label), o, st);
  });
}

int ht_softmax_cross_entropy_gradient(const HtArray* pred, const HtArray* label, const HtArray* grad_loss,
                                      HtArray* out, int stream_index) {
  return guarded([&] {
    NDArray o = wrap(out);
    const Stream st = stream_of(pred, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_softmax_cross_entropy_gradient",
                                    hetu::impl::SoftmaxCrossEntropyGradient, wrap(pred), wrap(label), wrap(grad_loss),
                                    o, st);
  });
}

int ht_softmax_cross_entropy_sparse(const HtArray* pred, const HtArray* label, HtArray* loss,
                                    int64_t ignored_index, int stream_index) {
  return guarded([&] {
    NDArray o = wrap(loss);
    const Stream st = stream_of(pred, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_softmax_cross_entropy_sparse",
                                    hetu::impl::SoftmaxCrossEntropySparse, wrap(pred), wrap(label), o,
                                    ignored_index, st);
  });
}

int ht_softmax_cross_entropy_sparse_gradient(const HtArray* pred, const HtArray* label, const HtArray* grad_loss,
                                             HtArray* out, int64_t ignored_index, int stream_index) {
  return guarded([&] {
    NDArray o = wrap(out);
    const Stream st = stream_of(pred, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_softmax_cross_entropy_sparse_gradient",
                                    hetu::impl::SoftmaxCrossEntropySparseGradient, wrap(pred), wrap(label),
                                    wrap(grad_loss), o, ignored_index, st);
  });
}

int ht_nll_loss(const HtArray* pred, const HtArray* label, HtArray* loss, int stream_index) {
  return guarded([&] {
    NDArray o = wrap(loss);
    const Stream st = stream_of(pred, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_nll_loss", hetu::impl::NLLLoss, wrap(pred), wrap(label), o,
                                    st);
  });
}

int ht_nll_loss_gradient(const HtArray* pred, const HtArray* label, const HtArray* grad_loss, HtArray* out,
                         int stream_index) {
  return guarded([&] {
    NDArray o = wrap(out);
    const Stream st = stream_of(pred, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_nll_loss_gradient", hetu::impl::NLLLossGradient, wrap(pred),
                                    wrap(label), wrap(grad_loss), o, st);
  });
}

int ht_reduce(const HtArray* in, HtArray* out, const int64_t* axes, int naxes, int red_type, int stream_index) {
  return guarded([&] {
    NDArray o = wrap(out);
    HTAxes ax(axes, axes + naxes);
    const Stream st = stream_of(in, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_reduce", hetu::impl::Reduce, wrap(in), o, ax,
                                    static_cast<ReductionType>(red_type), st);
  });
}

int ht_binary(int op, const HtArray* a, const HtArray* b, HtArray* out, int stream_index) {
  return guarded([&] {
    NDArray o = wrap(out);
    const Stream st = stream_of(a, stream_index);
    switch (op) {
      case 0:
        HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_binary", hetu::impl::AddElewise, wrap(a), wrap(b), o, st);
        break;
      case 1:
        HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_binary", hetu::impl::SubElewise, wrap(a), wrap(b), o, st);
        break;
      case 2:
        HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_binary", hetu::impl::MulElewise, wrap(a), wrap(b), o, st);
        break;
      case 3:
        HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_binary", hetu::impl::DivElewise, wrap(a), wrap(b), o, st);
        break;
      default: HT_VALUE_ERROR << "unknown binary op " << op;
    }
  });
}

int ht_binary_const(int op, const HtArray* in, double value, HtArray* out, int stream_index) {
  return guarded([&] {
    NDArray o = wrap(out);
    const Stream st = stream_of(in, stream_index);
    switch (op) {
      case 0:
        HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_binary_const", hetu::impl::AddConst, wrap(in), value, o, st);
        break;
      case 1:
        HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_binary_const", hetu::impl::SubConst, wrap(in), value, o, st);
        break;
      case 2:
        HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_binary_const", hetu::impl::MulConst, wrap(in), value, o, st);
        break;
      case 3:
        HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_binary_const", hetu::impl::DivConst, wrap(in), value, o, st);
        break;
      default: HT_VALUE_ERROR << "unknown binary op " << op;
    }
  });
}

int ht_unary(int op, const HtArray* in, HtArray* out, int stream_index) {
  return guarded([&] {
    NDArray o = wrap(out);
    const Stream st = stream_of(in, stream_index);
    switch (op) {
      case 0: HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_unary", hetu::impl::Exp, wrap(in), o, st); break;
      case 1: HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_unary", hetu::impl::Log, wrap(in), o, st); break;
      case 2: HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_unary", hetu::impl::Opposite, wrap(in), o, st); break;
      case 3: HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_unary", hetu::impl::Sqrt, wrap(in), o, st); break;
      default: HT_VALUE_ERROR << "unknown unary op " << op;
    }
  });
}

int ht_ndarray_binary(int op, const HtArray* a, const HtArray* b, HtArray* out, int in_place, int stream_index) {
  return guarded([&] {
    NDArray x = wrap(a), y = wrap(b), r, none;
    NDArray& dst = in_place ? x : none;
    switch (op) {
      case 0: r = NDArray::add(x, y, stream_index, dst); break;
      case 1: r = NDArray::sub(x, y, stream_index, dst); break;
      case 2: r = NDArray::mul(x, y, stream_index, dst); break;
      case 3: r = NDArray::div(x, y, stream_index, dst); break;
      default: HT_VALUE_ERROR << "unknown binary op " << op;
    }
    if (!in_place) copy_out(r, out, stream_of(a, stream_index));
  });
}

int ht_ndarray_unary(int op, const HtArray* in, HtArray* out, int in_place, int stream_index) {
  return guarded([&] {
    NDArray x = wrap(in), r, none;
    NDArray& dst = in_place ? x : none;
    switch (op) {
      case 0: r = NDArray::exp(x, stream_index, dst); break;
      case 1: r = NDArray::log(x, stream_index, dst); break;
      case 2: r = NDArray::neg(x, stream_index, dst); break;
      case 3: r = NDArray::sqrt(x, stream_index, dst); break;
      default: HT_VALUE_ERROR << "unknown unary op " << op;
    }
    if (!in_place) copy_out(r, out, stream_of(in, stream_index));
  });
}

int ht_batch_norm(const HtArray* input_X, const HtArray* bn_scale, const HtArray* bn_bias, HtArray* output_Y,
                  double momentum, double eps, HtArray* running_mean, HtArray* running_var, HtArray* save_mean,
                  HtArray* save_var, int stream_index) {
  return guarded([&] {
    NDArray y = wrap(output_Y), rm = wrap(running_mean), rv = wrap(running_var), sm = wrap(save_mean),
            sv = wrap(save_var);
    const Stream st = stream_of(input_X, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_batch_norm", hetu::impl::BatchNorm, wrap(input_X),
                                    wrap(bn_scale), wrap(bn_bias), y, momentum, eps, rm, rv, sm, sv, st);
  });
}

int ht_batch_norm_gradient(const HtArray* gradient_Y, const HtArray* input_X, const HtArray* bn_scale,
                           HtArray* gradient_X, HtArray* gradient_bn_scale, HtArray* gradient_bn_bias, double eps,
                           HtArray* save_mean, HtArray* save_var, int stream_index) {
  return guarded([&] {
    NDArray dx = wrap(gradient_X), ds = wrap(gradient_bn_scale), db = wrap(gradient_bn_bias), sm = wrap(save_mean),
            sv = wrap(save_var);
    const Stream st = stream_of(input_X, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_batch_norm_gradient", hetu::impl::BatchNormGradient,
                                    wrap(gradient_Y), wrap(input_X), wrap(bn_scale), dx, ds, db, eps, sm, sv, st);
  });
}

int ht_norm(const HtArray* input, HtArray* output, int64_t dim, int64_t p, int stream_index) {
  return guarded([&] {
    NDArray o = wrap(output);
    const Stream st = stream_of(input, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_norm", hetu::impl::Norm, wrap(input), o, dim, p, st);
  });
}

int ht_norm_gradient(const HtArray* input, const HtArray* output, const HtArray* output_grad, HtArray* input_grad,
                     int64_t dim, int64_t p, int stream_index) {
  return guarded([&] {
    NDArray g = wrap(input_grad);
    const Stream st = stream_of(input, stream_index);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_norm_gradient", hetu::impl::NormGradient, wrap(input),
                                    wrap(output), wrap(output_grad), g, dim, p, st);
  });
}

int ht_ndarray_norm(const HtArray* input, int64_t p, int64_t dim, int keepdim, HtArray* out, int stream_index) {
  return guarded([&] {
    NDArray r = NDArray::norm(wrap(input), p, dim, keepdim != 0, stream_index);
    copy_out(r, out, stream_of(input, stream_index));
  });
}

int ht_vocab_parallel_cross_entropy(const HtArray* vocab_parallel_logits, const HtArray* labels,
                                    int64_t vocab_start_index, int64_t vocab_end_index, int64_t ignored_index,
                                    HtArray* predicted_logits_partial, HtArray* log_sum_exp_logits,
                                    int stream_index) {
  return guarded([&] {
    NDArray p = wrap(predicted_logits_partial), l = wrap(log_sum_exp_logits);
    hetu::impl::VocabParallelCrossEntropyCuda(wrap(vocab_parallel_logits), wrap(labels), vocab_start_index,
                                              vocab_end_index, ignored_index, p, l,
                                              stream_of(vocab_parallel_logits, stream_index));
  });
}

int ht_vocab_parallel_cross_entropy_gradient(const HtArray* softmax, const HtArray* labels,
                                             int64_t vocab_start_index, int64_t vocab_end_index,
                                             int64_t ignored_index, const HtArray* grad_loss, HtArray* output,
                                             int stream_index) {
  return guarded([&] {
    NDArray o = wrap(output);
    hetu::impl::VocabParallelCrossEntropyGradientCuda(wrap(softmax), wrap(labels), vocab_start_index,
                                                      vocab_end_index, ignored_index, wrap(grad_loss), o,
                                                      stream_of(softmax, stream_index));
  });
}

int ht_ndarray_reduce(const HtArray* in, int red_type, const int64_t* axes, int naxes, int keepdims, HtArray* out,
                      int stream_index) {
  return guarded([&] {
    HTAxes ax(axes, axes + naxes);
    NDArray r = NDArray::reduce(wrap(in), static_cast<ReductionType>(red_type), ax, keepdims != 0, stream_index);
    copy_out(r, out, stream_of(in, stream_index));
  });
}

int ht_ndarray_softmax(const HtArray* in, int64_t dim, HtArray* out, int stream_index) {
  return guarded([&] {
    NDArray r = NDArray::softmax(wrap(in), dim, stream_index);
    copy_out(r, out, stream_of(in, stream_index));
  });
}

int ht_ndarray_layernorm(const HtArray* in, const HtArray* scale, const HtArray* bias, int normalized_ndim,
                         double eps, int fused, HtArray* out, HtArray* mean, HtArray* var, int stream_index) {
  return guarded([&] {
    NDArray x = wrap(in);
    HT_VALUE_ERROR_IF(normalized_ndim < 1 || size_t(normalized_ndim) > x->ndim()) << "bad normalized_ndim";
    HTShape normalized(x->shape().end() - normalized_ndim, x->shape().end());
    NDArrayList r = fused ? NDArray::fused_layernorm(x, wrap(scale), wrap(bias), normalized, eps, stream_index)
                          : NDArray::layernorm(x, wrap(scale), wrap(bias), normalized, eps, stream_index);
    const Stream s = stream_of(in, stream_index);
    copy_out(r[0], out, s);
    if (mean) copy_out(r[1], mean, s);
    if (var) copy_out(r[2], var, s);
  });
}

int ht_ndarray_sceloss(const HtArray* preds, const HtArray* labels, int sparse, int64_t ignored_index,
                       int reduction, HtArray* out, int stream_index) {
  return guarded([&] {
    const auto red = static_cast<ReductionType>(reduction);
    NDArray r = sparse ? NDArray::sceloss(wrap(preds), wrap(labels), ignored_index, red, stream_index)
                       : NDArray::sceloss(wrap(preds), wrap(labels), red, stream_index);
    copy_out(r, out, stream_of(preds, stream_index));
  });
}

int ht_broadcast_shape(const HtArray* input, int multiply, double const_value, HtArray* output,
                       const int64_t* add_axes, int n_add_axes, int stream_index) {
  return guarded([&] {
    NDArray out = wrap(output);
    HTShape axes(add_axes, add_axes + (add_axes ? n_add_axes : 0));
    const Stream st = stream_of(input, stream_index);
    if (multiply)
      HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_broadcast_shape", hetu::impl::BroadcastShapeMul,
                                      wrap(input), const_value, out, axes, st);
    else
      HT_DISPATCH_KERNEL_CPU_AND_CUDA(st.device_type(), "ht_broadcast_shape", hetu::impl::BroadcastShape, wrap(input),
                                      out, axes, st);
  });
}

int ht_reduce_gradient(const HtArray* grad_output, int reduction, const int64_t* axes, int naxes,
                       const int* keepdims, int n_keepdims, HtArray* output, int stream_index) {
  return guarded([&] {
    NDArray out = wrap(output);
    HTAxes ax(axes, axes + (axes ? naxes : 0));
    hetu::graph::HTKeepDims keep;
    for (int i = 0; i < n_keepdims; ++i) keep.push_back(keepdims[i] != 0);
    hetu::graph::ReduceGradientCompute(wrap(grad_output), out->shape(), static_cast<ReductionType>(reduction), ax,
                                       keep, stream_index, out);
  });
}

int ht_sceloss_gradient(const HtArray* preds, const HtArray* labels, const HtArray* grad_output, int sparse,
                        int64_t ignored_index, int reduction, int fused, HtArray* output, int stream_index) {
  return guarded([&] {
    NDArray out = wrap(output);
    const auto red = static_cast<ReductionType>(reduction);
    if (sparse)
      hetu::graph::SCESGradCompute(wrap(preds), wrap(labels), wrap(grad_output), ignored_index, red, stream_index,
                                   out, fused != 0);
    else
      hetu::graph::SCEGradCompute(wrap(preds), wrap(labels), wrap(grad_output), red, stream_index, out, fused != 0);
  });
}

int ht_stream_sync(int device_index, int stream_index) {
  return guarded([&] { Stream(Device(kCUDA, DeviceIndex(device_index)), StreamIndex(stream_index)).Sync(); });
}

int ht_synchronize_all(void) {
  return guarded([&] { SynchronizeAllStreams(); });
}

int ht_host_stream_sync(int stream_index) {
  return guarded([&] { Stream(Device(kCPU), StreamIndex(stream_index)).Sync(); });
}

int ht_set_host_async(int on) {
  const bool before = g_host_async.exchange(on != 0);
  return before ? 1 : 0;
}

int ht_set_host_threads(int threads) {
  hetu::impl::SetHostKernelThreads(threads);
#ifdef _OPENMP
  return threads > 0 ? threads : omp_get_max_threads();
#else
  return threads > 0 ? threads : 1;
#endif
}

int ht_pool_alloc(int device_index, size_t bytes, int stream_index, void** ptr, uint64_t* id,
                  size_t* granted_bytes) {
  return guarded([&] {
    const Device dev(kCUDA, DeviceIndex(device_index));
    DataPtr p = AllocFromMemoryPool(dev, bytes, Stream(dev, StreamIndex(stream_index)));
    *ptr = p.ptr;
    *id = p.id;
    *granted_bytes = p.size;
  });
}

int ht_pool_free(int device_index, void* ptr, uint64_t id, size_t granted_bytes) {
  return guarded([&] { FreeToMemoryPool(DataPtr(ptr, granted_bytes, Device(kCUDA, DeviceIndex(device_index)), id)); });
}

int ht_pool_mark_used(int device_index, void* ptr, uint64_t id, size_t granted_bytes, int stream_index) {
  return guarded([&] {
    const Device dev(kCUDA, DeviceIndex(device_index));
    GetMemoryPool(dev)->MarkDataSpaceUsedByStream(DataPtr(ptr, granted_bytes, dev, id),
                                                  Stream(dev, StreamIndex(stream_index)));
  });
}

int ht_pool_empty_cache(int device_index) {
  return guarded([&] { GetMemoryPool(Device(kCUDA, DeviceIndex(device_index)))->EmptyCache(); });
}

int ht_pool_stats(int device_index, uint64_t* values, int n_values) {
  return guarded([&] {
    auto s = caching_pool(device_index).stats();
    const uint64_t all[14] = {s.allocated, s.peak_allocated, s.reserved, s.peak_reserved, s.alloc_cnt, s.free_cnt,
                              s.mark_cnt, s.segment_allocs, s.segment_frees, s.cache_hits, s.cross_stream_takes,
                              s.parked, s.splits, s.merges};
    for (int i = 0; i < n_values && i < 14; ++i) values[i] = all[i];
  });
}

} // extern "C"
