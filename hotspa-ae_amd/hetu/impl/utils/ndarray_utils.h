// Argument-check macros of the kernel entry points
// (hetu/impl/utils/ndarray_utils.h of the reference).
#pragma once

#include "hetu/core/ndarray.h"

#define HT_ASSERT_CUDA_DEVICE(x) HT_ASSERT(x->is_cuda()) << "Data " << #x << " is not on an accelerator device."
#define HT_ASSERT_CPU_DEVICE(x) HT_ASSERT(x->is_cpu()) << "Data " << #x << " is not on a host device."
#define HT_ASSERT_SAME_SHAPE(x, y)                                                                  \
  HT_ASSERT(x->shape() == y->shape()) << "Data are not with the same shape: (" << #x << ") "         \
                                      << x->shape() << " vs. (" << #y << ") " << y->shape() << "."
#define HT_ASSERT_SAME_DTYPE(x, y)                                                                  \
  HT_ASSERT(x->dtype() == y->dtype()) << "Data are not with the same data type: (" << #x << ") "     \
                                      << x->dtype() << " vs. (" << #y << ") " << y->dtype() << "."
#define HT_ASSERT_SAME_DEVICE(x, y)                                                                 \
  HT_ASSERT(x->device() == y->device()) << "Data are not on the same device: (" << #x << ") "        \
                                        << x->device() << " vs. (" << #y << ") " << y->device() << "."
#define HT_ASSERT_NDIM(x, nd)                                                                       \
  HT_ASSERT(x->ndim() == size_t(nd)) << "Data " << #x << " expected to be with " << (nd)            \
                                     << " dimensions but got " << x->ndim() << "."
#define HT_ASSERT_CONTIGUOUS(x)                                                                     \
  HT_ASSERT(x->is_contiguous()) << "Data " << #x << " is not contiguous. Shape: " << x->shape()      \
                                << ". Strides: " << x->stride() << "."
