// dtype switch macros (names of hetu/impl/utils/dispatch.h:9-64 in the
// reference).  An unsupported dtype reaches the default case and throws
// hetu::not_implemented.
#pragma once

#include "hetu/core/dtype.h"

#define HT_DISPATH_CASE(DATA_TYPE, SPEC_TYPE, ...)                                                  \
  case DATA_TYPE: {                                                                                 \
    using SPEC_TYPE = hetu::DataType2SpecMeta<DATA_TYPE>::spec_type;                                \
    __VA_ARGS__();                                                                                  \
    break;                                                                                          \
  }

#define HT_DISPATH_SWITCH(DTYPE, NAME, ...)                                                         \
  do {                                                                                              \
    const auto& _dtype = DTYPE;                                                                     \
    switch (_dtype) {                                                                               \
      __VA_ARGS__                                                                                   \
      default:                                                                                      \
        HT_NOT_IMPLEMENTED << "\"" << NAME << "\" is not implemented for \"" << _dtype << "\"";     \
    }                                                                                               \
  } while (0)

#define HT_DISPATH_CASE_FLOATING_TYPES(SPEC_TYPE, ...)                                              \
  HT_DISPATH_CASE(hetu::DataType::FLOAT16, SPEC_TYPE, __VA_ARGS__)                                  \
  HT_DISPATH_CASE(hetu::DataType::BFLOAT16, SPEC_TYPE, __VA_ARGS__)                                 \
  HT_DISPATH_CASE(hetu::DataType::FLOAT32, SPEC_TYPE, __VA_ARGS__)                                  \
  HT_DISPATH_CASE(hetu::DataType::FLOAT64, SPEC_TYPE, __VA_ARGS__)

#define HT_DISPATH_CASE_INTEGER_TYPES(SPEC_TYPE, ...)                                               \
  HT_DISPATH_CASE(hetu::DataType::UINT8, SPEC_TYPE, __VA_ARGS__)                                    \
  HT_DISPATH_CASE(hetu::DataType::INT8, SPEC_TYPE, __VA_ARGS__)                                     \
  HT_DISPATH_CASE(hetu::DataType::INT16, SPEC_TYPE, __VA_ARGS__)                                    \
  HT_DISPATH_CASE(hetu::DataType::INT32, SPEC_TYPE, __VA_ARGS__)                                    \
  HT_DISPATH_CASE(hetu::DataType::INT64, SPEC_TYPE, __VA_ARGS__)

#define HT_DISPATCH_FLOATING_TYPES(DTYPE, SPEC_TYPE, NAME, ...)                                     \
  HT_DISPATH_SWITCH(DTYPE, NAME, HT_DISPATH_CASE_FLOATING_TYPES(SPEC_TYPE, __VA_ARGS__))

#define HT_DISPATCH_INTEGER_TYPES(DTYPE, SPEC_TYPE, NAME, ...)                                      \
  HT_DISPATH_SWITCH(DTYPE, NAME, HT_DISPATH_CASE_INTEGER_TYPES(SPEC_TYPE, __VA_ARGS__))

#define HT_DISPATCH_INTEGER_AND_FLOATING_TYPES(DTYPE, SPEC_TYPE, NAME, ...)                         \
  HT_DISPATH_SWITCH(DTYPE, NAME,                                                                    \
                    HT_DISPATH_CASE_FLOATING_TYPES(SPEC_TYPE, __VA_ARGS__)                          \
                      HT_DISPATH_CASE_INTEGER_TYPES(SPEC_TYPE, __VA_ARGS__))
