// dtype/op dispatch shared by the launchers: maps the run-time (fa_dtype, fa_op)
// pair onto a template instantiation FN<T, Op>(args...).
#pragma once
#include "common.hip.h"

using namespace fa;

#define FA_DISPATCH_TYPE_OP(FN, t, op, ...)                                          \
  switch (t) {                                                                       \
    case FA_I32:                                                                     \
      switch (op) {                                                                  \
        case FA_ADD: return FN<int32_t, OpAdd<int32_t>>(__VA_ARGS__);                \
        case FA_MAX: return FN<int32_t, OpMax<int32_t>>(__VA_ARGS__);                \
        case FA_MIN: return FN<int32_t, OpMin<int32_t>>(__VA_ARGS__);                \
        case FA_AND: return FN<int32_t, OpAnd<int32_t>>(__VA_ARGS__);                \
        case FA_OR: return FN<int32_t, OpOr<int32_t>>(__VA_ARGS__);                  \
        case FA_XOR: return FN<int32_t, OpXor<int32_t>>(__VA_ARGS__);                \
        default: return FA_ENOTSUP;                                                  \
      }                                                                              \
    case FA_I64:                                                                     \
      switch (op) {                                                                  \
        case FA_ADD: return FN<int64_t, OpAdd<int64_t>>(__VA_ARGS__);                \
        case FA_MAX: return FN<int64_t, OpMax<int64_t>>(__VA_ARGS__);                \
        case FA_MIN: return FN<int64_t, OpMin<int64_t>>(__VA_ARGS__);                \
        case FA_AND: return FN<int64_t, OpAnd<int64_t>>(__VA_ARGS__);                \
        case FA_OR: return FN<int64_t, OpOr<int64_t>>(__VA_ARGS__);                  \
        case FA_XOR: return FN<int64_t, OpXor<int64_t>>(__VA_ARGS__);                \
        default: return FA_ENOTSUP;                                                  \
      }                                                                              \
    case FA_U32:                                                                     \
      switch (op) {                                                                  \
        case FA_ADD: return FN<uint32_t, OpAdd<uint32_t>>(__VA_ARGS__);              \
        case FA_MAX: return FN<uint32_t, OpMax<uint32_t>>(__VA_ARGS__);              \
        case FA_MIN: return FN<uint32_t, OpMin<uint32_t>>(__VA_ARGS__);              \
        case FA_AND: return FN<uint32_t, OpAnd<uint32_t>>(__VA_ARGS__);              \
        case FA_OR: return FN<uint32_t, OpOr<uint32_t>>(__VA_ARGS__);                \
        case FA_XOR: return FN<uint32_t, OpXor<uint32_t>>(__VA_ARGS__);              \
        default: return FA_ENOTSUP;                                                  \
      }                                                                              \
    case FA_U64:                                                                     \
      switch (op) {                                                                  \
        case FA_ADD: return FN<uint64_t, OpAdd<uint64_t>>(__VA_ARGS__);              \
        case FA_MAX: return FN<uint64_t, OpMax<uint64_t>>(__VA_ARGS__);              \
        case FA_MIN: return FN<uint64_t, OpMin<uint64_t>>(__VA_ARGS__);              \
        case FA_AND: return FN<uint64_t, OpAnd<uint64_t>>(__VA_ARGS__);              \
        case FA_OR: return FN<uint64_t, OpOr<uint64_t>>(__VA_ARGS__);                \
        case FA_XOR: return FN<uint64_t, OpXor<uint64_t>>(__VA_ARGS__);              \
        default: return FA_ENOTSUP;                                                  \
      }                                                                              \
    case FA_F32:                                                                     \
      switch (op) {                                                                  \
        case FA_ADD: return FN<float, OpAdd<float>>(__VA_ARGS__);                    \
        case FA_MAX: return FN<float, OpMax<float>>(__VA_ARGS__);                    \
        case FA_MIN: return FN<float, OpMin<float>>(__VA_ARGS__);                    \
        default: return FA_ENOTSUP;                                                  \
      }                                                                              \
    case FA_F64:                                                                     \
      switch (op) {                                                                  \
        case FA_ADD: return FN<double, OpAdd<double>>(__VA_ARGS__);                  \
        case FA_MAX: return FN<double, OpMax<double>>(__VA_ARGS__);                  \
        case FA_MIN: return FN<double, OpMin<double>>(__VA_ARGS__);                  \
        default: return FA_ENOTSUP;                                                  \
      }                                                                              \
    default: return FA_ENOTSUP;                                                      \
  }

static inline size_t dtype_size(fa_dtype t) {
  switch (t) {
    case FA_I32: case FA_U32: case FA_F32: return 4;
    case FA_I64: case FA_U64: case FA_F64: case FA_I32X2: return 8;
    case FA_F16: case FA_BF16: case FA_I16: case FA_U16: return 2;
    case FA_I8: case FA_U8: return 1;
    default: return 0;
  }
}

