// Entry-point macros of the binary, comparison, logical and in-place families: one `hip_<op>_<dtype>` per
// `cuda_<op>_<dtype>` of crates/maidenx_cuda/src/ops/binary.rs:12-161 (same argument order); metadata is a HOST
// pointer, as on the reference's CPU arm.
#pragma once
#include "elementwise.hpp"
#include "ops.hpp"

using namespace mxh;

#define MXH_BINARY(NAME, OP, T, SUF, O)                                                                       \
    extern "C" void hip_##NAME##_##SUF(size_t num_els, size_t num_dims, const size_t* md, const T* lhs,       \
                                       const T* rhs, O* out) { MXH_API;                                       \
        ew_binary(num_els, num_dims, md, lhs, rhs, out, OP<T>{}, false);                                      \
    }
#define MXH_INPLACE(NAME, OP, T, SUF)                                                                         \
    extern "C" void hip_##NAME##_inplace_##SUF(size_t num_els, size_t num_dims, const size_t* md, T* lhs,     \
                                               const T* rhs) { MXH_API;                                       \
        ew_binary(num_els, num_dims, md, lhs, rhs, nullptr, OP<T>{}, true);                                   \
    }

#define MXH_ALL_FOR(T, SUF)                      \
    MXH_BINARY(add, OpAdd, T, SUF, T)            \
    MXH_BINARY(sub, OpSub, T, SUF, T)            \
    MXH_BINARY(mul, OpMul, T, SUF, T)            \
    MXH_BINARY(div, OpDiv, T, SUF, T)            \
    MXH_BINARY(maximum, OpMaximum, T, SUF, T)    \
    MXH_BINARY(minimum, OpMinimum, T, SUF, T)    \
    MXH_BINARY(logical_and, OpLogicalAnd, T, SUF, bool_t) \
    MXH_BINARY(logical_or, OpLogicalOr, T, SUF, bool_t)   \
    MXH_BINARY(logical_xor, OpLogicalXor, T, SUF, bool_t) \
    MXH_BINARY(eq, OpEq, T, SUF, bool_t)         \
    MXH_BINARY(ne, OpNe, T, SUF, bool_t)         \
    MXH_BINARY(lt, OpLt, T, SUF, bool_t)         \
    MXH_BINARY(le, OpLe, T, SUF, bool_t)         \
    MXH_BINARY(gt, OpGt, T, SUF, bool_t)         \
    MXH_BINARY(ge, OpGe, T, SUF, bool_t)         \
    MXH_INPLACE(add, OpAdd, T, SUF)              \
    MXH_INPLACE(sub, OpSub, T, SUF)              \
    MXH_INPLACE(mul, OpMul, T, SUF)              \
    MXH_INPLACE(div, OpDiv, T, SUF)

