// The functor dispatch of the fused chains and the resident step programs: position in EwProgOps -> functor, applied to a
// thread's elements.
#pragma once
#include <cstring>
#include <type_traits>
#include <utility>

#include "elementwise.hpp"
#include "mxh.hpp"
#include "ops.hpp"

namespace mxh {

// The functors whose evaluation is long (the libm restatements: dozens to hundreds of instructions per element).  A chain
// kernel runs for a few microseconds on code that is not in the instruction cache when it starts, so what its loops
// execute has to be compact: the short functors are dispatched by a switch of their own, whose cases are a few
// instructions each and sit next to each other, and the long ones by a second switch that is laid out after the loops.
template <class Op> struct IsLongOp { static constexpr bool value = false; };
#define MXH_LONG_OP(NAME) template <> struct IsLongOp<NAME<float>> { static constexpr bool value = true; };
MXH_LONG_OP(OpSigmoid) MXH_LONG_OP(OpTanh) MXH_LONG_OP(OpGelu) MXH_LONG_OP(OpSin) MXH_LONG_OP(OpCos) MXH_LONG_OP(OpTan) MXH_LONG_OP(OpLn)
MXH_LONG_OP(OpLog10) MXH_LONG_OP(OpLog2) MXH_LONG_OP(OpExp) MXH_LONG_OP(OpExp10) MXH_LONG_OP(OpExp2) MXH_LONG_OP(OpSoftplus) MXH_LONG_OP(OpPow)
MXH_LONG_OP(OpElu)
#undef MXH_LONG_OP
template <int I>
constexpr uint64_t long_op_bit() {
    if constexpr (I < EwProgOps::size) return IsLongOp<typename TypeAt<I, EwProgOps>::type>::value ? (1ull << I) : 0ull;
    else return 0ull;
}
template <int... Is>
constexpr uint64_t long_op_mask(std::integer_sequence<int, Is...>) { return (long_op_bit<Is>() | ... | 0ull); }
constexpr uint64_t LONG_OPS = long_op_mask(std::make_integer_sequence<int, 64>{});
__device__ __forceinline__ bool is_long_op(uint32_t op) { return (LONG_OPS >> (op & 63u)) & 1ull; }

// the functor at position I of EwProgOps applied to a thread's elements (only those that map float to float are
// recorded; the others compile to nothing), when it is of the wanted kind
template <int I, int VEC, bool LONG>
__device__ __forceinline__ void fuse_case(const float (&a)[VEC], const float (&b)[VEC], float (&r)[VEC], const uint32_t (&payload)[2]) {
    if constexpr (I < EwProgOps::size) {
        using Op = typename TypeAt<I, EwProgOps>::type;
        if constexpr (std::is_same<typename Op::Out, float>::value && std::is_same<typename Op::In, float>::value && sizeof(Op) <= 8 &&
                      IsLongOp<Op>::value == LONG) {
            Op o;
            __builtin_memcpy((void*)&o, payload, sizeof(Op));
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                if constexpr (Op::NIN == 1) r[e] = o(a[e]);
                else r[e] = o(a[e], b[e]);
            }
        }
    }
}
#define MXH_FC(I) case I: fuse_case<I, VEC, LONG>(a, b, r, payload); break;
#define MXH_FC8(B) MXH_FC(B + 0) MXH_FC(B + 1) MXH_FC(B + 2) MXH_FC(B + 3) MXH_FC(B + 4) MXH_FC(B + 5) MXH_FC(B + 6) MXH_FC(B + 7)
static_assert(EwProgOps::size <= 64, "the dispatch below has 64 cases");
template <int VEC, bool LONG>
__device__ __forceinline__ void fuse_switch(uint32_t op, const float (&a)[VEC], const float (&b)[VEC], float (&r)[VEC], const uint32_t (&payload)[2]) {
    switch (op) {      // uniform: one scalar dispatch per member, not per element
        MXH_FC8(0) MXH_FC8(8) MXH_FC8(16) MXH_FC8(24) MXH_FC8(32) MXH_FC8(40) MXH_FC8(48) MXH_FC8(56)
        default: break;
    }
}
#undef MXH_FC
#undef MXH_FC8
template <int VEC>
__device__ __forceinline__ void fuse_apply(uint32_t op, const float (&a)[VEC], const float (&b)[VEC], float (&r)[VEC], const uint32_t (&payload)[2]) {
    if (__builtin_expect(is_long_op(op), 0)) fuse_switch<VEC, true>(op, a, b, r, payload);
    else fuse_switch<VEC, false>(op, a, b, r, payload);
}

// A command of the chain from LDS into scalar registers: whole 16-byte pieces read back to back (one LDS latency for
// the lot, where field-by-field reads behind branches cost one each) and made uniform, so that the branches and the
// address arithmetic on its fields run on the scalar unit.
template <class S>
__device__ __forceinline__ S lds_uniform(const void* p) {
    constexpr int N = (sizeof(S) + 15) / 16;      // (the source is readable up to the next multiple of 16 bytes)
    typedef uint32_t Piece __attribute__((ext_vector_type(4)));
    Piece q[N];
#pragma unroll
    for (int i = 0; i < N; ++i) q[i] = ((const Piece*)p)[i];
    uint32_t w[N * 4];
#pragma unroll
    for (int i = 0; i < N; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) w[i * 4 + e] = (uint32_t)__builtin_amdgcn_readfirstlane((int)q[i][e]);
    S s;
    __builtin_memcpy((void*)&s, w, sizeof(S));
    return s;
}

}  // namespace mxh
