// The elementwise functors a recorded program can replay, as a type list: the position of a functor in
// the list is its instantiation number in a program command (low bit: vector or scalar form of ew_nd).
#pragma once
#include <type_traits>

#include "mxh.hpp"

namespace mxh {

template <class T> struct OpAdd;
template <class T> struct OpSub;
template <class T> struct OpMul;
template <class T> struct OpDiv;
template <class T> struct OpMaximum;
template <class T> struct OpMinimum;
template <class T> struct OpLogicalAnd;
template <class T> struct OpLogicalOr;
template <class T> struct OpLogicalXor;
template <class T> struct OpEq;
template <class T> struct OpNe;
template <class T> struct OpLt;
template <class T> struct OpLe;
template <class T> struct OpGt;
template <class T> struct OpGe;
template <class T> struct OpNeg;
template <class T> struct OpAbs;
template <class T> struct OpSign;
template <class T> struct OpSquare;
template <class T> struct OpSqrt;
template <class T> struct OpRelu;
template <class T> struct OpSigmoid;
template <class T> struct OpTanh;
template <class T> struct OpGelu;
template <class T> struct OpSin;
template <class T> struct OpCos;
template <class T> struct OpTan;
template <class T> struct OpLn;
template <class T> struct OpLog10;
template <class T> struct OpLog2;
template <class T> struct OpExp;
template <class T> struct OpExp10;
template <class T> struct OpExp2;
template <class T> struct OpSoftplus;
template <class T> struct OpRecip;
template <class T> struct OpLogicalNot;
template <class T> struct OpAddScalar;
template <class T> struct OpSubScalar;
template <class T> struct OpMulScalar;
template <class T> struct OpDivScalar;
template <class T> struct OpMaximumScalar;
template <class T> struct OpMinimumScalar;
template <class T> struct OpPow;
template <class T> struct OpLeakyRelu;
template <class T> struct OpElu;
template <class T> struct OpEqScalar;
template <class T> struct OpNeScalar;
template <class T> struct OpLtScalar;
template <class T> struct OpLeScalar;
template <class T> struct OpGtScalar;
template <class T> struct OpGeScalar;
template <class T> struct OpFill;
template <class T> struct OpIdentity;
template <class T> struct OpZeroPlus;
template <class T> struct OpSgdStep;
template <class T> struct OpMseGradUnit;

template <class... Ts> struct TypeList { static constexpr int size = (int)sizeof...(Ts); };
template <class T, class L> struct IndexOf;
template <class T> struct IndexOf<T, TypeList<>> { static constexpr int value = -1; };
template <class T, class H, class... R> struct IndexOf<T, TypeList<H, R...>> {
    static constexpr int rest = IndexOf<T, TypeList<R...>>::value;
    static constexpr int value = std::is_same<T, H>::value ? 0 : (rest < 0 ? -1 : rest + 1);
};
template <int I, class L> struct TypeAt;
template <class H, class... R> struct TypeAt<0, TypeList<H, R...>> { using type = H; };
template <int I, class H, class... R> struct TypeAt<I, TypeList<H, R...>> { using type = typename TypeAt<I - 1, TypeList<R...>>::type; };

#define MXH_PROG_EW_OPS(T)                                                                                            \
    OpAdd<T>, OpSub<T>, OpMul<T>, OpDiv<T>, OpMaximum<T>, OpMinimum<T>, OpLogicalAnd<T>, OpLogicalOr<T>,              \
        OpLogicalXor<T>, OpEq<T>, OpNe<T>, OpLt<T>, OpLe<T>, OpGt<T>, OpGe<T>, OpNeg<T>, OpAbs<T>, OpSign<T>,         \
        OpSquare<T>, OpSqrt<T>, OpRelu<T>, OpSigmoid<T>, OpTanh<T>, OpGelu<T>, OpSin<T>, OpCos<T>, OpTan<T>, OpLn<T>, \
        OpLog10<T>, OpLog2<T>, OpExp<T>, OpExp10<T>, OpExp2<T>, OpSoftplus<T>, OpRecip<T>, OpLogicalNot<T>,           \
        OpAddScalar<T>, OpSubScalar<T>, OpMulScalar<T>, OpDivScalar<T>, OpMaximumScalar<T>, OpMinimumScalar<T>,       \
        OpPow<T>, OpLeakyRelu<T>, OpElu<T>, OpEqScalar<T>, OpNeScalar<T>, OpLtScalar<T>, OpLeScalar<T>,               \
        OpGtScalar<T>, OpGeScalar<T>, OpFill<T>, OpIdentity<T>, OpZeroPlus<T>, OpSgdStep<T>, OpMseGradUnit<T>
// f32: the dtype of the small training loops this is for
using EwProgOps = TypeList<MXH_PROG_EW_OPS(float)>;

}  // namespace mxh
