// Conversions between the plain-number dtypes on the device, with the results of the reference's host conversion
// (crates/maidenx_core/src/buffer/mod.rs:155-196, table :414-560): Rust's `as` between primitives — a float becomes
// the integer obtained by dropping its fraction, clamped to the target's range, NaN becomes 0; an integer becomes the
// nearest float (ties to even); integer to integer keeps the low bits; anything to bool is `!= 0`; bool is 0 or 1.
#pragma once
#include "elementwise.hpp"
#include "ops.hpp"

namespace mxh {

template <class TO, class F> __device__ inline TO float_to_int(F x) {
    using L = std::numeric_limits<TO>;
    if (x != x) return (TO)0;
    const F lo = (F)L::min();                             // 0 or a power of two: exact in F
    const F hi_excl = (F)(L::max() / 2 + 1) * (F)2;       // max + 1, a power of two: exact in F
    if (x <= lo) return L::min();
    if (x >= hi_excl) return L::max();
    return (TO)x;                                         // inside the range: truncation toward zero
}

template <class TI, class TO> struct OpCast {
    using In = TI; using Out = TO; static constexpr int NIN = 1;
    __device__ TO operator()(TI x) const {
        constexpr bool fin = std::is_floating_point<TI>::value, fout = std::is_floating_point<TO>::value;
        if constexpr (std::is_same<TO, b8_t>::value) return b8_t{(uint8_t)(x != (TI)0)};
        else if constexpr (std::is_same<TI, b8_t>::value) return (TO)(x.bits ? 1 : 0);
        else if constexpr (fin && !fout) return float_to_int<TO>(x);
        else return (TO)x;
    }
};

}  // namespace mxh

#define MXH_CAST_WIDE(TI, PI, SI, TO, PO, SO)                                                              \
    extern "C" void hip_cast_##SI##_##SO(size_t n, const PI* in, PO* out) { MXH_API;                       \
        if (!in) { mxh::set_status(mxh::ERR_INVALID, "cast: null input"); return; }                        \
        mxh::ew_unary(n, 1, nullptr, (const TI*)in, (TO*)out, mxh::OpCast<TI, TO>{});                      \
    }
