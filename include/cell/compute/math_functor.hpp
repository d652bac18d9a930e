// Scalar functors used by the element-wise, broadcast and reduce templates.
// Same functor names and call shapes as the reference's
// include/cell/compute/math_functor.hpp:7-176.
#pragma once

#include <type_traits>

#include "config.hpp"

namespace tiledcuda::cell::compute {

namespace detail {
DEVICE float to_f32(float v) { return v; }
DEVICE float to_f32(__half v) { return __half2float(v); }
template <typename T>
DEVICE T from_f32(float v) {
    if constexpr (std::is_same_v<T, float>) return v; else return __float2half(v);
}
}  // namespace detail

#define TCU_BINARY_FUNCTOR(Name, expr)                                                          \
    template <typename Element>                                                                  \
    struct Name {                                                                                \
        DEVICE Element operator()(Element a, Element b) const { return (expr); }                 \
        DEVICE void operator()(const Element& a, const Element& b, Element& dst) { dst = (expr); } \
    }

TCU_BINARY_FUNCTOR(Add, a + b);
TCU_BINARY_FUNCTOR(Sub, a - b);
TCU_BINARY_FUNCTOR(Mul, a * b);
TCU_BINARY_FUNCTOR(Div, a / b);
TCU_BINARY_FUNCTOR(Max, a > b ? a : b);
TCU_BINARY_FUNCTOR(Min, a < b ? a : b);
#undef TCU_BINARY_FUNCTOR

template <typename Element>
struct Exp {
    DEVICE Element operator()(Element a) const { return detail::from_f32<Element>(__expf(detail::to_f32(a))); }
    DEVICE void operator()(const Element& src, Element& dst) { dst = (*this)(src); }
};

template <>
struct Exp<__half> {
    DEVICE __half operator()(__half a) const { return hexp(a); }
    DEVICE void operator()(const __half& src, __half& dst) { dst = hexp(src); }
};

template <typename Element>
struct Log {
    DEVICE Element operator()(Element a) const { return detail::from_f32<Element>(__logf(detail::to_f32(a))); }
    DEVICE void operator()(const Element& src, Element& dst) { dst = (*this)(src); }
};

template <>
struct Log<__half> {
    DEVICE __half operator()(__half a) const { return hlog(a); }
    DEVICE void operator()(const __half& src, __half& dst) { dst = hlog(src); }
};

template <typename Element>
struct Relu {
    DEVICE Element operator()(Element a) const { return a > Element(0.f) ? a : Element(0.f); }
    DEVICE void operator()(const Element& src, Element& dst) { dst = (*this)(src); }
};

template <typename SrcElement, typename DstElement>
struct Convert {
    DEVICE DstElement operator()(SrcElement a) const { return detail::from_f32<DstElement>(detail::to_f32(a)); }
    DEVICE void operator()(const SrcElement& src, DstElement& dst) { dst = (*this)(src); }
};

/// 2^x as ONE v_exp_f32, no range fix-ups (arguments of a softmax in the log2 domain are bounded above, and results
/// below 2^-126 may flush to zero): the transcendental that hides under a matrix instruction of the same wavefront.
template <typename Element>
struct Exp2Raw {
    static_assert(std::is_same_v<Element, float>);
    DEVICE float operator()(float a) const { return __builtin_amdgcn_exp2f(a); }
    DEVICE void operator()(const float& src, float& dst) { dst = __builtin_amdgcn_exp2f(src); }
};

/// Two f32 -> two adjacent 2-byte elements at dst (round to nearest even), as one v_cvt_pk_f16_f32 issued WHERE IT IS
/// WRITTEN: left to the compiler, the conversions of a whole step of a scheduled kernel sink to their first use and run
/// as one block that no matrix instruction hides. The sources may be results of v_exp_f32: at least one other
/// instruction must have been issued since (in a scheduled kernel a matrix instruction is).
DEVICE void convert_pair_here(float a, float b, __half* dst) {
    unsigned int r;
    asm volatile("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    __builtin_memcpy(dst, &r, sizeof(r));
}

}  // namespace tiledcuda::cell::compute
