// Scalar functors used by the element-wise, broadcast and reduce templates.
// Same functor names and call shapes as the reference's
// include/cell/compute/math_functor.hpp:7-176.
#pragma once

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

}  // namespace tiledcuda::cell::compute
