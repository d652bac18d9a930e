// Fixed-width vector moves between memory and per-lane register arrays.
#pragma once

#include "config.hpp"

namespace tiledcuda::cell::copy {

template <int kBytes>
struct VecOf;
template <>
struct VecOf<2> { using type = unsigned short; };
template <>
struct VecOf<4> { using type = unsigned; };
template <>
struct VecOf<8> { using type = u32x2; };
template <>
struct VecOf<16> { using type = u32x4; };

/// Copy kN contiguous elements memory -> registers with one access of kN*sizeof(T) bytes.
/// `src` must be aligned to the access width.
template <int kN, typename T>
DEVICE void vec_load(const T* src, T* dst) {
    using V = typename VecOf<kN * sizeof(T)>::type;
    V v = *reinterpret_cast<const V*>(src);
    __builtin_memcpy(dst, &v, sizeof(V));
}

/// Copy kN contiguous elements registers -> memory with one access.
template <int kN, typename T>
DEVICE void vec_store(const T* src, T* dst) {
    using V = typename VecOf<kN * sizeof(T)>::type;
    V v;
    __builtin_memcpy(&v, src, sizeof(V));
    *reinterpret_cast<V*>(dst) = v;
}

/// The same with a non-temporal store: the data is streamed to memory instead of staying dirty in the XCD's L2 until
/// the kernel's end (whole lines written by neighbouring lanes only: pieces of lines are better gathered by the L2).
template <int kN, typename T>
DEVICE void vec_store_stream(const T* src, T* dst) {
    using V = typename VecOf<kN * sizeof(T)>::type;
    V v;
    __builtin_memcpy(&v, src, sizeof(V));
    __builtin_nontemporal_store(v, reinterpret_cast<V*>(dst));
}

}  // namespace tiledcuda::cell::copy
