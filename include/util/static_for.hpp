// A loop whose index is a constant expression: f(integral_constant<int, 0>) ... f(integral_constant<int, kN - 1>).
// For kernels that place every instruction themselves: tile coordinates, wait counts and instruction offsets that
// depend on the iteration are template arguments and immediates.
#pragma once

#include <type_traits>
#include <utility>

#include "config.hpp"

namespace tiledcuda {

template <int kN, typename F>
DEVICE void static_for(F&& f) {
    [&]<int... kIs>(std::integer_sequence<int, kIs...>) {
        (f(std::integral_constant<int, kIs>{}), ...);
    }(std::make_integer_sequence<int, kN>{});
}

}  // namespace tiledcuda
