// Static shape tuple, `dim_size` and the slicing placeholder `_`.
// Same surface as the reference's include/types/tile_shape.hpp:8-28, without CuTe.
#pragma once

#include "config.hpp"

#include <array>
#include <cstddef>
#include <cstdint>

namespace tiledcuda::cell {

template <size_t... Ns>
struct TileShape {
    static constexpr size_t kRank = sizeof...(Ns);
    static constexpr std::array<size_t, sizeof...(Ns)> shape = {Ns...};

    static constexpr size_t get_numel() {
        size_t product = 1;
        for (size_t n : shape) product *= n;
        return product;
    }

    static constexpr size_t kNumel = get_numel();
};

template <typename TileShape>
inline constexpr int64_t get_numel = TileShape::kNumel;

template <const size_t I, typename TileShape>
inline constexpr size_t dim_size = TileShape::shape[I];

struct Underscore {};                   // placeholder type for slicing
inline constexpr Underscore _ = {};     // usable on host and device

}  // namespace tiledcuda::cell
