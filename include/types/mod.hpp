#pragma once

#include "types/global.hpp"
#include "types/global_tile_iterator.hpp"
#include "types/layout.hpp"
#include "types/mfma_tile.hpp"
#include "types/register.hpp"
#include "types/shared.hpp"
#include "types/shared_tile_iterator.hpp"
#include "types/tile_shape.hpp"
#include "util/tile_print.hpp"

namespace tiledcuda::cell {

namespace detail {
template <class Tile, class ChunkShape, bool kShared>
struct TileIteratorSelect { using type = GTileIterator<Tile, ChunkShape>; };
template <class Tile, class ChunkShape>
struct TileIteratorSelect<Tile, ChunkShape, true> { using type = STileIterator<Tile, ChunkShape>; };
}  // namespace detail

/// `TileIterator` (the spelling used in the reference's README.md:70-76): picks the global
/// or the shared iterator from the tile type.
template <class Tile, class ChunkShape>
using TileIterator =
    typename detail::TileIteratorSelect<Tile, ChunkShape, requires { Tile::kSwizzled; }>::type;

}  // namespace tiledcuda::cell
