// Row / column softmax of a register tile. Same functor as the reference's
// include/cell/compute/softmax.hpp:27-78 (Softmax<RegTile, kLayout>::operator()(tile, reduce_tile)).
// The reference exponentiates without subtracting the maximum (its header says so); here
// the line maximum is subtracted first, which changes nothing mathematically and removes
// the overflow. `reduce_tile` receives the sum of exponentials per line.
#pragma once

#include "cell/compute/broadcast.hpp"
#include "cell/compute/map.hpp"
#include "cell/compute/reduce.hpp"

namespace tiledcuda::cell::compute {

template <typename RegTile, const tl::Layout kLayout>
struct Softmax {
    using DType = typename RegTile::DType::DType;

    template <typename ReduceTile>
    DEVICE void operator()(RegTile& tile, ReduceTile& reduce_tile) {
        MaxReduce<RegTile, kLayout> line_max;
        line_max(tile, reduce_tile);

        BroadcastSub<ReduceTile, RegTile, kLayout> sub_max;
        sub_max(reduce_tile, tile);

        RegTileExp<RegTile> exp;
        exp(tile, tile);

        SumReduce<RegTile, kLayout> line_sum;
        line_sum(tile, reduce_tile);

        BroadcastDiv<ReduceTile, RegTile, kLayout> div_sum;
        div_sum(reduce_tile, tile);
    }
};

}  // namespace tiledcuda::cell::compute
