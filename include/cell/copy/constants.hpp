// Enumerations of the copy layer. WarpReuse keeps the reference's names and values
// (include/cell/copy/constants.hpp:14-26); a "warp" is a 64-lane wavefront here.
// CopyInst names the gfx950 instructions the loaders map to instead of ldmatrix/stmatrix.
#pragma once

#include "config.hpp"

namespace tiledcuda::cell::copy {

enum class CopyInst {
    kLdsRead64 = 0,      // ds_read_b64: one 4 x f16 BaseTile share per lane
    kLdsRead128 = 1,     // ds_read_b128: one 4 x f32 BaseTile share (or two K-adjacent f16 shares)
    kLdsWrite64 = 2,     // ds_write_b64
    kLdsWrite128 = 3,    // ds_write_b128
    kGlobalLoad128 = 4,  // global_load_dwordx4 (coalesced 16 B per lane)
    kLdsReadTr16 = 5     // ds_read_b64_tr_b16: transposing LDS read
};

enum class WarpReuse {
    kCont = 0,          // the tile is split evenly over all wavefronts, no reuse
    kCir = 1,           // circular split, no reuse (not implemented, as in the reference)
    kRowReuseCont = 2,  // wavefronts of one wavefront-row load the same rows (operand A)
    kRowReuseCir = 3,   // (not implemented)
    kColReuseCont = 4,  // wavefronts of one wavefront-column load the same columns (operand B)
    kColReuseCir = 5    // (not implemented)
};

}  // namespace tiledcuda::cell::copy
