// Cross-lane primitives. Same names as the reference's include/cell/warp.hpp:13-26
// (shuffle_sync / shuffle_down_sync), 64 lanes wide; plus the XOR butterfly the reductions
// over a BaseTile row use (a row is spread over lanes l, l^16, l^32, l^48).
#pragma once

#include "config.hpp"

namespace tiledcuda::cell {

constexpr unsigned long long MASK_ALL = 0xFFFFFFFFFFFFFFFFull;

DEVICE float shuffle_sync(unsigned long long, float value, int src_lane) { return __shfl(value, src_lane, kWaveSize); }
DEVICE float shuffle_down_sync(unsigned long long, float value, int delta) { return __shfl_down(value, delta, kWaveSize); }
DEVICE float shuffle_xor(float value, int mask) { return __shfl_xor(value, mask, kWaveSize); }

DEVICE __half shuffle_sync(unsigned long long, __half value, int src_lane) {
    return __float2half(__shfl(__half2float(value), src_lane, kWaveSize));
}
DEVICE __half shuffle_down_sync(unsigned long long, __half value, int delta) {
    return __float2half(__shfl_down(__half2float(value), delta, kWaveSize));
}
DEVICE __half shuffle_xor(__half value, int mask) {
    return __float2half(__shfl_xor(__half2float(value), mask, kWaveSize));
}

}  // namespace tiledcuda::cell
