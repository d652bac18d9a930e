// Debug predicates; same names as the reference's util/debug.hpp:9-30.
#pragma once

#include "config.hpp"

namespace tiledcuda {

DEVICE bool block(int bid) {
    int id = blockIdx.x + blockIdx.y * gridDim.x + blockIdx.z * gridDim.x * gridDim.y;
    return id == bid;
}

DEVICE bool thread(int tid, int bid) {
    int id = threadIdx.x + threadIdx.y * blockDim.x + threadIdx.z * blockDim.x * blockDim.y;
    return id == tid && block(bid);
}

DEVICE bool thread(int tid) { return thread(tid, 0); }
DEVICE bool thread0() { return thread(0, 0); }
DEVICE bool block0() { return block(0); }

}  // namespace tiledcuda
