// Host-side helpers. Replaces the reference's include/cuda_utils.hpp:15-47
// (CeilDiv, CudaCheck). Unlike the reference's check, a failed HIP call throws
// instead of calling exit(): the C-ABI layer turns it into a status code.
#pragma once

#include "config.hpp"

#include <sstream>
#include <stdexcept>

namespace tiledcuda {

template <int a, int b>
inline constexpr int CeilDiv = (a + b - 1) / b;

HOST_DEVICE constexpr int ceil_div(int a, int b) { return (a + b - 1) / b; }

inline void hip_check_impl(hipError_t code, const char* file, int line) {
    if (code != hipSuccess) {
        std::ostringstream ss;
        ss << "HIP error " << static_cast<int>(code) << " (" << hipGetErrorString(code) << ") at " << file << ":"
           << line;
        throw std::runtime_error(ss.str());
    }
}

#define HipCheck(call) ::tiledcuda::hip_check_impl((call), __FILE__, __LINE__)

}  // namespace tiledcuda
