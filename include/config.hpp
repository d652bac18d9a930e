// Platform macros for the gfx950 (CDNA4) build.
// Replaces the reference's include/config.hpp:3-11 (HOST_DEVICE / DEVICE / HOST).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#define HOST_DEVICE __forceinline__ __host__ __device__
#define DEVICE __forceinline__ __device__
#define HOST inline

namespace tiledcuda {

// A wavefront on CDNA4 is 64 lanes wide; every "warp" of the tile API is one wavefront.
inline constexpr int kWaveSize = 64;

// LDS budget per workgroup on gfx950 (160 KiB per CU).
inline constexpr int kMaxLdsBytes = 160 * 1024;

// Vector register types used to talk to the MFMA / LDS builtins.
using f16x4 = _Float16 __attribute__((ext_vector_type(4)));
using f16x8 = _Float16 __attribute__((ext_vector_type(8)));
using f32x4 = float __attribute__((ext_vector_type(4)));
using f32x16 = float __attribute__((ext_vector_type(16)));
using u32x2 = unsigned __attribute__((ext_vector_type(2)));
using u32x4 = unsigned __attribute__((ext_vector_type(4)));
using u32x16 = unsigned __attribute__((ext_vector_type(16)));

DEVICE int lane_id() { return static_cast<int>(threadIdx.x) & (kWaveSize - 1); }
DEVICE int wave_id() { return static_cast<int>(threadIdx.x) >> 6; }

}  // namespace tiledcuda
