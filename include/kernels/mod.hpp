#pragma once

#include "kernels/b2b_gemm.hpp"
#include "kernels/flash_attn.hpp"
#include "kernels/gemm.hpp"
#include "kernels/lstm.hpp"
#include "kernels/scatter_nd.hpp"
