#pragma once

#include "cell/compute/mod.hpp"
#include "cell/copy/mod.hpp"
#include "cell/sync.hpp"
#include "cell/traits/base.hpp"
#include "cell/warp.hpp"
#include "types/mod.hpp"
