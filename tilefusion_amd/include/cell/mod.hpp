// Umbrella header of the cell primitives (counterpart of include/cell/mod.hpp:6-11).
#pragma once

#include "cell/compute/mod.hpp"
#include "cell/copy/mod.hpp"
#include "cell/mask.hpp"
#include "cell/pipeline.hpp"
#include "cell/warp.hpp"
