// Umbrella header of the tile types (counterpart of include/types/mod.hpp:6-16).
#pragma once

#include "types/base.hpp"
#include "types/base_tile.hpp"
#include "types/global.hpp"
#include "types/global_tile_iterator.hpp"
#include "types/layout.hpp"
#include "types/packing.hpp"
#include "types/register.hpp"
#include "types/shared.hpp"
#include "types/shared_tile_iterator.hpp"
#include "types/swizzle.hpp"
#include "types/tile_shape.hpp"
