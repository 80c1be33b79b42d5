// Umbrella header of the tile types.
// The list of headers and their names follow microsoft/TileFusion (MIT License,
// Copyright (c) Microsoft Corporation), include/types/mod.hpp:6-16;
// everything they include is written for gfx950.
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
