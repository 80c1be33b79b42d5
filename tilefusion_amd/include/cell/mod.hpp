// Umbrella header of the cell primitives.
// The list of headers and their names follow microsoft/TileFusion (MIT License,
// Copyright (c) Microsoft Corporation), include/cell/mod.hpp:6-11;
// everything they include is written for gfx950.
#pragma once

#include "cell/compute/mod.hpp"
#include "cell/copy/mod.hpp"
#include "cell/mask.hpp"
#include "cell/pipeline.hpp"
#include "cell/warp.hpp"
