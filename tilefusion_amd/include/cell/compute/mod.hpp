// Umbrella header of the compute primitives.
// The list of headers and their names follow microsoft/TileFusion (MIT License,
// Copyright (c) Microsoft Corporation), include/cell/compute/mod.hpp;
// everything they include is written for gfx950.
#pragma once

#include "cell/compute/broadcast.hpp"
#include "cell/compute/gemm.hpp"
#include "cell/compute/map.hpp"
#include "cell/compute/math_functor.hpp"
#include "cell/compute/reduce.hpp"
