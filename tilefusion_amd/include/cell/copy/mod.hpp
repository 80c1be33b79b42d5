// Umbrella header of the copy primitives.
// The list of headers and their names follow microsoft/TileFusion (MIT License,
// Copyright (c) Microsoft Corporation), include/cell/copy/mod.hpp:6-14;
// everything they include is written for gfx950.
#pragma once

#include "cell/copy/constants.hpp"
#include "cell/copy/copy_atom.hpp"
#include "cell/copy/global_to_register.hpp"
#include "cell/copy/global_to_shared.hpp"
#include "cell/copy/register.hpp"
#include "cell/copy/shared_to_register.hpp"
#include "cell/copy/sync.hpp"
#include "cell/copy/vectorize.hpp"
#include "cell/copy/warp.hpp"
