#pragma once

#include "jit/common.hpp"
#include "jit/compiler.hpp"
#include "jit/config.hpp"
