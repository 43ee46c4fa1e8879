#pragma once
// Kept so that sources written against the reference layout keep compiling:
// every device entry point of this name lives in gpu.hpp.
#include "gpu.hpp"
