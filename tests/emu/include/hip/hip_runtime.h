// Stands in for <hip/hip_runtime.h> when the flash-attention sources are compiled for the host
// (see ../../wave_emu.h): test infrastructure, never part of the GPU build.
#pragma once
#include "../../wave_emu.h"
