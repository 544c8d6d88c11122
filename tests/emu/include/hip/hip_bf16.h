// Stands in for the HIP header of the same name in the host build of the kernels (../../wave_emu.h).
#pragma once
#include "../../wave_emu.h"
