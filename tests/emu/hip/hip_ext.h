// Stands in for the HIP header of the same name when the kernels are built for the CPU emulation.
#pragma once
#include "../emu.h"
