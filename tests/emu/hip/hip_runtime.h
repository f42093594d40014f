// Stand-in for <hip/hip_runtime.h> in the host build of the kernels' logic (tests/emu): the
// device code's include of the HIP runtime lands here.
#pragma once
#include "../amdgcn_emu.hpp"
