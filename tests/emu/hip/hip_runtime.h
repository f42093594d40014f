// Stand-in for <hip/hip_runtime.h> in the host build of the library's source (tests/emu): the
// includes of the HIP runtime land here.
#pragma once
#include "../emu_runtime.hpp"
