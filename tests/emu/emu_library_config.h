// Forced into every translation unit of libhomcomp_emu.so: the size of the array that stands for
// dynamic LDS (four waves of the library's largest budget).
#pragma once
#define EMU_DYN_LDS (4 * 2 * (8192 + 64))
