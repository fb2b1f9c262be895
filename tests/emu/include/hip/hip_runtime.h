// Test infrastructure, not part of the library: the few HIP names the kernel sources and their launchers use, mapped
// onto the wave64 emulator of tests/emu so that the UNCHANGED kernel sources compile for the host.  Only the build of
// tests/emu/libflashck_fmha_emu.so sees this directory; the shipped library is built by hipcc against the real headers.
#pragma once
#include "../../emu_runtime.h"
