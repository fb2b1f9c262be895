// Emulated twin of flashck_amd/csrc/gfx950_ops.hpp (test infrastructure): the same names, implemented on the wave64
// emulator instead of inline assembly.  It defines that header's include guard, so the kernel sources, which include
// the real one, get these definitions when they are compiled for the host.
#ifndef FCK_GFX950_OPS_HPP
#define FCK_GFX950_OPS_HPP

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fck {

#define FCK_LDS
#define FCK_CONST
#define FCK_DYNAMIC_LDS(name) char* const name = emu::dynamic_lds()

// the emulated LDS lives below 4 GiB, so its addresses fit the 32 bits the kernels keep them in
inline uint32_t lds_address(const void* p) { return (uint32_t)(uintptr_t)p; }

// v_permlane32_swap: lanes 32..63 of a <-> lanes 0..31 of b, from two copies of x
inline void swap32(float x, float& a, float& b)
{
    const char* all = emu::exchange(&x, 4);
    const int l = emu::cur->lane;
    a = emu::lane_value<float>(all, l & 31);
    b = emu::lane_value<float>(all, (l & 31) + 32);
}
// v_permlane16_swap: odd 16-lane rows of a <-> even rows of b, from two copies of x
inline void swap16(float x, float& a, float& b)
{
    const char* all = emu::exchange(&x, 4);
    const int l = emu::cur->lane;
    a = emu::lane_value<float>(all, l & ~16);
    b = emu::lane_value<float>(all, l | 16);
}

// global -> LDS: lane l copies 16 bytes to byte l * 16 of the 1 KiB block at dst; when the copy lands: emu::late_loads()
inline void load_to_lds(uint32_t dst, const void* base, uint32_t off)
{
    emu::request_copy((char*)(uintptr_t)dst + emu::cur->lane * 16, (const char*)base + off);
}
inline void load_to_lds(uint32_t dst, const void* src) { emu::request_copy((char*)(uintptr_t)dst + emu::cur->lane * 16, (const char*)src); }

// a masked-off lane of an issued instruction: an empty entry in the lane's queue
#define FCK_LOAD_TO_LDS_MASKED() emu::request_copy(nullptr, nullptr)

// the kernels count only their own global -> LDS instructions; so does this
template <int N>
inline void wait_vm()
{
    emu::land_copies(N);
}

#define FCK_ACC_SCALE(acc, f) ((acc) *= (f))
#define FCK_PIN_VGPR(x) ((void)0)
#define FCK_PIN_VGPR4(a, b, c, d) ((void)0)
#define FCK_PIN_SGPR(x) ((void)0)

// lanes run one after the other here: all of them must have made their LDS stores before any goes on to read
#define FCK_WAVE_LDS_ORDER() ((void)emu::exchange("", 1))

inline int const_load(const int32_t* table, int i) { return table[i]; }

}  // namespace fck

#endif  // FCK_GFX950_OPS_HPP
