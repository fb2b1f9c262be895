// The gfx950 instructions the kernels use that have no compiler builtin, written as inline assembly, plus the address
// space qualifiers of LDS and constant memory.  Every piece of assembly in the library lives in this file.
#ifndef FCK_GFX950_OPS_HPP
#define FCK_GFX950_OPS_HPP

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fck {

#define FCK_LDS __attribute__((address_space(3)))
#define FCK_CONST __attribute__((address_space(4)))
// the workgroup's dynamic LDS allocation, as a generic pointer named `name`
#define FCK_DYNAMIC_LDS(name) extern __shared__ __attribute__((aligned(16))) char name[]

// LDS byte address of a pointer into the workgroup's allocation (what m0 and the DS instructions take)
__device__ __forceinline__ uint32_t lds_address(const void FCK_LDS* p) { return (uint32_t)(uintptr_t)p; }

// Cross-lane exchange on the VALU (no LDS round trip).
// v_permlane32_swap a, b exchanges lanes 32..63 of a with lanes 0..31 of b; v_permlane16_swap does the same between the
// odd 16-lane rows of a and the even rows of b.  Started from two copies of x they leave (x[l % 32], x[l % 32 + 32]) resp.
// (x[even row of l], x[odd row of l]) in every lane.  The instructions are written as inline assembly because they
// update both operands in place; the s_nop covers the wait states a VALU write needs before a lane permute reads it.
__device__ __forceinline__ void swap32(float x, float& a, float& b)
{
    a = x;
    b = x;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap16(float x, float& a, float& b)
{
    a = x;
    b = x;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}

// One global -> LDS instruction: every lane copies 16 bytes from base + off (base uniform, off per lane, in bytes) to
// the 1 KiB block at LDS address dst (uniform), lane l to byte l*16 of it.  Written as assembly on purpose: a load the
// compiler knows about makes it drain the whole load queue before the next LDS read it cannot prove disjoint, and no
// register is a load destination, so nothing the compiler schedules can wait on these loads by accident.  m0 carries
// the LDS address and is put back afterwards, since the compiler does not expect it to change.
__device__ __forceinline__ void load_to_lds(uint32_t dst, const void* base, uint32_t off)
{
    uint32_t m0_saved;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3\n\ts_mov_b32 m0, %0"
                 : "=&s"(m0_saved)
                 : "s"(dst), "v"(off), "s"(base)
                 : "memory");
}
// the same with a full address per lane
__device__ __forceinline__ void load_to_lds(uint32_t dst, const void* src)
{
    uint32_t m0_saved;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(m0_saved)
                 : "s"(dst), "v"(src)
                 : "memory");
}

// A lane that sits out a global -> LDS instruction which other lanes of its wave issue (it is masked off for that
// instruction): nothing to do on the hardware, where the wave's counter of outstanding operations counts the instruction
// once for all lanes; the emulated twin keeps the lane's own count in step with it.
#define FCK_LOAD_TO_LDS_MASKED() ((void)0)

// wait until at most N of this wave's vector-memory operations are outstanding (they complete in order)
template <int N>
__device__ __forceinline__ void wait_vm()
{
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// acc *= f for a value that lives in the accumulation half of the register file, without moving it out for longer
// than the multiply.  (Macros: elements of the vector types the MFMA builtins use cannot be bound to references.)
#define FCK_ACC_SCALE(acc, f)                                             \
    do {                                                                  \
        float x_;                                                         \
        asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(x_) : "a"(acc));  \
        x_ *= (f);                                                        \
        asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(acc) : "v"(x_)); \
    } while (0)

// Optimisation fences: the value is treated as read and rewritten here, in a vector / scalar register, so the
// instructions that produce it cannot be moved past this point.
#define FCK_PIN_VGPR(x) asm volatile("" : "+v"(x))
#define FCK_PIN_VGPR4(a, b, c, d) asm volatile("" : "+v"(a), "+v"(b), "+v"(c), "+v"(d))
#define FCK_PIN_SGPR(x) asm volatile("" : "+s"(x))

// Marks a point where lanes of one wave read LDS data that other lanes of the same wave wrote before it.  A wave's LDS
// operations execute in order and its lanes run in lockstep, so no instruction is needed and none is emitted (even a
// compiler-only wave barrier here changes the instruction schedule of the streaming loop).
#define FCK_WAVE_LDS_ORDER() ((void)0)

// table[i] through the scalar data path (the table is an input that no kernel writes): the load waits on its own counter
// and does not disturb the queue of vector loads
__device__ __forceinline__ int const_load(const int32_t* table, int i) { return ((const FCK_CONST int32_t*)table)[i]; }

}  // namespace fck

#endif  // FCK_GFX950_OPS_HPP
