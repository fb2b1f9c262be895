// Wave64 emulator for the host: test infrastructure, never loaded by the library or its Python layer.
//
// The kernel sources under flashck_amd/csrc are compiled unchanged as C++ for the host.  Every thread of a workgroup runs
// as a fiber (a stack of its own, switched cooperatively); an instruction that exchanges data between the lanes of a
// wave (MFMA, lane permutes, readlane, ballot, the transposing LDS read) is a rendezvous of the wave's 64 fibers, and
// __syncthreads a rendezvous of the workgroup.  Loads into LDS complete at once, so what this cannot show is a missing
// wait on an asynchronous load or a race between waves; what it does show is every index, swizzle, mask, table lookup
// and arithmetic step of the kernels, against the same oracle the GPU tests use.
#pragma once

#include <math.h>
#include <stddef.h>
#include <stdio.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include <cmath>
#include <functional>
#include <typeinfo>
#include <type_traits>

// ---- language keywords ------------------------------------------------------------------------------------------------
#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))
// statically sized LDS variables: one instance per kernel is enough, workgroups run one after the other
#define __shared__ static

struct dim3 {
    unsigned x, y, z;
    constexpr dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};

// ---- runtime API subset -----------------------------------------------------------------------------------------------
typedef void* hipStream_t;
enum hipError_t { hipSuccess = 0, hipErrorInvalidValue = 1, hipErrorInvalidDevice = 101, hipErrorLaunchFailure = 719 };
enum hipFuncAttribute { hipFuncAttributeMaxDynamicSharedMemorySize = 8 };
struct hipDeviceProp_t {
    int multiProcessorCount;
};
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
// 256 compute units as on the real device; EMU_NUM_CU=<n> emulates a smaller chip, on which the small problems of the
// tests "fill the chip" and take the branches the launchers keep for that (head pairs, longest-first dealing, wide
// combine workgroups) without being asked to
inline hipError_t hipGetDeviceProperties(hipDeviceProp_t* p, int)
{
    const char* e = getenv("EMU_NUM_CU");
    p->multiProcessorCount = e && atoi(e) > 0 ? atoi(e) : 256;
    return hipSuccess;
}
inline hipError_t hipFuncSetAttribute(const void*, hipFuncAttribute, int) { return hipSuccess; }
inline hipError_t hipGetSymbolAddress(void** p, const void* sym) { *p = const_cast<void*>(sym); return hipSuccess; }
#define HIP_SYMBOL(x) (&(x))
inline const char* hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : "emulated launch failed"; }

namespace emu {

// A global -> LDS copy a lane has requested and that has not landed yet (see late_loads()).
struct PendingCopy {
    char* dst;
    const char* src;
};

struct Lane {
    dim3 tid;  // threadIdx of the fiber that is running
    dim3 bid, bdim, gdim;
    int lane, wave;
    PendingCopy pending[256];  // FIFO: vector-memory operations complete in order
    int pending_head, pending_count;
    unsigned requests;  // global -> LDS requests this lane has made so far (real or masked)
};
extern thread_local Lane* cur;

// last launch failed (a kernel broke a rule of the emulator: see emu_runtime.cpp); cleared by the read
hipError_t take_error();
void launch(dim3 grid, dim3 block, size_t lds_bytes, const std::function<void()>& body);
// EMU_COVERAGE=<file>: the first launch of every kernel instantiation in a process appends the mangled name of
// KernelTag<&kernel<...>> to the file (c++filt turns it into the instantiation): what a test run has launched.
template <auto Kernel>
struct KernelTag {};
void note_launch(const char* tag);
// How the asynchronous global -> LDS copies are modelled.  true (default): a copy lands at the LAST moment the
// program allows - when the lane that requested it waits for its outstanding copies to drop below the copy's place in
// the queue, or when the lane ends - so a read that is not covered by the proper wait sees stale (poisoned) LDS and the
// parity test fails.  false (EMU_LATE_LOADS=0): copies land at once, the earliest moment, which is what exposes a
// request into a buffer that is still being read.
bool late_loads();
// the lane's part of one global -> LDS instruction: 16 bytes from src to dst
void request_copy(char* dst, const char* src);
// leave at most `keep` of the lane's copies outstanding (the oldest land first)
void land_copies(int keep);
char* dynamic_lds();
void barrier();
// Rendezvous of the wave: deposits n <= 256 bytes, returns when every live lane of the wave has deposited; the
// result points at 64 slots of 256 bytes (slot i = lane i), valid until the lane's next rendezvous.
const char* exchange(const void* mine, size_t n);

template <typename T>
inline T lane_value(const char* all, int lane)
{
    T v;
    memcpy(&v, all + (size_t)lane * 256, sizeof(T));
    return v;
}

}  // namespace emu

inline hipError_t hipGetLastError() { return emu::take_error(); }
#define hipLaunchKernelGGL(kern, grid, block, lds, stream, ...) \
    (emu::note_launch(typeid(emu::KernelTag<kern>).name()), emu::launch((grid), (block), (lds), [=]() { kern(__VA_ARGS__); }))

#define threadIdx (emu::cur->tid)
#define blockIdx (emu::cur->bid)
#define blockDim (emu::cur->bdim)
#define gridDim (emu::cur->gdim)
#define __syncthreads() emu::barrier()

// ---- device library functions -----------------------------------------------------------------------------------------
template <typename A, typename B>
constexpr typename std::common_type<A, B>::type min(A a, B b)
{
    typedef typename std::common_type<A, B>::type C;
    return (C)b < (C)a ? (C)b : (C)a;
}
template <typename A, typename B>
constexpr typename std::common_type<A, B>::type max(A a, B b)
{
    typedef typename std::common_type<A, B>::type C;
    return (C)a < (C)b ? (C)b : (C)a;
}
inline float __expf(float x) { return expf(x); }
inline int atomicAdd(int* p, int v) { return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); }
inline int atomicMin(int* p, int v)
{
    const int old = *p;  // fibers switch only at a rendezvous: nothing runs between the read and the write
    if (v < old) *p = v;
    return old;
}

// ---- target builtins ----------------------------------------------------------------------------------------------------
typedef float emu_f32x2 __attribute__((ext_vector_type(2)));
typedef float emu_f32x4 __attribute__((ext_vector_type(4)));
typedef float emu_f32x16 __attribute__((ext_vector_type(16)));
typedef short emu_s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 emu_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 emu_f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 emu_f16x4 __attribute__((ext_vector_type(4)));

namespace emu {

inline float bf16_bits_to_f32(uint16_t b)
{
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
inline float f16_bits_to_f32(uint16_t b)
{
    _Float16 h;
    memcpy(&h, &b, 2);
    return (float)h;
}

// D = A.B + C for one MFMA shape.  Operand layout (lane l, element j of the lane's E packed values):
//   A[i][k], B[k][n]:  i (or n) = l % M,  k = (l / M) * E + j
//   C/D[i][n]:         n = l % M,  i = (v / 4) * (4 * 64 / M) + (l / M) * 4 + v % 4   for accumulator register v
// (M = 32: 16 registers, rows (v/4)*8 + (l/32)*4 + v%4;  M = 16: 4 registers, rows (l/16)*4 + v)
template <int M, int E, bool kBf16, typename Acc>
inline Acc mfma(const void* a_bits, const void* b_bits, Acc c)
{
    struct Ops {
        uint16_t a[E], b[E];
    } mine;
    memcpy(mine.a, a_bits, E * 2);
    memcpy(mine.b, b_bits, E * 2);
    const char* all = exchange(&mine, sizeof(mine));
    const int l = cur->lane;
    const int n = l % M;
    constexpr int G = 64 / M;                       // lane groups along k
    constexpr int NV = M * M / 64;                  // accumulator registers
    Acc d = c;
    if (getenv("EMU_TRACE_NAN")) {
        static int reported = 0;
        for (int j = 0; j < E && reported < 8; ++j) {
            const float x = kBf16 ? bf16_bits_to_f32(mine.a[j]) : f16_bits_to_f32(mine.a[j]);
            const float y = kBf16 ? bf16_bits_to_f32(mine.b[j]) : f16_bits_to_f32(mine.b[j]);
            if (x != x || y != y) {
                ++reported;
                fprintf(stderr, "emu: NaN operand in mfma<%d,%d> lane %d wave %d block %u: a=%g b=%g (element %d)\n", M, E, l, cur->wave, cur->bid.x, x, y, j);
            }
        }
    }
    for (int v = 0; v < NV; ++v) {
        const int i = (v / 4) * (4 * G) + (l / M) * 4 + v % 4;
        float acc = 0.f;
        for (int kg = 0; kg < G; ++kg) {
            const Ops oa = lane_value<Ops>(all, kg * M + i);
            const Ops ob = lane_value<Ops>(all, kg * M + n);
            for (int j = 0; j < E; ++j) {
                const float x = kBf16 ? bf16_bits_to_f32(oa.a[j]) : f16_bits_to_f32(oa.a[j]);
                const float y = kBf16 ? bf16_bits_to_f32(ob.b[j]) : f16_bits_to_f32(ob.b[j]);
                acc += x * y;
            }
        }
        d[v] = c[v] + acc;
    }
    return d;
}

inline int readlane(int x, int i) { return lane_value<int>(exchange(&x, 4), i & 63); }
int readfirstlane(int x);
uint64_t ballot(bool p);

}  // namespace emu

#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) emu::mfma<32, 8, true, emu_f32x16>(&(a), &(b), (c))
#define __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, x, y, z) emu::mfma<32, 8, false, emu_f32x16>(&(a), &(b), (c))
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, x, y, z) emu::mfma<16, 8, true, emu_f32x4>(&(a), &(b), (c))
#define __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, x, y, z) emu::mfma<16, 8, false, emu_f32x4>(&(a), &(b), (c))
#define __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, x, y, z) emu::mfma16k16_(true, (a), (b), (c))
#define __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, x, y, z) emu::mfma16k16_(false, (a), (b), (c))

namespace emu {
template <typename V>
inline emu_f32x4 mfma16k16_(bool bf16, V a, V b, emu_f32x4 c)
{
    return bf16 ? mfma<16, 4, true, emu_f32x4>(&a, &b, c) : mfma<16, 4, false, emu_f32x4>(&a, &b, c);
}
// ds_read_tr16_b64: within each group of 16 lanes, lane i receives, for k = 0..3, element i % 4 of the 8 bytes that
// lane 4k + i / 4 of the group addressed
inline emu_s16x4 ds_read_tr16(const void* p)
{
    const char* all = exchange(&p, sizeof(p));
    const int l = cur->lane, base = l & ~15, i = l & 15;
    emu_s16x4 r;
    for (int k = 0; k < 4; ++k) {
        const char* src = lane_value<const char*>(all, base + 4 * k + i / 4);
        short e;
        memcpy(&e, src + (i % 4) * 2, 2);
        r[k] = e;
    }
    return r;
}
// OCP e4m3 -> fp32 (no infinities; S.1111.111 is NaN)
inline float e4m3_to_f32(uint8_t b)
{
    const int s = b >> 7, e = (b >> 3) & 15, m = b & 7;
    float v;
    if (e == 15 && m == 7)
        v = NAN;
    else if (e == 0)
        v = ldexpf((float)m, -9);
    else
        v = ldexpf((float)(8 + m), e - 10);
    return s ? -v : v;
}
// fp32 -> e4m3, round to nearest even by search over the 127 positive finite codes (ties go to the even code, which
// for adjacent codes is the even mantissa); beyond the largest finite value and for NaN / inf: NaN
inline uint8_t f32_to_e4m3(float f)
{
    const uint8_t sign = std::signbit(f) ? 0x80 : 0;
    const float a = fabsf(f);
    if (!(a == a) || std::isinf(a)) return sign | 0x7f;
    if (a >= 464.f) return sign | 0x7f;  // rounds past 448: not representable without saturation
    int best = 0;
    float best_err = a;  // code 0 = zero
    for (int c = 1; c <= 0x7e; ++c) {
        const float err = fabsf(e4m3_to_f32((uint8_t)c) - a);
        if (err < best_err || (err == best_err && (c & 1) == 0)) {
            best = c;
            best_err = err;
        }
    }
    return sign | (uint8_t)best;
}
inline int cvt_pk_fp8_f32(float a, float b, int old, bool hi)
{
    const uint32_t two = (uint32_t)f32_to_e4m3(a) | ((uint32_t)f32_to_e4m3(b) << 8);
    const uint32_t o = (uint32_t)old;
    return (int)(hi ? ((o & 0xffffu) | (two << 16)) : ((o & 0xffff0000u) | two));
}
inline emu_f32x2 cvt_pk_f32_fp8(int v, bool hi)
{
    const uint32_t u = (uint32_t)v >> (hi ? 16 : 0);
    return emu_f32x2{e4m3_to_f32(u & 255), e4m3_to_f32((u >> 8) & 255)};
}
}  // namespace emu

#define __builtin_amdgcn_ds_read_tr16_b64_v4i16(p) emu::ds_read_tr16((const void*)(p))
#define __builtin_amdgcn_readlane(x, i) emu::readlane((int)(x), (i))
#define __builtin_amdgcn_readfirstlane(x) emu::readfirstlane((int)(x))
#define __builtin_amdgcn_ballot_w64(p) emu::ballot(p)
#define __ballot(p) emu::ballot(p)
#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __builtin_amdgcn_s_setprio(x) ((void)0)
#define __builtin_amdgcn_s_waitcnt(x) ((void)0)
#define __builtin_amdgcn_fence(order, scope) __atomic_thread_fence(__ATOMIC_SEQ_CST)
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_logf(x) log2f(x)
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))
#define __builtin_amdgcn_cvt_pk_f32_fp8(v, hi) emu::cvt_pk_f32_fp8((v), (hi))
#define __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, hi) emu::cvt_pk_fp8_f32((a), (b), (old), (hi))
#define __HIP_MEMORY_SCOPE_AGENT 0
#define __hip_atomic_fetch_add(p, v, order, scope) __atomic_fetch_add((p), (v), __ATOMIC_SEQ_CST)
