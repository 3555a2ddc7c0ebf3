// LDS access by absolute byte address and asynchronous global -> LDS copies, shared by the
// row-batch kernels that stage their operands (prefill.hip, rows_q4k.hip). The kernels that use
// these place their dynamic LDS block at address 0 and check that they got it.
#pragma once
#include "common.hpp"

namespace yvex {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

__device__ __forceinline__ void lds_write_uint4(unsigned address, uint4 v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    *reinterpret_cast<__attribute__((address_space(3))) uint4 *>(address) = v;
#else
    (void)address;
    (void)v;
#endif
}
__device__ __forceinline__ void lds_write_uint2(unsigned address, uint2 v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    *reinterpret_cast<__attribute__((address_space(3))) uint2 *>(address) = v;
#else
    (void)address;
    (void)v;
#endif
}
__device__ __forceinline__ void lds_write_u32(unsigned address, unsigned v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    *reinterpret_cast<__attribute__((address_space(3))) unsigned *>(address) = v;
#else
    (void)address;
    (void)v;
#endif
}
__device__ __forceinline__ void lds_write_u16(unsigned address, unsigned v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    *reinterpret_cast<__attribute__((address_space(3))) unsigned short *>(address) = (unsigned short)v;
#else
    (void)address;
    (void)v;
#endif
}
// One 16-byte LDS read as a vector value (a struct of four words may reach the backend as four
// scalar loads and come out as two 8-byte reads).
__device__ __forceinline__ v4i lds_read_v4i(unsigned address)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return *reinterpret_cast<__attribute__((address_space(3))) const v4i *>(address);
#else
    (void)address;
    return v4i{0, 0, 0, 0};
#endif
}
__device__ __forceinline__ unsigned lds_read_u16(unsigned address)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return *reinterpret_cast<__attribute__((address_space(3))) const unsigned short *>(address);
#else
    (void)address;
    return 0u;
#endif
}
__device__ __forceinline__ unsigned lds_read_u32(unsigned address)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return *reinterpret_cast<__attribute__((address_space(3))) const unsigned *>(address);
#else
    (void)address;
    return 0u;
#endif
}

// The copies below write m0. The compiler reserves m0 and reloads it before every use of its
// own, but it may merge two of its own loads of the same value across code that sits between
// them; naming m0 as written by the assembly keeps it from doing that across a copy. It answers
// the clobber with a diagnostic about reserved registers, silenced here.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"

// Asynchronous copy global -> LDS (GLOBAL_LOAD_LDS): lane l of the wave writes `bytes` bytes at
// lds_base + l * bytes; nothing passes through registers. Written as assembly so the compiler
// does not put a conservative wait in front of every later LDS read: the kernel waits with
// vmcnt(0) (loads retire in order, so the compiler's own counted waits stay correct) before
// the barrier that publishes the data.
__device__ __forceinline__ void copy_to_lds_16(const void *global, unsigned lds_base)
{
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :: "s"(lds_base), "v"(global) : "memory", "m0");   // (m0 named: a value the compiler keeps there is reloaded)
#else
    (void)global;
    (void)lds_base;
#endif
}
__device__ __forceinline__ void copy_to_lds_4(const void *global, unsigned lds_base)
{
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off"
                 :: "s"(lds_base), "v"(global) : "memory", "m0");   // (m0 named: a value the compiler keeps there is reloaded)
#else
    (void)global;
    (void)lds_base;
#endif
}

// A workgroup barrier that orders LDS traffic only. __syncthreads() also waits for every global
// load and store the compiler knows to be in flight (a kernel's output stores among them: their
// acknowledgement takes as long as a load), which a barrier between two users of an LDS region
// has no need of.
__device__ __forceinline__ void lds_barrier()
{
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#endif
}

// The same 16-byte copy for lanes 0-31 only (the other lanes neither read nor write).
__device__ __forceinline__ void copy_to_lds_16_first32(const void *global, unsigned lds_base)
{
#if defined(__HIP_DEVICE_COMPILE__)
    unsigned long long saved;
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b32 exec_hi, 0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %2, off\n\ts_mov_b64 exec, %0"
                 : "=&s"(saved) : "s"(lds_base), "v"(global) : "memory", "m0");
#else
    (void)global;
    (void)lds_base;
#endif
}

#pragma clang diagnostic pop

}  // namespace yvex
