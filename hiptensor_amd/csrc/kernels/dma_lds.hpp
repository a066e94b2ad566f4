// Loads from global memory straight into LDS (global_load_lds_*), as inline assembly, and the waits
// that go with them.  Shared by the 16-bit (contract_hd.hpp) and the 32/64-bit (contract_wd.hpp)
// direct-load kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hiptk
{
    // Direct load, in two halves so that another instruction (an MFMA) can sit between the write of
    // M0 and the load that reads it (one wait state is required there):
    //   dma_dst:  M0 <- LDS byte address lds_base + off (wave-uniform)
    //   dma_load: 16 bytes per lane from global memory (base + 32-bit byte offset voff) to LDS address
    //             M0 + 16 * lane (dma_load1: 4 bytes per lane to M0 + 4 * lane).  Counted by vmcnt.
    // Nothing else in these kernels uses M0.  M0 cannot be named in a clobber list (the compiler treats it as a reserved
    // register and warns that clobbering it is undefined), so that nothing the compiler generates between the two halves
    // touches M0 is checked in the device assembly instead (tests/test_kernel_codegen.py).
    // The compiler's hazard recognizer does not look inside inline assembly, so the wait states an
    // instruction needs are provided here: a VMEM instruction must not read an SGPR within 5 wait
    // states of a VALU instruction writing it (the compiler reloads spilled SGPRs with v_readlane,
    // possibly right in front of the asm statement), and M0 needs 1 wait state before the load that
    // reads it: s_nop 4 in front of the load covers both.
    // The operands that must be scalar are passed through readfirstlane: an "s" constraint does not
    // make the compiler move a (wave-uniform) value that it chose to compute in vector registers, and
    // readfirstlane of a value that is in scalar registers already costs nothing.
    __device__ __forceinline__ uint32_t hd_scalar(uint32_t v)
    {
        return (uint32_t)__builtin_amdgcn_readfirstlane((int)v);
    }
    __device__ __forceinline__ const void* hd_scalar(const void* p)
    {
        const uint64_t v = (uint64_t)p;
        return (const void*)(((uint64_t)hd_scalar((uint32_t)(v >> 32)) << 32) | (uint64_t)hd_scalar((uint32_t)v));
    }
    template <int OFF>
    __device__ __forceinline__ void dma_dst(uint32_t lds_base)
    {
        asm volatile("s_add_u32 m0, %0, %1" : : "s"(hd_scalar(lds_base)), "n"(OFF) : "scc");
    }
    __device__ __forceinline__ void dma_dst_at(uint32_t lds_base, uint32_t off)
    {
        asm volatile("s_add_u32 m0, %0, %1" : : "s"(hd_scalar(lds_base)), "s"(hd_scalar(off)) : "scc");
    }
    __device__ __forceinline__ void dma_load(uint32_t voff, const void* base)
    {
        asm volatile("s_nop 4\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(hd_scalar(base)) : "memory");
    }
    // The same load without the wait states in front of it, for the inside of a hand-ordered main loop:
    // an s_nop N holds the wave's issue slot for N + 1 rounds of 4 cycles, longer than a 16-cycle MFMA
    // runs.  To be used only where (1) another instruction sits between the write of M0 and this load
    // and (2) no VALU instruction writes a scalar register anywhere near: the loops that use it are
    // checked for that in their device assembly (tests/test_kernel_codegen.py).
    __device__ __forceinline__ void dma_load_in_loop(uint32_t voff, const void* base)
    {
        asm volatile("global_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(hd_scalar(base)) : "memory");
    }
    // The instruction's offset field moves the global address AND the LDS destination (found by a probe on the device: with
    // offset:1024 lane l's 16 bytes came from base + voff + 1024 and landed at M0 + 1024 + 16 l).  So up to four loads into
    // consecutive KiB of LDS share one write of M0 (the field is 13 bits, signed), when each lane's offset is lowered by the
    // same amount beforehand: the callers keep voff + DMA_BIAS - OFF in their registers and base - DMA_BIAS in the scalars, so
    // that no lane offset goes below zero.
    constexpr int DMA_BIAS = 3072;
    template <int OFF>
    __device__ __forceinline__ void dma_load_off(uint32_t voff, const void* base)
    {
        static_assert(OFF >= 0 && OFF <= DMA_BIAS && OFF % 1024 == 0, "one of four consecutive KiB");
        asm volatile("s_nop 4\n\tglobal_load_lds_dwordx4 %0, %1 offset:%2" : : "v"(voff), "s"(hd_scalar(base)), "n"(OFF) : "memory");
    }
    template <int OFF>
    __device__ __forceinline__ void dma_load_in_loop_off(uint32_t voff, const void* base)
    {
        static_assert(OFF >= 0 && OFF <= DMA_BIAS && OFF % 1024 == 0, "one of four consecutive KiB");
        asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" : : "v"(voff), "s"(hd_scalar(base)), "n"(OFF) : "memory");
    }
    // ... with a full address per lane (no scalar base): for loads some lanes of which must look elsewhere
    __device__ __forceinline__ void dma_load_at(const void* lane_address)
    {
        asm volatile("s_nop 4\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(lane_address) : "memory");
    }
    __device__ __forceinline__ void dma_load1(uint32_t voff, const void* base)
    {
        asm volatile("s_nop 4\n\tglobal_load_lds_dword %0, %1" : : "v"(voff), "s"(hd_scalar(base)) : "memory");
    }

    // The 4-byte load without wait states in front of it: under the conditions of dma_load_in_loop
    __device__ __forceinline__ void dma_load1_bare(uint32_t voff, const void* base)
    {
        asm volatile("global_load_lds_dword %0, %1" : : "v"(voff), "s"(hd_scalar(base)) : "memory");
    }

    // s_waitcnt immediates (gfx9 encoding): vmcnt(N) with the other counters left alone
    constexpr int waitcnt_vm(int n)
    {
        return (n & 15) | ((n >> 4) << 14) | 0x0F70;
    }
    // vmcnt(N) and lgkmcnt(0) in one: what a wave waits for before the barrier that hands a ring stage on (its
    // loads of the tile the next step reads have landed; its own LDS reads of the tile just multiplied are done,
    // so that the stage may be overwritten).  Written out because the wait the workgroup fence implies was
    // found missing in front of the first barrier of an unrolled loop body.
    constexpr int waitcnt_vm_lgkm0(int n)
    {
        return (n & 15) | ((n >> 4) << 14) | 0x0070;
    }
    // lgkmcnt(0) with the other counters left alone
    constexpr int waitcnt_lgkm0 = 0xC07F;

}
