// Direct global -> LDS staging (gfx950 global_load_lds_dwordx4) for 16-bit tiles whose rows are
// 128 bytes (64 elements): the loading wave's 64 lanes each fetch 16 bytes and the hardware
// writes lane i's bytes at (wave-uniform LDS base) + 16*i, i.e. one instruction fills 8
// consecutive dense tile rows.  No registers hold the data and no LDS store is issued.
//
// Dense 128-byte rows would put every row on the same banks, so 16-byte chunk c of row r is
// stored at chunk position c ^ f(r).  Two swizzles, by how an MFMA operand read walks the tile:
//   swz_perm : lane n reads row key_of_row(n) (the permuted K1-style A operand)
//   swz_seq  : lane n reads row n (B operands, and every other consecutive-row access)
// Both give 16 consecutive lanes 16 distinct (row parity, chunk position) pairs and 8 consecutive
// lanes 8 distinct chunk positions.
#pragma once
#include "common.hpp"

namespace tritt {

__device__ __forceinline__ constexpr int swz_perm(int r) {
    return ((r >> 1) & 1) | (((r >> 3) & 1) << 1) | (((r ^ (r >> 2)) & 1) << 2);
}
__device__ __forceinline__ constexpr int swz_seq(int r) { return (r & 7) ^ ((r >> 3) & 1); }
// one 1 KB block: `gbase` is wave-uniform, `byte_off` per lane, `lds_dst` wave-uniform.
// Written as inline assembly on purpose.  The compiler treats the builtin form of this load as an access that may
// touch both global memory and LDS, and while one is outstanding its wait-count insertion turns every wait for an
// LDS read into lgkmcnt(0): in loops that keep stage loads in flight all the time (every kernel here) an operand
// read issued a phase ahead was then waited for together with the reads issued after it, and the prefetch bought
// nothing.  Seen as an opaque statement, the load leaves the compiler's counting of LDS reads exact; the callers
// wait for these loads themselves (wait_vmcnt / barrier_keep_loads), as they had to before.  A wait that the
// compiler computes for its own vector-memory loads can only become more conservative by loads it does not know.
// M0 (the LDS base of the load) is a reserved register that nothing else in these kernels uses.
__device__ __forceinline__ void direct_load_16(const void* gbase, unsigned byte_off, void* lds_dst) {
    const unsigned lds = (unsigned)(size_t)(__attribute__((address_space(3))) char*)lds_dst;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds), "v"(byte_off), "s"(gbase)
                 : "memory");
}

// the same with 4 bytes per lane: one instruction fills 256 consecutive bytes.  (Both wave-uniform operands are made
// scalar here: callers that pick the destination from a ring slot do not always get them as scalars.)
__device__ __forceinline__ void direct_load_4(const void* gbase, unsigned byte_off, void* lds_dst) {
    const unsigned lds =
        __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) char*)lds_dst);
    const unsigned long long a = reinterpret_cast<unsigned long long>(gbase);
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)a), hi = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32));
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :
                 : "s"(lds), "v"(byte_off), "s"(((unsigned long long)hi << 32) | lo)
                 : "memory");
}

// make a wave-uniform pointer provably scalar (keeps it in SGPRs instead of spilled VGPR pairs)
template <typename T>
__device__ __forceinline__ const T* uniform_ptr(const T* p) {
    const unsigned long long a = reinterpret_cast<unsigned long long>(p);
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)a);
    const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32));
    return reinterpret_cast<const T*>(((unsigned long long)hi << 32) | lo);
}

// s_waitcnt vmcnt(N) only (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[15:14])
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// Workgroup barrier for kernels that keep direct loads in flight: waits for this wave's LDS
// traffic and for all but its newest N vector-memory operations, then s_barrier.  (__syncthreads
// would wait for every outstanding load, i.e. also for the stages fetched ahead.)
template <int N>
__device__ __forceinline__ void barrier_keep_loads() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (0 << 8) | ((N >> 4) << 14));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

}  // namespace tritt
