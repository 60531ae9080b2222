// qm_resident.h — what the kernels whose blocks stay resident and talk to each other share (gfx950): agent-scope
// words for the hand-offs between blocks, LDS accesses the compiler does not see for the waves that have weight
// pieces under way, and the wait for all but the last N of a wave's memory operations.
#pragma once

#include "qm_device.h"

namespace qm {

// A value handed from block to block: relaxed, agent scope (it bypasses the per-XCD L2s).
__device__ __forceinline__ uint32_t agent_load(const uint32_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void agent_store(uint32_t* p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Waits until at most N of this wave's memory operations are outstanding (they complete in the order they were
// made: what is outstanding then was requested last).
template <int N>
__device__ __forceinline__ void wait_vm_at_most() {
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// LDS accesses written out.  The compiler makes every LDS access of its own wait until ALL global_load_lds
// requests of the wave have landed (it cannot tell which bytes a read touches); a wave that has such requests
// under way reads and writes LDS through these, with the waits the hardware needs: lds_wait() before the first
// use of what lds_read_* requested, then pin() on every register read into, so that no use is scheduled above
// the wait.
__device__ __forceinline__ uint32_t lds_at(const void* p) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void*)p));
}
template <int J, int N, int STRIDE>
__device__ __forceinline__ void lds_read_b32(uint32_t at, uint32_t (&v)[N]) {
    if constexpr (J < N) {
        asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v[J]) : "v"(at), "n"(J * STRIDE));
        lds_read_b32<J + 1, N, STRIDE>(at, v);
    }
}
template <int J, int N, int STRIDE>
__device__ __forceinline__ void lds_read_u16(uint32_t at, uint32_t (&v)[N]) {
    if constexpr (J < N) {
        asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(v[J]) : "v"(at), "n"(J * STRIDE));
        lds_read_u16<J + 1, N, STRIDE>(at, v);
    }
}
__device__ __forceinline__ void lds_wait() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
template <int J, int N>
__device__ __forceinline__ void pin(uint32_t (&v)[N]) {
    if constexpr (J < N) {
        asm volatile("" : "+v"(v[J]));
        pin<J + 1, N>(v);
    }
}
__device__ __forceinline__ uint32_t lds_word(const void* p) {
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(lds_at(p)) : "memory");
    return v;
}
// four counters that lie together, 16-byte aligned, with one instruction
typedef int lds_int4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ lds_int4 lds_four(const void* p) {
    lds_int4 v;
    asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(lds_at(p)) : "memory");
    return v;
}
__device__ __forceinline__ void lds_store(void* p, uint32_t v) {
    asm volatile("ds_write_b32 %0, %1" : : "v"(lds_at(p)), "v"(v) : "memory");
}
__device__ __forceinline__ void lds_add_one(void* p) {
    asm volatile("ds_add_u32 %0, %1" : : "v"(lds_at(p)), "v"(1u) : "memory");
}

}  // namespace qm
