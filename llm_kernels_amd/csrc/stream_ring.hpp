// Hand-issued global loads for the weight-streaming (decode) kernels.
//
// A persistent workgroup keeps the weights of several tiles in flight in a ring of registers.  With ordinary
// loads the compiler has to guess how many loads are outstanding at the top of the loop and, the ring being
// filled under loop-carried control flow, guesses "wait for all of them": the load just requested included,
// which serialises every tile behind a full memory round trip.  The loads of the ring are therefore issued
// from inline asm (wave-uniform 64-bit base in scalar registers + one 32-bit offset per lane + immediate) and
// waited for by hand with s_waitcnt vmcnt(n), n = the number of LOADS issued after the ones needed (loads
// return in order; stores in flight only make the wait longer, never shorter).
//
// The compiler takes a destination register for ready as soon as the load is issued.  The registers pass
// through the wait as read-write operands, so every use comes after it; that the compiler neither copies,
// spills nor reuses them between load and wait is proved on the assembly of every build by check_asm.py.
#pragma once
#include "common.hpp"

namespace llmk {

// The base pointer of hand-issued loads: the same in every lane, held in scalar registers, and settled.
//
// The compiler may carry a wave-uniform pointer in vector registers (64-bit multiplies have no scalar form, and
// behind divergent control flow anything can end up there) and move it to scalar registers with
// v_readfirstlane_b32 right in front of the use.  A vector-memory instruction that reads a scalar register
// needs five wait states after a VALU instruction wrote it; the hardware does not interlock, the compiler
// inserts them for the loads it emits itself and knows nothing about the ones inside an asm statement, which
// would then take their base from whatever the register held before: a wild address.  ring_base() therefore
// ends in "s_nop 4" that names both halves as read-write operands, so every load that uses the base is at
// least five wait states behind the last VALU write to it.  The loads take nothing but a RingBase, and
// check_asm.py proves the distance on the assembly of every build.
struct RingBase {
    const void* p;
};
__device__ __forceinline__ RingBase ring_base(const void* p) {
    const uint64_t u = (uint64_t)(uintptr_t)p;
    uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)u);
    uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(u >> 32));
    asm volatile("s_nop 4 ; scalar base settled" : "+s"(lo), "+s"(hi));
    return RingBase{(const void*)(uintptr_t)(((uint64_t)hi << 32) | lo)};
}

template <int IMM>
__device__ __forceinline__ v4i ring_load_b128(uint32_t voff, RingBase base) {
    static_assert(IMM >= 0 && IMM < 4096, "13-bit signed immediate");
    v4i v;
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(v) : "v"(voff), "s"(base.p), "n"(IMM) : "memory");
    return v;
}
template <int IMM>
__device__ __forceinline__ v2i ring_load_b64(uint32_t voff, RingBase base) {
    static_assert(IMM >= 0 && IMM < 4096, "13-bit signed immediate");
    v2i v;
    asm volatile("global_load_dwordx2 %0, %1, %2 offset:%3" : "=v"(v) : "v"(voff), "s"(base.p), "n"(IMM) : "memory");
    return v;
}
template <int IMM>
__device__ __forceinline__ int ring_load_b32(uint32_t voff, RingBase base) {
    static_assert(IMM >= 0 && IMM < 4096, "13-bit signed immediate");
    int v;
    asm volatile("global_load_dword %0, %1, %2 offset:%3" : "=v"(v) : "v"(voff), "s"(base.p), "n"(IMM) : "memory");
    return v;
}

// Every load of the wave has landed (end of a ring kernel: requests that nobody consumed are drained).  ID ends
// up in the statement's text, which keeps the compiler from merging several such sites into one block.
template <int ID>
__device__ __forceinline__ void ring_drain() { asm volatile("s_waitcnt vmcnt(0) ; ring exit %0" ::"n"(ID) : "memory"); }

template <int IMM>
__device__ __forceinline__ int ring_load_u16(uint32_t voff, RingBase base) {
    static_assert(IMM >= 0 && IMM < 4096, "13-bit signed immediate");
    int v;
    asm volatile("global_load_ushort %0, %1, %2 offset:%3" : "=v"(v) : "v"(voff), "s"(base.p), "n"(IMM) : "memory");
    return v;
}

// s_waitcnt vmcnt(N) that names the registers it releases
template <int N>
__device__ __forceinline__ void ring_wait(v4i& a, v4i& b) {
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void ring_wait(int& a, int& b, int& c) {
    asm volatile("s_waitcnt vmcnt(%3)" : "+v"(a), "+v"(b), "+v"(c) : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void ring_wait(v4i& a, v4i& b, v4i& c, v4i& d) {
    asm volatile("s_waitcnt vmcnt(%4)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void ring_wait(v4i& a, v4i& b, v4i& c, v4i& d, v2i& e) {
    asm volatile("s_waitcnt vmcnt(%5)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e) : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void ring_wait(v4i& a, v4i& b, v4i& c, v4i& d, v4i& e, v4i& f, v4i& g, v4i& h) {
    asm volatile("s_waitcnt vmcnt(%8)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e), "+v"(f), "+v"(g), "+v"(h) : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void ring_wait16(v4i (&a)[16]) {
    asm volatile("s_waitcnt vmcnt(%16)"
                 : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]),
                   "+v"(a[8]), "+v"(a[9]), "+v"(a[10]), "+v"(a[11]), "+v"(a[12]), "+v"(a[13]), "+v"(a[14]), "+v"(a[15])
                 : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void ring_wait(int& a, int& b, int& c, int& d) {
    asm volatile("s_waitcnt vmcnt(%4)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N) : "memory");
}

}  // namespace llmk
