// LDS and streaming helpers shared by the MFMA attention kernels (internal).
#pragma once
#include "bgtq_common.h"

namespace {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) uint8_t* lds_ptr_t;

// (a & mask) | c in one instruction; the mask travels in a scalar register
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t c) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(c));
    return r;
}
// two consecutive dwords at a 4-byte aligned LDS address (one ds_read2_b32; a plain load, so that the
// compiler places the wait for it)
typedef uint32_t dword_pair __attribute__((ext_vector_type(2), aligned(4)));
__device__ __forceinline__ void lds_read2(uint32_t addr, uint32_t& lo, uint32_t& hi) {
    const dword_pair r = *(const __attribute__((address_space(3))) dword_pair*)(uintptr_t)addr;
    lo = r.x;
    hi = r.y;
}

// 4 / 8 bytes from any LDS byte address: aligned dword reads and a byte funnel shift (unaligned LDS
// reads are legal on this target but several times slower)
__device__ __forceinline__ uint32_t lds_codes4(uint32_t addr) {
    uint32_t lo, hi;
    lds_read2(addr & ~3u, lo, hi);
    return __builtin_amdgcn_alignbyte(hi, lo, addr & 3u);
}
__device__ __forceinline__ uint2v lds_codes8(uint32_t addr) {
    uint32_t lo, hi;
    lds_read2(addr & ~3u, lo, hi);
    const uint32_t hi2 = *(const __attribute__((address_space(3))) uint32_t*)(uintptr_t)((addr & ~3u) + 8);
    return (uint2v){__builtin_amdgcn_alignbyte(hi, lo, addr & 3u), __builtin_amdgcn_alignbyte(hi2, hi, addr & 3u)};
}

// Read through an absolute LDS address (the kernel has no static LDS, so the dynamic block
// starts at LDS address 0 and offsets into it are addresses).
template <class T>
__device__ __forceinline__ T lds_at(uint32_t addr) {
    return *(const __attribute__((address_space(3))) T*)(uintptr_t)addr;
}
template <class T>
__device__ __forceinline__ void lds_put(uint32_t addr, T v) {
    *(__attribute__((address_space(3))) T*)(uintptr_t)addr = v;
}

// A wave-uniform pointer as a scalar register pair, also where the compiler computed it in vector registers
__device__ __forceinline__ const uint8_t* uniform_ptr(const uint8_t* p) {
    const uint64_t v = (uint64_t)(uintptr_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const uint8_t*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

// 16 bytes per lane from sbase + voff into LDS at lds_addr + lane * 16, for the lanes
// set in `lanes`.  The execution mask is switched inside the block, so the copy needs
// no divergent branch around it.
__device__ __forceinline__ void dma16(uint32_t voff, const uint8_t* sbase, uint32_t lds_addr, uint64_t lanes) {
    uint64_t saved;
    sbase = uniform_ptr(sbase);
    asm volatile("" : "+s"(lanes));          // (a mask known at compile time must still arrive in a register pair)
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %4\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, %0\n"
                 : "=&s"(saved) : "v"(voff), "s"(sbase), "s"(lds_addr), "s"(lanes) : "memory", "m0");
}
// Same for all 64 lanes of a 1 KB chunk at a compile-time distance from sbase / lds_addr:
// the instruction offset moves the global and the LDS address together.
template <int OFF>
__device__ __forceinline__ void dma_chunk(uint32_t voff, const uint8_t* sbase, uint32_t lds_addr) {
    sbase = uniform_ptr(sbase);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3\n"
                 :: "v"(voff), "s"(sbase), "s"(lds_addr), "n"(OFF) : "memory", "m0");
}

// How a byte range [src_al, src_al + total) is cut into 1 KB load instructions: every
// chunk but the last runs with all lanes, the last one with the lanes whose aligned
// 16-byte piece still starts inside the range.  Pieces are aligned, so a piece that holds
// at least one wanted byte never crosses into a page the range itself does not touch.
struct DmaShape {
    int nfull;          // chunks before the last
    uint64_t last;      // lanes of the last chunk
};
__device__ __forceinline__ DmaShape dma_shape(int total, uint32_t voff) {
    DmaShape d;
    d.nfull = ((total + 1023) >> 10) - 1;
    d.last = __builtin_amdgcn_ballot_w64((int)voff < total - d.nfull * 1024);
    return d;
}
// The same from wave-uniform values only (scalar arithmetic, no lane compare)
__device__ __forceinline__ DmaShape dma_shape_uniform(int total) {
    DmaShape d;
    d.nfull = ((total + 1023) >> 10) - 1;
    const int pieces = (total - d.nfull * 1024 + 15) >> 4;           // 1..64 lanes
    d.last = pieces >= 64 ? ~0ull : ((1ull << pieces) - 1ull);
    return d;
}
// Issues the nfull + 1 loads of a range of at most NCH chunks.
template <int NCH>
__device__ __forceinline__ void dma_region(const uint8_t* src_al, uint32_t lds_addr, const DmaShape& d, uint32_t voff) {
#pragma unroll
    for (int c = 0; c + 1 < NCH; c++)
        if (c < d.nfull) {
            if ((c & 3) == 0) dma_chunk<0>(voff, src_al + (c >> 2) * 4096, lds_addr + (c >> 2) * 4096);
            if ((c & 3) == 1) dma_chunk<1024>(voff, src_al + (c >> 2) * 4096, lds_addr + (c >> 2) * 4096);
            if ((c & 3) == 2) dma_chunk<2048>(voff, src_al + (c >> 2) * 4096, lds_addr + (c >> 2) * 4096);
            if ((c & 3) == 3) dma_chunk<3072>(voff, src_al + (c >> 2) * 4096, lds_addr + (c >> 2) * 4096);
        }
    dma16(voff, src_al + d.nfull * 1024, lds_addr + d.nfull * 1024, d.last);
}

// N (1..4) whole 1 KB chunks that follow each other, through one setting of M0: lane l copies the 16
// bytes at sbase + voff (+ 1024 a chunk; voff = 16 l + the tile's distance from sbase) to lds + 16 l.
template <int N>
__device__ __forceinline__ void dma_full(uint32_t voff, const uint8_t* sbase, uint32_t lds) {
    static_assert(N >= 1 && N <= 4, "the instruction offset reaches 4 chunks");
    if (N == 1) asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1\n" :: "v"(voff), "s"(sbase), "s"(lds) : "memory", "m0");
    if (N == 2) asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1\n\tglobal_load_lds_dwordx4 %0, %1 offset:1024\n"
                             :: "v"(voff), "s"(sbase), "s"(lds) : "memory", "m0");
    if (N == 3) asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1\n\tglobal_load_lds_dwordx4 %0, %1 offset:1024\n\t"
                             "global_load_lds_dwordx4 %0, %1 offset:2048\n" :: "v"(voff), "s"(sbase), "s"(lds) : "memory", "m0");
    if (N == 4) asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1\n\tglobal_load_lds_dwordx4 %0, %1 offset:1024\n\t"
                             "global_load_lds_dwordx4 %0, %1 offset:2048\n\tglobal_load_lds_dwordx4 %0, %1 offset:3072\n"
                             :: "v"(voff), "s"(sbase), "s"(lds) : "memory", "m0");
}
// n (0..8) whole chunks
__device__ __forceinline__ void dma_chunks(uint32_t voff, const uint8_t* sbase, uint32_t lds, int n) {
    sbase = uniform_ptr(sbase);
    if (n >= 4) {
        dma_full<4>(voff, sbase, lds);
        if (n == 4) return;
        voff += 4096;
        lds += 4096;
        n -= 4;
    }
    switch (n) {
    case 1: dma_full<1>(voff, sbase, lds); break;
    case 2: dma_full<2>(voff, sbase, lds); break;
    case 3: dma_full<3>(voff, sbase, lds); break;
    case 4: dma_full<4>(voff, sbase, lds); break;
    default: break;
    }
}
// One chunk each of up to three ranges, for the lanes of its mask: the execution mask is saved and
// restored once around all of them.
struct DmaTail { const uint8_t* src; uint32_t lds; uint64_t lanes; };
__device__ __forceinline__ void dma_tails(uint32_t v0, const DmaTail& t0, uint32_t v1, const DmaTail& t1, uint32_t v2, const DmaTail& t2) {
    uint64_t saved;
    const uint8_t *s0 = uniform_ptr(t0.src), *s1 = uniform_ptr(t1.src), *s2 = uniform_ptr(t2.src);
    uint64_t m0 = t0.lanes, m1 = t1.lanes, m2 = t2.lanes;
    asm volatile("" : "+s"(m0), "+s"(m1), "+s"(m2));
    asm volatile("s_mov_b64 %0, exec\n\t"
                 "s_mov_b64 exec, %3\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %10, %1\n\t"
                 "s_mov_b64 exec, %6\n\ts_mov_b32 m0, %5\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %11, %4\n\t"
                 "s_mov_b64 exec, %9\n\ts_mov_b32 m0, %8\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %12, %7\n\t"
                 "s_mov_b64 exec, %0\n"
                 : "=&s"(saved)
                 : "s"(s0), "s"(t0.lds), "s"(m0), "s"(s1), "s"(t1.lds), "s"(m1), "s"(s2), "s"(t2.lds), "s"(m2), "v"(v0), "v"(v1), "v"(v2)
                 : "memory", "m0");
}
__device__ __forceinline__ void dma_tail(uint32_t v0, const DmaTail& t0) {
    uint64_t saved;
    const uint8_t* s0 = uniform_ptr(t0.src);
    uint64_t m0 = t0.lanes;
    asm volatile("" : "+s"(m0));
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %3\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %4, %1\n\ts_mov_b64 exec, %0\n"
                 : "=&s"(saved) : "s"(s0), "s"(t0.lds), "s"(m0), "v"(v0) : "memory", "m0");
}

// Waits until at most n of the loads issued so far are still in flight.
__device__ __forceinline__ void wait_loads(int n) {
#define BGTQ_WAIT_CASE(k) case k: asm volatile("s_waitcnt vmcnt(" #k ")" ::: "memory"); break;
    switch (n) {
    BGTQ_WAIT_CASE(0) BGTQ_WAIT_CASE(1) BGTQ_WAIT_CASE(2) BGTQ_WAIT_CASE(3) BGTQ_WAIT_CASE(4) BGTQ_WAIT_CASE(5)
    BGTQ_WAIT_CASE(6) BGTQ_WAIT_CASE(7) BGTQ_WAIT_CASE(8) BGTQ_WAIT_CASE(9) BGTQ_WAIT_CASE(10) BGTQ_WAIT_CASE(11)
    BGTQ_WAIT_CASE(12) BGTQ_WAIT_CASE(13) BGTQ_WAIT_CASE(14) BGTQ_WAIT_CASE(15) BGTQ_WAIT_CASE(16) BGTQ_WAIT_CASE(17)
    BGTQ_WAIT_CASE(18) BGTQ_WAIT_CASE(19) BGTQ_WAIT_CASE(20) BGTQ_WAIT_CASE(21) BGTQ_WAIT_CASE(22) BGTQ_WAIT_CASE(23)
    default: asm volatile("s_waitcnt vmcnt(24)" ::: "memory"); break;
    }
#undef BGTQ_WAIT_CASE
}


// (a & mask) | c with all three operands in vector registers
__device__ __forceinline__ uint32_t and_or_v(uint32_t a, uint32_t mask, uint32_t c) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(mask), "v"(c));
    return r;
}

}  // namespace
