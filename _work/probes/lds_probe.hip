// LDS access-pattern probe for gfx950: time per LDS instruction when lane l of a half-wave accesses byte
// l * stride (the upper half-wave a given distance behind), for the access widths the attention kernels use,
// with one wave per CU (latency of a run of independent accesses) and with eight (throughput of the CU's LDS).
//   hipcc --offload-arch=gfx950 -O2 lds_probe.hip -o lds_probe && ./lds_probe
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdint.h>
#include <vector>
#include <algorithm>
#define REP4(x) x x x x
#define REP16(x) REP4(REP4(x))
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));
__global__ __launch_bounds__(1024) void k(uint64_t* out, int iters, uint32_t* sink, int kind, int stride_bytes, int half_off) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int i = tid; i < 16384; i += blockDim.x) ((uint32_t*)smem)[i] = i * 2654435761u;
    __syncthreads();
    // lanes 32..63 get an extra offset so that the two halves can be placed independently
    const uint32_t addr = (uint32_t)((lane & 31) * stride_bytes + (lane >> 5) * half_off) & 0xFFFCu;
    uint32_t a0 = 0, a1 = 0;
    u4 w0 = {0, 0, 0, 0}, w1 = w0;
    u2 d0 = {0, 0}, d1 = d0;
    uint32_t val = tid;
    uint64_t t0 = __builtin_readcyclecounter();
    for (int it = 0; it < iters; it++) {
        switch (kind) {
        case 0: asm volatile(REP16("ds_read_b32 %0, %2\n ds_read_b32 %1, %2 offset:4096\n") "s_waitcnt lgkmcnt(0)" : "+v"(a0), "+v"(a1) : "v"(addr) : "memory"); break;
        case 1: asm volatile(REP16("ds_write_b32 %0, %1\n ds_write_b32 %0, %1 offset:4096\n") "s_waitcnt lgkmcnt(0)" :: "v"(addr), "v"(val) : "memory"); break;
        case 2: asm volatile(REP16("ds_read_b128 %0, %2\n ds_read_b128 %1, %2 offset:4096\n") "s_waitcnt lgkmcnt(0)" : "+v"(w0), "+v"(w1) : "v"(addr & 0xFFF0u) : "memory"); break;
        case 3: asm volatile(REP16("ds_read_b64 %0, %2\n ds_read_b64 %1, %2 offset:4096\n") "s_waitcnt lgkmcnt(0)" : "+v"(d0), "+v"(d1) : "v"(addr & 0xFFF8u) : "memory"); break;
        case 4: asm volatile(REP16("ds_read_u16 %0, %2\n ds_read_u16 %1, %2 offset:4096\n") "s_waitcnt lgkmcnt(0)" : "+v"(a0), "+v"(a1) : "v"(addr) : "memory"); break;
        case 5: asm volatile(REP16("ds_read2_b32 %0, %2 offset1:1\n ds_read2_b32 %1, %2 offset0:16 offset1:17\n") "s_waitcnt lgkmcnt(0)" : "+v"(d0), "+v"(d1) : "v"(addr) : "memory"); break;
        case 6: asm volatile(REP16("ds_write_b128 %0, %1\n ds_write_b128 %0, %1 offset:4096\n") "s_waitcnt lgkmcnt(0)" :: "v"(addr & 0xFFF0u), "v"(w0) : "memory"); break;
        case 7: asm volatile(REP16("ds_read2_b64 %0, %2 offset1:2\n ds_read2_b64 %1, %2 offset0:64 offset1:66\n") "s_waitcnt lgkmcnt(0)" : "+v"(w0), "+v"(w1) : "v"(addr & 0xFFF8u) : "memory"); break;
        }
    }
    uint64_t t1 = __builtin_readcyclecounter();
    if (lane == 0) out[blockIdx.x * (blockDim.x >> 6) + wave] = t1 - t0;
    sink[blockIdx.x * blockDim.x + tid] = a0 ^ a1 ^ w0.x ^ w1.y ^ d0.x ^ d1.y;
}
int main() {
    uint64_t* dout; uint32_t* dsink;
    hipMalloc(&dout, 256 * 16 * 8); hipMalloc(&dsink, 256 * 1024 * 4);
    const char* names[] = {"ds_read_b32", "ds_write_b32", "ds_read_b128", "ds_read_b64", "ds_read_u16", "ds_read2_b32", "ds_write_b128", "ds_read2_b64"};
    struct Case { int kind, stride, half; };
    std::vector<Case> cases;
    for (int s : {4, 8, 12, 16, 32, 48, 64, 76, 96, 128, 144, 272}) { cases.push_back({0, s, 32 * s}); cases.push_back({1, s, 32 * s}); }
    for (int s : {4, 128}) { cases.push_back({0, s, 0}); cases.push_back({0, s, 128}); cases.push_back({0, s, 4096 + 128}); }   // halves on the same / other banks
    for (int s : {16, 32, 144, 272}) { cases.push_back({2, s, 32 * s}); cases.push_back({6, s, 32 * s}); }
    for (int s : {8, 16, 144, 272}) { cases.push_back({3, s, 32 * s}); cases.push_back({7, s, 32 * s}); }
    for (int s : {2, 4, 12}) cases.push_back({4, s, 32 * s});
    for (int s : {4, 48, 76, 96}) cases.push_back({5, s, 32 * s});
    for (int nw : {1, 8}) {
        for (auto c : cases) {
            const int iters = 200;
            k<<<256, nw * 64, 64 * 1024>>>(dout, 5, dsink, c.kind, c.stride, c.half);
            hipDeviceSynchronize();
            k<<<256, nw * 64, 64 * 1024>>>(dout, iters, dsink, c.kind, c.stride, c.half);
            hipError_t e = hipDeviceSynchronize();
            std::vector<uint64_t> h(256 * nw);
            hipMemcpy(h.data(), dout, h.size() * 8, hipMemcpyDeviceToHost);
            std::sort(h.begin(), h.end());
            double per_wave = (double)h[h.size() / 2] / (iters * 32.0);
            printf("%-14s lane stride %4d B, upper half +%5d B, waves/CU %d: %7.2f ticks per instr per wave, %6.2f per instr per CU  err=%d\n",
                   names[c.kind], c.stride, c.half, nw, per_wave, per_wave / nw, (int)e);
            fflush(stdout);
        }
    }
    return 0;
}
