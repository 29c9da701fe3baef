// Do vector ALU instructions issue while matrix instructions execute on gfx950?  Time of a run of
// v_mfma_f32_32x32x16_f16 alone, of dependent vector ALU instructions alone, of both interleaved in one wave,
// and of both in different waves of one SIMD (waves w and w + 4 of a work-group share a SIMD).
//   hipcc --offload-arch=gfx950 -O2 mfma_valu_probe.hip -o mfma_valu_probe && ./mfma_valu_probe
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdint.h>
#include <vector>
#include <algorithm>
#define REP4(x) x x x x
#define REP16(x) REP4(REP4(x))
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
#define MF "v_mfma_f32_32x32x16_f16 %0, %4, %5, %0\n v_mfma_f32_32x32x16_f16 %1, %4, %5, %1\n"
#define VA "v_and_or_b32 %2, %3, %2, %3\n v_and_or_b32 %3, %2, %3, %2\n v_and_or_b32 %2, %3, %2, %3\n v_and_or_b32 %3, %2, %3, %2\n"
#define VA8 VA VA
__global__ __launch_bounds__(1024) void k(uint64_t* out, int iters, uint32_t* sink, int kind) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    half8 ha, hb;
    for (int i = 0; i < 8; i++) { ha[i] = (_Float16)(tid * 0.001f + i); hb[i] = (_Float16)(i * 0.5f); }
    float16v c0 = {0}, c1 = {0};
    uint32_t a0 = tid, a1 = tid * 3 + 1;
    uint64_t t0 = __builtin_readcyclecounter();
    for (int it = 0; it < iters; it++) {
        switch (kind) {
        case 0: asm volatile(REP16(MF) : "+v"(c0), "+v"(c1), "+v"(a0), "+v"(a1) : "v"(ha), "v"(hb)); break;              // 32 MFMA
        case 1: asm volatile(REP16(VA8) : "+v"(c0), "+v"(c1), "+v"(a0), "+v"(a1) : "v"(ha), "v"(hb)); break;             // 128 VALU
        case 2: asm volatile(REP16(MF VA8) : "+v"(c0), "+v"(c1), "+v"(a0), "+v"(a1) : "v"(ha), "v"(hb)); break;          // 32 MFMA + 128 VALU interleaved in one wave
        case 3:                                                                                                           // even waves MFMA, odd waves VALU
            if (wave & 1) asm volatile(REP16(VA8) : "+v"(c0), "+v"(c1), "+v"(a0), "+v"(a1) : "v"(ha), "v"(hb));
            else asm volatile(REP16(MF) : "+v"(c0), "+v"(c1), "+v"(a0), "+v"(a1) : "v"(ha), "v"(hb));
            break;
        case 4:                                                                                                           // waves 0..3 MFMA, waves 4..7 VALU
            if (wave & 4) asm volatile(REP16(VA8) : "+v"(c0), "+v"(c1), "+v"(a0), "+v"(a1) : "v"(ha), "v"(hb));
            else asm volatile(REP16(MF) : "+v"(c0), "+v"(c1), "+v"(a0), "+v"(a1) : "v"(ha), "v"(hb));
            break;
        case 5: asm volatile(REP16(MF VA) : "+v"(c0), "+v"(c1), "+v"(a0), "+v"(a1) : "v"(ha), "v"(hb)); break;           // 32 MFMA + 64 VALU
        }
    }
    uint64_t t1 = __builtin_readcyclecounter();
    if (lane == 0) out[blockIdx.x * (blockDim.x >> 6) + wave] = t1 - t0;
    sink[blockIdx.x * blockDim.x + tid] = a0 ^ a1 ^ (uint32_t)(c0[0] + c1[1]);
}
int main() {
    uint64_t* dout; uint32_t* dsink;
    hipMalloc(&dout, 256 * 16 * 8); hipMalloc(&dsink, 256 * 1024 * 4);
    const char* names[] = {"32 MFMA 32x32x16", "128 VALU", "32 MFMA + 128 VALU, one wave", "even waves MFMA, odd waves VALU", "waves 0-3 MFMA, 4-7 VALU", "32 MFMA + 64 VALU, one wave"};
    for (int nw : {4, 8}) for (int kind = 0; kind < 6; kind++) {
        const int iters = 300;
        k<<<256, nw * 64>>>(dout, 5, dsink, kind);
        hipDeviceSynchronize();
        hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
        hipEventRecord(e0);
        k<<<256, nw * 64>>>(dout, iters, dsink, kind);
        hipEventRecord(e1);
        hipError_t e = hipDeviceSynchronize();
        float ms; hipEventElapsedTime(&ms, e0, e1);
        std::vector<uint64_t> h(256 * nw);
        hipMemcpy(h.data(), dout, h.size() * 8, hipMemcpyDeviceToHost);
        std::sort(h.begin(), h.end());
        printf("%-34s waves/CU %d: %8.1f ticks per loop body per wave (median), max %8.1f, kernel %.3f ms  err=%d\n", names[kind], nw,
               (double)h[h.size() / 2] / iters, (double)h.back() / iters, ms, (int)e);
    }
    return 0;
}
