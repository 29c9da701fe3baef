// Issue-rate probe for gfx950: every wave of a work-group runs the same instruction mix, one
// work-group per CU, 4 or 12 waves per CU (1 or 3 per SIMD).  Prints the time per instruction seen
// by one wave and the resulting time per instruction per SIMD, in ticks of the shader's cycle
// counter, and the counter's rate against wall time.  It prices the instruction classes the
// decode-attention kernel is made of (VOP2 / VOP3 vector ALU, scalar ALU, 4-byte and 16-byte LDS
// reads, MFMA) alone and mixed.
//   hipcc --offload-arch=gfx950 -O2 issue_probe.hip -o issue_probe && ./issue_probe
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdint.h>
#include <vector>
#include <algorithm>
#define REP4(x) x x x x
#define REP16(x) REP4(REP4(x))
#define V "v_and_or_b32 %0, %1, %2, %3\n v_and_or_b32 %1, %2, %3, %0\n"
#define VF "v_add_u32 %0, %1, %2\n v_add_u32 %1, %2, %3\n"
#define S "s_add_u32 s20, s20, 1\n s_add_u32 s21, s21, 3\n"
#define L "ds_read_b32 %4, %6\n ds_read_b32 %5, %6 offset:256\n"
#define L4 "ds_read_b128 %0, %2\n ds_read_b128 %1, %2 offset:1024\n"
#define M "v_mfma_f32_16x16x32_f16 %0, %2, %3, %0\n v_mfma_f32_16x16x32_f16 %1, %2, %3, %1\n"
__global__ __launch_bounds__(1024) void k(uint64_t* out, int iters, uint32_t* sink, int kind) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int i = tid; i < 8192; i += blockDim.x) ((uint32_t*)smem)[i] = i * 2654435761u;
    __syncthreads();
    uint32_t a0 = tid, a1 = tid + 1, a2 = tid + 2, a3 = tid + 3, l0 = 0, l1 = 0;
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    typedef _Float16 half8 __attribute__((ext_vector_type(8)));
    typedef float float4v __attribute__((ext_vector_type(4)));
    u4 w0 = {0, 0, 0, 0}, w1 = w0;
    half8 ha, hb;
    for (int i = 0; i < 8; i++) { ha[i] = (_Float16)(tid * 0.001f + i); hb[i] = (_Float16)(i * 0.5f); }
    float4v c0 = {0, 0, 0, 0}, c1 = c0;
    const uint32_t addr16 = lane * 16;
    const uint32_t addr = lane * 4;
    uint64_t t0 = __builtin_readcyclecounter();
    for (int it = 0; it < iters; it++) {
#define BODY(X) asm volatile(REP16(X) : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(l0), "+v"(l1) : "v"(addr) : "memory", "s20", "s21", "scc")
        switch (kind) {
        case 0: BODY(V V); break;                 // 64 slow VALU
        case 1: BODY(S S); break;                 // 64 SALU
        case 2: BODY(V S); break;                 // 32 VALU + 32 SALU
        case 3: BODY(VF VF); break;               // 64 fast VALU
        case 4: BODY(VF S); break;
        case 5: BODY(L L) ; asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); break;   // 64 LDS
        case 6: BODY(V L); asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); break;    // 32 VALU + 32 LDS
        case 7: BODY(V S L V); asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); break; // 64 VALU + 32 SALU + 32 LDS = 128
        case 8: asm volatile(REP16(L4 L4) "s_waitcnt lgkmcnt(0)" : "+v"(w0), "+v"(w1) : "v"(addr16) : "memory"); break;   // 64 LDS b128
        case 9: asm volatile(REP16(M M) : "+v"(c0), "+v"(c1) : "v"(ha), "v"(hb)); break;                                    // 64 MFMA
        }
    }
    uint64_t t1 = __builtin_readcyclecounter();
    if (lane == 0) out[blockIdx.x * (blockDim.x >> 6) + wave] = t1 - t0;
    sink[blockIdx.x * blockDim.x + tid] = a0 ^ a1 ^ a2 ^ a3 ^ l0 ^ l1 ^ w0.x ^ w1.y ^ (uint32_t)(c0[0] + c1[1]);
}
void run(const char* name, int kind, int nwaves, int ninstr, uint64_t* dout, uint32_t* dsink) {
    const int iters = 500, blocks = 256;
    k<<<blocks, nwaves * 64, 64 * 1024>>>(dout, 10, dsink, kind);
    hipDeviceSynchronize();
    k<<<blocks, nwaves * 64, 64 * 1024>>>(dout, iters, dsink, kind);
    hipDeviceSynchronize();
    std::vector<uint64_t> h(blocks * nwaves);
    hipMemcpy(h.data(), dout, h.size() * 8, hipMemcpyDeviceToHost);
    std::sort(h.begin(), h.end());
    double per_wave = (double)h[h.size() / 2] / iters / ninstr;
    printf("%-34s waves/CU %2d: %6.2f counter ticks per instr per wave, %6.2f per instr per SIMD  err=%d\n", name, nwaves, per_wave,
           per_wave / (nwaves / 4.0), (int)hipGetLastError());
}
int main() {
    uint64_t* dout; uint32_t* dsink;
    hipMalloc(&dout, 256 * 16 * 8); hipMalloc(&dsink, 256 * 1024 * 4);
    const char* names[] = {"VOP3 VALU (v_and_or_b32)", "SALU (s_add_u32)", "VOP3 VALU + SALU 1:1", "VOP2 VALU (v_add_u32)", "VOP2 VALU + SALU 1:1",
                           "LDS ds_read_b32", "VOP3 VALU + LDS b32 1:1", "VALU 2 : SALU 1 : LDS b32 1", "LDS ds_read_b128", "MFMA 16x16x32 f16"};
    const int n[] = {64, 64, 64, 64, 64, 64, 64, 128, 64, 64};
    for (int nw : {4, 12})
        for (int kd = 0; kd < 10; kd++) run(names[kd], kd, nw, n[kd], dout, dsink);
    // clock ratio: wall time of a known count
    hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
    hipEventRecord(e0); k<<<256, 768, 64 * 1024>>>(dout, 2000, dsink, 0); hipEventRecord(e1); hipDeviceSynchronize();
    float ms; hipEventElapsedTime(&ms, e0, e1);
    std::vector<uint64_t> h(256 * 12); hipMemcpy(h.data(), dout, h.size() * 8, hipMemcpyDeviceToHost);
    std::sort(h.begin(), h.end());
    printf("counter ticks %llu in %.3f ms -> %.1f MHz counter\n", (unsigned long long)h[h.size() / 2], ms, h[h.size() / 2] / ms / 1e3);
    return 0;
}
