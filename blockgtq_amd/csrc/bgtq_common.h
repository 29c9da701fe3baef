// Shared device/host helpers of the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/bgtq.h"

#define BGTQ_D BGTQ_HEAD_DIM

#define BGTQ_CHECK_ARG(cond) do { if (!(cond)) return BGTQ_EINVAL; } while (0)

static inline int bgtq_launch_status() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? BGTQ_OK : (int)e;
}

// Bytes a K segment of `len` codes of width `bw` occupies in the bit-packed record.
__host__ __device__ static inline int bgtq_seg_bytes(int bw, int len) {
    switch (bw) {
    case 1: return (len + 7) >> 3;
    case 2: return (len + 3) >> 2;
    case 3: return ((len + 7) >> 3) * 3;
    case 4: return (len + 1) >> 1;
    default: return len;
    }
}

__device__ static inline float bgtq_h2f(uint16_t h) {
    return __half2float(__ushort_as_half(h));
}
__device__ static inline uint16_t bgtq_f2h(float f) {
    return __half_as_ushort(__float2half_rn(f));
}
