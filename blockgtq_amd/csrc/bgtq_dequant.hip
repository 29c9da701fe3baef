// Packed records back to fp16 vectors (gfx950).
//
// K comes back in the packed-dim order and rotated space the records were
// encoded in (value = fp16(codebook[code] * group norm), 0 on 0-bit dims), V
// in its rotated space (value = fp16(centroid[code] * norm)).  Attention over
// these tensors with rotated queries, followed by the V un-rotation, is
// attention over the packed cache; the prompt phase uses it where many query
// tokens share every K/V tile and the dequantised tile is worth keeping.
//
// One work-group of 128 threads handles TOK consecutive tokens of one (batch
// row, KV head): records and norms are staged in LDS with coalesced loads,
// then thread d extracts dim d of every token, so each token row goes out as
// one 256-byte store.
#include "bgtq_common.h"

namespace {

constexpr int D = BGTQ_D;
constexpr int TOK = 32;                 // tokens per work-group
constexpr int ROW_PAD = 4;              // 2 bytes of over-read by the 16-bit field window + alignment

struct DequantArgs {
    const bgtq_head_plan* plans;
    const uint8_t* kp;  int64_t kp_sb, kp_sh, kp_st;
    const uint16_t* kn; int64_t kn_sb, kn_sh, kn_st;
    const uint8_t* vp;  int64_t vp_sb, vp_sh, vp_st;
    const uint16_t* vn; int64_t vn_sb, vn_sh, vn_st;
    uint16_t* ko; int64_t ko_sb, ko_sh, ko_st;
    uint16_t* vo; int64_t vo_sb, vo_sh, vo_st;
    int T, k_layout, v_layout, k_row_width, v_row_width;
};

__device__ inline unsigned take_bits(const uint8_t* row, int bit, int bw) {
    const int byte = bit >> 3;
    const unsigned w = (unsigned)row[byte] | ((unsigned)row[byte + 1] << 8);
    return (w >> (bit & 7)) & ((1u << bw) - 1u);
}

__global__ __launch_bounds__(D) void dequant_kernel(DequantArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int d = threadIdx.x;
    const int h = blockIdx.y, b = blockIdx.z;
    const int t0 = blockIdx.x * TOK, nt = min(TOK, a.T - t0);
    const bgtq_head_plan& P = a.plans[h];

    const int krow = (a.k_row_width + ROW_PAD + 3) & ~3, vrow = (a.v_row_width + ROW_PAD + 3) & ~3;
    float* kn_s = (float*)smem;                          // [TOK][8]
    float* vn_s = kn_s + TOK * BGTQ_MAX_SEGMENTS;        // [TOK]
    uint8_t* krow_s = (uint8_t*)(vn_s + TOK);            // [TOK][krow]
    uint8_t* vrow_s = krow_s + TOK * krow;               // [TOK][vrow]

    const int n_seg = P.n_seg;
    const int kbytes = min(a.k_layout == BGTQ_K_MIXED ? P.k_mixed_bytes : P.k_row_bytes, a.k_row_width);
    const int vbw = a.v_layout == BGTQ_V_NIBBLE ? 4 : P.v_bits;
    const int vbytes = min(bgtq_seg_bytes(vbw, D), a.v_row_width);
    const uint8_t* kp = a.kp + b * a.kp_sb + h * a.kp_sh + (int64_t)t0 * a.kp_st;
    const uint8_t* vp = a.vp + b * a.vp_sb + h * a.vp_sh + (int64_t)t0 * a.vp_st;
    const uint16_t* kn = a.kn + b * a.kn_sb + h * a.kn_sh + (int64_t)t0 * a.kn_st;
    const uint16_t* vn = a.vn + b * a.vn_sb + h * a.vn_sh + (int64_t)t0 * a.vn_st;
    for (int i = d; i < nt * kbytes; i += D) {
        const int t = i / kbytes, o = i - t * kbytes;
        krow_s[t * krow + o] = kp[(int64_t)t * a.kp_st + o];
    }
    for (int i = d; i < nt * vbytes; i += D) {
        const int t = i / vbytes, o = i - t * vbytes;
        vrow_s[t * vrow + o] = vp[(int64_t)t * a.vp_st + o];
    }
    for (int i = d; i < nt * n_seg; i += D) {
        const int t = i / n_seg, g = i - t * n_seg;
        kn_s[t * BGTQ_MAX_SEGMENTS + g] = bgtq_h2f(kn[(int64_t)t * a.kn_st + g]);
    }
    if (d < nt) vn_s[d] = bgtq_h2f(vn[(int64_t)d * a.vn_st]);

    // where dim d sits in a K record
    const int g = P.group_of[d];
    int kbit = 0, kxbw = 0;
    if (g >= 0) {
        const int bw = P.seg_bw[g], rel = d - P.seg_start[g];
        if (a.k_layout == BGTQ_K_MIXED) {
            if (bw <= 4) { kbit = (d - P.n_zero_dims) * 4; kxbw = 4; }
            else         { kbit = (P.seg_mixed_off[g] + rel) * 8; kxbw = 8; }
        } else {
            if (bw <= 4) { kbit = P.seg_pack_off[g] * 8 + rel * bw; kxbw = bw; }
            else         { kbit = (P.seg_pack_off[g] + rel) * 8; kxbw = 8; }
        }
    }
    const uint16_t* cb = P.k_codebook_f16[g < 0 ? 0 : g];
    const int vbit = d * vbw;
    __syncthreads();

    uint16_t* ko = a.ko + b * a.ko_sb + h * a.ko_sh + (int64_t)t0 * a.ko_st + d;
    uint16_t* vo = a.vo + b * a.vo_sb + h * a.vo_sh + (int64_t)t0 * a.vo_st + d;
    for (int t = 0; t < nt; t++) {
        float kv = 0.f;
        if (g >= 0) kv = bgtq_h2f(cb[take_bits(krow_s + t * krow, kbit, kxbw)]) * kn_s[t * BGTQ_MAX_SEGMENTS + g];
        ko[(int64_t)t * a.ko_st] = bgtq_f2h(kv);
        const float vv = bgtq_h2f(P.v_lut_f16[take_bits(vrow_s + t * vrow, vbit, vbw)]) * vn_s[t];
        vo[(int64_t)t * a.vo_st] = bgtq_f2h(vv);
    }
}

}  // namespace

extern "C" int bgtq_dequant_kv(const bgtq_head_plan* plans,
                               const void* k_packed, int64_t kp_sb, int64_t kp_sh, int64_t kp_st, int k_row_width,
                               const void* k_norms, int64_t kn_sb, int64_t kn_sh, int64_t kn_st,
                               const void* v_packed, int64_t vp_sb, int64_t vp_sh, int64_t vp_st, int v_row_width,
                               const void* v_norms, int64_t vn_sb, int64_t vn_sh, int64_t vn_st,
                               int B, int n_kv, int T, int k_layout, int v_layout,
                               void* k_out, int64_t ko_sb, int64_t ko_sh, int64_t ko_st,
                               void* v_out, int64_t vo_sb, int64_t vo_sh, int64_t vo_st,
                               void* stream) {
    BGTQ_CHECK_ARG(plans && k_packed && k_norms && v_packed && v_norms && k_out && v_out);
    BGTQ_CHECK_ARG(B >= 0 && n_kv >= 0 && T >= 0);
    BGTQ_CHECK_ARG(k_row_width >= 1 && k_row_width <= 2 * D && v_row_width >= 1 && v_row_width <= D);
    BGTQ_CHECK_ARG(k_layout == BGTQ_K_BITPACKED || k_layout == BGTQ_K_MIXED);
    BGTQ_CHECK_ARG(v_layout == BGTQ_V_BITPACKED || v_layout == BGTQ_V_NIBBLE);
    if (B == 0 || n_kv == 0 || T == 0) return BGTQ_OK;
    if (n_kv > 65535 || B > 65535) return BGTQ_ELIMIT;
    DequantArgs a;
    a.plans = plans;
    a.kp = (const uint8_t*)k_packed; a.kp_sb = kp_sb; a.kp_sh = kp_sh; a.kp_st = kp_st;
    a.kn = (const uint16_t*)k_norms; a.kn_sb = kn_sb; a.kn_sh = kn_sh; a.kn_st = kn_st;
    a.vp = (const uint8_t*)v_packed; a.vp_sb = vp_sb; a.vp_sh = vp_sh; a.vp_st = vp_st;
    a.vn = (const uint16_t*)v_norms; a.vn_sb = vn_sb; a.vn_sh = vn_sh; a.vn_st = vn_st;
    a.ko = (uint16_t*)k_out; a.ko_sb = ko_sb; a.ko_sh = ko_sh; a.ko_st = ko_st;
    a.vo = (uint16_t*)v_out; a.vo_sb = vo_sb; a.vo_sh = vo_sh; a.vo_st = vo_st;
    a.T = T; a.k_layout = k_layout; a.v_layout = v_layout;
    a.k_row_width = k_row_width; a.v_row_width = v_row_width;
    const int krow = (k_row_width + ROW_PAD + 3) & ~3, vrow = (v_row_width + ROW_PAD + 3) & ~3;
    const size_t smem = (size_t)TOK * (BGTQ_MAX_SEGMENTS + 1) * 4 + (size_t)TOK * (krow + vrow);
    dim3 grid((unsigned)((T + TOK - 1) / TOK), (unsigned)n_kv, (unsigned)B);
    hipLaunchKernelGGL(dequant_kernel, grid, dim3(D), smem, (hipStream_t)stream, a);
    return bgtq_launch_status();
}
