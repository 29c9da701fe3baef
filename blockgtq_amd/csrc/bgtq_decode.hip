// Fused unpack + dequant + split-T decode attention, the partition merge, and
// the dense fp16 window partial, for gfx950.
//
// decode_generic_kernel is the layout-agnostic path: any segment table, both K
// layouts, both V layouts, any row stride.  One work-group of 256 threads owns
// one partition of one (batch row, KV head).  Per 256-token tile the packed K
// rows, K norms, packed V rows and V norms are staged into LDS with coalesced
// loads; thread t then scores token t against all query heads of the group
// (codes pulled out of the staged record with shift/mask, codebooks and the
// rotated queries read from LDS), the tile maximum is reduced across the
// work-group, and thread (d, half) accumulates output dim d for one half of
// the query heads over the tile's tokens.
#include "bgtq_common.h"
#include <mutex>

#include "bgtq_decode.h"

namespace {

constexpr int D = BGTQ_D;
constexpr int GT = 256;          // threads == tokens per tile of the generic kernel
constexpr int ROW_PAD = 4;       // slack bytes so a 2-byte window never leaves the tile


__device__ inline float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// code of width `bw` at absolute bit `bit` of a staged record
__device__ inline unsigned take_bits(const uint8_t* row, int bit, int bw) {
    int byte = bit >> 3;
    unsigned w = (unsigned)row[byte] | ((unsigned)row[byte + 1] << 8);
    return (w >> (bit & 7)) & ((1u << bw) - 1u);
}

template <int GQA_MAX>
__global__ __launch_bounds__(GT) void decode_generic_kernel(DecodeArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x;
    const int c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const bgtq_head_plan& P = a.plans[h];
    const int gqa = a.gqa;

    // (a length beyond the capacity the caller stated reads nothing past it)
    const int T = a.seq_lens ? min(max(a.seq_lens[b], 0), a.T) : a.T;
    const int chunk = (T + a.n_splits - 1) / a.n_splits;
    const int t0 = min(c * chunk, T);
    const int t1 = min(t0 + chunk, T);

    // ---- LDS carve-up ------------------------------------------------------
    const int krow = (a.k_row_width + ROW_PAD + 3) & ~3;
    const int vrow = (a.v_row_width + ROW_PAD + 3) & ~3;
    float* q_s = (float*)smem;                               // [GQA_MAX][D]
    float* cb_s = q_s + GQA_MAX * D;                         // [8][256]
    float* vlut_s = cb_s + BGTQ_MAX_SEGMENTS * BGTQ_MAX_CENTROIDS;  // [16]
    float* p_s = vlut_s + 16;                                // [GQA_MAX][GT]
    float* red_s = p_s + GQA_MAX * GT;                       // [GQA_MAX][4]
    float* alpha_s = red_s + GQA_MAX * 4;                    // [GQA_MAX] rescale of the tile
    float* fin_s = alpha_s + GQA_MAX;                        // [2][GQA_MAX] final m, l
    float* kn_s = fin_s + 2 * GQA_MAX;                       // [GT][8]
    float* vn_s = kn_s + GT * BGTQ_MAX_SEGMENTS;             // [GT]
    uint32_t* dim_s = (uint32_t*)(vn_s + GT);                // [D] bit | bw<<16 | seg<<24
    uint8_t* krow_s = (uint8_t*)(dim_s + D);                 // [GT][krow]
    uint8_t* vrow_s = krow_s + (size_t)GT * krow;            // [GT][vrow]

    // ---- static tables -----------------------------------------------------
    for (int i = tid; i < gqa * D; i += GT) {
        int hq = i / D, d = i - hq * D;
        q_s[i] = bgtq_h2f(a.q[b * a.q_sb + (h * gqa + hq) * a.q_sh + d]);
    }
    for (int i = tid; i < BGTQ_MAX_SEGMENTS * BGTQ_MAX_CENTROIDS; i += GT)
        cb_s[i] = bgtq_h2f(P.k_codebook_f16[i >> 8][i & 255]);
    if (tid < 16) vlut_s[tid] = bgtq_h2f(P.v_lut_f16[tid]);
    if (tid < D) {
        int g = P.group_of[tid];
        uint32_t e = 0xFFFFFFFFu;
        if (g >= 0) {
            int bw = P.seg_bw[g], rel = tid - P.seg_start[g];
            int bit, xbw;
            if (a.k_layout == BGTQ_K_MIXED) {
                if (bw <= 4) { bit = (tid - P.n_zero_dims) * 4; xbw = 4; }
                else         { bit = (P.seg_mixed_off[g] + rel) * 8; xbw = 8; }
            } else {
                if (bw <= 4) { bit = P.seg_pack_off[g] * 8 + rel * bw; xbw = bw; }
                else         { bit = (P.seg_pack_off[g] + rel) * 8; xbw = 8; }
            }
            e = (uint32_t)bit | ((uint32_t)xbw << 16) | ((uint32_t)g << 24);
        }
        dim_s[tid] = e;
    }
    const int n_seg = P.n_seg;
    const int kbytes = min((a.k_layout == BGTQ_K_MIXED) ? P.k_mixed_bytes : P.k_row_bytes,
                           a.k_row_width);
    const int vbw = (a.v_layout == BGTQ_V_NIBBLE) ? 4 : P.v_bits;
    const int vbytes = min(bgtq_seg_bytes(vbw, D), a.v_row_width);

    const uint8_t* kp_base = a.kp + b * a.kp_sb + h * a.kp_sh;
    const uint16_t* kn_base = a.kn + b * a.kn_sb + h * a.kn_sh;
    const uint8_t* vp_base = a.vp + b * a.vp_sb + h * a.vp_sh;
    const uint16_t* vn_base = a.vn + b * a.vn_sb + h * a.vn_sh;

    // running softmax state (replicated in every thread) and output accumulators
    float m_run[GQA_MAX], l_run[GQA_MAX];
    const int hhalf = (GQA_MAX + 1) / 2;         // heads per PV thread
    float acc[(GQA_MAX + 1) / 2];
#pragma unroll
    for (int i = 0; i < GQA_MAX; i++) { m_run[i] = -INFINITY; l_run[i] = 0.f; }
#pragma unroll
    for (int i = 0; i < hhalf; i++) acc[i] = 0.f;
    const int pv_d = tid & (D - 1);
    const int pv_h0 = (tid >> 7) * hhalf;

    for (int tile = t0; tile < t1; tile += GT) {
        const int nt = min(GT, t1 - tile);
        __syncthreads();   // previous tile fully consumed (also orders the static tables)
        // ---- stage the tile -----------------------------------------------
        for (int i = tid; i < nt * kbytes; i += GT) {
            int t = i / kbytes, o = i - t * kbytes;
            krow_s[t * krow + o] = kp_base[(int64_t)(tile + t) * a.kp_st + o];
        }
        for (int i = tid; i < nt * vbytes; i += GT) {
            int t = i / vbytes, o = i - t * vbytes;
            vrow_s[t * vrow + o] = vp_base[(int64_t)(tile + t) * a.vp_st + o];
        }
        for (int i = tid; i < nt * n_seg; i += GT) {
            int t = i / n_seg, g = i - t * n_seg;
            kn_s[t * BGTQ_MAX_SEGMENTS + g] = bgtq_h2f(kn_base[(int64_t)(tile + t) * a.kn_st + g]);
        }
        if (tid < nt) vn_s[tid] = bgtq_h2f(vn_base[(int64_t)(tile + tid) * a.vn_st]);
        __syncthreads();

        // ---- scores: thread = token ------------------------------------------
        float logit[GQA_MAX];
#pragma unroll
        for (int i = 0; i < GQA_MAX; i++) logit[i] = -INFINITY;
        if (tid < nt) {
            const uint8_t* row = krow_s + tid * krow;
            float tot[GQA_MAX], part[GQA_MAX];
#pragma unroll
            for (int i = 0; i < GQA_MAX; i++) { tot[i] = 0.f; part[i] = 0.f; }
            int cur = -1;
            for (int d = P.n_zero_dims; d < D; d++) {
                uint32_t e = dim_s[d];
                int g = (int)(e >> 24);
                if (g != cur) {
                    if (cur >= 0) {
                        float n = kn_s[tid * BGTQ_MAX_SEGMENTS + cur];
#pragma unroll
                        for (int i = 0; i < GQA_MAX; i++) { tot[i] += part[i] * n; part[i] = 0.f; }
                    }
                    cur = g;
                }
                unsigned code = take_bits(row, (int)(e & 0xFFFFu), (int)((e >> 16) & 0xFFu));
                float cv = cb_s[g * BGTQ_MAX_CENTROIDS + code];
#pragma unroll
                for (int i = 0; i < GQA_MAX; i++)
                    if (i < gqa) part[i] += q_s[i * D + d] * cv;
            }
            if (cur >= 0) {
                float n = kn_s[tid * BGTQ_MAX_SEGMENTS + cur];
#pragma unroll
                for (int i = 0; i < GQA_MAX; i++) tot[i] += part[i] * n;
            }
#pragma unroll
            for (int i = 0; i < GQA_MAX; i++) logit[i] = tot[i] * a.scale;
        }

        // ---- tile maximum per head (work-group reduce) -------------------------
#pragma unroll
        for (int i = 0; i < GQA_MAX; i++) {
            float m = wave_max(logit[i]);
            if ((tid & 63) == 0) red_s[i * 4 + (tid >> 6)] = m;
        }
        __syncthreads();
        float alpha[GQA_MAX];
#pragma unroll
        for (int i = 0; i < GQA_MAX; i++) {
            float m = fmaxf(fmaxf(red_s[i * 4], red_s[i * 4 + 1]),
                            fmaxf(red_s[i * 4 + 2], red_s[i * 4 + 3]));
            float m_new = fmaxf(m_run[i], m);
            alpha[i] = (m_run[i] == -INFINITY) ? 0.f : __expf(m_run[i] - m_new);
            m_run[i] = m_new;
            float p = (tid < nt && i < gqa) ? __expf(logit[i] - m_new) : 0.f;
            p_s[i * GT + tid] = p * ((tid < nt) ? vn_s[tid] : 0.f);   // V norm folded into p
            logit[i] = p;
            if (tid == 0) alpha_s[i] = alpha[i];
        }
        __syncthreads();   // red_s consumed, p_s visible
#pragma unroll
        for (int i = 0; i < GQA_MAX; i++) {
            float s = wave_sum(logit[i]);
            if ((tid & 63) == 0) red_s[i * 4 + (tid >> 6)] = s;
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < GQA_MAX; i++) {
            float s = red_s[i * 4] + red_s[i * 4 + 1] + red_s[i * 4 + 2] + red_s[i * 4 + 3];
            l_run[i] = l_run[i] * alpha[i] + s;
        }

        // ---- values: thread = (dim, half of the heads) ------------------------
#pragma unroll
        for (int i = 0; i < hhalf; i++)
            if (pv_h0 + i < GQA_MAX) acc[i] *= alpha_s[pv_h0 + i];
        for (int t = 0; t < nt; t++) {
            unsigned code = take_bits(vrow_s + t * vrow, pv_d * vbw, vbw);
            float val = vlut_s[code];
#pragma unroll
            for (int i = 0; i < hhalf; i++)
                if (pv_h0 + i < GQA_MAX) acc[i] += p_s[(pv_h0 + i) * GT + t] * val;
        }
    }

    // ---- partition result --------------------------------------------------------
    __syncthreads();
    if (tid == 0) {
#pragma unroll
        for (int i = 0; i < GQA_MAX; i++) { fin_s[i] = m_run[i]; fin_s[GQA_MAX + i] = l_run[i]; }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < hhalf; i++) {
        int hq = pv_h0 + i;
        if (hq < gqa) {
            float l = fin_s[GQA_MAX + hq];
            float o = (t1 > t0) ? acc[i] / l : 0.f;
            size_t row = ((size_t)b * a.n_kv * gqa + (size_t)h * gqa + hq) * a.n_splits + c;
            a.part_out[row * D + pv_d] = o;
        }
    }
    if (tid < gqa) {
        float lse = (t1 > t0) ? fin_s[tid] + __logf(fin_s[GQA_MAX + tid]) : -INFINITY;
        size_t row = ((size_t)b * a.n_kv * gqa + (size_t)h * gqa + tid) * a.n_splits + c;
        a.part_lse[row] = lse;
    }
}

size_t generic_smem_bytes(int gqa_max, int krow_bytes, int vrow_bytes) {
    size_t krow = (size_t)((krow_bytes + ROW_PAD + 3) & ~3);
    size_t vrow = (size_t)((vrow_bytes + ROW_PAD + 3) & ~3);
    size_t f = (size_t)gqa_max * D + BGTQ_MAX_SEGMENTS * BGTQ_MAX_CENTROIDS + 16 +
               (size_t)gqa_max * GT + (size_t)gqa_max * 7 + (size_t)GT * BGTQ_MAX_SEGMENTS + GT + D;
    return f * 4 + (size_t)GT * (krow + vrow) + 16;
}

template <int GQA_MAX>
int launch_generic(const DecodeArgs& a, hipStream_t st) {
    size_t smem = generic_smem_bytes(GQA_MAX, a.k_row_width, a.v_row_width);
    auto kern = decode_generic_kernel<GQA_MAX>;
    if (smem > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)kern,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return (int)e;
    }
    dim3 grid((unsigned)a.n_splits, (unsigned)a.n_kv, (unsigned)a.B);
    hipLaunchKernelGGL(kern, grid, dim3(GT), smem, st, a);
    return bgtq_launch_status();
}

// ---- partition merge + V un-rotation ------------------------------------------
// One work-group of NTHR threads per (batch row, query head).  Its loads are 16 bytes a lane
// and contiguous across the wave: thread t holds columns 4(t & 31) .. +3 of the rows
// r = t >> 5 (mod NTHR / 32) of the partial vectors and of the un-rotation, sums over its own
// rows, and the NTHR / 32 row classes are added through LDS (in a fixed order, so the result
// does not depend on timing).  Every load that does not depend on a computed value
// (the first round of partial vectors, the whole un-rotation) is issued up front, so the
// kernel pays for about one memory round trip.  512 threads (16 classes: 8 rows of the
// un-rotation a thread instead of 32) where the launch has at most one work-group per compute
// unit, 128 threads where work-groups queue up.
static_assert(offsetof(bgtq_head_plan, v_rot) % 16 == 0 && sizeof(bgtq_head_plan) % 16 == 0,
              "the un-rotation is read 16 bytes at a time");
template <int RT_THREADS>
__global__ __launch_bounds__(RT_THREADS) void lse_reduce_kernel(
    const bgtq_head_plan* plans, const float* part_out, const float* part_lse, int n_splits,
    const float* extra_out, const float* extra_lse, int n_extra,
    int n_q, int gqa, int unrotate, uint16_t* out, int64_t o_sb, int64_t o_sh, float* lse_out) {
    constexpr int RT_CLASSES = RT_THREADS / 32;
    __shared__ __align__(16) float cls_sum[RT_CLASSES][D];
    __shared__ float vec[D];
    __shared__ float wgt[BGTQ_MAX_SPLITS];
    __shared__ float red[RT_THREADS / 64];
    __shared__ float dsum[RT_CLASSES];
    const int j = threadIdx.x;
    const int cls = j >> 5, c4 = (j & 31) * 4;
    const int hq = blockIdx.x, b = blockIdx.y;
    const size_t row = (size_t)b * n_q + hq;
    const float* pl = part_lse + row * n_splits;
    const float* el = extra_lse ? extra_lse + row * n_extra : nullptr;
    const float* R = plans[hq / gqa].v_rot;
    const float* po = part_out + row * n_splits * D + c4;

    // loads land in issue order: the partitions' log-sum-exps go first, so that the maximum and
    // the weights are worked out while the vectors and the un-rotation are still on their way
    const float l_first = j < n_splits ? pl[j] : -INFINITY;
    constexpr int NB = 16 / RT_CLASSES;        // rounds of partial vectors fetched before anything else (16 vectors)
    float4 pv[NB];
#pragma unroll
    for (int i = 0; i < NB; i++) pv[i] = *(const float4*)(po + (size_t)min(RT_CLASSES * i + cls, n_splits - 1) * D);
    float4 rv[D / RT_CLASSES];                 // rows 16 i + cls of the un-rotation, this thread's four columns
    if (unrotate) {
#pragma unroll
        for (int i = 0; i < D / RT_CLASSES; i++) rv[i] = *(const float4*)(R + (RT_CLASSES * i + cls) * D + c4);
    }

    float m = l_first;
    if (j < n_splits) wgt[j] = l_first;
    for (int c = j + RT_THREADS; c < n_splits; c += RT_THREADS) { float l = pl[c]; wgt[c] = l; m = fmaxf(m, l); }
    for (int c = j; c < n_extra; c += RT_THREADS) m = fmaxf(m, el[c]);
    m = wave_max(m);
    if ((j & 63) == 0) red[j >> 6] = m;
    __syncthreads();
    m = red[0];
#pragma unroll
    for (int i = 1; i < RT_THREADS / 64; i++) m = fmaxf(m, red[i]);
    if (m == -INFINITY) {                      // nothing visible at all
        if (j < D) out[b * o_sb + hq * o_sh + j] = 0;
        if (lse_out && j == 0) lse_out[row] = -INFINITY;
        return;
    }
    // weights: exp(lse - m), 0 for empty partitions (their vectors are undefined)
    for (int c = j; c < n_splits; c += RT_THREADS) { float l = wgt[c]; wgt[c] = (l == -INFINITY) ? 0.f : __expf(l - m); }
    __syncthreads();
    float dcl = 0.f;                           // weight sum of this thread's row class
    float4 a4 = {0.f, 0.f, 0.f, 0.f};
    auto add = [&](float w, const float4& v) {
        dcl += w;
        if (w != 0.f) { a4.x += w * v.x; a4.y += w * v.y; a4.z += w * v.z; a4.w += w * v.w; }
    };
#pragma unroll
    for (int i = 0; i < NB; i++)
        if (RT_CLASSES * i + cls < n_splits) add(wgt[RT_CLASSES * i + cls], pv[i]);
    for (int c = RT_CLASSES * NB + cls; c < n_splits; c += RT_CLASSES) add(wgt[c], *(const float4*)(po + (size_t)c * D));
    *(float4*)&cls_sum[cls][c4] = a4;
    if ((j & 31) == 0) dsum[cls] = dcl;
    float acce = 0.f, den = 0.f;
    if (j < D)
        for (int e = 0; e < n_extra; e++) {
            float l = el[e];
            if (l == -INFINITY) continue;
            float w = __expf(l - m);
            den += w;
            acce += w * extra_out[(row * n_extra + e) * D + j];
        }
    __syncthreads();
    // the classes are added pairwise in a fixed order
    auto fold = [&](const float (*t)[D], int col) {
        float s[RT_CLASSES];
#pragma unroll
        for (int i = 0; i < RT_CLASSES; i++) s[i] = t[i][col];
#pragma unroll
        for (int w = RT_CLASSES / 2; w >= 1; w >>= 1)
#pragma unroll
            for (int i = 0; i < w; i++) s[i] = s[2 * i] + s[2 * i + 1];
        return s[0];
    };
    float res = 0.f;
    if (j < D) {
        float ds[RT_CLASSES];
#pragma unroll
        for (int i = 0; i < RT_CLASSES; i++) ds[i] = dsum[i];
#pragma unroll
        for (int w = RT_CLASSES / 2; w >= 1; w >>= 1)
#pragma unroll
            for (int i = 0; i < w; i++) ds[i] = ds[2 * i] + ds[2 * i + 1];
        den += ds[0];
        res = fold(cls_sum, j);
    }
    if (unrotate) {
        if (j < D) vec[j] = res;
        __syncthreads();                       // also: every read of cls_sum above is done
        float4 r4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < D / RT_CLASSES; i++) {
            const float x = vec[RT_CLASSES * i + cls];
            r4.x += x * rv[i].x; r4.y += x * rv[i].y; r4.z += x * rv[i].z; r4.w += x * rv[i].w;
        }
        *(float4*)&cls_sum[cls][c4] = r4;
        __syncthreads();
        if (j < D) res = fold(cls_sum, j);
    }
    if (j < D) {
        out[b * o_sb + hq * o_sh + j] = bgtq_f2h((res + acce) / den);
        if (lse_out && j == 0) lse_out[row] = m + __logf(den);
    }
}


// ---- dense fp16 partial over the sink + recent-window tokens ------------------
constexpr int WT = 256;
__global__ __launch_bounds__(WT) void window_attn_generic_kernel(
    const uint16_t* q, int64_t q_sb, int64_t q_sh,
    const uint16_t* kbuf, const uint16_t* vbuf, int64_t w_sb, int64_t w_sh, int64_t w_st,
    const int32_t* lens, int W, int n_q, int gqa, float scale, float* part_out, float* part_lse) {
    extern __shared__ float wlog[];            // [W] logits, then weights
    __shared__ float q_s[D];
    __shared__ float red[WT / 64];
    const int tid = threadIdx.x;
    const int hq = blockIdx.x, b = blockIdx.y, h = hq / gqa;
    const int n = lens ? min(lens[b], W) : W;
    const size_t row = (size_t)b * n_q + hq;
    if (tid < D) q_s[tid] = bgtq_h2f(q[b * q_sb + hq * q_sh + tid]);
    __syncthreads();
    const uint16_t* kb = kbuf + b * w_sb + h * w_sh;
    const uint16_t* vb = vbuf + b * w_sb + h * w_sh;
    float m = -INFINITY;
    for (int t = tid; t < n; t += WT) {
        const uint16_t* kr = kb + (int64_t)t * w_st;
        float acc = 0.f;
        for (int d = 0; d < D; d++) acc += q_s[d] * bgtq_h2f(kr[d]);
        acc *= scale;
        wlog[t] = acc;
        m = fmaxf(m, acc);
    }
    m = wave_max(m);
    if ((tid & 63) == 0) red[tid >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float l = 0.f;
    for (int t = tid; t < n; t += WT) {
        float p = __expf(wlog[t] - m);
        wlog[t] = p;
        l += p;
    }
    l = wave_sum(l);
    if ((tid & 63) == 0) red[tid >> 6] = l;
    __syncthreads();
    l = red[0] + red[1] + red[2] + red[3];
    if (tid < D) {
        float acc = 0.f;
        for (int t = 0; t < n; t++) acc += wlog[t] * bgtq_h2f(vb[(int64_t)t * w_st + tid]);
        part_out[row * D + tid] = n > 0 ? acc / l : 0.f;
    }
    if (tid == 0) part_lse[row] = n > 0 ? m + __logf(l) : -INFINITY;
}


// The same partial for buffers whose rows start on 16-byte boundaries (the manager's do): one
// work-group per (batch row, KV head) serves all its query heads, HG at a time, so the window is
// read once per HG heads, and every load is contiguous across the wave.  Scores: 16 lanes share a
// token (8 dims each, one 16-byte load), 4 tokens per wave instruction; values: a wave covers
// one token row per load (2 dims a lane), the four waves take every fourth token and their sums
// meet in LDS.  wlog holds HG rows of W scores, then weights.
// sum over the 16 lanes of a row, in every lane of it (rotations within the row: no LDS traffic)
__device__ __forceinline__ float row16_sum(float x) {
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x128, 0xf, 0xf, false));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x124, 0xf, 0xf, false));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x122, 0xf, 0xf, false));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x121, 0xf, 0xf, false));
    return x;
}

template <int HG>
__global__ __launch_bounds__(WT) void window_attn_kernel(
    const uint16_t* q, int64_t q_sb, int64_t q_sh,
    const uint16_t* kbuf, const uint16_t* vbuf, int64_t w_sb, int64_t w_sh, int64_t w_st,
    const int32_t* lens, int W, int n_q, int gqa, float scale, float* part_out, float* part_lse) {
    extern __shared__ float wlog[];            // [HG][W]
    __shared__ float red_m[HG], red_l[HG];
    __shared__ float osum[WT / 64][HG][D];
    constexpr int NW = WT / 64;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int h = blockIdx.x, b = blockIdx.y;
    const int n = lens ? min(lens[b], W) : W;
    const uint16_t* kb = kbuf + b * w_sb + h * w_sh;
    const uint16_t* vb = vbuf + b * w_sb + h * w_sh;
    const int sub = lane & 15, tq = lane >> 4;  // scores: dim chunk and token within a wave load
    // Loads run one batch ahead of the arithmetic that uses them (a batch waited for on the spot
    // costs a trip to memory each); small batches in rolled loops measured as fast as large
    // unrolled ones.
    constexpr int SB = 3;                       // score passes (4 tokens per wave each) per batch
    constexpr int PB = 8;                       // value rows per batch
    auto fetch_k = [&](uint4 (&k4)[SB], const int t0) {
#pragma unroll
        for (int u = 0; u < SB; u++) {
            const int t = t0 + u * 4 * NW + tq;
            k4[u] = uint4{0, 0, 0, 0};
            if (t < n) k4[u] = *(const uint4*)(kb + (int64_t)t * w_st + sub * 8);
        }
    };
    auto fetch_v = [&](uint32_t (&vv)[PB], const int t0) {
#pragma unroll
        for (int u = 0; u < PB; u++) {
            const int t = t0 + u * NW;
            vv[u] = t < n ? *(const uint32_t*)(vb + (int64_t)t * w_st + 2 * lane) : 0u;
        }
    };
    for (int g0 = 0; g0 < gqa; g0 += HG) {
        const int ng = min(HG, gqa - g0);
        // ---- scores: 16 lanes share a token ------------------------------------------------
        float qf[HG][8];
#pragma unroll
        for (int g = 0; g < HG; g++) {
            uint4 w4 = {0, 0, 0, 0};
            if (g < ng) w4 = *(const uint4*)(q + b * q_sb + (int64_t)(h * gqa + g0 + g) * q_sh + sub * 8);
            const uint32_t ws[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                qf[g][2 * i] = bgtq_h2f((uint16_t)(ws[i] & 0xFFFFu)) * scale;
                qf[g][2 * i + 1] = bgtq_h2f((uint16_t)(ws[i] >> 16)) * scale;
            }
        }
        uint4 kc[SB], kn[SB];
        uint32_t vc[PB], vn[PB];
        fetch_k(kc, wave * 4);
        fetch_v(vc, wave);                      // the first value rows do not wait for the scores
#pragma unroll 1
        for (int t0 = wave * 4; t0 < n; t0 += SB * 4 * NW) {
            fetch_k(kn, t0 + SB * 4 * NW);
#pragma unroll
            for (int u = 0; u < SB; u++) {
                const int t = t0 + u * 4 * NW + tq;
                const uint32_t ks[4] = {kc[u].x, kc[u].y, kc[u].z, kc[u].w};
                float kf[8];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    kf[2 * i] = bgtq_h2f((uint16_t)(ks[i] & 0xFFFFu));
                    kf[2 * i + 1] = bgtq_h2f((uint16_t)(ks[i] >> 16));
                }
#pragma unroll
                for (int g = 0; g < HG; g++) {
                    float acc = 0.f;
#pragma unroll
                    for (int i = 0; i < 8; i++) acc += qf[g][i] * kf[i];
                    acc = row16_sum(acc);
                    if (sub == 0 && t < n && g < ng) wlog[g * W + t] = acc;
                }
            }
#pragma unroll
            for (int u = 0; u < SB; u++) kc[u] = kn[u];
        }
        __syncthreads();
        // ---- softmax weights: wave w owns heads w, w + 4, ... ----------------------------------
        for (int g = wave; g < ng; g += NW) {
            float mm = -INFINITY;
            for (int t = lane; t < n; t += 64) mm = fmaxf(mm, wlog[g * W + t]);
            mm = wave_max(mm);
            float ll = 0.f;
            for (int t = lane; t < n; t += 64) {
                const float p = __expf(wlog[g * W + t] - mm);
                wlog[g * W + t] = p;
                ll += p;
            }
            ll = wave_sum(ll);
            if (lane == 0) { red_m[g] = mm; red_l[g] = ll; }
        }
        __syncthreads();
        // ---- values: wave w takes tokens w, w + 4, ...; lane = dims 2 lane, 2 lane + 1 -------
        float o0[HG], o1[HG];
#pragma unroll
        for (int g = 0; g < HG; g++) o0[g] = o1[g] = 0.f;
#pragma unroll 1
        for (int t0 = wave; t0 < n; t0 += PB * NW) {
            fetch_v(vn, t0 + PB * NW);
            float pw[PB][HG];                   // the batch's weights, read together
#pragma unroll
            for (int u = 0; u < PB; u++)
#pragma unroll
                for (int g = 0; g < HG; g++) {
                    const int t = min(t0 + u * NW, n - 1);
                    pw[u][g] = wlog[min(g, ng - 1) * W + t];
                }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < PB; u++) {
                const bool live = t0 + u * NW < n;
                const float v0 = bgtq_h2f((uint16_t)(vc[u] & 0xFFFFu)), v1 = bgtq_h2f((uint16_t)(vc[u] >> 16));
#pragma unroll
                for (int g = 0; g < HG; g++) {
                    const float p = (g < ng && live) ? pw[u][g] : 0.f;
                    o0[g] += p * v0;
                    o1[g] += p * v1;
                }
            }
#pragma unroll
            for (int u = 0; u < PB; u++) vc[u] = vn[u];
        }
#pragma unroll
        for (int g = 0; g < HG; g++) { osum[wave][g][2 * lane] = o0[g]; osum[wave][g][2 * lane + 1] = o1[g]; }
        __syncthreads();
        for (int i = tid; i < ng * D; i += WT) {
            const int g = i / D, d = i - g * D;
            const float acc = (osum[0][g][d] + osum[1][g][d]) + (osum[2][g][d] + osum[3][g][d]);
            const size_t row = (size_t)b * n_q + h * gqa + g0 + g;
            const float mg = red_m[g], lg = red_l[g];
            part_out[row * D + d] = n > 0 ? acc / lg : 0.f;
            if (d == 0) part_lse[row] = n > 0 ? mg + __logf(lg) : -INFINITY;
        }
        __syncthreads();                        // wlog, red_* and osum are reused by the next heads
    }
}

// ---- with-buffer append: the token in ring slot slot[b] leaves, this step's token enters -----
// One work-group per (KV head, batch row), thread j moves dim j of K and of V.  A slot outside
// [0, W) moves nothing and leaves zeros in the outputs.
__global__ __launch_bounds__(D) void window_swap_kernel(
    uint16_t* kbuf, uint16_t* vbuf, int64_t w_sb, int64_t w_sh, int64_t w_st,
    const uint16_t* new_k, const uint16_t* new_v, int64_t n_sb, int64_t n_sh,
    const int32_t* slot, int W, int n_kv, uint16_t* old_k, uint16_t* old_v) {
    const int j = threadIdx.x, h = blockIdx.x, b = blockIdx.y;
    const int sl = slot[b];
    const int64_t o = ((int64_t)b * n_kv + h) * D + j;
    if (sl < 0 || sl >= W) { old_k[o] = 0; old_v[o] = 0; return; }
    const int64_t at = b * w_sb + h * w_sh + (int64_t)sl * w_st + j;
    const int64_t nw = b * n_sb + h * n_sh + j;
    const uint16_t nk = new_k[nw], nv = new_v[nw];
    old_k[o] = kbuf[at];
    old_v[o] = vbuf[at];
    kbuf[at] = nk;
    vbuf[at] = nv;
}

}  // namespace

static int g_decode_path = 0;
static int g_last_path = 0;      // kernel the last attention call ran: 1 layout-agnostic, 2 MFMA

// ---- partition results of bgtq_decode_attend_static ------------------------------------------
// The partial vectors and log-sum-exps of the entry point that allocates nothing live in
// this array: one copy per GPU the library runs on, held until the process ends.  Host code
// never uses the array's name as an address; it asks the runtime once per device for the
// device address of that GPU's copy and passes that to the kernels.
static __device__ __align__(256) unsigned char scratch[BGTQ_STATIC_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[MAX_DEVICES];        // device address of `scratch` on device i, once known

// Device address of the current device's scratch array (asked for on the first call on
// that device, with that device current).
int scratch_of_current_device(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES) return BGTQ_ELIMIT;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return BGTQ_EINVAL;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return BGTQ_OK;
}
}  // namespace

extern "C" {

int bgtq_last_decode_path(void) { return g_last_path; }

int bgtq_set_decode_path(int path) {
    if (path < 0 || path > 2) return BGTQ_EINVAL;
    g_decode_path = path;
    return BGTQ_OK;
}

size_t bgtq_workspace_bytes(int B, int n_q, int n_splits) {
    if (B <= 0 || n_q <= 0 || n_splits <= 0) return 0;
    return (size_t)B * n_q * n_splits * (D + 1) * sizeof(float);
}

int bgtq_default_splits(int B, int n_kv, int max_T) {
    // One work-group per partition and the fast kernel keeps a whole CU busy with
    // one work-group, so aim for one partition per CU (256 of them), but never
    // fewer than 128 tokens per partition.
    if (B <= 0 || n_kv <= 0 || max_T <= 0) return 1;
    int by_tokens = (max_T + 127) / 128;
    int want = (256 + B * n_kv - 1) / (B * n_kv);
    int s = want < by_tokens ? want : by_tokens;
    if (s < 1) s = 1;
    if (s > BGTQ_MAX_SPLITS) s = BGTQ_MAX_SPLITS;
    return s;
}

int bgtq_decode_attn(const bgtq_head_plan* plans,
                     const void* q_rot, int64_t q_sb, int64_t q_sh,
                     const void* k_packed, int64_t kp_sb, int64_t kp_sh, int64_t kp_st, int k_row_width,
                     const void* k_norms, int64_t kn_sb, int64_t kn_sh, int64_t kn_st,
                     const void* v_packed, int64_t vp_sb, int64_t vp_sh, int64_t vp_st, int v_row_width,
                     const void* v_norms, int64_t vn_sb, int64_t vn_sh, int64_t vn_st,
                     const int32_t* seq_lens, int T,
                     int B, int n_kv, int gqa, int n_splits,
                     float* partial_out, float* partial_lse,
                     int k_layout, int v_layout, float scale, void* stream) {
    BGTQ_CHECK_ARG(plans && q_rot && k_packed && k_norms && v_packed && v_norms);
    BGTQ_CHECK_ARG(partial_out && partial_lse);
    BGTQ_CHECK_ARG(B >= 0 && n_kv >= 0 && T >= 0);
    BGTQ_CHECK_ARG(gqa >= 1 && gqa <= BGTQ_MAX_GQA);
    BGTQ_CHECK_ARG(k_layout == BGTQ_K_BITPACKED || k_layout == BGTQ_K_MIXED);
    BGTQ_CHECK_ARG(v_layout == BGTQ_V_BITPACKED || v_layout == BGTQ_V_NIBBLE);
    if (n_splits > BGTQ_MAX_SPLITS) return BGTQ_ELIMIT;
    BGTQ_CHECK_ARG(n_splits >= 1);
    if (B == 0 || n_kv == 0) return BGTQ_OK;
    DecodeArgs a{};
    a.plans = plans;
    a.q = (const uint16_t*)q_rot; a.q_sb = q_sb; a.q_sh = q_sh;
    a.kp = (const uint8_t*)k_packed; a.kp_sb = kp_sb; a.kp_sh = kp_sh; a.kp_st = kp_st;
    a.kn = (const uint16_t*)k_norms; a.kn_sb = kn_sb; a.kn_sh = kn_sh; a.kn_st = kn_st;
    a.vp = (const uint8_t*)v_packed; a.vp_sb = vp_sb; a.vp_sh = vp_sh; a.vp_st = vp_st;
    a.vn = (const uint16_t*)v_norms; a.vn_sb = vn_sb; a.vn_sh = vn_sh; a.vn_st = vn_st;
    a.seq_lens = seq_lens; a.T = T;
    a.B = B; a.n_kv = n_kv; a.gqa = gqa; a.n_splits = n_splits;
    a.part_out = partial_out; a.part_lse = partial_lse;
    a.k_layout = k_layout; a.v_layout = v_layout; a.scale = scale;
    BGTQ_CHECK_ARG(k_row_width >= 1 && k_row_width <= BGTQ_D);
    BGTQ_CHECK_ARG(v_row_width >= 1 && v_row_width <= BGTQ_D / 2);
    a.k_row_width = k_row_width; a.v_row_width = v_row_width;
    hipStream_t st = (hipStream_t)stream;
    if (g_decode_path != 1) {
        int rc = bgtq_launch_decode_seg(a, st);
        if (rc != BGTQ_EUNSUPPORTED) { g_last_path = 2; return rc; }
        if (g_decode_path == 2) return rc;        // forced fast path: report why it refused
    }
    g_last_path = 1;
    if (gqa <= 4) return launch_generic<4>(a, st);
    if (gqa <= 8) return launch_generic<8>(a, st);
    return launch_generic<16>(a, st);
}

int bgtq_lse_reduce(const bgtq_head_plan* plans,
                    const float* partial_out, const float* partial_lse, int n_splits,
                    const float* extra_out, const float* extra_lse, int n_extra,
                    int B, int n_kv, int gqa, int unrotate,
                    void* out, int64_t o_sb, int64_t o_sh,
                    float* lse_out, void* stream) {
    BGTQ_CHECK_ARG(plans && partial_out && partial_lse && out);
    BGTQ_CHECK_ARG(B >= 0 && n_kv >= 0 && gqa >= 1 && n_splits >= 1 && n_extra >= 0);
    BGTQ_CHECK_ARG(n_extra == 0 || (extra_out && extra_lse));
    // the kernel reads the partial vectors and the plan 16 bytes at a time
    BGTQ_CHECK_ARG(((uintptr_t)partial_out & 15) == 0 && ((uintptr_t)plans & 15) == 0);
    if (n_splits > BGTQ_MAX_SPLITS) return BGTQ_ELIMIT;
    if (B == 0 || n_kv == 0) return BGTQ_OK;
    dim3 grid((unsigned)(n_kv * gqa), (unsigned)B);
    if ((int64_t)B * n_kv * gqa <= 256)
        hipLaunchKernelGGL(lse_reduce_kernel<512>, grid, dim3(512), 0, (hipStream_t)stream,
                           plans, partial_out, partial_lse, n_splits,
                           n_extra ? extra_out : nullptr, n_extra ? extra_lse : nullptr, n_extra,
                           n_kv * gqa, gqa, unrotate, (uint16_t*)out, o_sb, o_sh, lse_out);
    else
        hipLaunchKernelGGL(lse_reduce_kernel<128>, grid, dim3(128), 0, (hipStream_t)stream,
                           plans, partial_out, partial_lse, n_splits,
                           n_extra ? extra_out : nullptr, n_extra ? extra_lse : nullptr, n_extra,
                           n_kv * gqa, gqa, unrotate, (uint16_t*)out, o_sb, o_sh, lse_out);
    return bgtq_launch_status();
}

int bgtq_decode_attend_static(const bgtq_head_plan* plans,
                              const void* q_rot, int64_t q_sb, int64_t q_sh,
                              const void* k_packed, int64_t kp_sb, int64_t kp_sh, int64_t kp_st, int k_row_width,
                              const void* k_norms, int64_t kn_sb, int64_t kn_sh, int64_t kn_st,
                              const void* v_packed, int64_t vp_sb, int64_t vp_sh, int64_t vp_st, int v_row_width,
                              const void* v_norms, int64_t vn_sb, int64_t vn_sh, int64_t vn_st,
                              const int32_t* seq_lens, int T,
                              int B, int n_kv, int gqa, int n_splits,
                              int k_layout, int v_layout, float scale, int unrotate,
                              void* out, int64_t o_sb, int64_t o_sh, float* lse_out, void* stream) {
    BGTQ_CHECK_ARG(out);
    BGTQ_CHECK_ARG(B >= 0 && n_kv >= 0 && gqa >= 1 && gqa <= BGTQ_MAX_GQA);
    if (n_splits <= 0) n_splits = bgtq_default_splits(B, n_kv, T > 0 ? T : 1);
    if (n_splits > BGTQ_MAX_SPLITS) return BGTQ_ELIMIT;
    if (B == 0 || n_kv == 0) return BGTQ_OK;
    const size_t rows = (size_t)B * n_kv * gqa * n_splits;         // (batch row, query head, partition)
    if (bgtq_workspace_bytes(B, n_kv * gqa, n_splits) > (size_t)BGTQ_STATIC_SCRATCH_BYTES) return BGTQ_ELIMIT;
    void* base = nullptr;
    int rc = scratch_of_current_device(&base);
    if (rc != BGTQ_OK) return rc;
    float* part_out = (float*)base;                                 // [rows][128], 16-byte aligned
    float* part_lse = part_out + rows * D;                          // [rows]
    rc = bgtq_decode_attn(plans, q_rot, q_sb, q_sh, k_packed, kp_sb, kp_sh, kp_st, k_row_width,
                          k_norms, kn_sb, kn_sh, kn_st, v_packed, vp_sb, vp_sh, vp_st, v_row_width,
                          v_norms, vn_sb, vn_sh, vn_st, seq_lens, T, B, n_kv, gqa, n_splits,
                          part_out, part_lse, k_layout, v_layout, scale, stream);
    if (rc != BGTQ_OK) return rc;
    return bgtq_lse_reduce(plans, part_out, part_lse, n_splits, nullptr, nullptr, 0,
                           B, n_kv, gqa, unrotate, out, o_sb, o_sh, lse_out, stream);
}

int bgtq_window_attn(const void* q, int64_t q_sb, int64_t q_sh,
                     const void* kbuf, const void* vbuf,
                     int64_t w_sb, int64_t w_sh, int64_t w_st,
                     const int32_t* lens, int W,
                     int B, int n_kv, int gqa, float scale,
                     float* part_out, float* part_lse, void* stream) {
    BGTQ_CHECK_ARG(q && kbuf && vbuf && part_out && part_lse);
    BGTQ_CHECK_ARG(B >= 0 && n_kv >= 0 && gqa >= 1 && W >= 0);
    if (W > 8192) return BGTQ_ELIMIT;
    if (B == 0 || n_kv == 0) return BGTQ_OK;
    const size_t wbytes = (size_t)(W > 0 ? W : 1) * sizeof(float);
    // rows and query vectors on 16-byte boundaries: one work-group per (row, KV head)
    const bool wide = (((uintptr_t)q | (uintptr_t)kbuf | (uintptr_t)vbuf) & 15) == 0 &&
                      ((q_sb | q_sh | w_sb | w_sh | w_st) & 7) == 0;
    if (wide) {
        dim3 grid((unsigned)n_kv, (unsigned)B);
        if (gqa > 1 && 4 * wbytes <= 48 * 1024)
            hipLaunchKernelGGL((window_attn_kernel<4>), grid, dim3(WT), 4 * wbytes,
                               (hipStream_t)stream, (const uint16_t*)q, q_sb, q_sh,
                               (const uint16_t*)kbuf, (const uint16_t*)vbuf, w_sb, w_sh, w_st,
                               lens, W, n_kv * gqa, gqa, scale, part_out, part_lse);
        else
            hipLaunchKernelGGL((window_attn_kernel<1>), grid, dim3(WT), wbytes,
                               (hipStream_t)stream, (const uint16_t*)q, q_sb, q_sh,
                               (const uint16_t*)kbuf, (const uint16_t*)vbuf, w_sb, w_sh, w_st,
                               lens, W, n_kv * gqa, gqa, scale, part_out, part_lse);
        return bgtq_launch_status();
    }
    dim3 grid((unsigned)(n_kv * gqa), (unsigned)B);
    hipLaunchKernelGGL(window_attn_generic_kernel, grid, dim3(WT), wbytes,
                       (hipStream_t)stream, (const uint16_t*)q, q_sb, q_sh,
                       (const uint16_t*)kbuf, (const uint16_t*)vbuf, w_sb, w_sh, w_st,
                       lens, W, n_kv * gqa, gqa, scale, part_out, part_lse);
    return bgtq_launch_status();
}

int bgtq_window_swap(void* kbuf, void* vbuf, int64_t w_sb, int64_t w_sh, int64_t w_st,
                     const void* new_k, const void* new_v, int64_t n_sb, int64_t n_sh,
                     const int32_t* slot, int W, int B, int n_kv,
                     void* old_k, void* old_v, void* stream) {
    BGTQ_CHECK_ARG(kbuf && vbuf && new_k && new_v && slot && old_k && old_v);
    BGTQ_CHECK_ARG(B >= 0 && n_kv >= 0 && W >= 1);
    if (B == 0 || n_kv == 0) return BGTQ_OK;
    hipLaunchKernelGGL(window_swap_kernel, dim3((unsigned)n_kv, (unsigned)B), dim3(D), 0, (hipStream_t)stream,
                       (uint16_t*)kbuf, (uint16_t*)vbuf, w_sb, w_sh, w_st,
                       (const uint16_t*)new_k, (const uint16_t*)new_v, n_sb, n_sh, slot, W, n_kv,
                       (uint16_t*)old_k, (uint16_t*)old_v);
    return bgtq_launch_status();
}

size_t bgtq_plan_sizeof(void) { return sizeof(bgtq_head_plan); }
int bgtq_abi_version(void) { return 7; }
int bgtq_decode_kernel_revision(void) { return 7; }

const char* bgtq_strerror(int code) {
    switch (code) {
    case BGTQ_OK: return "ok";
    case BGTQ_EINVAL: return "invalid argument";
    case BGTQ_EUNSUPPORTED: return "not supported by this build";
    case BGTQ_ELIMIT: return "size beyond a documented maximum";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error";
    }
}


}  // extern "C"
