// MFMA decode attention over bit-packed K and V records (gfx950).
//
// One work-group of 4 waves owns one partition of one (batch row, KV head);
// every wave walks its own 64-token tiles with a private online softmax and the
// four results are merged through LDS at the end.
//
// Dequantisation is table driven.  A "unit" is 8 consecutive codes of one
// token (bw bytes of the record).  For every bit width <= 4 the work-group
// builds a pair table in LDS: entry (c0 | c1 << bw) holds the two fp16
// centroids of a code pair, replicated across LDS banks so that lanes with
// different indices do not collide (32 copies, 8 for the 256-entry 4-bit table).
// A unit costs one raw read, four {bit-field extract, shift-add, table read}
// triples and yields the eight fp16 operands of one MFMA k-group.
//
// QK^T:  v_mfma_f32_16x16x32_f16, A = dequantised K (row = token, lane group g
//        supplies unit 4m+g of step m; a step never mixes segments, so field
//        width and table are the same for the whole wave), B = rotated queries
//        laid out per step in LDS (zero on padding dims), D[token][head].  Each
//        segment accumulates on its own and is scaled by the fp32 group norm of
//        its token row when the segment ends.
// PV:    the D layout of two 16-token blocks is exactly the A layout of a
//        K=32 step (row = head, lane group g holds 8 tokens), so P never leaves
//        its lane; B = dequantised V where lane (j, g) decodes unit j of its 8
//        tokens and hands dim 8j+e to MFMA e.  The V norm is folded into P in
//        fp32 before P is rounded to fp16.
#include "bgtq_decode.h"

namespace {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef int int4v __attribute__((ext_vector_type(4)));

constexpr int D = BGTQ_D;
constexpr int MW = 4;              // waves per work-group
constexpr int NT = MW * 64;
constexpr int MT = 64;             // tokens per wave tile = 4 MFMA row blocks
constexpr int NBLK = MT / 16;
constexpr int MAX_STEPS = BGTQ_MAX_STEPS;
constexpr int KR = 6;              // 128-bit prefetch registers per lane for a K tile (row <= 95 B)
constexpr int VR = 5;              // same for a V tile (row <= 64 B)

// ---- LDS layout (bytes) -----------------------------------------------------------
constexpr int KLUT1 = 0;                       // 4 entries   x 128 B
constexpr int KLUT2 = KLUT1 + 4 * 128;         // 16 entries  x 128 B
constexpr int KLUT3 = KLUT2 + 16 * 128;        // 64 entries  x 128 B
constexpr int KLUT4 = KLUT3 + 64 * 128;        // 256 entries x 32 B
constexpr int KRAW = KLUT4 + 256 * 32;         // 4 tables x 256 fp16 (bw 5..8)
constexpr int VLUT = KRAW + 4 * 512;
__host__ __device__ constexpr int vlut_bytes(int vbw) { return vbw == 4 ? 256 * 32 : (1 << (2 * vbw)) * 128; }
__host__ __device__ constexpr int steps_off(int vbw) { return VLUT + vlut_bytes(vbw); }   // MAX_STEPS x 32 B
__host__ __device__ constexpr int qop_off(int vbw) { return steps_off(vbw) + MAX_STEPS * 32; }  // MAX_STEPS x 1 KB
__host__ __device__ constexpr int wave_off(int vbw) { return qop_off(vbw) + MAX_STEPS * 1024; }

__device__ inline uint32_t lds_u32(const uint8_t* base, uint32_t off) {
    return *(const uint32_t*)(base + off);
}

// A tile of packed records is one contiguous byte range.  It is fetched with
// aligned 128-bit loads (the 16-byte phase of the source is kept in LDS), first
// into registers while the previous tile is being processed, then into LDS.
template <int NR>
struct TileRegs {
    uint4 r[NR];
    uint32_t phase;
    int total;      // phase + valid bytes
};

template <int NR>
__device__ inline void tile_issue(TileRegs<NR>& t, const uint8_t* src, int nbytes, int lane) {
    t.phase = (uint32_t)((uintptr_t)src & 15);
    t.total = (int)t.phase + nbytes;
    const uint8_t* al = src - t.phase;
#pragma unroll
    for (int i = 0; i < NR; i++) {
        const int off = lane * 16 + i * 1024;
        uint4 v = {0, 0, 0, 0};
        if (off + 16 <= t.total) {
            v = *(const uint4*)(al + off);
        } else if (off < t.total) {            // last, partial chunk: never read past the tile
            const uint32_t* w = (const uint32_t*)(al + off);
            v.x = w[0];
            if (off + 8 <= t.total) v.y = w[1];
            if (off + 12 <= t.total) v.z = w[2];
        }
        t.r[i] = v;
    }
}

template <int NR>
__device__ inline void tile_commit(const TileRegs<NR>& t, uint8_t* dst, int lane) {
#pragma unroll
    for (int i = 0; i < NR; i++) {
        const int off = lane * 16 + i * 1024;
        if (off < t.total) *(uint4*)(dst + off) = t.r[i];
    }
}

template <int VBW>
__global__ __launch_bounds__(NT) void decode_mfma_kernel(DecodeArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const bgtq_head_plan& P = a.plans[h];
    const int gqa = a.gqa;
    const int li = lane & 15, lg = lane >> 4;           // MFMA row/col index, lane group

    const int T = a.seq_lens ? a.seq_lens[b] : a.T;
    int chunk = (T + a.n_splits - 1) / a.n_splits;
    chunk = (chunk + MT - 1) / MT * MT;
    const int t0 = min(c * chunk, T), t1 = min(t0 + chunk, T);

    // ---- LDS carve-up --------------------------------------------------------
    const int krow = a.k_row_width, vrow = a.v_row_width;
    const int kt_bytes = (MT * krow + 16 + 12 + 15) & ~15;
    const int vt_bytes = (MT * vrow + 16 + 12 + 15) & ~15;
    constexpr int kn_bytes = BGTQ_MAX_SEGMENTS * MT * 4;  // fp32 norms, [segment][token]
    const int wave_bytes = kt_bytes + vt_bytes + kn_bytes + MT * 2;
    uint8_t* vlut = smem + VLUT;
    int4v* steps_s = (int4v*)(smem + steps_off(VBW));
    uint8_t* qop_s = smem + qop_off(VBW);
    uint8_t* wbuf0 = smem + wave_off(VBW);
    uint8_t* kt_s = wbuf0 + wave * wave_bytes;
    uint8_t* vt_s = kt_s + kt_bytes;
    float* kn_s = (float*)(vt_s + vt_bytes);
    uint16_t* vn_s = (uint16_t*)((uint8_t*)kn_s + kn_bytes);

    // ---- init 1: plan header, step schedule, codebooks and queries into LDS scratch --
    // (scratch lives in the tile buffers, which are idle until the main loop)
    int* hdr_s = (int*)wbuf0;                             // first 56 ints of the plan
    uint16_t* cb_s = (uint16_t*)(wbuf0 + 256);            // [8][16] K codebooks + [16] V
    int* stp_s = (int*)(wbuf0 + 576);                     // n_steps, 3 pad, step[12][8]
    uint16_t* q_s = (uint16_t*)(wbuf0 + 1024);            // [16][128] rotated queries
    if (tid < 56) hdr_s[tid] = ((const int*)&P)[tid];
    if (tid >= 64 && tid < 64 + 4 + MAX_STEPS * 8) stp_s[tid - 64] = (&P.n_steps)[tid - 64];
    for (int i = tid; i < BGTQ_MAX_SEGMENTS * 16; i += NT) cb_s[i] = P.k_codebook_f16[i >> 4][i & 15];
    if (tid < 16) cb_s[BGTQ_MAX_SEGMENTS * 16 + tid] = P.v_lut_f16[tid];
    for (int i = tid; i < 16 * D / 2; i += NT) {
        int hq = i / (D / 2), d2 = i - hq * (D / 2);
        uint32_t v = 0;
        if (hq < gqa) v = *(const uint32_t*)(a.q + b * a.q_sb + (h * gqa + hq) * a.q_sh + d2 * 2);
        ((uint32_t*)q_s)[i] = v;
    }
    __syncthreads();
    const int n_seg = hdr_s[0];
    const int* seg_bw = hdr_s + 8;
    const int* seg_start = hdr_s + 16;
    const int* seg_len = hdr_s + 24;
    const int n_steps = min(stp_s[0], MAX_STEPS);

    // ---- init 2: pair tables, step table -------------------------------------------
    for (int s = 0; s < n_seg; s++) {
        const int bw = seg_bw[s];
        if (bw <= 4) {
            const int n = 1 << (2 * bw);
            const int rep = bw == 4 ? 8 : 32;
            uint8_t* tb = smem + (bw == 1 ? KLUT1 : bw == 2 ? KLUT2 : bw == 3 ? KLUT3 : KLUT4);
            for (int i = tid; i < n * rep; i += NT) {
                int e = i / rep;
                uint32_t v = (uint32_t)cb_s[s * 16 + (e & ((1 << bw) - 1))] |
                             ((uint32_t)cb_s[s * 16 + (e >> bw)] << 16);
                *(uint32_t*)(tb + i * 4) = v;
            }
        } else {
            // every byte value needs a finite entry: the last unit of a segment also
            // decodes bytes of its neighbour (their products meet a zero query)
            uint16_t* tb = (uint16_t*)(smem + KRAW) + (bw - 5) * 256;
            for (int i = tid; i < 256; i += NT) tb[i] = i < (1 << bw) ? P.k_codebook_f16[s][i] : (uint16_t)0;
        }
    }
    {
        constexpr int n = 1 << (2 * VBW);
        constexpr int rep = VBW == 4 ? 8 : 32;
        for (int i = tid; i < n * rep; i += NT) {
            int e = i / rep;
            uint32_t v = (uint32_t)cb_s[BGTQ_MAX_SEGMENTS * 16 + (e & ((1 << VBW) - 1))] |
                         ((uint32_t)cb_s[BGTQ_MAX_SEGMENTS * 16 + (e >> VBW)] << 16);
            *(uint32_t*)(vlut + i * 4) = v;
        }
    }
    // step m: {unit0 byte offset, bytes per unit, bits per pair (0 = raw bytes), table offset}
    //         {table shift, table lane mask, norm row | last-of-segment << 8, real units in the step}
    if (tid < n_steps) {
        const int* sp = stp_s + 4 + tid * 8;
        const int bw = sp[3];
        int4v p0, p1;
        p0.x = sp[0];
        p0.y = sp[1];
        p0.z = sp[2];
        p0.w = bw == 1 ? KLUT1 : bw == 2 ? KLUT2 : bw == 3 ? KLUT3 : bw == 4 ? KLUT4
                                                            : KRAW + (bw - 5) * 512;
        p1.x = bw == 4 ? 5 : 7;
        p1.y = bw == 4 ? 7 * 4 : 31 * 4;
        p1.z = sp[4] | (sp[5] ? 256 : 0);
        p1.w = sp[6];
        steps_s[2 * tid] = p0;
        steps_s[2 * tid + 1] = p1;
    }

    // ---- init 3: query B operands per step, [step][lane][8 halves] ------------------
    for (int i = tid; i < n_steps * 64 * 4; i += NT) {
        int m = i >> 8, l = (i >> 2) & 63, p = i & 3;          // p: pair of halves
        int d = 8 * (l >> 4) + 2 * p;                          // dim inside the step
        const int* sp = stp_s + 4 + m * 8;
        int left = seg_start[sp[4]] + seg_len[sp[4]] - sp[7];   // dims of the segment from this step on
        const uint16_t* row = q_s + (l & 15) * D + sp[7] + d;
        uint32_t lo = d < left ? row[0] : 0, hi = d + 1 < left ? row[1] : 0;
        ((uint32_t*)qop_s)[i] = lo | (hi << 16);
    }
    __syncthreads();                                        // scratch is dead from here
    if (lane < MT / 2) ((uint32_t*)vn_s)[lane] = 0;

    const uint8_t* kp_base = a.kp + b * a.kp_sb + h * a.kp_sh;
    const uint16_t* kn_base = a.kn + b * a.kn_sb + h * a.kn_sh;
    const uint8_t* vp_base = a.vp + b * a.vp_sb + h * a.vp_sh;
    const uint16_t* vn_base = a.vn + b * a.vn_sb + h * a.vn_sh;
    const float c2 = a.scale * 1.44269504088896340736f;      // logits go through exp2
    const uint32_t lane4 = (uint32_t)lane * 4;
    const uint32_t vbank = VBW == 4 ? (lane4 & 28u) : (lane4 & 124u);
    constexpr int vshift = VBW == 4 ? 5 : 7;

    float m_ref = -INFINITY;        // running max of head li, in exp2 units
    float l_part = 0.f;             // this lane's share of the softmax denominator
    float4v acc[8];
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = (float4v){0, 0, 0, 0};

    TileRegs<KR> kreg;
    TileRegs<VR> vreg;
    uint16_t nreg[BGTQ_MAX_SEGMENTS];
    uint16_t vnreg = 0;
    auto issue = [&](int tile) {
        const int nt = min(MT, t1 - tile);
        tile_issue(kreg, kp_base + (int64_t)tile * a.kp_st, nt * krow, lane);
        tile_issue(vreg, vp_base + (int64_t)tile * a.vp_st, nt * vrow, lane);
        const uint16_t* nr = kn_base + (int64_t)(tile + lane) * a.kn_st;    // lane = token
#pragma unroll
        for (int s = 0; s < BGTQ_MAX_SEGMENTS; s++) nreg[s] = (s < n_seg && lane < nt) ? nr[s] : (uint16_t)0;
        vnreg = lane < nt ? vn_base[tile + lane] : (uint16_t)0;
    };
    int tile = t0 + wave * MT;
    if (tile < t1) issue(tile);

    for (; tile < t1; tile += MW * MT) {
        const int nt = min(MT, t1 - tile);
        // ---- registers -> LDS (wave private), then start fetching the next tile ------
        const uint32_t kph = kreg.phase, vph = vreg.phase;
        tile_commit(kreg, kt_s, lane);
        tile_commit(vreg, vt_s, lane);
#pragma unroll
        for (int s = 0; s < BGTQ_MAX_SEGMENTS; s++)          // fp16 -> fp32, [segment][token]
            if (s < n_seg) kn_s[s * MT + lane] = bgtq_h2f(nreg[s]);
        vn_s[lane] = vnreg;
        if (tile + MW * MT < t1) issue(tile + MW * MT);
        // a wave's LDS operations execute in issue order; the clobber keeps the
        // compiler from moving the tile reads above the staging writes
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();

        // ---- scores ---------------------------------------------------------------
        float4v S[NBLK], dseg[NBLK];
        uint32_t rowb[NBLK];
#pragma unroll
        for (int k = 0; k < NBLK; k++) {
            S[k] = (float4v){0, 0, 0, 0};
            dseg[k] = (float4v){0, 0, 0, 0};
            rowb[k] = kph + (uint32_t)(k * 16 + li) * krow;
        }
        for (int m = 0; m < n_steps; m++) {
            const int4v p0 = steps_s[2 * m], p1 = steps_s[2 * m + 1];
            const half8 Q = *(const half8*)(qop_s + m * 1024 + lane * 16);
            const uint32_t off = (uint32_t)p0.x + (uint32_t)min(lg, p1.w - 1) * (uint32_t)p0.y;
            const int pw = __builtin_amdgcn_readfirstlane(p0.z);
            if (pw != 0) {
                const uint32_t lb = (uint32_t)p0.w + (lane4 & (uint32_t)p1.y);
                const uint32_t sh = (uint32_t)p1.x;
#pragma unroll
                for (int k = 0; k < NBLK; k++) {
                    uint32_t o = rowb[k] + off;
                    uint32_t lo = lds_u32(kt_s, o & ~3u), hi = lds_u32(kt_s, (o & ~3u) + 4);
                    uint32_t raw = __builtin_amdgcn_alignbyte(hi, lo, o & 3u);
                    half8 A;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        uint32_t idx = __builtin_amdgcn_ubfe(raw, e * pw, pw);
                        half2v pr = __builtin_bit_cast(half2v, lds_u32(smem, (idx << sh) + lb));
                        A[2 * e] = pr[0];
                        A[2 * e + 1] = pr[1];
                    }
                    dseg[k] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, Q, dseg[k], 0, 0, 0);
                }
            } else {
                const uint16_t* tb = (const uint16_t*)(smem + p0.w);
#pragma unroll
                for (int k = 0; k < NBLK; k++) {
                    uint32_t o = rowb[k] + off;
                    uint32_t lo = lds_u32(kt_s, o & ~3u), hi = lds_u32(kt_s, (o & ~3u) + 4);
                    uint32_t hi2 = lds_u32(kt_s, (o & ~3u) + 8);
                    uint32_t r0 = __builtin_amdgcn_alignbyte(hi, lo, o & 3u);
                    uint32_t r1 = __builtin_amdgcn_alignbyte(hi2, hi, o & 3u);
                    half8 A;
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        uint32_t r = e < 4 ? r0 : r1;
                        A[e] = __builtin_bit_cast(_Float16, tb[(r >> ((e & 3) * 8)) & 0xFF]);
                    }
                    dseg[k] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, Q, dseg[k], 0, 0, 0);
                }
            }
            const int sz = __builtin_amdgcn_readfirstlane(p1.z);
            if (sz & 256) {       // segment complete: scale by the token rows' group norms
                const float* nrm = kn_s + (sz & 255) * MT + lg * 4;
#pragma unroll
                for (int k = 0; k < NBLK; k++) {
                    const float4v n4 = *(const float4v*)(nrm + k * 16);
                    S[k] += dseg[k] * n4;
                    dseg[k] = (float4v){0, 0, 0, 0};
                }
            }
        }

        // ---- online softmax: lane (head li, group lg) holds tokens 16k + 4lg + r ------
        float sv[4 * NBLK];
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4 * NBLK; r++) {
            int tk = (r >> 2) * 16 + lg * 4 + (r & 3);
            float x = S[r >> 2][r & 3] * c2;
            x = tk < nt ? x : -INFINITY;
            sv[r] = x;
            mx = fmaxf(mx, x);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_ref, mx);
        if (__builtin_amdgcn_ballot_w64(m_new > m_ref)) {          // wave-uniform: rescale only when needed
            const float alpha = (m_ref == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_ref - m_new);
            // acc rows are heads 4lg+r, not this lane's head: fetch their factors
            float al[4];
#pragma unroll
            for (int r = 0; r < 4; r++) al[r] = __shfl(alpha, lg * 4 + r, 64);
#pragma unroll
            for (int e = 0; e < 8; e++)
#pragma unroll
                for (int r = 0; r < 4; r++) acc[e][r] *= al[r];
            l_part *= alpha;
            m_ref = m_new;
        }

#pragma unroll
        for (int half = 0; half < NBLK / 2; half++) {
            // P * v_norm is formed in fp32 and rounded to fp16 once
            half8 Pm;
            {
                const uint2 vlo = *(const uint2*)(vn_s + half * 32 + lg * 4);        // tokens 4lg .. 4lg+3
                const uint2 vhi = *(const uint2*)(vn_s + half * 32 + 16 + lg * 4);   // tokens 16+4lg ..
                const uint32_t vnn[4] = {vlo.x, vlo.y, vhi.x, vhi.y};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    half2v vn2 = __builtin_bit_cast(half2v, vnn[e]);
                    float p0 = __builtin_amdgcn_exp2f(sv[half * 8 + 2 * e] - m_ref);
                    float p1 = __builtin_amdgcn_exp2f(sv[half * 8 + 2 * e + 1] - m_ref);
                    l_part += p0 + p1;
                    Pm[2 * e] = (_Float16)(p0 * (float)vn2[0]);
                    Pm[2 * e + 1] = (_Float16)(p1 * (float)vn2[1]);
                }
            }
            // values: lane (j = li, group lg) decodes unit j of its 8 tokens
            uint32_t W[8][4];
#pragma unroll
            for (int r = 0; r < 8; r++) {
                const int tk = half * 32 + (r >> 2) * 16 + lg * 4 + (r & 3);
                uint32_t o = vph + (uint32_t)tk * vrow + (uint32_t)li * VBW;
                uint32_t lo = lds_u32(vt_s, o & ~3u), hi = lds_u32(vt_s, (o & ~3u) + 4);
                uint32_t raw = __builtin_amdgcn_alignbyte(hi, lo, o & 3u);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    uint32_t idx = __builtin_amdgcn_ubfe(raw, e * 2 * VBW, 2 * VBW);
                    W[r][e] = lds_u32(vlut, (idx << vshift) + vbank);
                }
            }
#pragma unroll
            for (int e = 0; e < 8; e++) {
                half8 Bv;
                const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;   // high or low halves
#pragma unroll
                for (int p = 0; p < 4; p++) {
                    uint32_t x = __builtin_amdgcn_perm(W[2 * p + 1][e >> 1], W[2 * p][e >> 1], sel);
                    half2v hv = __builtin_bit_cast(half2v, x);
                    Bv[2 * p] = hv[0];
                    Bv[2 * p + 1] = hv[1];
                }
                acc[e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Pm, Bv, acc[e], 0, 0, 0);
            }
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();     // tile buffers are rewritten next iteration
    }

    // ---- merge the four waves ------------------------------------------------------
    float l_tot = l_part;
    l_tot += __shfl_xor(l_tot, 16, 64);
    l_tot += __shfl_xor(l_tot, 32, 64);
    __syncthreads();                         // tables and tile buffers are dead from here
    float* mg_m = (float*)smem;              // [MW][16]
    float* mg_l = mg_m + MW * 16;            // [MW][16]
    float* mg_o = mg_l + MW * 16;            // [MW][16][D]
    if (lane < 16) { mg_m[wave * 16 + lane] = m_ref; mg_l[wave * 16 + lane] = l_tot; }
#pragma unroll
    for (int e = 0; e < 8; e++)
#pragma unroll
        for (int r = 0; r < 4; r++)
            mg_o[(wave * 16 + lg * 4 + r) * D + li * 8 + e] = acc[e][r];
    __syncthreads();
    for (int i = tid; i < gqa * D; i += NT) {
        int hq = i / D, d = i - hq * D;
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < MW; w++) m = fmaxf(m, mg_m[w * 16 + hq]);
        float den = 0.f, num = 0.f;
#pragma unroll
        for (int w = 0; w < MW; w++) {
            float mw = mg_m[w * 16 + hq];
            float f = (mw == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mw - m);
            den += f * mg_l[w * 16 + hq];
            num += f * mg_o[(w * 16 + hq) * D + d];
        }
        size_t row = ((size_t)b * a.n_kv * gqa + (size_t)h * gqa + hq) * a.n_splits + c;
        a.part_out[row * D + d] = (t1 > t0) ? num / den : 0.f;
        if (d == 0) a.part_lse[row] = (t1 > t0) ? (m + log2f(den)) * 0.69314718055994530942f : -INFINITY;
    }
}

size_t mfma_smem_bytes(int vbw, int krow, int vrow) {
    size_t kt = (size_t)((MT * krow + 16 + 12 + 15) & ~15);
    size_t vt = (size_t)((MT * vrow + 16 + 12 + 15) & ~15);
    size_t wave = kt + vt + (size_t)BGTQ_MAX_SEGMENTS * MT * 4 + MT * 2;
    size_t need = (size_t)wave_off(vbw) + wave * MW;
    size_t merge = (size_t)(MW * 16 * 2 + MW * 16 * D) * 4;
    return need > merge ? need : merge;
}

template <int VBW>
int launch(const DecodeArgs& a, hipStream_t st) {
    size_t smem = mfma_smem_bytes(VBW, a.k_row_width, a.v_row_width);
    auto kern = decode_mfma_kernel<VBW>;
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return (int)e;
    dim3 grid((unsigned)a.n_splits, (unsigned)a.n_kv, (unsigned)a.B);
    hipLaunchKernelGGL(kern, grid, dim3(NT), smem, st, a);
    return bgtq_launch_status();
}

}  // namespace

int bgtq_launch_decode_mfma(const DecodeArgs& a, hipStream_t stream) {
    // layout requirements of the fast path; anything else takes the generic kernel
    if (a.k_layout != BGTQ_K_BITPACKED || a.v_layout != BGTQ_V_BITPACKED) return BGTQ_EUNSUPPORTED;
    if (a.gqa > 16) return BGTQ_EUNSUPPORTED;
    if ((a.kp_st & 3) || (a.kp_sb & 3) || (a.kp_sh & 3) || ((uintptr_t)a.kp & 3)) return BGTQ_EUNSUPPORTED;
    if ((a.vp_st & 3) || (a.vp_sb & 3) || (a.vp_sh & 3) || ((uintptr_t)a.vp & 3)) return BGTQ_EUNSUPPORTED;
    if (a.kp_st != a.k_row_width || a.vp_st != a.v_row_width) return BGTQ_EUNSUPPORTED;   // records contiguous
    if (a.vn_st != 1) return BGTQ_EUNSUPPORTED;
    if (MT * a.k_row_width + 12 > KR * 1024 || MT * a.v_row_width + 12 > VR * 1024) return BGTQ_EUNSUPPORTED;
    if ((a.q_sb & 1) || (a.q_sh & 1) || ((uintptr_t)a.q & 3)) return BGTQ_EUNSUPPORTED;
    // a bit-packed V record of 128 dims is 16 bytes per bit of code width
    switch (a.v_row_width) {
    case 16: return launch<1>(a, stream);
    case 32: return launch<2>(a, stream);
    case 48: return launch<3>(a, stream);
    case 64: return launch<4>(a, stream);
    default: return BGTQ_EUNSUPPORTED;
    }
}
