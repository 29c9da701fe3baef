// MFMA decode attention over bit-packed K and V records (gfx950).
//
// One work-group of 4 waves owns one partition of one (batch row, KV head);
// every wave walks its own 32-token tiles with a private online softmax and the
// four results are merged through LDS at the end.
//
// Dequantisation is table driven.  A "unit" is 8 consecutive codes of one
// token (bw bytes of the record).  For every bit width <= 4 the work-group
// builds a pair table in LDS: entry (c0 | c1 << bw) holds the two fp16
// centroids of a code pair, replicated once per LDS bank so that 64 lanes with
// 64 different indices never collide (lane l reads the copy in bank l % 32).
// A unit therefore costs one raw read, four {bit-field extract, shift-add,
// table read} triples and gives the eight fp16 operands of one MFMA k-group.
//
// QK^T:  v_mfma_f32_16x16x32_f16 with A = dequantised K (row = token, lane group
//        g supplies unit 4m+g of MFMA step m, steps never mix segments so the
//        field widths are wave-uniform scalars), B = rotated queries (kept in
//        registers for the whole partition, zero on padding dims), D[token][head].
// PV:    the D layout of two 16-token blocks is exactly the A layout of a
//        K=32 step (row = head, lane group g holds 8 tokens), so P never leaves
//        its lane; B = dequantised V where lane (j, g) decodes unit j of its 8
//        tokens and hands dim 8j+e to MFMA e.
// K group norms are applied in fp32 to each segment's partial score, the V norm
// scales P before it is rounded to fp16.
#include "bgtq_decode.h"

namespace {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int D = BGTQ_D;
constexpr int MW = 4;              // waves per work-group
constexpr int NT = MW * 64;
constexpr int MT = 32;             // tokens per wave tile
constexpr int MAX_STEPS = 12;      // sum over segments of ceil(ceil(len/8)/4) <= 11
constexpr int REPL = 128;          // bytes per pair-table entry (32 banks x 4 B)

// LDS byte offsets of the K pair tables by bit width (each width occurs at most once)
__host__ __device__ constexpr int klut_off(int bw) {
    return bw == 1 ? 0 : bw == 2 ? 4 * REPL : bw == 3 ? (4 + 16) * REPL : (4 + 16 + 64) * REPL;
}
constexpr int KLUT_BYTES = (4 + 16 + 64 + 256) * REPL;          // 43520
constexpr int KRAW_OFF = KLUT_BYTES;                             // 4 tables x 256 fp16
constexpr int KRAW_BYTES = 4 * 256 * 2;
constexpr int VLUT_OFF = KRAW_OFF + KRAW_BYTES;
__host__ __device__ constexpr int vlut_bytes(int vbw) { return (1 << (2 * vbw)) * REPL; }

struct StepTable {            // wave-uniform description of the MFMA steps of QK^T
    int n_steps;
    int bw[MAX_STEPS];        // code width (5..8 = raw bytes)
    int seg[MAX_STEPS];       // segment index (norm column)
    int unit0[MAX_STEPS];     // first unit of the step inside its segment
    int n_units[MAX_STEPS];   // units of the whole segment
};

__device__ inline uint32_t lds_u32(const uint8_t* base, uint32_t off) {
    return *(const uint32_t*)(base + off);
}
__device__ inline float wave_xor_max(float v, int m) { return fmaxf(v, __shfl_xor(v, m, 64)); }

// copy nbytes (multiple of 4) from 4-byte aligned global memory into LDS keeping
// the 16-byte phase of the source, so full 128-bit loads stay aligned
__device__ inline uint32_t stage_bytes(const uint8_t* src, int nbytes, uint8_t* dst, int lane) {
    uint32_t phase = (uint32_t)((uintptr_t)src & 15);
    const uint8_t* al = src - phase;
    int total = (int)phase + nbytes;
    int full = total & ~15;
    for (int off = lane * 16; off < full; off += 64 * 16)
        *(uint4*)(dst + off) = *(const uint4*)(al + off);
    int tail = (total - full) >> 2;           // 0..3 dwords
    if (lane < tail) *(uint32_t*)(dst + full + lane * 4) = *(const uint32_t*)(al + full + lane * 4);
    return phase;
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
    const int kt_bytes = (MT * krow + 16 + 8 + 15) & ~15;
    const int vt_bytes = (MT * vrow + 16 + 8 + 15) & ~15;
    constexpr int kn_bytes = BGTQ_MAX_SEGMENTS * MT * 4;  // fp32 norms, [segment][token]
    const int wave_bytes = kt_bytes + vt_bytes + kn_bytes + 64;
    uint8_t* klut = smem;
    uint8_t* vlut = smem + VLUT_OFF;
    uint8_t* wbuf = smem + VLUT_OFF + vlut_bytes(VBW) + wave * wave_bytes;
    uint8_t* kt_s = wbuf;
    uint8_t* vt_s = kt_s + kt_bytes;
    float* kn_s = (float*)(vt_s + vt_bytes);
    uint8_t* vn_s = (uint8_t*)kn_s + kn_bytes;            // 32 fp16

    // ---- tables -----------------------------------------------------------------
    for (int s = 0; s < P.n_seg; s++) {
        const int bw = P.seg_bw[s];
        if (bw <= 4) {
            const int n = 1 << (2 * bw);
            uint8_t* tb = klut + klut_off(bw);
            for (int i = tid; i < n * 32; i += NT) {
                int e = i >> 5, bank = i & 31;
                uint32_t v = (uint32_t)P.k_codebook_f16[s][e & ((1 << bw) - 1)] |
                             ((uint32_t)P.k_codebook_f16[s][e >> bw] << 16);
                *(uint32_t*)(tb + e * REPL + bank * 4) = v;
            }
        } else {
            uint16_t* tb = (uint16_t*)(smem + KRAW_OFF) + (bw - 5) * 256;
            // every byte value needs a finite entry: the last unit of a segment also
            // decodes bytes that belong to its neighbour (their products meet a zero query)
            for (int i = tid; i < 256; i += NT) tb[i] = i < (1 << bw) ? P.k_codebook_f16[s][i] : (uint16_t)0;
        }
    }
    for (int i = tid; i < (1 << (2 * VBW)) * 32; i += NT) {
        int e = i >> 5, bank = i & 31;
        uint32_t v = (uint32_t)P.v_lut_f16[e & ((1 << VBW) - 1)] | ((uint32_t)P.v_lut_f16[e >> VBW] << 16);
        *(uint32_t*)(vlut + e * REPL + bank * 4) = v;
    }
    if (lane < 16) ((uint32_t*)vn_s)[lane] = 0;

    // ---- step table (identical in every lane, lives in scalar registers) -------
    StepTable st;
    st.n_steps = 0;
#pragma unroll
    for (int m = 0; m < MAX_STEPS; m++) { st.bw[m] = 1; st.seg[m] = 0; st.unit0[m] = 0; st.n_units[m] = 0; }
    {
        int m = 0;
        for (int s = 0; s < P.n_seg; s++) {
            int nu = (P.seg_len[s] + 7) >> 3;
            for (int u0 = 0; u0 < nu; u0 += 4) {
#pragma unroll
                for (int k = 0; k < MAX_STEPS; k++)
                    if (k == m) { st.bw[k] = P.seg_bw[s]; st.seg[k] = s; st.unit0[k] = u0; st.n_units[k] = nu; }
                m++;
            }
        }
        st.n_steps = m;
    }

    // ---- rotated queries as B operands, one per step (zero on padding dims) ----
    half8 qB[MAX_STEPS];
#pragma unroll
    for (int m = 0; m < MAX_STEPS; m++) {
        half8 v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (m < st.n_steps && li < gqa) {
            int s = st.seg[m];
            int u = st.unit0[m] + lg;
            const uint16_t* qp = a.q + b * a.q_sb + (h * gqa + li) * a.q_sh + P.seg_start[s] + u * 8;
            int left = P.seg_len[s] - u * 8;
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (i < left) v[i] = __builtin_bit_cast(_Float16, qp[i]);
        }
        qB[m] = v;
    }
    // per-lane byte offset of this lane's unit inside a K record, per step
    int koff[MAX_STEPS];
#pragma unroll
    for (int m = 0; m < MAX_STEPS; m++) {
        int s = st.seg[m];
        int u = min(st.unit0[m] + lg, max(st.n_units[m] - 1, 0));     // clamp: padding units re-read a real one
        int ub = st.bw[m] <= 4 ? st.bw[m] : 8;
        koff[m] = P.seg_pack_off[s] + u * ub;
    }
    __syncthreads();

    const uint8_t* kp_base = a.kp + b * a.kp_sb + h * a.kp_sh;
    const uint16_t* kn_base = a.kn + b * a.kn_sb + h * a.kn_sh;
    const uint8_t* vp_base = a.vp + b * a.vp_sb + h * a.vp_sh;
    const uint16_t* vn_base = a.vn + b * a.vn_sb + h * a.vn_sh;
    const int n_seg = P.n_seg;
    const float c2 = a.scale * 1.44269504088896340736f;      // logits go through exp2
    const uint32_t bank4 = (uint32_t)(lane & 31) * 4;

    float m_ref = -INFINITY;        // running max of head li, in exp2 units
    float l_part = 0.f;             // this lane's share of the softmax denominator
    float4v acc[8];
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = (float4v){0, 0, 0, 0};

    for (int tile = t0 + wave * MT; tile < t1; tile += MW * MT) {
        const int nt = min(MT, t1 - tile);
        // ---- stage the tile (wave private) -------------------------------------
        uint32_t kph = stage_bytes(kp_base + (int64_t)tile * a.kp_st, nt * krow, kt_s, lane);
        uint32_t vph = stage_bytes(vp_base + (int64_t)tile * a.vp_st, nt * vrow, vt_s, lane);
        // group norms: fp16 -> fp32, transposed to [segment][token] so that a lane
        // later fetches the four tokens of its MFMA rows with one 128-bit read
        if (lane < MT) {
            const uint16_t* nr = kn_base + (int64_t)(tile + lane) * a.kn_st;
            for (int s = 0; s < n_seg; s++)
                kn_s[s * MT + lane] = lane < nt ? bgtq_h2f(nr[s]) : 0.f;
        }
        if (lane < MT) ((uint16_t*)vn_s)[lane] = lane < nt ? vn_base[tile + lane] : (uint16_t)0;
        // a wave's LDS operations execute in issue order; the clobber keeps the
        // compiler from moving the tile reads above the staging writes
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();

        // ---- scores ---------------------------------------------------------------
        // Per segment: MFMA over its unscaled fp16 centroids, then the fp32 group norm
        // of each token row scales the segment's partial sum.
        float4v S[2];
#pragma unroll
        for (int blk = 0; blk < 2; blk++) {
            float4v s4 = {0, 0, 0, 0}, dseg = {0, 0, 0, 0};
            const uint32_t rowb = kph + (uint32_t)(blk * 16 + li) * krow;
#pragma unroll
            for (int m = 0; m < MAX_STEPS; m++) {
                if (m < st.n_steps) {
                    const int bw = st.bw[m];
                    uint32_t o = rowb + (uint32_t)koff[m];
                    uint32_t lo = lds_u32(kt_s, o & ~3u), hi = lds_u32(kt_s, (o & ~3u) + 4);
                    uint32_t w[4];
                    if (bw <= 4) {
                        uint32_t raw = __builtin_amdgcn_alignbyte(hi, lo, o & 3u);
                        const uint32_t tboff = bw == 1 ? klut_off(1) : bw == 2 ? klut_off(2)
                                             : bw == 3 ? klut_off(3) : klut_off(4);
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            uint32_t idx = __builtin_amdgcn_ubfe(raw, e * 2 * bw, 2 * bw);
                            w[e] = lds_u32(klut, tboff + (idx << 7) + bank4);
                        }
                    } else {
                        // raw bytes: 8 single-code look-ups
                        uint32_t hi2 = lds_u32(kt_s, (o & ~3u) + 8);
                        uint32_t r0 = __builtin_amdgcn_alignbyte(hi, lo, o & 3u);
                        uint32_t r1 = __builtin_amdgcn_alignbyte(hi2, hi, o & 3u);
                        const uint16_t* tb = (const uint16_t*)(smem + KRAW_OFF) + (bw - 5) * 256;
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            uint32_t r = e < 2 ? r0 : r1;
                            uint32_t ca = (r >> ((e & 1) * 16)) & 0xFF, cb = (r >> ((e & 1) * 16 + 8)) & 0xFF;
                            w[e] = (uint32_t)tb[ca] | ((uint32_t)tb[cb] << 16);
                        }
                    }
                    half8 A;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        half2v pr = __builtin_bit_cast(half2v, w[e]);
                        A[2 * e] = pr[0];
                        A[2 * e + 1] = pr[1];
                    }
                    const bool first = (m == 0) || (st.seg[m] != st.seg[m > 0 ? m - 1 : 0]);
                    const bool last = (m + 1 >= st.n_steps) || (st.seg[m] != st.seg[m + 1 < MAX_STEPS ? m + 1 : m]);
                    if (first) dseg = (float4v){0, 0, 0, 0};
                    dseg = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, qB[m], dseg, 0, 0, 0);
                    if (last) {
                        const float4v n4 = *(const float4v*)(kn_s + st.seg[m] * MT + blk * 16 + lg * 4);
                        s4 += dseg * n4;
                    }
                }
            }
            S[blk] = s4;
        }

        // ---- online softmax: lane (head li, group lg) holds tokens 4lg+r, 16+4lg+r --
        float sv[8];
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 8; r++) {
            int tk = (r >> 2) * 16 + lg * 4 + (r & 3);
            float x = S[r >> 2][r & 3] * c2;
            x = tk < nt ? x : -INFINITY;
            sv[r] = x;
            mx = fmaxf(mx, x);
        }
        mx = wave_xor_max(wave_xor_max(mx, 16), 32);
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
        // P * v_norm is formed in fp32 and rounded to fp16 once
        half8 Pm;
        {
            const uint2 vlo = *(const uint2*)(vn_s + (lg * 4) * 2);          // tokens 4lg .. 4lg+3
            const uint2 vhi = *(const uint2*)(vn_s + (16 + lg * 4) * 2);     // tokens 16+4lg ..
            const uint32_t vnn[4] = {vlo.x, vlo.y, vhi.x, vhi.y};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                half2v vn2 = __builtin_bit_cast(half2v, vnn[e]);
                float p0 = __builtin_amdgcn_exp2f(sv[2 * e] - m_ref);
                float p1 = __builtin_amdgcn_exp2f(sv[2 * e + 1] - m_ref);
                l_part += p0 + p1;
                Pm[2 * e] = (_Float16)(p0 * (float)vn2[0]);
                Pm[2 * e + 1] = (_Float16)(p1 * (float)vn2[1]);
            }
        }

        // ---- values: lane (j = li, group lg) decodes unit j of its 8 tokens -----------
        uint32_t W[8][4];
#pragma unroll
        for (int r = 0; r < 8; r++) {
            const int tk = (r >> 2) * 16 + lg * 4 + (r & 3);
            uint32_t o = vph + (uint32_t)tk * vrow + (uint32_t)li * VBW;
            uint32_t lo = lds_u32(vt_s, o & ~3u), hi = lds_u32(vt_s, (o & ~3u) + 4);
            uint32_t raw = __builtin_amdgcn_alignbyte(hi, lo, o & 3u);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                uint32_t idx = __builtin_amdgcn_ubfe(raw, e * 2 * VBW, 2 * VBW);
                W[r][e] = lds_u32(vlut, (idx << 7) + bank4);
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
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();     // tile buffers are rewritten next iteration
    }

    // ---- merge the four waves ------------------------------------------------------
    // denominators: sum the lane groups of each head
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
            float f = (mw == -INFINITY) ? 0.f : exp2f(mw - m);
            den += f * mg_l[w * 16 + hq];
            num += f * mg_o[(w * 16 + hq) * D + d];
        }
        size_t row = ((size_t)b * a.n_kv * gqa + (size_t)h * gqa + hq) * a.n_splits + c;
        a.part_out[row * D + d] = (t1 > t0) ? num / den : 0.f;
        if (d == 0) a.part_lse[row] = (t1 > t0) ? (m + log2f(den)) * 0.69314718055994530942f : -INFINITY;
    }
}

size_t mfma_smem_bytes(int vbw, int krow, int vrow) {
    size_t kt = (size_t)((MT * krow + 16 + 8 + 15) & ~15);
    size_t vt = (size_t)((MT * vrow + 16 + 8 + 15) & ~15);
    size_t kn = (size_t)BGTQ_MAX_SEGMENTS * MT * 4;
    size_t tables = (size_t)VLUT_OFF + vlut_bytes(vbw);
    size_t waves = (kt + vt + kn + 64) * MW;
    size_t merge = (size_t)(MW * 16 * 2 + MW * 16 * D) * 4;
    size_t need = tables + waves;
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
    // a bit-packed V record of 128 dims is 16 bytes per bit of code width
    switch (a.v_row_width) {
    case 16: return launch<1>(a, stream);
    case 32: return launch<2>(a, stream);
    case 48: return launch<3>(a, stream);
    case 64: return launch<4>(a, stream);
    default: return BGTQ_EUNSUPPORTED;
    }
}
