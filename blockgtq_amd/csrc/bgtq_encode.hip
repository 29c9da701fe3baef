// K / V quantise-and-pack kernels and the query rotation for gfx950.
//
// Arithmetic contract (what "bit-exact" means for the packed bytes): every
// reduction over coordinates is a chain of fused multiply-adds in ascending
// packed-dim order starting from +0, square roots and divisions are IEEE
// correctly rounded, and the rotation of coordinate j of a group spanning dims
// [s, e) is fma(xhat[k], R_T[k][j], acc) for k = s .. e-1 (skipped altogether,
// y = xhat, when the group's rotation block is the identity).  This file is
// compiled with floating-point contraction off so nothing else fuses.
//
// One work-group of 128 threads encodes ROWS token rows of one KV head:
// thread j owns packed dim j during normalise / rotate / quantise and output
// byte j while packing.  The rotation matrix is read once per work-group
// (coalesced across j, served from L2) and reused for all ROWS rows out of
// registers; rows are staged in LDS so the k-loop reads them as broadcasts.
#include <type_traits>

#include "bgtq_common.h"

namespace {

constexpr int D = BGTQ_D;
constexpr int NT = 128;  // threads per work-group


struct EncodeArgs {
    const bgtq_head_plan* plans;
    const uint16_t* x;          // fp16 [B][n_kv][S][128]
    int64_t x_sb, x_sh, x_ss;
    int B, n_kv, S;
    uint8_t* packed;            // cache records, or nullptr
    int64_t p_sb, p_sh, p_st;
    int row_width;
    uint16_t* norms;            // fp16 cache norms, or nullptr
    int64_t n_sb, n_sh, n_st;
    int norm_width;
    const int32_t* t_pos;
    int t_pos_scalar;
    int max_T;                  // token capacity of the cache: records at positions outside [0, max_T) are dropped
    int layout;
    int quant_mode;
    uint8_t* codes_out;         // [N][128] unpacked codes, or nullptr
    float* norms_f32_out;       // K: [N][norm_width] fp32; or nullptr
    int corrected;              // K codes path: emit corrected norms
};

// One byte of the LSB-first stream of bw-bit codes (bw <= 4) covers the codes first .. first + n - 1,
// the first of them from its bit `skip` on.  None of this depends on the row: the plan holds it per
// record byte (enc_byte, enc_vbyte).
struct StreamSlot { int first, n, skip; };
__device__ inline unsigned stream_byte(const uint8_t* codes, StreamSlot s, int bw) {
    unsigned w = 0;
    for (int i = 0; i < s.n; i++) w |= (unsigned)codes[s.first + i] << (i * bw);
    return (w >> s.skip) & 0xFFu;
}
// The same byte with all (at most 8) code reads issued at once: for the latency-bound append of
// a few rows, where one LDS round trip per code is what the loop above would cost.
__device__ inline unsigned stream_byte_batched(const uint8_t* codes, StreamSlot s, int bw) {
    unsigned c[8];
#pragma unroll
    for (int i = 0; i < 8; i++) c[i] = codes[s.first + min(i, s.n - 1)];
    unsigned w = 0;
#pragma unroll
    for (int i = 0; i < 8; i++)
        if (i < s.n) w |= c[i] << (i * bw);
    return (w >> s.skip) & 0xFFu;
}

// Row n of the [B][S] input is (batch b, step s).  The row count fits 32 bits (the launchers
// check), so this is one 32-bit division instead of the 64-bit software routine.
__device__ inline void split_row(int64_t n, int S, int& b, int& s) {
    const unsigned q = (unsigned)n / (unsigned)S;
    b = (int)q;
    s = (int)((unsigned)n - q * (unsigned)S);
}

// Plan tables a work-group needs, copied to LDS with one burst of independent loads:
// every later table access is an LDS read instead of one more dependent trip to memory.
struct StagedK {
    int hdr[56];                 // n_seg .. seg_identity, as at the start of bgtq_head_plan
    uint8_t code_lut[BGTQ_MAX_SEGMENTS * BGTQ_LUT_BINS];
    float centroids[BGTQ_MAX_SEGMENTS * 32];   // first 32 levels of every segment (bw <= 5)
};
struct StagedV {
    int v_bits;
    float centroids[16];
    float boundaries[16];
};
constexpr int H_NSEG = 0, H_NZERO = 1, H_NOPACK_START = 4, H_NOPACK_LEN = 5, H_VBITS = 6;
constexpr int H_BW = 8, H_START = 16, H_LEN = 24, H_PACK_OFF = 32, H_IDENT = 48;

// The 128 x 128 fp32 rotation as 4096 pieces of 16 bytes: thread j fetches pieces j, j + 128, ...
// (a wave reads 1 KB of consecutive addresses per instruction) and later parks them at the same
// offsets in LDS, where thread j reads column j (consecutive lanes, consecutive banks).
static_assert(offsetof(bgtq_head_plan, k_rot_T) % 16 == 0 && offsetof(bgtq_head_plan, v_rot_T) % 16 == 0 &&
              sizeof(bgtq_head_plan) % 16 == 0, "rotations are read 16 bytes at a time");
typedef float rot_piece __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void fetch_rotation(const float* M, const int j, rot_piece (&st)[D / 4]) {
#pragma unroll
    for (int i = 0; i < D / 4; i++) st[i] = ((const rot_piece*)M)[i * NT + j];
}
__device__ __forceinline__ void park_rotation(float* rot_s, const int j, const rot_piece (&st)[D / 4]) {
#pragma unroll
    for (int i = 0; i < D / 4; i++) ((rot_piece*)rot_s)[i * NT + j] = st[i];
}

// Sum of x[k]^2 over a whole row of D values in LDS (V) as ONE fmaf chain in increasing k.  The reads
// of a batch are all issued before its first fmaf (left to itself the compiler waits for every few
// reads in turn); the chain itself runs at the 8 clocks of a dependent instruction.
__device__ __forceinline__ float chain_sumsq_row(const float* x) {
    float ss = 0.f;
#pragma unroll
    for (int k0 = 0; k0 < D; k0 += 32) {
        float4 v[8];
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = *(const float4*)&x[k0 + 4 * i];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            ss = __builtin_fmaf(v[i].x, v[i].x, ss);
            ss = __builtin_fmaf(v[i].y, v[i].y, ss);
            ss = __builtin_fmaf(v[i].z, v[i].z, ss);
            ss = __builtin_fmaf(v[i].w, v[i].w, ss);
        }
    }
    return ss;
}

template <int ROWS, bool IS_V>
__device__ __forceinline__ void encode_rows(const EncodeArgs& a, const int bx, const int h,
                                            const int64_t n_tiles, const int tile_stride,
                                            float* rot_s) {
    __shared__ __align__(16) float xs[ROWS + 1][D];     // (one more row of zeros: the compact rotation reads up to BGTQ_ROT_COL values past a segment's start)
    __shared__ float nrm[ROWS][BGTQ_MAX_SEGMENTS];
    __shared__ float nrm_out[ROWS][BGTQ_MAX_SEGMENTS];
    __shared__ uint8_t cds[ROWS][D];
    __shared__ uint16_t xraw[ROWS][D];
    __shared__ typename std::conditional<IS_V, StagedV, StagedK>::type sp;

    const int j = threadIdx.x;
    const bgtq_head_plan& P = a.plans[h];
    const int64_t N = (int64_t)a.B * a.S;
    const float* RT = IS_V ? P.v_rot_T : P.k_rot_T;

    // ---- 0. one burst: plan tables, the first tile's raw rows, and (V) the rotation column ----
    // A work-group stages the plan once and then walks tiles bx, bx + tile_stride, ...
    if constexpr (IS_V) {
        if (j == 0) sp.v_bits = P.v_bits;
        if (j < 16) { sp.centroids[j] = P.v_centroids[j]; sp.boundaries[j] = P.v_boundaries[j]; }
    } else {
        if (j < 56) sp.hdr[j] = ((const int*)&P)[j];
#pragma unroll
        for (int i = 0; i < 4; i++)
            ((uint32_t*)sp.code_lut)[j + i * NT] = ((const uint32_t*)&P.code_lut[0][0])[j + i * NT];
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int e = j + i * NT;                        // segment e / 32, level e % 32
            sp.centroids[e] = P.k_centroids[e >> 5][e & 31];
        }
    }
    xs[ROWS][j] = 0.f;
    uint16_t xr[ROWS];                 // raw rows of the tile about to be processed
    int tp[2];         // decode append: their cache positions, fetched with them
    auto fetch_rows = [&](int64_t tile) {
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            int64_t n = tile * ROWS + r;
            uint16_t v = 0;
            int t = 0;
            if (n < N) {
                int b, s;
                split_row(n, a.S, b, s);
                v = a.x[b * a.x_sb + h * a.x_sh + s * a.x_ss + j];
                if (ROWS <= 2) t = (a.t_pos ? a.t_pos[b] : a.t_pos_scalar) + s;
            }
            xr[r] = v;
            if (ROWS <= 2) tp[r] = t;
        }
    };
    fetch_rows(bx);
    int4 k_dim = {0, 0, 0, 0};
    uint2 k_byte = {0u, 0u};
    float k_lut_off = 0.f, k_lut_scale = 0.f;
    if constexpr (!IS_V) {
        k_dim = *(const int4*)P.enc_dim[j];
        k_byte = *(const uint2*)P.enc_byte[a.layout == BGTQ_K_MIXED ? 1 : 0][j];
        k_lut_off = P.lut_offset[j];
        k_lut_scale = P.lut_inv_scale[j];
    } else if (j < D / 2) {
        k_byte = *(const uint2*)P.enc_vbyte[a.layout == BGTQ_V_NIBBLE ? 1 : 0][j];
    }
    // Decode append (tiles of one or two rows) is latency bound.  K: the whole rotation matrix is requested now,
    // before anything else is known (which rows a thread needs is only known once the plan is in
    // LDS), 16 bytes a lane and contiguous across the wave (32 loads a thread), and parked in LDS
    // (rot_s) ahead of the rotation, which then reads its column from there.  16-row tiles fetch
    // their column slices per tile instead.
    // V's rotation is dense and is needed later than its rows: its column comes straight into
    // registers, one 4-byte load per matrix row (the wide loads of the whole matrix land later).
    constexpr bool STAGED = ROWS <= 2 && !IS_V;
    constexpr int PF = (ROWS <= 2 && IS_V) ? D : 0;
    rot_piece rst[STAGED ? D / 4 : 1];
    float rpre[PF > 0 ? PF : 1];
    // K, where no rotated segment is longer than BGTQ_ROT_COL dims: the plan also holds every dim's
    // rotation column cut down to its segment, which goes straight into registers (12 wide loads
    // instead of 32 and no trip through LDS)
    constexpr int RC = STAGED ? BGTQ_ROT_COL : 4;
    float rc[RC];
    bool compact = false;
    if constexpr (STAGED) {
        compact = P.rot_compact[0] != 0;                 // (uniform)
        if (compact) {
#pragma unroll
            for (int i = 0; i < RC / 4; i++) {
                const float4 v = *(const float4*)&P.k_rot_cols[j][4 * i];
                rc[4 * i] = v.x; rc[4 * i + 1] = v.y; rc[4 * i + 2] = v.z; rc[4 * i + 3] = v.w;
            }
        } else {
            fetch_rotation(RT, j, rst);
        }
    }
    if constexpr (PF > 0) {
        // (the plan holds v_rot_T four rows interleaved: 16-byte loads, contiguous across the threads)
#pragma unroll
        for (int i = 0; i < PF / 4; i++) {
            const float4 v = *(const float4*)P.v_rot_T4[i][j];
            rpre[4 * i] = v.x; rpre[4 * i + 1] = v.y; rpre[4 * i + 2] = v.z; rpre[4 * i + 3] = v.w;
        }
    }
    if constexpr (!IS_V) __syncthreads();     // (K reads the staged header next; V's staged tables are first read three barriers on)

    // ---- per-thread static data, read ready-made from the plan (requested in the first burst) ----
    int n_seg = 1, g = 0, gs = 0, ge = D, ident = 0, src_dim = j;
    float lut_off_j = 0.f, lut_scale_j = 0.f;          // K: this dim's cell-search parameters
    if constexpr (!IS_V) {
        lut_off_j = k_lut_off;
        lut_scale_j = k_lut_scale;
        n_seg = sp.hdr[H_NSEG];
        g = k_dim.x;
        gs = k_dim.y;
        ge = k_dim.z;
        ident = k_dim.w & 0xFF;
        src_dim = k_dim.w >> 8;
    }
    // output byte j: 0: zero fill, 1: bit stream, 2: raw byte copy
    const int mode = (int)(k_byte.x & 3u);
    const int bw = (int)((k_byte.x >> 2) & 15u);
    const StreamSlot slot{0, (int)(k_byte.x >> 8), (int)((k_byte.x >> 6) & 3u)};
    const int c0 = (int)k_byte.y;                       // (the slot's first code is folded into the base)

    for (int64_t tile = bx; tile < n_tiles; tile += tile_stride) {
    const int64_t row0 = tile * ROWS;
    int tcur[2] = {0, 0};              // this tile's positions (the prefetch below overwrites tp)
    if (ROWS <= 2) { tcur[0] = tp[0]; tcur[1] = tp[ROWS == 2 ? 1 : 0]; }
    // ---- 1. rows to LDS, next tile's rows on their way, gather by head_perm (K) -------------
    if constexpr (IS_V) {              // (no gather: a thread converts its own value)
#pragma unroll
        for (int r = 0; r < ROWS; r++) xs[r][j] = bgtq_h2f(xr[r]);
        if (tile + tile_stride < n_tiles) fetch_rows(tile + tile_stride);
    } else {
#pragma unroll
        for (int r = 0; r < ROWS; r++) xraw[r][j] = xr[r];
        __syncthreads();
        if (tile + tile_stride < n_tiles) fetch_rows(tile + tile_stride);
#pragma unroll
        for (int r = 0; r < ROWS; r++) xs[r][j] = bgtq_h2f(xraw[r][src_dim]);
    }
    __syncthreads();

    // ---- 2. group norms: thread (r, grp) runs one sequential chain ---------
    if (j < ROWS * BGTQ_MAX_SEGMENTS) {
        int r = j / BGTQ_MAX_SEGMENTS, gg = j % BGTQ_MAX_SEGMENTS;
        float n = 0.f;
        if (gg < n_seg) {
            int s = 0, e = D;
            if constexpr (!IS_V) { s = sp.hdr[H_START + gg]; e = s + sp.hdr[H_LEN + gg]; }
            float ss = 0.f;
            if constexpr (IS_V) {
                ss = chain_sumsq_row(xs[r]);
            } else {                           // short ranges: the batches would mostly run masked
#pragma unroll 8
                for (int k = s; k < e; k++) ss = __builtin_fmaf(xs[r][k], xs[r][k], ss);
            }
            n = __builtin_sqrtf(ss + 1e-30f);
        }
        nrm[r][gg] = n;
    }
    __syncthreads();

    // ---- 3. normalise -------------------------------------------------------
    float xh[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        float v = 0.f;
        if (g >= 0) {
            float n = nrm[r][g];
            float safe = (n > (IS_V ? 1e-8f : 1e-10f)) ? n : 1.0f;
            v = xs[r][j] / safe;
        }
        xh[r] = v;
        xs[r][j] = v;     // only this thread ever touched xs[r][j] since the barrier
    }
    if constexpr (STAGED) { if (!compact) park_rotation(rot_s, j, rst); }   // (every tile of the walk: the registers stay as they are)
    __syncthreads();

    // ---- 4. rotate ------------------------------------------------------------
    // Same chain as written in the contract above; the matrix column is fetched in
    // batches of RB independent loads so the chain never waits on one load at a time.
    float y[ROWS];
    if (ident || g < 0) {
#pragma unroll
        for (int r = 0; r < ROWS; r++) y[r] = xh[r];
    } else {
#pragma unroll
        for (int r = 0; r < ROWS; r++) y[r] = 0.f;
        if constexpr (STAGED) {
            if (compact) {
                // The column is in registers and is zero past the segment's end, so the chain runs over
                // BGTQ_ROT_COL terms for every dim without a length test: a term x * 0 leaves the sum as it
                // is (the row is followed by zeros, so every x read is finite).  The row values of a batch
                // are read ahead of the chain.
                constexpr int CB = 16;
#pragma unroll
                for (int i0 = 0; i0 < RC; i0 += CB) {
                    float xv[ROWS][CB];
#pragma unroll
                    for (int i = 0; i < CB; i++)
#pragma unroll
                        for (int r = 0; r < ROWS; r++) xv[r][i] = (&xs[r][0])[gs + i0 + i];
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int i = 0; i < CB; i++)
#pragma unroll
                        for (int r = 0; r < ROWS; r++) y[r] = __builtin_fmaf(xv[r][i], rc[i0 + i], y[r]);
                }
            } else
            // column j of the parked rotation against the rows, the LDS reads a batch ahead of
            // the chain that consumes them
            {
                constexpr int CB = 16;
                for (int k0 = gs; k0 < ge; k0 += CB) {
                    float rk[CB], xv[ROWS][CB];
#pragma unroll
                    for (int i = 0; i < CB; i++) {
                        const int k = min(k0 + i, ge - 1);
                        rk[i] = rot_s[k * D + j];
#pragma unroll
                        for (int r = 0; r < ROWS; r++) xv[r][i] = xs[r][k];
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int i = 0; i < CB; i++)
                        if (k0 + i < ge) {
#pragma unroll
                            for (int r = 0; r < ROWS; r++) y[r] = __builtin_fmaf(xv[r][i], rk[i], y[r]);
                        }
                }
            }
        }
        if constexpr (PF > 0) {                 // V: the column fetched at the top of the kernel
            // row values come from LDS a batch of 32 dims ahead of the chain that consumes them
            constexpr int CB = 32;
            float4 xv[2][ROWS][CB / 4];
            auto load = [&](const int b) {
#pragma unroll
                for (int r = 0; r < ROWS; r++)
#pragma unroll
                    for (int i = 0; i < CB / 4; i++) xv[b & 1][r][i] = *(const float4*)&xs[r][b * CB + 4 * i];
            };
            load(0);
#pragma unroll
            for (int b = 0; b < PF / CB; b++) {
                if (b + 1 < PF / CB) load(b + 1);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < CB / 4; i++)
#pragma unroll
                    for (int r = 0; r < ROWS; r++) {
                        const float4 x4 = xv[b & 1][r][i];
                        const int k = b * CB + 4 * i;
                        y[r] = __builtin_fmaf(x4.x, rpre[k], y[r]);
                        y[r] = __builtin_fmaf(x4.y, rpre[k + 1], y[r]);
                        y[r] = __builtin_fmaf(x4.z, rpre[k + 2], y[r]);
                        y[r] = __builtin_fmaf(x4.w, rpre[k + 3], y[r]);
                    }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        constexpr int RB = IS_V ? 32 : 16;
        for (int k0 = (STAGED || PF > 0) ? ge : gs; k0 < ge; k0 += RB) {
            float rt[RB];
#pragma unroll
            for (int i = 0; i < RB; i++) rt[i] = RT[min(k0 + i, ge - 1) * D + j];
            if (IS_V) {
                // dense rotation: the range is the whole row, so the row values can be
                // read four at a time (same chain order)
#pragma unroll
                for (int i = 0; i < RB; i += 4) {
#pragma unroll
                    for (int r = 0; r < ROWS; r++) {
                        const float4 x4 = *(const float4*)&xs[r][k0 + i];
                        y[r] = __builtin_fmaf(x4.x, rt[i], y[r]);
                        y[r] = __builtin_fmaf(x4.y, rt[i + 1], y[r]);
                        y[r] = __builtin_fmaf(x4.z, rt[i + 2], y[r]);
                        y[r] = __builtin_fmaf(x4.w, rt[i + 3], y[r]);
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < RB; i++) {
                    if (k0 + i < ge) {
#pragma unroll
                        for (int r = 0; r < ROWS; r++) y[r] = __builtin_fmaf(xs[r][k0 + i], rt[i], y[r]);
                    }
                }
            }
        }
    }

    // ---- 5. scalar quantise ---------------------------------------------------
    const bool need_cent = IS_V || a.layout == BGTQ_K_MIXED || a.corrected;
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        int code = 0;
        if (IS_V) {
            if constexpr (IS_V) {
                // (all 15 slots are read at once; those past the codebook's last boundary are skipped)
                const int nb = (1 << sp.v_bits) - 1;
                float bd[15];
#pragma unroll
                for (int b = 0; b < 15; b++) bd[b] = sp.boundaries[b];
#pragma unroll
                for (int b = 0; b < 15; b++) code += (b < nb && y[r] > bd[b]) ? 1 : 0;
            }
        } else if (g >= 0) {
            if constexpr (!IS_V) {
                if (a.quant_mode == BGTQ_QUANT_EXACT) {
                    int nb = (1 << sp.hdr[H_BW + g]) - 1;
                    for (int b = 0; b < nb; b++) code += (P.k_boundaries[g][b] < y[r]) ? 1 : 0;
                } else {
                    float t = (y[r] - lut_off_j) * lut_scale_j;
                    t = fminf(fmaxf(t, 0.0f), (float)(BGTQ_LUT_BINS - 1));
                    code = sp.code_lut[g * BGTQ_LUT_BINS + (int)t];
                }
            }
        }
        cds[r][j] = (uint8_t)code;
        // centroid of the chosen code for the norm correction below; it is parked in xs
        // after the barrier (other threads may still be reading xs in their rotation)
        if (need_cent) {
            if constexpr (IS_V) y[r] = sp.centroids[code];
            else y[r] = g < 0 ? 0.f : code < 32 ? sp.centroids[g * 32 + code] : P.k_centroids[g][code];
        }
    }
    __syncthreads();
    if (need_cent) {
#pragma unroll
        for (int r = 0; r < ROWS; r++) xs[r][j] = y[r];
    }
    __syncthreads();

    // ---- 6. norms to store (raw or divided by ||centroids[codes]||) ---------
    // Single-row tiles give this chain to the second wave: the first one packs the record meanwhile
    // (neither needs anything of the other: the barrier between them is left out below).
    const int jn = ROWS == 1 ? j - 64 : j;
    if (jn >= 0 && jn < ROWS * BGTQ_MAX_SEGMENTS) {
        int r = jn / BGTQ_MAX_SEGMENTS, gg = jn % BGTQ_MAX_SEGMENTS;
        float out = 0.f;
        if (gg < n_seg) {
            float n = nrm[r][gg];
            if (IS_V) {
                const float cs = chain_sumsq_row(xs[r]);
                float cn = __builtin_sqrtf(cs + 1e-20f);
                out = n / (cn > 1e-10f ? cn : 1.0f);
            } else if (a.layout == BGTQ_K_MIXED || a.corrected) {
                int s = 0, e = 0;
                if constexpr (!IS_V) { s = sp.hdr[H_START + gg]; e = s + sp.hdr[H_LEN + gg]; }
                float cs = 0.f;
                for (int k = s; k < e; k++) {
                    float c = xs[r][k];
                    cs = __builtin_fmaf(c, c, cs);
                }
                out = n / fmaxf(__builtin_sqrtf(cs), 1e-10f);
            } else {
                out = n;
            }
        }
        nrm_out[r][gg] = out;
    }
    if (ROWS > 1 || a.codes_out) __syncthreads();       // (uniform; the cache norms below are stored by the thread that made them)

    // ---- 7a. unpacked outputs (codes path) ------------------------------------
    if (a.codes_out) {
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            int64_t n = row0 + r;
            if (n < N) a.codes_out[n * D + j] = cds[r][j];
        }
        if (IS_V) {
            if (j < ROWS && row0 + j < N && a.norms)
                a.norms[row0 + j] = bgtq_f2h(nrm_out[j][0]);
        } else if (a.norms_f32_out && j < ROWS * BGTQ_MAX_SEGMENTS) {
            int r = j / BGTQ_MAX_SEGMENTS, gg = j % BGTQ_MAX_SEGMENTS;
            if (row0 + r < N && gg < a.norm_width)
                a.norms_f32_out[(row0 + r) * a.norm_width + gg] = nrm_out[r][gg];
        }
    }

    // ---- 7b. cache norms --------------------------------------------------------
    if (!a.codes_out && jn >= 0 && jn < ROWS * BGTQ_MAX_SEGMENTS) {
        int r = jn / BGTQ_MAX_SEGMENTS, gg = jn % BGTQ_MAX_SEGMENTS;
        int64_t n = row0 + r;
        int width = IS_V ? 1 : a.norm_width;
        if (n < N && gg < width) {
            int b, s;
            split_row(n, a.S, b, s);
            int64_t t = ROWS <= 2 ? tcur[r & 1] : (a.t_pos ? a.t_pos[b] : a.t_pos_scalar) + s;
            if (t >= 0 && t < a.max_T)
                a.norms[b * a.n_sb + h * a.n_sh + t * a.n_st + gg] = bgtq_f2h(nrm_out[r][gg]);
        }
    }

    // ---- 8. pack: thread j produces output byte j of every row ---------------
    if (!a.codes_out && j < a.row_width) {
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            int64_t n = row0 + r;
            if (n >= N) break;
            int b, s;
            split_row(n, a.S, b, s);
            int64_t t = ROWS <= 2 ? tcur[r & 1] : (a.t_pos ? a.t_pos[b] : a.t_pos_scalar) + s;
            if (t < 0 || t >= a.max_T) continue;
            unsigned v = 0;
            if (mode == 1)      v = ROWS <= 2 ? stream_byte_batched(&cds[r][c0], slot, bw) : stream_byte(&cds[r][c0], slot, bw);
            else if (mode == 2) v = cds[r][c0];
            a.packed[b * a.p_sb + h * a.p_sh + t * a.p_st + j] = (uint8_t)v;
        }
    }
    __syncthreads();            // the tile buffers are rewritten by the next tile
    }
}

template <int ROWS, bool IS_V>
__global__ __launch_bounds__(NT) void encode_kernel(EncodeArgs a) {
    const int64_t N = (int64_t)a.B * a.S;
    __shared__ __align__(16) float rot_s[(ROWS <= 2 && !IS_V) ? D * D : 4];
    encode_rows<ROWS, IS_V>(a, blockIdx.x, blockIdx.y, (N + ROWS - 1) / ROWS, gridDim.x, rot_s);
}
// The prefill-sized encoder is throughput bound: at least 4 waves per SIMD (128 registers a
// lane), which the register allocator does not aim for by itself.
template <bool IS_V>
__global__ __launch_bounds__(NT, 4) void encode_kernel16(EncodeArgs a) {
    const int64_t N = (int64_t)a.B * a.S;
    encode_rows<16, IS_V>(a, blockIdx.x, blockIdx.y, (N + 15) / 16, gridDim.x, nullptr);
}

template <bool IS_V>
int launch_encode(const EncodeArgs& a, hipStream_t st) {
    int64_t N = (int64_t)a.B * a.S;
    if (N == 0 || a.n_kv == 0) return BGTQ_OK;
    if (N > INT32_MAX) return BGTQ_EINVAL;        // the kernels index rows with 32 bits
    // Few rows (decode append): small tiles so every row gets its own work-group
    // and the step stays latency-bound; many rows (prefill): 16-row tiles so the
    // rotation matrix is amortised.
    if (N <= 32) {               // one row a work-group: the shortest chain of dependent stages
        dim3 grid((unsigned)N, (unsigned)a.n_kv);
        hipLaunchKernelGGL((encode_kernel<1, IS_V>), grid, dim3(NT), 0, st, a);
    } else if (N <= 64) {
        dim3 grid((unsigned)((N + 1) / 2), (unsigned)a.n_kv);
        hipLaunchKernelGGL((encode_kernel<2, IS_V>), grid, dim3(NT), 0, st, a);
    } else {
        // a work-group stages its head's plan once and walks several tiles: about 10
        // work-groups per CU in total
        int64_t tiles = (N + 15) / 16;
        int64_t want = (256 * 10 + a.n_kv - 1) / a.n_kv;
        dim3 grid((unsigned)(tiles < want ? tiles : want), (unsigned)a.n_kv);
        hipLaunchKernelGGL((encode_kernel16<IS_V>), grid, dim3(NT), 0, st, a);
    }
    return bgtq_launch_status();
}

// ---- query permute + rotate ---------------------------------------------------
struct RotQArgs {
    const bgtq_head_plan* plans;
    const uint16_t* q;  int64_t q_sr, q_sh;
    uint16_t* q_rot;    int64_t qr_sr, qr_sh;
    int n_rows, n_q, gqa;
    int group;          // query heads per work-group: 1 or 4
};

// QG query heads (h_first ..) of one (row, KV head): the rotation is fetched and parked once for
// all of them, the rows come in with the same round of loads (un-permuted, so that their
// addresses do not wait for head_perm; the gather by head_perm then runs through LDS), and a
// batch of the rotation column read from LDS serves every row.  Each row's chain is the one
// written in the contract above; rows past the group's last head are zeros and are not stored.
template <int QG>
__device__ __forceinline__ void rotate_q_group(const RotQArgs& a, const int64_t row, const int h,
                                               const int h_first, float* rot_s) {
    __shared__ uint16_t qraw[QG][D];
    __shared__ float xs[QG + 1][D];                 // (one more row of zeros, see the compact chain below)
    const int j = threadIdx.x;
    const bgtq_head_plan& P = a.plans[h];
    // what thread j needs of the segment table comes ready-made (enc_dim), and so does its column of
    // the rotation where the plan holds it by columns (no rotated segment longer than BGTQ_ROT_COL)
    const int4 dim = *(const int4*)P.enc_dim[j];
    const int g = dim.x, s = dim.y, e = dim.z, ident = dim.w & 0xFF, src = dim.w >> 8;
    const bool compact = P.rot_compact[0] != 0;      // (uniform)
    rot_piece rst[D / 4];
    float rc[BGTQ_ROT_COL];
    if (compact) {
#pragma unroll
        for (int i = 0; i < BGTQ_ROT_COL / 4; i++) {
            const float4 v = *(const float4*)&P.k_rot_cols[j][4 * i];
            rc[4 * i] = v.x; rc[4 * i + 1] = v.y; rc[4 * i + 2] = v.z; rc[4 * i + 3] = v.w;
        }
    } else {
        fetch_rotation(P.k_rot_T, j, rst);
    }
    const int gqa = a.gqa;
#pragma unroll
    for (int r = 0; r < QG; r++)
        qraw[r][j] = h_first + r < gqa ? a.q[row * a.q_sr + (int64_t)(h * gqa + h_first + r) * a.q_sh + j] : (uint16_t)0;
    xs[QG][j] = 0.f;
    if (!compact) park_rotation(rot_s, j, rst);
    __syncthreads();
#pragma unroll
    for (int r = 0; r < QG; r++) xs[r][j] = bgtq_h2f(qraw[r][src]);
    __syncthreads();
    float acc[QG];
#pragma unroll
    for (int r = 0; r < QG; r++) acc[r] = 0.f;
    if (g >= 0) {
        if (ident) {
#pragma unroll
            for (int r = 0; r < QG; r++) acc[r] = xs[r][j];
        } else if (compact) {
            // the column is zero past the segment's end: BGTQ_ROT_COL terms for every dim, no length test
            // (a term x * 0 leaves the sum as it is; the values read past the row are finite)
            constexpr int CB = QG == 1 ? 16 : 8;
#pragma unroll
            for (int i0 = 0; i0 < BGTQ_ROT_COL; i0 += CB) {
                float xv[QG][CB];
#pragma unroll
                for (int i = 0; i < CB; i++)
#pragma unroll
                    for (int r = 0; r < QG; r++) xv[r][i] = (&xs[r][0])[s + i0 + i];
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < CB; i++)
#pragma unroll
                    for (int r = 0; r < QG; r++) acc[r] = __builtin_fmaf(xv[r][i], rc[i0 + i], acc[r]);
            }
        } else {
            constexpr int CB = QG == 1 ? 16 : 8;    // LDS reads a batch ahead of the chains
            for (int k0 = s; k0 < e; k0 += CB) {
                float rk[CB], xv[QG][CB];
#pragma unroll
                for (int i = 0; i < CB; i++) {
                    const int k = min(k0 + i, e - 1);
                    rk[i] = rot_s[k * D + j];
#pragma unroll
                    for (int r = 0; r < QG; r++) xv[r][i] = xs[r][k];
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < CB; i++)
                    if (k0 + i < e) {
#pragma unroll
                        for (int r = 0; r < QG; r++) acc[r] = __builtin_fmaf(xv[r][i], rk[i], acc[r]);
                    }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < QG; r++)
        if (h_first + r < gqa)
            a.q_rot[row * a.qr_sr + (int64_t)(h * gqa + h_first + r) * a.qr_sh + j] = bgtq_f2h(acc[r]);
}

// Work-group `bid` of the query part: a.group heads of one (row, KV head).  One head per
// work-group where that still leaves the chip partly idle (every work-group fetches the 64 KB
// rotation), four where the rows are many.
__device__ __forceinline__ void rotate_q_block(const RotQArgs& a, const int bid, float* rot_s) {
    const int n_kv = a.n_q / a.gqa;
    const int per = (a.gqa + a.group - 1) / a.group;            // work-groups per (row, KV head)
    const int rowh = bid / per, part = bid - rowh * per;
    if (a.group == 1) rotate_q_group<1>(a, rowh / n_kv, rowh % n_kv, part, rot_s);
    else              rotate_q_group<4>(a, rowh / n_kv, rowh % n_kv, part * 4, rot_s);
}
__host__ inline int rotate_q_group_size(int64_t n_rows, int n_q) { return n_rows * n_q > 256 ? 4 : 1; }
__host__ inline unsigned rotate_q_blocks(int64_t n_rows, int n_kv, int gqa, int group) {
    return (unsigned)(n_rows * n_kv * ((gqa + group - 1) / group));
}

__global__ __launch_bounds__(NT) void rotate_q_kernel(RotQArgs a) {
    __shared__ __align__(16) float rot_s[D * D];
    rotate_q_block(a, blockIdx.x, rot_s);
}

constexpr int PREP_ROWS = 1;       // rows of a work-group in the one-launch preparation

// ---- decode-step preparation: append-encode K and V and rotate the queries, one launch ----
// Work-groups [0, nv) encode one V row each (the longest chain of the three goes out first),
// [nv, nv + nk) one K row each, the rest rotate one or four query heads each.
__global__ __launch_bounds__(NT) void prepare_kernel(EncodeArgs ak, EncodeArgs av, RotQArgs aq,
                                                     int k_tiles, int v_tiles) {
    __shared__ __align__(16) float rot_s[D * D];       // the work-group's rotation, whatever its role
    int bid = blockIdx.x;
    const int nk = k_tiles * ak.n_kv, nv = v_tiles * av.n_kv;
    if (bid < nv) {
        encode_rows<PREP_ROWS, true>(av, bid % v_tiles, bid / v_tiles, v_tiles, v_tiles, rot_s);
    } else if (bid < nk + nv) {
        bid -= nv;
        encode_rows<PREP_ROWS, false>(ak, bid % k_tiles, bid / k_tiles, k_tiles, k_tiles, rot_s);
    } else {
        rotate_q_block(aq, bid - (nk + nv), rot_s);
    }
}

// argument checks + EncodeArgs assembly shared by the separate and the fused entry points
int fill_k_args(EncodeArgs& a, const bgtq_head_plan* plans,
                const void* k, int64_t k_sb, int64_t k_sh, int64_t k_ss, int B, int n_kv, int S,
                void* k_packed, int64_t kp_sb, int64_t kp_sh, int64_t kp_st, int k_row_width,
                void* k_norms, int64_t kn_sb, int64_t kn_sh, int64_t kn_st, int norm_width,
                const int32_t* t_pos, int t_pos_scalar, int max_T, int k_layout, int quant_mode) {
    BGTQ_CHECK_ARG(plans && k && k_packed && k_norms);
    BGTQ_CHECK_ARG(k_row_width >= 0 && k_row_width <= NT);
    BGTQ_CHECK_ARG(norm_width >= 0 && norm_width <= BGTQ_MAX_SEGMENTS);
    BGTQ_CHECK_ARG(k_layout == BGTQ_K_BITPACKED || k_layout == BGTQ_K_MIXED);
    BGTQ_CHECK_ARG(quant_mode == BGTQ_QUANT_LUT256 || quant_mode == BGTQ_QUANT_EXACT);
    BGTQ_CHECK_ARG(t_pos || t_pos_scalar >= 0);
    BGTQ_CHECK_ARG(max_T >= 0);
    if (!t_pos && (int64_t)t_pos_scalar + S > max_T) return BGTQ_ELIMIT;   // would run past the cache
    a.max_T = max_T;
    a.plans = plans; a.x = (const uint16_t*)k; a.x_sb = k_sb; a.x_sh = k_sh; a.x_ss = k_ss;
    a.B = B; a.n_kv = n_kv; a.S = S;
    a.packed = (uint8_t*)k_packed; a.p_sb = kp_sb; a.p_sh = kp_sh; a.p_st = kp_st;
    a.row_width = k_row_width;
    a.norms = (uint16_t*)k_norms; a.n_sb = kn_sb; a.n_sh = kn_sh; a.n_st = kn_st;
    a.norm_width = norm_width;
    a.t_pos = t_pos; a.t_pos_scalar = t_pos_scalar;
    a.layout = k_layout; a.quant_mode = quant_mode;
    return BGTQ_OK;
}

int fill_v_args(EncodeArgs& a, const bgtq_head_plan* plans,
                const void* v, int64_t v_sb, int64_t v_sh, int64_t v_ss, int B, int n_kv, int S,
                void* v_packed, int64_t vp_sb, int64_t vp_sh, int64_t vp_st, int v_row_width,
                void* v_norms, int64_t vn_sb, int64_t vn_sh, int64_t vn_st,
                const int32_t* t_pos, int t_pos_scalar, int max_T, int v_layout) {
    BGTQ_CHECK_ARG(plans && v && v_packed && v_norms);
    BGTQ_CHECK_ARG(v_row_width >= 0 && v_row_width <= NT);
    BGTQ_CHECK_ARG(v_layout == BGTQ_V_BITPACKED || v_layout == BGTQ_V_NIBBLE);
    BGTQ_CHECK_ARG(t_pos || t_pos_scalar >= 0);
    BGTQ_CHECK_ARG(max_T >= 0);
    if (!t_pos && (int64_t)t_pos_scalar + S > max_T) return BGTQ_ELIMIT;
    a.max_T = max_T;
    a.plans = plans; a.x = (const uint16_t*)v; a.x_sb = v_sb; a.x_sh = v_sh; a.x_ss = v_ss;
    a.B = B; a.n_kv = n_kv; a.S = S;
    a.packed = (uint8_t*)v_packed; a.p_sb = vp_sb; a.p_sh = vp_sh; a.p_st = vp_st;
    a.row_width = v_row_width;
    a.norms = (uint16_t*)v_norms; a.n_sb = vn_sb; a.n_sh = vn_sh; a.n_st = vn_st;
    a.norm_width = 1;
    a.t_pos = t_pos; a.t_pos_scalar = t_pos_scalar;
    a.layout = v_layout;
    return BGTQ_OK;
}

}  // namespace

extern "C" {

int bgtq_encode_k(const bgtq_head_plan* plans,
                  const void* k, int64_t k_sb, int64_t k_sh, int64_t k_ss,
                  int B, int n_kv, int S,
                  void* k_packed, int64_t kp_sb, int64_t kp_sh, int64_t kp_st, int k_row_width,
                  void* k_norms, int64_t kn_sb, int64_t kn_sh, int64_t kn_st, int norm_width,
                  const int32_t* t_pos, int t_pos_scalar, int max_T,
                  int k_layout, int quant_mode, void* stream) {
    BGTQ_CHECK_ARG(B >= 0 && n_kv >= 0 && S >= 0);
    if (B == 0 || n_kv == 0 || S == 0) return BGTQ_OK;     // nothing to encode
    EncodeArgs a{};
    int rc = fill_k_args(a, plans, k, k_sb, k_sh, k_ss, B, n_kv, S, k_packed, kp_sb, kp_sh, kp_st, k_row_width,
                         k_norms, kn_sb, kn_sh, kn_st, norm_width, t_pos, t_pos_scalar, max_T, k_layout, quant_mode);
    if (rc != BGTQ_OK) return rc;
    return launch_encode<false>(a, (hipStream_t)stream);
}

int bgtq_encode_v(const bgtq_head_plan* plans,
                  const void* v, int64_t v_sb, int64_t v_sh, int64_t v_ss,
                  int B, int n_kv, int S,
                  void* v_packed, int64_t vp_sb, int64_t vp_sh, int64_t vp_st, int v_row_width,
                  void* v_norms, int64_t vn_sb, int64_t vn_sh, int64_t vn_st,
                  const int32_t* t_pos, int t_pos_scalar, int max_T,
                  int v_layout, void* stream) {
    BGTQ_CHECK_ARG(B >= 0 && n_kv >= 0 && S >= 0);
    if (B == 0 || n_kv == 0 || S == 0) return BGTQ_OK;
    EncodeArgs a{};
    int rc = fill_v_args(a, plans, v, v_sb, v_sh, v_ss, B, n_kv, S, v_packed, vp_sb, vp_sh, vp_st, v_row_width,
                         v_norms, vn_sb, vn_sh, vn_st, t_pos, t_pos_scalar, max_T, v_layout);
    if (rc != BGTQ_OK) return rc;
    return launch_encode<true>(a, (hipStream_t)stream);
}

int bgtq_compress_k_codes(const bgtq_head_plan* plan, const void* k, int64_t N,
                          void* codes, float* norms, int norm_width,
                          int corrected, int quant_mode, void* stream) {
    BGTQ_CHECK_ARG(plan && k && codes && norms);
    BGTQ_CHECK_ARG(N >= 0 && N < (int64_t)1 << 31);
    BGTQ_CHECK_ARG(norm_width >= 1 && norm_width <= BGTQ_MAX_SEGMENTS);
    BGTQ_CHECK_ARG(quant_mode == BGTQ_QUANT_LUT256 || quant_mode == BGTQ_QUANT_EXACT);
    EncodeArgs a{};
    a.plans = plan; a.x = (const uint16_t*)k; a.x_sb = 0; a.x_sh = 0; a.x_ss = D;
    a.B = 1; a.n_kv = 1; a.S = (int)N;
    a.codes_out = (uint8_t*)codes; a.norms_f32_out = norms; a.norm_width = norm_width;
    a.corrected = corrected; a.layout = BGTQ_K_BITPACKED; a.quant_mode = quant_mode;
    return launch_encode<false>(a, (hipStream_t)stream);
}

int bgtq_compress_v_codes(const bgtq_head_plan* plan, const void* v, int64_t N,
                          void* codes, void* norms_f16, void* stream) {
    BGTQ_CHECK_ARG(plan && v && codes && norms_f16);
    BGTQ_CHECK_ARG(N >= 0 && N < (int64_t)1 << 31);
    EncodeArgs a{};
    a.plans = plan; a.x = (const uint16_t*)v; a.x_sb = 0; a.x_sh = 0; a.x_ss = D;
    a.B = 1; a.n_kv = 1; a.S = (int)N;
    a.codes_out = (uint8_t*)codes; a.norms = (uint16_t*)norms_f16; a.norm_width = 1;
    return launch_encode<true>(a, (hipStream_t)stream);
}

int bgtq_rotate_q(const bgtq_head_plan* plans,
                  const void* q, int64_t q_sr, int64_t q_sh,
                  void* q_rot, int64_t qr_sr, int64_t qr_sh,
                  int n_rows, int n_kv, int gqa, void* stream) {
    BGTQ_CHECK_ARG(plans && q && q_rot);
    BGTQ_CHECK_ARG(n_rows >= 0 && n_kv >= 0 && gqa >= 1);
    if (n_rows == 0 || n_kv == 0) return BGTQ_OK;
    const int group = rotate_q_group_size(n_rows, n_kv * gqa);
    RotQArgs a{plans, (const uint16_t*)q, q_sr, q_sh, (uint16_t*)q_rot, qr_sr, qr_sh, n_rows, n_kv * gqa, gqa, group};
    hipLaunchKernelGGL(rotate_q_kernel, dim3(rotate_q_blocks(n_rows, n_kv, gqa, group)), dim3(NT), 0,
                       (hipStream_t)stream, a);
    return bgtq_launch_status();
}

int bgtq_decode_prepare(const bgtq_head_plan* plans,
                        const void* k, int64_t k_sb, int64_t k_sh, int64_t k_ss,
                        const void* v, int64_t v_sb, int64_t v_sh, int64_t v_ss,
                        int B, int n_kv, int S,
                        void* k_packed, int64_t kp_sb, int64_t kp_sh, int64_t kp_st, int k_row_width,
                        void* k_norms, int64_t kn_sb, int64_t kn_sh, int64_t kn_st, int norm_width,
                        void* v_packed, int64_t vp_sb, int64_t vp_sh, int64_t vp_st, int v_row_width,
                        void* v_norms, int64_t vn_sb, int64_t vn_sh, int64_t vn_st,
                        const int32_t* t_pos, int t_pos_scalar, int max_T,
                        int k_layout, int v_layout, int quant_mode,
                        const void* q, int64_t q_sr, int64_t q_sh,
                        void* q_rot, int64_t qr_sr, int64_t qr_sh, int gqa, void* stream) {
    BGTQ_CHECK_ARG(B >= 0 && n_kv >= 0 && S >= 0 && gqa >= 1);
    if (B == 0 || n_kv == 0) return BGTQ_OK;
    EncodeArgs ak{}, av{};
    int rc = fill_k_args(ak, plans, k, k_sb, k_sh, k_ss, B, n_kv, S, k_packed, kp_sb, kp_sh, kp_st, k_row_width,
                         k_norms, kn_sb, kn_sh, kn_st, norm_width, t_pos, t_pos_scalar, max_T, k_layout, quant_mode);
    if (rc != BGTQ_OK) return rc;
    rc = fill_v_args(av, plans, v, v_sb, v_sh, v_ss, B, n_kv, S, v_packed, vp_sb, vp_sh, vp_st, v_row_width,
                     v_norms, vn_sb, vn_sh, vn_st, t_pos, t_pos_scalar, max_T, v_layout);
    if (rc != BGTQ_OK) return rc;
    BGTQ_CHECK_ARG((q == nullptr) == (q_rot == nullptr));     // both, or neither (queries rotated elsewhere)
    const bool with_q = q != nullptr;
    const int64_t N = (int64_t)B * S;
    if (N > 64) {          // prefill-sized append: the three stages are big enough on their own
        rc = launch_encode<false>(ak, (hipStream_t)stream);
        if (rc != BGTQ_OK) return rc;
        rc = launch_encode<true>(av, (hipStream_t)stream);
        if (rc != BGTQ_OK || !with_q) return rc;
        return bgtq_rotate_q(plans, q, q_sr, q_sh, q_rot, qr_sr, qr_sh, B, n_kv, gqa, stream);
    }
    const int group = rotate_q_group_size(B, n_kv * gqa);
    RotQArgs aq{plans, (const uint16_t*)q, q_sr, q_sh, (uint16_t*)q_rot, qr_sr, qr_sh, B, n_kv * gqa, gqa, group};
    const int tiles = (int)((N + PREP_ROWS - 1) / PREP_ROWS);
    const unsigned blocks = (unsigned)(2 * tiles * n_kv) + (with_q ? rotate_q_blocks(B, n_kv, gqa, group) : 0u);
    hipLaunchKernelGGL(prepare_kernel, dim3(blocks), dim3(NT), 0, (hipStream_t)stream, ak, av, aq, tiles, tiles);
    return bgtq_launch_status();
}


}  // extern "C"
