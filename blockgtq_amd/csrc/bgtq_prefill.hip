// Prompt-phase (many query tokens) attention over packed K and V records (gfx950).
//
// One work-group of 8 waves owns 256 query rows of one (batch row, KV head): BQ = 256 / gqa
// consecutive query tokens of every query head of the group, 32 rows per wave.  It walks the
// 64-token tiles its rows can see.  Per tile the raw records come from HBM straight into LDS
// (global_load_lds_dwordx4), all waves dequantise them once through the plan's pair tables
// into an fp16 K tile [token][dim] (packed-dim order, fp16(centroid * group norm): what
// bgtq_dequant_kv writes) and a transposed fp16 V tile [dim][token], and then every wave runs
// both products on v_mfma_f32_32x32x16_f16 for its own rows:
//
//   S^T = K Q^T   A = K tile rows (tokens), B = the wave's rotated queries (kept in registers).
//                 In the result a lane holds one query (column) and 16 tokens of each 32-token
//                 block, so the softmax statistics of a query are in-lane up to one exchange
//                 between the two halves of the wave.
//   O^T = V^T P^T A = transposed V tile rows (dims), B = P straight from the score registers:
//                 the token order of a lane's score registers is a fixed permutation of the
//                 contraction index, and the V reads follow the same permutation.
//
// The exponentials are taken relative to a per-query reference that is only moved when a score
// exceeds it (to the maximum + 4 in log2 units), so the accumulators are rescaled rarely.  At the
// end O is normalised and un-rotated against the plan's fp32 V rotation, again on the fp16 matrix
// cores: both factors are split into an fp16 head and an fp16 remainder and three of the four
// products are summed in fp32 (operands once more taken from the accumulator registers under a
// permutation of the contraction index), then stored as fp16.  No fp16 K/V tensor of the layer
// is written.
//
// Work-groups are numbered so that every (batch row, KV head) pair of the query block that sees
// most tokens starts first and the short blocks fill the tail of the launch.
//
// Reference behaviour: blockgtq/kernels/fused_packed_attention.py:1876-2594 (prefill kernel),
// driver blockgtq/prefill.py:66-101.
#include <atomic>

#include "bgtq_lds.h"

namespace {

typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int D = BGTQ_D;
constexpr int MT = 64;                       // tokens per tile
constexpr int NWAVES = 8;                    // (4 waves and 128 rows: 13 % slower, the tile is dequantised twice as often per row)
constexpr int ROWS = 32 * NWAVES;            // query rows per work-group (32 per wave)
constexpr int NTHR = 64 * NWAVES;
constexpr int V_UNITS_PER_THREAD = 16 * 32 / NTHR;   // V tile: 32 token pairs x 16 units over the threads
constexpr int MAX_UNITS = BGTQ_MAX_UNITS;
constexpr int MAX_KN = 8;
constexpr int UPW = (MAX_UNITS + NWAVES - 1) / NWAVES;   // K units per wave
constexpr float REFRESH = 4.0f;
constexpr int KROW = D * 2 + 16;             // bytes of a K tile row: rows 4 banks apart
constexpr int VTROW = MT * 2 + 16;           // bytes of a transposed V tile row (one dim, 64 tokens)

// LDS layout (bytes): [V table | K tables | 2 x (raw K | K norms | V norms | raw V) | 2 x (K tile | V^T tile)]
constexpr int VTAB_OFF = 0;
constexpr int KTAB_OFF = BGTQ_VLUT_BYTES;
constexpr int RAW_OFF = KTAB_OFF + BGTQ_LUT_IMAGE_BYTES;

struct PrefillArgs {
    const bgtq_head_plan* plans;
    const uint16_t* q;  int64_t q_sb, q_sh, q_ss;
    const uint8_t* kp;  int64_t kp_sb, kp_sh, kp_st;
    const uint16_t* kn; int64_t kn_sb, kn_sh, kn_st;
    const uint8_t* vp;  int64_t vp_sb, vp_sh, vp_st;
    const uint16_t* vn; int64_t vn_sb, vn_sh;
    int B, n_kv, gqa, S, T, q_pos_offset, causal;
    int k_layout, v_layout;
    float scale;
    int unrotate;
    uint16_t* out; int64_t o_sb, o_sh, o_ss;
    int k_row_width, v_row_width, v_stride;
    int kt, knr, vnr, vt;      // raw tile areas
};

__host__ __device__ inline int raw_bytes(int krow, int vstride, int kn_st, int& kt, int& knr, int& vnr, int& vt) {
    kt = (MT * krow + 32 + 15) & ~15;
    knr = (MT * kn_st * 2 + 16 + 15) & ~15;
    vnr = MT * 2 + 16;
    vt = (MT * vstride + 32 + 15) & ~15;
    return kt + knr + vnr + vt;
}

__device__ __forceinline__ uint32_t pk_mul_f16(uint32_t a, uint32_t b) {
    uint32_t r;
    asm("v_pk_mul_f16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ uint32_t cvt_pk_f16(float lo, float hi) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2 r = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, r);
}

__global__ __launch_bounds__(NTHR, 8 / NWAVES) void prefill_mfma_kernel(PrefillArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = blockIdx.x, b = blockIdx.y;
    const bgtq_head_plan& P = a.plans[h];
    const int gqa = a.gqa, kl = a.k_layout;
    const bool vnib = a.v_layout == BGTQ_V_NIBBLE;
    const int BQ = ROWS / gqa;                                   // query tokens per work-group
    // work-groups start in the order of their index, x fastest: every (batch row, KV head) pair of the query
    // block that sees most tokens first, so that the short blocks fill the tail of the launch
    const int qb = (int)gridDim.z - 1 - (int)blockIdx.z;
    const int s0 = qb * BQ;
    const int krow = a.k_row_width, vrow = a.v_stride, kn_st = (int)a.kn_st;
    const int vbw = vnib ? 4 : (int)P.v_bits;                    // bits of a V code as stored
    const bool vrep = !vnib && vbw <= 3;                         // V pair table replicated over the banks

    // ---- the tiles this work-group walks
    const int s_last = min(s0 + BQ, a.S) - 1;
    const int t_end = a.causal ? min(a.T, a.q_pos_offset + s_last + 1) : a.T;
    const int n_tiles = (t_end + MT - 1) / MT;

    // ---- this lane's query row: row r = wave * 32 + (lane & 31); head r / BQ, token s0 + r % BQ
    const int li = lane & 31, lg = lane >> 5;
    const int row = wave * 32 + li;
    const int hq = row / BQ, sq = s0 + row - hq * BQ;
    const bool row_ok = hq < gqa && sq < a.S;
    // tokens t < lim are visible to this row
    const int lim = !row_ok ? 0 : a.causal ? min(a.T, a.q_pos_offset + sq + 1) : a.T;

    // ---- LDS areas
    // two sets of raw buffers and two sets of dequantised tiles: set (tile & 1)
    const uint32_t raw_set = (uint32_t)(a.kt + a.knr + a.vnr + a.vt);
    const uint32_t tile_set = MT * KROW + D * VTROW;
    const uint32_t tiles0 = RAW_OFF + 2 * raw_set;

    // ---- tables into LDS
    const uint32_t voff = (uint32_t)lane * 16;
    {
        const uint8_t* vimg = (const uint8_t*)P.vlut_image[vnib ? 1 : 0];
        const uint8_t* kimg = (const uint8_t*)P.lut_image[kl];
        const int vbytes = (vnib || vbw == 4) ? 1024 : (1 << (2 * vbw)) * 128;
        const int kbytes = kl == BGTQ_K_MIXED ? BGTQ_LUTM_KEND : BGTQ_LUT_KEND;
        const int vch = (vbytes + 1023) >> 10, kch = (kbytes + 1023) >> 10;
        for (int cc = wave; cc < vch + kch; cc += NTHR / 64) {
            const uint8_t* src;
            uint32_t dst;
            int left;
            if (cc < vch) { src = vimg + cc * 1024; dst = VTAB_OFF + cc * 1024; left = vbytes - cc * 1024; }
            else { src = kimg + (cc - vch) * 1024; dst = KTAB_OFF + (cc - vch) * 1024; left = kbytes - (cc - vch) * 1024; }
            dma16(voff, src, __builtin_amdgcn_readfirstlane(dst), __builtin_amdgcn_ballot_w64((int)voff < left));
        }
    }
    const int n_units = min(P.n_units[kl], MAX_UNITS), n_pair = min(P.n_pair_units[kl], n_units);
    const uint32_t kend = P.kend[kl], kfirst0 = P.kfirst[kl][0], kfirst1 = P.kfirst[kl][1];
    const int n_zero = min(max(P.n_zero_dims, 0), D);

    // ---- the wave's queries as B operands: lane (query li, half lg) holds dims 16 kk + 8 lg .. + 7 of step kk
    half8 Qb[8];
    {
        const uint16_t* qrow = a.q + b * a.q_sb + ((int64_t)h * gqa + (row_ok ? hq : 0)) * a.q_sh + (int64_t)(row_ok ? sq : 0) * a.q_ss;
#pragma unroll
        for (int kk = 0; kk < 8; kk++) {
            uint4v w = {0, 0, 0, 0};
            if (row_ok) w = *(const uint4v*)(qrow + 16 * kk + 8 * lg);
            Qb[kk] = __builtin_bit_cast(half8, w);
        }
    }

    // ---- streaming sources
    const uint8_t* kp_base = a.kp + b * a.kp_sb + h * a.kp_sh;
    const uint8_t* vp_base = a.vp + b * a.vp_sb + h * a.vp_sh;
    const uint8_t* kn_base = (const uint8_t*)(a.kn + b * a.kn_sb + h * a.kn_sh);
    const uint8_t* vn_base = (const uint8_t*)(a.vn + b * a.vn_sb + h * a.vn_sh);
    const uint32_t kph = (uint32_t)((uintptr_t)kp_base & 15), vph = (uint32_t)((uintptr_t)vp_base & 15);
    const uint32_t knph = (uint32_t)((uintptr_t)kn_base & 15), vnph = (uint32_t)((uintptr_t)vn_base & 15);
    // wave 0 fetches the K records, wave 1 the V records, wave 2 both norm arrays
    auto issue_tile = [&](int tile) {
        const int t = tile * MT, nt = min(MT, t_end - t);
        const uint32_t kraw = RAW_OFF + (uint32_t)(tile & 1) * raw_set, knraw = kraw + a.kt, vnraw = knraw + a.knr, vraw = vnraw + a.vnr;
        if (wave == 0) {
            dma_region<9>(kp_base - kph + (int64_t)t * krow, kraw, dma_shape((int)kph + nt * krow, voff), voff);
        } else if (wave == 1) {
            dma_region<9>(vp_base - vph + (int64_t)t * vrow, vraw, dma_shape((int)vph + nt * vrow, voff), voff);
        } else if (wave == 2) {
            dma_region<2>(kn_base - knph + (int64_t)t * kn_st * 2, knraw, dma_shape((int)knph + nt * kn_st * 2, voff), voff);
            dma_region<1>(vn_base - vnph + (int64_t)t * 2, vnraw, dma_shape((int)vnph + nt * 2, voff), voff);
        }
    };
    if (n_tiles > 0) issue_tile(0);

    // the K tile's columns of 0-bit dims are never written: zero them once
    for (int i = tid; i < 2 * MT * (n_zero / 2); i += NTHR) {
        const int t = i / (n_zero / 2), c = i - t * (n_zero / 2);        // t: row of set t / MT
        lds_put<uint32_t>(tiles0 + (uint32_t)(t / MT) * tile_set + (uint32_t)(t % MT) * KROW + c * 4, 0u);
    }

    const float c2 = a.scale * 1.44269504088896340736f;        // scores in log2 units
    const uint32_t rep = ((uint32_t)lane & 31u) * 4u;
    float16v O[4];                                              // O^T: block db = dims 32 db .., reg r -> dim 32 db + 8 (r / 4) + 4 lg + r % 4
#pragma unroll
    for (int db = 0; db < 4; db++) O[db] = (float16v){0};
    float m_ref = -INFINITY, l_part = 0.f;                       // per query (this half's share of the denominator)

    // K dequantisation: lane = token, wave w takes units w, w + NWAVES, ... (parameters: ku[] below)
    const uint32_t krow_l0 = RAW_OFF + kph + (uint32_t)lane * krow;                    // set 0; + raw_set for set 1
    const uint32_t knrow_l0 = RAW_OFF + a.kt + knph + (uint32_t)lane * kn_st * 2;
    // V dequantisation: thread (token pair tp, unit up); code pair e of a unit's raw word is brought to
    // the table-index position by a rotation (the V table sits at LDS address 0).  Neighbouring lanes take
    // neighbouring units of one token pair: a half-wave then reads 16 token pairs (records 96 bytes apart fall on
    // 8 banks) instead of 32
    const int tp = (tid >> 1) & 31, up = 2 * (tid >> 6) + (tid & 1);
    // Column order of the V^T tile: inside every group of 16 tokens, token x sits at position
    // 8 ((x >> 2) & 1) + 4 (x >> 3) + (x & 3), so that the 8 tokens {4 g + i, 8 + 4 g + i} a half-wave g contracts in
    // one MFMA step are 16 contiguous bytes.  Tokens 2 tp and 2 tp + 1 stay neighbours: byte offset of their dword
    const uint32_t vcol = (uint32_t)(8 * (tp >> 3) + 4 * ((tp >> 1) & 1) + 2 * ((tp >> 2) & 1) + (tp & 1)) * 4;
    const int vtsh = vrep ? 7 : 2;
    uint32_t vrot[4];
#pragma unroll
    for (int e = 0; e < 4; e++) vrot[e] = (uint32_t)(2 * vbw * e - vtsh) & 31u;
    const uint32_t vfmask = ((1u << (2 * vbw)) - 1u) << vtsh, vbase = vrep ? rep : 0u;

    // The K units of this wave (w, w + NWAVES, then the third round shifted by half): their parameters stay in scalar registers for the
    // whole walk.  A unit the wave does not have reads valid addresses and stores nothing (len 0).
    struct KUnit { uint32_t rot[4], mask, tab, repm, off, d0x2, seg2; int len; bool raw; };
    KUnit ku[UPW];
#pragma unroll
    for (int i = 0; i < UPW; i++) {
        // the third round starts at wave NWAVES / 2: the first waves also issue the tile loads
        const int u = i < 2 ? wave + i * NWAVES : i * NWAVES + (wave + NWAVES / 2) % NWAVES;
        const bool have = u < n_units;
        const int uu = have ? u : 0;
        const uint32_t dsc = P.kunit[kl][uu];
        ku[i].len = have ? (int)(dsc >> 8) & 0xFF : 0;
        ku[i].d0x2 = (dsc & 0xFF) * 2;
        ku[i].raw = have && ku[i].len > 0 && u >= n_pair;
        const bool pair = have && ku[i].len > 0 && u < n_pair;
#pragma unroll
        for (int e = 0; e < 4; e++) ku[i].rot[e] = pair ? P.kprog[kl][uu][e] : 0u;
        ku[i].mask = pair ? P.kprog[kl][uu][4] : 0u;
        ku[i].tab = ku[i].len > 0 ? P.kprog[kl][uu][5] : (uint32_t)KTAB_OFF;
        ku[i].repm = pair ? P.kprog[kl][uu][6] : 0u;
        ku[i].off = ku[i].len == 0 ? 0u : uu == 0 ? kfirst0 : uu == 1 ? kfirst1 : P.kprog[kl][uu - 2][7];
        ku[i].seg2 = ku[i].len == 0 ? 0u : 2u * (uint32_t)__builtin_popcount(kend & ((1u << uu) - 1u));
    }

    // Dequantise raw tile `tile` (set tile & 1) into the K and V^T tiles of the same set.
    auto dequant_tile = [&](int tile) {
        const int nt = min(MT, t_end - tile * MT);               // records of this tile; the rows behind them hold stale bytes
        const uint32_t set = (uint32_t)(tile & 1);
        const uint32_t krow_l = krow_l0 + set * raw_set, knrow_l = knrow_l0 + set * raw_set;
        const uint32_t vnraw = RAW_OFF + set * raw_set + a.kt + a.knr, vraw = vnraw + a.vnr;
        const uint32_t ktile = tiles0 + set * tile_set, vtile = ktile + MT * KROW;
        // K tile [token][dim] (packed-dim order) and V^T tile [dim][token], both fp16(centroid * norm).  K: lane =
        // token, the wave's own units; V: thread = tokens 2 tp, 2 tp + 1 of V_UNITS_PER_THREAD units.  Both go
        // through the same three stages together, without a branch between them, so that all LDS round trips
        // of a stage overlap: codes and norms, table lookups, products and stores.
        uint32_t nn[UPW], kw[UPW][4];
        uint2v rr[UPW];
        uint32_t nrm[2], vr[V_UNITS_PER_THREAD][2], vw[V_UNITS_PER_THREAD][2][4];
        // ---- stage 1
#pragma unroll
        for (int i = 0; i < UPW; i++) {
            // rows past the tile's last record get norm 0: their products must stay finite (P is 0 there)
            const uint32_t n16 = lds_at<uint16_t>(knrow_l + ku[i].seg2);
            nn[i] = lane < nt ? n16 | (n16 << 16) : 0u;
            rr[i] = lds_codes8(krow_l + ku[i].off);
        }
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint32_t n16 = lds_at<uint16_t>(vnraw + vnph + (uint32_t)(2 * tp + j) * 2);
            nrm[j] = 2 * tp + j < nt ? n16 | (n16 << 16) : 0u;
        }
#pragma unroll
        for (int uu = 0; uu < V_UNITS_PER_THREAD; uu++)
#pragma unroll
            for (int j = 0; j < 2; j++)
                vr[uu][j] = lds_codes4(vraw + vph + (uint32_t)(2 * tp + j) * vrow + (uint32_t)((V_UNITS_PER_THREAD * up + uu) * vbw));
        // ---- stage 2
#pragma unroll
        for (int i = 0; i < UPW; i++) {
            const uint32_t r = rr[i].x;
            const uint32_t base = and_or(rep, ku[i].repm, ku[i].tab);
#pragma unroll
            for (int e = 0; e < 4; e++)
                kw[i][e] = lds_at<uint32_t>(and_or(__builtin_amdgcn_alignbit(r, r, ku[i].rot[e]), ku[i].mask, base));
        }
#pragma unroll
        for (int uu = 0; uu < V_UNITS_PER_THREAD; uu++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int e = 0; e < 4; e++)
                    vw[uu][j][e] = lds_at<uint32_t>(and_or_v(__builtin_amdgcn_alignbit(vr[uu][j], vr[uu][j], vrot[e]), vfmask, vbase));
#pragma unroll
        for (int i = 0; i < UPW; i++) {
            if (ku[i].raw) {                                     // (wave-uniform) one byte per code, one fp16 per table entry
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const uint32_t x = e < 2 ? rr[i].x : rr[i].y;
                    const uint32_t c0 = ku[i].tab + ((x >> ((e & 1) * 16)) & 0xFF) * 2;
                    const uint32_t c1 = ku[i].tab + ((x >> ((e & 1) * 16 + 8)) & 0xFF) * 2;
                    kw[i][e] = (uint32_t)lds_at<uint16_t>(c0) | ((uint32_t)lds_at<uint16_t>(c1) << 16);
                }
            }
        }
        // ---- stage 3.  A dim pair past the unit's last dim goes to the 16 spare bytes at the end of the lane's
        // K tile row, which nothing reads.
        const uint32_t krow_t = ktile + (uint32_t)lane * KROW;
#pragma unroll
        for (int i = 0; i < UPW; i++)
#pragma unroll
            for (int e = 0; e < 4; e++)
                lds_put<uint32_t>(krow_t + (2 * e < ku[i].len ? ku[i].d0x2 + e * 4 : (uint32_t)(D * 2)), pk_mul_f16(kw[i][e], nn[i]));
#pragma unroll
        for (int uu = 0; uu < V_UNITS_PER_THREAD; uu++) {
            const int u = V_UNITS_PER_THREAD * up + uu;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const uint32_t w0 = pk_mul_f16(vw[uu][0][e], nrm[0]), w1 = pk_mul_f16(vw[uu][1][e], nrm[1]);
                // (dim 8u + 2e of both tokens), (dim 8u + 2e + 1 of both tokens)
                const uint32_t lo = __builtin_amdgcn_perm(w1, w0, 0x05040100u);
                const uint32_t hi = __builtin_amdgcn_perm(w1, w0, 0x07060302u);
                lds_put<uint32_t>(vtile + (uint32_t)(8 * u + 2 * e) * VTROW + vcol, lo);
                lds_put<uint32_t>(vtile + (uint32_t)(8 * u + 2 * e + 1) * VTROW + vcol, hi);
            }
        }
    };

    // Pipeline: while the products of tile i run, tile i + 1 is dequantised into the other set of tiles and the
    // raw records of tile i + 2 stream into the set tile i's came from; one barrier per tile.
    if (n_tiles > 0) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");        // this wave's share of raw tile 0 and of the tables
        __syncthreads();
        dequant_tile(0);
        if (n_tiles > 1) issue_tile(1);
    }
    for (int tile = 0; tile < n_tiles; tile++) {
        const int t0 = tile * MT;
        const uint32_t ktile = tiles0 + (uint32_t)(tile & 1) * tile_set, vtile = ktile + MT * KROW;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");        // this wave's share of raw tile + 1
        __syncthreads();    // raw tile + 1 and tiles `tile` complete; everyone is done with the products of tile - 1
        if (tile + 1 < n_tiles) dequant_tile(tile + 1);
        if (tile + 2 < n_tiles) issue_tile(tile + 2);           // (its raw set was last read before this barrier)

        // ---- S^T = K Q^T for the wave's 32 queries: 2 token blocks x 8 steps of 16 dims
        float16v Sc[2];
#pragma unroll
        for (int tb = 0; tb < 2; tb++) {
            Sc[tb] = (float16v){0};
            const uint32_t arow = ktile + (uint32_t)(32 * tb + li) * KROW + (uint32_t)lg * 16;
#pragma unroll
            for (int kk = 0; kk < 8; kk++) {
                const half8 A = lds_at<half8>(arow + kk * 32);
                Sc[tb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A, Qb[kk], Sc[tb], 0, 0, 0);
            }
        }
        // ---- softmax, lane = query; reg r of block tb is token t0 + 32 tb + 8 (r / 4) + 4 lg + r % 4
        // (raw scores stay in the registers; the scale goes into the exponent's multiply-add)
        float mx = -INFINITY;
        if (__builtin_amdgcn_ballot_w64(t0 + MT > lim)) {        // (wave-uniform) some row of the wave has masked tokens in this tile
#pragma unroll
            for (int tb = 0; tb < 2; tb++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    if (t0 + 32 * tb + 8 * (r >> 2) + 4 * lg + (r & 3) >= lim) Sc[tb][r] = -INFINITY;
                    mx = fmaxf(mx, Sc[tb][r]);
                }
        } else {
#pragma unroll
            for (int tb = 0; tb < 2; tb++)
#pragma unroll
                for (int r = 0; r < 16; r++) mx = fmaxf(mx, Sc[tb][r]);
        }
        mx *= c2;                                                // c2 > 0: the maximum commutes with the scale
        if (__builtin_amdgcn_ballot_w64(mx > m_ref)) {           // wave-uniform, rare after the first tiles
            const float other = __shfl_xor(mx, 32, 64);
            const float top = fmaxf(mx, other);
            const float m_new = top > m_ref ? top + REFRESH : m_ref;
            const float alpha = (m_ref == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_ref - m_new);
            l_part *= alpha;
#pragma unroll
            for (int db = 0; db < 4; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) O[db][r] *= alpha;
            m_ref = m_new;
        }
        // rows that have seen no record yet keep every exponential at 0 (no inf - inf)
        const float mneg = m_ref == -INFINITY ? 0.f : -m_ref;
        uint32_t Pw[2][8];                                        // fp16 pairs: Pw[tb][j] = regs 2j, 2j + 1
#pragma unroll
        for (int tb = 0; tb < 2; tb++)
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const float p0 = __builtin_amdgcn_exp2f(fmaf(Sc[tb][2 * j], c2, mneg));
                const float p1 = __builtin_amdgcn_exp2f(fmaf(Sc[tb][2 * j + 1], c2, mneg));
                l_part += p0 + p1;
                Pw[tb][j] = cvt_pk_f16(p0, p1);
            }
        // ---- O^T += V^T P^T: step (tb, hf) contracts the 16 tokens 32 tb + 16 hf + {4 lg + i, 8 + 4 lg + i}
#pragma unroll
        for (int tb = 0; tb < 2; tb++)
#pragma unroll
            for (int hf = 0; hf < 2; hf++) {
                const uint4v pw = {Pw[tb][4 * hf], Pw[tb][4 * hf + 1], Pw[tb][4 * hf + 2], Pw[tb][4 * hf + 3]};
                const half8 Bp = __builtin_bit_cast(half8, pw);
                const uint32_t col = (uint32_t)(32 * tb + 16 * hf + 8 * lg) * 2;
#pragma unroll
                for (int db = 0; db < 4; db++) {
                    const half8 av = lds_at<half8>(vtile + (uint32_t)(32 * db + li) * VTROW + col);
                    O[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, Bp, O[db], 0, 0, 0);
                }
            }
    }

    // ---- normalise; un-rotate: out^T = R^T O^T on the fp16 matrix cores with both factors split into an
    // fp16 head and an fp16 remainder (x = hi + lo up to 2^-22 |x|; the lo * lo product is dropped), fp32 sums
    const float l_tot = l_part + __shfl_xor(l_part, 32, 64);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) O[db][r] *= inv;
    float16v R[4];
    if (a.unrotate) {
        // R^T goes through LDS (the tiles are dead): row o = output dim, 128 fp16 heads in the order the MFMA
        // wants its contraction slots, position 32 db + 16 s + 8 g + e <-> dim 32 db + 16 s + 8 (e / 4) + 4 g + e % 4
        // (what register 8 s + e of accumulator block db holds in half-wave g); the remainders follow at RT_LO.
        constexpr uint32_t RT_ROW = D * 2 + 16, RT_LO = D * RT_ROW;
        static_assert(2 * RT_LO <= 2 * (MT * KROW + D * VTROW), "both halves of R^T fit into the tile sets");
        __syncthreads();                                        // every wave is done with the tiles
        const float* rot = P.v_rot;
        for (int idx = tid; idx < D * 4; idx += NTHR) {
            const int o = idx & (D - 1), dq = idx >> 7;         // this thread: column o of rows 32 dq .. 32 dq + 31
            float x[32];
#pragma unroll
            for (int i = 0; i < 32; i++) x[i] = rot[(32 * dq + i) * D + o];
#pragma unroll
            for (int g8 = 0; g8 < 4; g8++) {                    // positions 8 g8 .. 8 g8 + 7 of the block: s = g8 / 2, g = g8 % 2
                uint32_t hi[4], lo[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int e0 = 2 * j, e1 = 2 * j + 1;
                    const float x0 = x[16 * (g8 >> 1) + 8 * (e0 >> 2) + 4 * (g8 & 1) + (e0 & 3)];
                    const float x1 = x[16 * (g8 >> 1) + 8 * (e1 >> 2) + 4 * (g8 & 1) + (e1 & 3)];
                    const _Float16 h0 = (_Float16)x0, h1 = (_Float16)x1;
                    hi[j] = cvt_pk_f16((float)h0, (float)h1);
                    lo[j] = cvt_pk_f16(x0 - (float)h0, x1 - (float)h1);
                }
                const uint32_t dst = (uint32_t)o * RT_ROW + (uint32_t)(32 * dq + 8 * g8) * 2;
                lds_put<uint4v>(dst, (uint4v){hi[0], hi[1], hi[2], hi[3]});
                lds_put<uint4v>(RT_LO + dst, (uint4v){lo[0], lo[1], lo[2], lo[3]});
            }
        }
        // the wave's O^T as B operands: step (db, s) takes registers 8 s .. 8 s + 7 of block db
        half8 Bh[8], Bl[8];
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int sst = 0; sst < 2; sst++) {
                uint32_t hi[4], lo[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float x0 = O[db][8 * sst + 2 * j], x1 = O[db][8 * sst + 2 * j + 1];
                    const _Float16 h0 = (_Float16)x0, h1 = (_Float16)x1;
                    hi[j] = cvt_pk_f16((float)h0, (float)h1);
                    lo[j] = cvt_pk_f16(x0 - (float)h0, x1 - (float)h1);
                }
                Bh[2 * db + sst] = __builtin_bit_cast(half8, (uint4v){hi[0], hi[1], hi[2], hi[3]});
                Bl[2 * db + sst] = __builtin_bit_cast(half8, (uint4v){lo[0], lo[1], lo[2], lo[3]});
            }
        __syncthreads();
#pragma unroll
        for (int ob = 0; ob < 4; ob++) R[ob] = (float16v){0};
#pragma unroll
        for (int st = 0; st < 8; st++) {                        // four independent accumulators per pass
            half8 Ah[4], Al[4];
#pragma unroll
            for (int ob = 0; ob < 4; ob++) {
                const uint32_t arow = (uint32_t)(32 * ob + li) * RT_ROW + (uint32_t)lg * 16 + st * 32;
                Ah[ob] = lds_at<half8>(arow);
                Al[ob] = lds_at<half8>(RT_LO + arow);
            }
#pragma unroll
            for (int ob = 0; ob < 4; ob++) R[ob] = __builtin_amdgcn_mfma_f32_32x32x16_f16(Ah[ob], Bh[st], R[ob], 0, 0, 0);
#pragma unroll
            for (int ob = 0; ob < 4; ob++) R[ob] = __builtin_amdgcn_mfma_f32_32x32x16_f16(Al[ob], Bh[st], R[ob], 0, 0, 0);
#pragma unroll
            for (int ob = 0; ob < 4; ob++) R[ob] = __builtin_amdgcn_mfma_f32_32x32x16_f16(Ah[ob], Bl[st], R[ob], 0, 0, 0);
        }
    } else {
#pragma unroll
        for (int ob = 0; ob < 4; ob++) R[ob] = O[ob];
    }
    if (row_ok) {
        uint16_t* orow = a.out + b * a.o_sb + ((int64_t)h * gqa + hq) * a.o_sh + (int64_t)sq * a.o_ss;
#pragma unroll
        for (int ob = 0; ob < 4; ob++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                uint2v w = {cvt_pk_f16(R[ob][4 * j], R[ob][4 * j + 1]), cvt_pk_f16(R[ob][4 * j + 2], R[ob][4 * j + 3])};
                *(uint2v*)(orow + 32 * ob + 8 * j + 4 * lg) = w;
            }
    }
}

}  // namespace

extern "C" int bgtq_prefill_attn(const bgtq_head_plan* plans,
                                 const void* q_rot, int64_t q_sb, int64_t q_sh, int64_t q_ss,
                                 const void* k_packed, int64_t kp_sb, int64_t kp_sh, int64_t kp_st, int k_row_width,
                                 const void* k_norms, int64_t kn_sb, int64_t kn_sh, int64_t kn_st,
                                 const void* v_packed, int64_t vp_sb, int64_t vp_sh, int64_t vp_st, int v_row_width,
                                 const void* v_norms, int64_t vn_sb, int64_t vn_sh, int64_t vn_st,
                                 int B, int n_kv, int gqa, int S, int T, int q_pos_offset, int is_causal,
                                 int k_layout, int v_layout, float scale, int unrotate,
                                 void* out, int64_t o_sb, int64_t o_sh, int64_t o_ss, void* stream) {
    BGTQ_CHECK_ARG(plans && q_rot && k_packed && k_norms && v_packed && v_norms && out);
    BGTQ_CHECK_ARG(B >= 0 && n_kv > 0 && gqa > 0 && S >= 0 && T >= 0 && q_pos_offset >= 0);
    if (B == 0 || S == 0) return BGTQ_OK;            // no query rows: nothing to write
    BGTQ_CHECK_ARG(k_layout == BGTQ_K_BITPACKED || k_layout == BGTQ_K_MIXED);
    BGTQ_CHECK_ARG(v_layout == BGTQ_V_BITPACKED || v_layout == BGTQ_V_NIBBLE);
    // layout requirements of this kernel; callers copy their records into rows that meet them
    if (gqa > ROWS || !(scale > 0.f)) return BGTQ_EUNSUPPORTED;
    if ((kp_st & 3) || (kp_sb & 3) || (kp_sh & 3) || ((uintptr_t)k_packed & 3)) return BGTQ_EUNSUPPORTED;
    if ((vp_st & 3) || (vp_sb & 3) || (vp_sh & 3) || ((uintptr_t)v_packed & 3)) return BGTQ_EUNSUPPORTED;
    if (kp_st != k_row_width || k_row_width < 4 || k_row_width > 128) return BGTQ_EUNSUPPORTED;
    if (vn_st != 1 || kn_st < 1 || kn_st > MAX_KN) return BGTQ_EUNSUPPORTED;
    if (v_row_width != 16 && v_row_width != 32 && v_row_width != 48 && v_row_width != 64) return BGTQ_EUNSUPPORTED;
    if (vp_st < v_row_width || vp_st > v_row_width + 4) return BGTQ_EUNSUPPORTED;
    if (v_layout == BGTQ_V_NIBBLE && v_row_width != 64) return BGTQ_EUNSUPPORTED;
    if ((q_ss & 7) || (q_sh & 7) || (q_sb & 7) || ((uintptr_t)q_rot & 15)) return BGTQ_EUNSUPPORTED;   // 16-byte query loads
    if ((o_ss & 3) || (o_sh & 3) || (o_sb & 3) || ((uintptr_t)out & 7)) return BGTQ_EUNSUPPORTED;      // 8-byte output stores
    if (T == 0) return BGTQ_EUNSUPPORTED;
    PrefillArgs a;
    a.plans = plans;
    a.q = (const uint16_t*)q_rot; a.q_sb = q_sb; a.q_sh = q_sh; a.q_ss = q_ss;
    a.kp = (const uint8_t*)k_packed; a.kp_sb = kp_sb; a.kp_sh = kp_sh; a.kp_st = kp_st;
    a.kn = (const uint16_t*)k_norms; a.kn_sb = kn_sb; a.kn_sh = kn_sh; a.kn_st = kn_st;
    a.vp = (const uint8_t*)v_packed; a.vp_sb = vp_sb; a.vp_sh = vp_sh; a.vp_st = vp_st;
    a.vn = (const uint16_t*)v_norms; a.vn_sb = vn_sb; a.vn_sh = vn_sh;
    a.B = B; a.n_kv = n_kv; a.gqa = gqa; a.S = S; a.T = T; a.q_pos_offset = q_pos_offset; a.causal = is_causal != 0;
    a.k_layout = k_layout; a.v_layout = v_layout; a.scale = scale; a.unrotate = unrotate != 0;
    a.out = (uint16_t*)out; a.o_sb = o_sb; a.o_sh = o_sh; a.o_ss = o_ss;
    a.k_row_width = k_row_width; a.v_row_width = v_row_width; a.v_stride = (int)vp_st;
    const int raw = raw_bytes(k_row_width, (int)vp_st, (int)kn_st, a.kt, a.knr, a.vnr, a.vt);
    const size_t smem = (size_t)RAW_OFF + 2 * ((size_t)raw + (size_t)MT * KROW + (size_t)D * VTROW);
    static std::atomic<int> ready{0};
    if (ready.load(std::memory_order_acquire) == 0) {
        // offsets into the dynamic LDS block are used as LDS addresses: holds only without static LDS
        hipFuncAttributes fa;
        hipError_t e = hipFuncGetAttributes(&fa, (const void*)prefill_mfma_kernel);
        if (e != hipSuccess) return (int)e;
        e = hipFuncSetAttribute((const void*)prefill_mfma_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return (int)e;
        ready.store(fa.sharedSizeBytes == 0 ? 1 : -1, std::memory_order_release);
    }
    if (ready.load(std::memory_order_acquire) < 0 || smem > 160 * 1024) return BGTQ_EUNSUPPORTED;
    const int BQ = ROWS / gqa;
    if ((S + BQ - 1) / BQ > 65535 || B > 65535) return BGTQ_EUNSUPPORTED;
    dim3 grid((unsigned)n_kv, (unsigned)B, (unsigned)((S + BQ - 1) / BQ));
    hipLaunchKernelGGL(prefill_mfma_kernel, grid, dim3(NTHR), smem, (hipStream_t)stream, a);
    return bgtq_launch_status();
}
