// MFMA decode attention over packed K and V records (gfx950), query groups of at most 8 heads.
//
// One work-group of up to 12 waves (3 per SIMD, as many as the tile buffers leave
// room for in LDS) owns one partition of one (batch row, KV head).  The 64-token
// tiles of a (batch row, KV head) are dealt to the partitions as evenly as whole
// tiles allow and round-robin to the waves inside a partition; every wave walks
// its tiles with a private online softmax and the waves are merged through LDS at
// the end.
//
// Data movement.  A tile of packed records is one contiguous byte range of the
// cache.  It goes from HBM straight into LDS with global_load_lds_dwordx4
// (aligned 16-byte pieces, the 16-byte phase of the source is kept), into the
// wave's own K buffer as soon as QK^T of the previous tile has read it, V
// likewise after PV.  The fp16 norms of the tile travel the same way.  Nothing
// on the streaming path passes through vector registers.
//
// Dequantisation is table driven.  A "unit" is 8 consecutive codes of one token.
// For every bit width <= 4 the plan carries a pair table that the work-group copies
// into LDS: entry (c0 | c1 << bw) holds the two fp16 centroids of a code pair.
// Tables of at most 64 entries are replicated 32 times (entry stride 128 bytes), so
// that the 32 lanes of a half-wave, which LDS serves together, always read 32
// different banks; the 256-entry tables are not replicated (8 or 16 copies collide
// more often than none).  A unit costs one raw read, four {rotate, and-or, table read}
// triples and yields the eight fp16 operands of one MFMA k-group.
//
// QK^T:  lane = token.  Every lane decodes the same unit of its own token, so the field
//        positions, masks and tables of a unit are the same in every lane: the plan's
//        per-unit parameter rows are copied to LDS once and read (all lanes one address)
//        as the units go by, together with the unit's query operands, through one
//        running pointer.  v_mfma_f32_16x16x32_f16 with B = dequantised K (column j of
//        lane group g is token 16g + j) and A = the unit's rotated queries, zero outside
//        lane group g for rows 4g..4g+3: D[4g + r][j] is then q_head(r) . k_token(16g + j),
//        i.e. every lane receives the scores of its own token, 4 heads per MFMA.  The
//        units of a segment accumulate in the MFMA and the segment's sum is scaled by
//        the token's fp16 norm of that segment in fp32: one multiply-add per head and lane.
// Softmax: lane = token, exponentials relative to a per-head reference (wave-uniform) that
//        is kept above every score seen so far.  It is only moved (to the new maximum
//        plus a headroom of 4 in log2 units) when a score of the tile exceeds it;
//        otherwise the tile needs no cross-lane traffic at all.
// PV:    P * v_norm goes through LDS once (2 bytes per head and token) into the A layout of
//        the value product.  That product runs over (token, dim parity) pairs: A row
//        (head h, parity e) holds P[h][t] in slot (t, e), B column c holds the V table word
//        of token t, so a table word is an MFMA operand as it comes.
// Merge: every wave leaves its reference, denominator and sums in its own (then dead) tile
//        buffers; after one barrier the first 32 * gqa threads fold the waves.
#include <atomic>

#include "bgtq_decode.h"
#include "bgtq_lds.h"

namespace {


constexpr int D = BGTQ_D;
constexpr int MT = 64;             // tokens per wave tile = 4 MFMA row blocks
constexpr int MAX_UNITS = BGTQ_MAX_UNITS;
constexpr int MAX_WAVES = 12;
constexpr int MAX_KN = 8;          // norm columns per token row
constexpr int LDS_LIMIT = 160 * 1024;
constexpr float REFRESH = 4.0f;
//    // log2 headroom put above the largest score when the reference is refreshed

// ---- LDS layout (bytes) -----------------------------------------------------------
// [ V pair table | K tables of the record layout in use | query units | per wave: K tile + K norms + V norms,
//   V tile, P ]
// (query units are followed by the segment parameters)
constexpr int VTAB_BYTES = BGTQ_VLUT_BYTES;
constexpr int KTAB_BYTES = BGTQ_LUT_IMAGE_BYTES;
constexpr int UROW = (MAX_UNITS + 2) * 16;                      // one 16-byte slot per unit (+ 2: the look-ahead of the last units)
// What a lane reads per unit sits behind one pointer: its A rows for both MFMAs and the unit's
// parameters.  One struct per A row 0..3 (heads r and r + 4) and one whose A rows are zero (for the
// lanes outside the unit's lane group); the parameters are repeated in each.  The stride puts the
// five structs on different banks.
constexpr int QS_A2 = UROW, QS_PA = 2 * UROW, QS_PB = 3 * UROW;
constexpr int QSTRUCT = 4 * UROW + 16;
constexpr int QS_OFF = VTAB_BYTES + KTAB_BYTES;
constexpr int N_QJOBS = 8 * MAX_UNITS + 5 * 2 * MAX_UNITS + 2 * MAX_UNITS;   // query units, parameter halves, zero rows
constexpr int WAVES_OFF = QS_OFF + 5 * QSTRUCT;
constexpr int PROW = MT * 4 + 32;                                // bytes from one head's P row to the next: rows land 8 banks apart
constexpr int PBUF_BYTES = 8 * PROW;                          // P of a tile: [head][token], fp16 in the low half of a dword

__host__ __device__ constexpr int kimg_bytes(int k_layout) { return k_layout == BGTQ_K_MIXED ? BGTQ_LUTM_KEND : BGTQ_LUT_KEND; }
__host__ __device__ constexpr int vlut_bytes(int vbw, bool nibble) {
    return (nibble || vbw == 4) ? 1024 : (1 << (2 * vbw)) * 128;
}

constexpr int MERGE_BYTES = 64 + 8 * 32 * 16;                    // what a wave leaves for the merge: m, l, 8 heads x 128 floats

__host__ __device__ inline TileLayout tile_layout(int krow, int vrow, int kn_st) {
    TileLayout t;
    t.kt = (MT * krow + 32 + 15) & ~15;
    t.vt = (MT * vrow + 32 + 15) & ~15;
    t.knr = (MT * kn_st * 2 + 16 + 15) & ~15;
    t.vnr = MT * 2 + 16;
    t.kbuf = t.kt + t.knr + t.vnr;
    return t;
}

// LDS bytes of one wave: its tile buffers, which also take its contribution to the merge
__host__ __device__ inline int wave_lds_bytes(const TileLayout& t) {
    const int tiles = t.kbuf + t.vt + PBUF_BYTES;
    return tiles > MERGE_BYTES ? tiles : MERGE_BYTES;
}

static_assert(offsetof(bgtq_head_plan, kprog) % 16 == 0 && offsetof(bgtq_head_plan, lut_image) % 16 == 0 &&
              offsetof(bgtq_head_plan, vlut_image) % 16 == 0 && BGTQ_LUT_IMAGE_BYTES % 16 == 0 && BGTQ_VLUT_BYTES % 16 == 0,
              "plan tables are copied 16 bytes at a time");


// Wave-wide sums / maxima of 8 values at once through the DPP lane crossbar (no LDS traffic): quads,
// half rows, rows of 16, then the row results travel to the rows behind them; lane 63 ends up with
// the totals.  The 8 values go through every stage together, so that no instruction reads what the
// one before it wrote (a DPP source needs two idle issue slots after its producer).
#define BGTQ_DPP8(op, ctrl)                                                                       \
    op " %0, %0, %0 " ctrl "\n\t" op " %1, %1, %1 " ctrl "\n\t" op " %2, %2, %2 " ctrl "\n\t"     \
    op " %3, %3, %3 " ctrl "\n\t" op " %4, %4, %4 " ctrl "\n\t" op " %5, %5, %5 " ctrl "\n\t"     \
    op " %6, %6, %6 " ctrl "\n\t" op " %7, %7, %7 " ctrl "\n\t"
#define BGTQ_DPP_REDUCE8(op)                                                                      \
    "s_nop 1\n\t"                                                                                 \
    BGTQ_DPP8(op, "quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf")                               \
    BGTQ_DPP8(op, "quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf")                               \
    BGTQ_DPP8(op, "row_half_mirror row_mask:0xf bank_mask:0xf")                                   \
    BGTQ_DPP8(op, "row_mirror row_mask:0xf bank_mask:0xf")                                        \
    BGTQ_DPP8(op, "row_bcast:15 row_mask:0xa bank_mask:0xf")                                      \
    BGTQ_DPP8(op, "row_bcast:31 row_mask:0xc bank_mask:0xf")                                      \
    "s_nop 1\n\t"
__device__ __forceinline__ void wave_sum8(float (&x)[8]) {            // totals in lane 63
    asm volatile(BGTQ_DPP_REDUCE8("v_add_f32_dpp")
                 : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7]));
}
__device__ __forceinline__ void wave_max8(float (&x)[8]) {            // maxima in lane 63
    asm volatile(BGTQ_DPP_REDUCE8("v_max_f32_dpp")
                 : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7]));
}

// VBW: bits per V code; VST: bytes from one V record to the next (the record itself is
// 16 * VBW bytes; a padded stride keeps the rows of a tile on different LDS banks)
// TWO: more than 4 query heads per KV head (a second MFMA per unit for heads 4..7)
template <int VBW, int VST, bool TWO>
__global__ __launch_bounds__(MAX_WAVES * 64) void decode_mfma_kernel(DecodeArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nw = a.nw, nthr = nw * 64;
    const int c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const bgtq_head_plan& P = a.plans[h];
    const int gqa = a.gqa;
    const int li = lane & 15, lg = lane >> 4;           // MFMA row/col index, lane group
    const int kl = a.k_layout;
    const bool vnib = a.v_layout == BGTQ_V_NIBBLE;

    // ---- this partition's tiles: the tiles of the row are dealt to the partitions as evenly as
    // whole tiles allow (partition sizes differ by at most one tile)
    int T = a.T, per = a.per_tiles, rem = a.rem_tiles;        // (the launcher divides when every row has T records)
    if (a.seq_lens) {
        T = a.seq_lens[b];
        const int n_tiles = (T + MT - 1) / MT;
        per = n_tiles / a.n_splits;
        rem = n_tiles - per * a.n_splits;
    }
    const int tile_lo = c * per + min(c, rem), tile_hi = tile_lo + per + (c < rem ? 1 : 0);
    const int t0 = tile_lo * MT, t1 = min(tile_hi * MT, T);

    const int krow = a.k_row_width;
    constexpr int vrow = VST;
    const int kn_st = (int)a.kn_st;
    const TileLayout tl = a.tl;
    // byte offset of (row b, KV head h) of a tensor whose strides (in elements of `elem` bytes) the launcher
    // has checked to fit 32 bits
    auto at_bh = [&](int64_t sb, int64_t sh, int elem) -> uint64_t {
        return ((uint64_t)(uint32_t)b * (uint32_t)sb + (uint64_t)(uint32_t)h * (uint32_t)sh) * (uint32_t)elem;
    };
    const uint16_t* q_src = (const uint16_t*)((const uint8_t*)a.q + ((uint64_t)(uint32_t)b * (uint32_t)a.q_sb + (uint64_t)(uint32_t)(h * gqa) * (uint32_t)a.q_sh) * 2u);
    const int n_units = min(P.n_units[kl], MAX_UNITS);
    const int n_pair = min(P.n_pair_units[kl], n_units);
    const uint32_t kend = P.kend[kl], kfirst0 = P.kfirst[kl][0], kfirst1 = P.kfirst[kl][1];
    // Job j < N_QJOBS fills one 16-byte slot of the structs: a query unit (head j / MAX_UNITS), one half
    // of a unit's parameters for one struct, or a slot of the all-zero A rows.  The loads of a thread's
    // first job go out here, the slots are written once the streaming loads have been issued.
    auto job_load = [&](int j) -> uint4v {
        uint4v w = {0, 0, 0, 0};
        if (j < 8 * MAX_UNITS) {
            const int jh = j / MAX_UNITS, ju = j - jh * MAX_UNITS;
            const uint32_t dsc = P.kunit[kl][ju];
            const int d0 = (int)(dsc & 0xFF), len = (int)(dsc >> 8);
            if (jh < gqa && len > 0) {
                const uint32_t* row = (const uint32_t*)(q_src + jh * a.q_sh + d0);        // d0 is even
#pragma unroll
                for (int pp = 0; pp < 4; pp++)
                    w[pp] = row[min(pp, (D - d0) / 2 - 1)] &
                            ((2 * pp < len ? 0xFFFFu : 0u) | (2 * pp + 1 < len ? 0xFFFF0000u : 0u));
            }
        } else if (j < 8 * MAX_UNITS + 10 * MAX_UNITS) {
            const int r = (j - 8 * MAX_UNITS) % (2 * MAX_UNITS);
            w = *(const uint4v*)&P.kprog[kl][r >> 1][(r & 1) * 4];
        }
        return w;
    };
    auto job_slot = [&](int j) -> uint32_t {
        if (j < 8 * MAX_UNITS) {
            const int jh = j / MAX_UNITS, ju = j - jh * MAX_UNITS;
            return QS_OFF + (jh & 3) * QSTRUCT + (jh >> 2) * QS_A2 + ju * 16;
        }
        if (j < 8 * MAX_UNITS + 10 * MAX_UNITS) {
            const int s5 = (j - 8 * MAX_UNITS) / (2 * MAX_UNITS), r = (j - 8 * MAX_UNITS) % (2 * MAX_UNITS);
            return QS_OFF + s5 * QSTRUCT + ((r & 1) ? QS_PB : QS_PA) + (r >> 1) * 16;
        }
        return QS_OFF + 4 * QSTRUCT + (j - 18 * MAX_UNITS) * 16;
    };
    uint4v job0 = {0, 0, 0, 0};
    if (tid < N_QJOBS) job0 = job_load(tid);

    // ---- tables by DMA: V table at LDS offset 0, K tables behind it; the chunks are dealt round-robin
    // to the waves
    const uint32_t voff = (uint32_t)lane * 16;
    {
        const uint8_t* vimg = (const uint8_t*)P.vlut_image[vnib ? 1 : 0];
        const uint8_t* kimg_src = (const uint8_t*)P.lut_image[kl];
        const int vbytes = vlut_bytes(VBW, vnib), kbytes = kimg_bytes(kl);
        const int vch = (vbytes + 1023) >> 10, kch = (kbytes + 1023) >> 10;
        for (int cc = wave; cc < vch + kch; cc += nw) {
            const uint8_t* src;
            uint32_t dst;
            int left;
            if (cc < vch) { src = vimg + cc * 1024; dst = cc * 1024; left = vbytes - cc * 1024; }
            else { src = kimg_src + (cc - vch) * 1024; dst = VTAB_BYTES + (cc - vch) * 1024; left = kbytes - (cc - vch) * 1024; }
            dma16(voff, src, __builtin_amdgcn_readfirstlane(dst), __builtin_amdgcn_ballot_w64((int)voff < left));
        }
    }

    // ---- per-wave buffers and streaming sources: 16-byte aligned bases and phases (constant per tile) ----
    const int wave_bytes = a.wave_bytes;
    const uint32_t kbuf = WAVES_OFF + wave * wave_bytes;                       // K records, K norms, V norms
    const uint32_t vbuf = kbuf + tl.kbuf;                                     // V records
    const uint32_t pbuf = vbuf + tl.vt;                                       // P * v_norm of the tile
    const uint8_t* kp_base = a.kp + at_bh(a.kp_sb, a.kp_sh, 1);
    const uint8_t* vp_base = a.vp + at_bh(a.vp_sb, a.vp_sh, 1);
    const uint8_t* kn_base = (const uint8_t*)a.kn + at_bh(a.kn_sb, a.kn_sh, 2);
    const uint8_t* vn_base = (const uint8_t*)a.vn + at_bh(a.vn_sb, a.vn_sh, 2);
    const uint32_t kph = (uint32_t)((uintptr_t)kp_base & 15), vph = (uint32_t)((uintptr_t)vp_base & 15);
    const uint32_t knph = (uint32_t)((uintptr_t)kn_base & 15), vnph = (uint32_t)((uintptr_t)vn_base & 15);
    // The shapes of a full tile are the same for every tile of the partition.
    const DmaShape full_k = dma_shape((int)kph + MT * krow, voff), full_kn = dma_shape((int)knph + MT * kn_st * 2, voff);
    const DmaShape full_vn = dma_shape((int)vnph + MT * 2, voff), full_v = dma_shape((int)vph + MT * vrow, voff);
    // Sources of the wave's next tile (16-byte aligned: the phase stays in the LDS offset); they move on by
    // the wave's tile stride after every issue.
    const int step_tiles = nw * MT;
    const uint32_t first = (uint32_t)(t0 + wave * MT);          // (a (row, head) slice is below 4 GB: checked by the launcher)
    const uint8_t* k_src = kp_base - kph + first * (uint32_t)krow;
    const uint8_t* kn_src = kn_base - knph + first * (uint32_t)(kn_st * 2);
    const uint8_t* vn_src = vn_base - vnph + first * 2u;
    const uint8_t* v_src = vp_base - vph + first * (uint32_t)vrow;
    const int k_step = step_tiles * krow, kn_step = step_tiles * kn_st * 2, vn_step = step_tiles * 2, v_step = step_tiles * vrow;
    // K records and both norm arrays of a tile go to the K buffer; returns the loads issued.
    auto issue_k = [&](int tile) -> int {
        const int nt = min(MT, t1 - tile);
        DmaShape sk = full_k, sn = full_kn, sv = full_vn;
        if (nt < MT) {
            sk = dma_shape((int)kph + nt * krow, voff);
            sn = dma_shape((int)knph + nt * kn_st * 2, voff);
            sv = dma_shape((int)vnph + nt * 2, voff);
        }
        dma_region<9>(k_src, kbuf, sk, voff);
        dma_region<2>(kn_src, kbuf + tl.kt, sn, voff);
        dma_region<1>(vn_src, kbuf + tl.kt + tl.knr, sv, voff);
        k_src += k_step;
        kn_src += kn_step;
        vn_src += vn_step;
        return sk.nfull + sn.nfull + sv.nfull + 3;
    };
    auto issue_v = [&](int tile) -> int {
        const int nt = min(MT, t1 - tile);
        DmaShape sv = full_v;
        if (nt < MT) sv = dma_shape((int)vph + nt * vrow, voff);
        dma_region<5>(v_src, vbuf, sv, voff);
        v_src += v_step;
        return sv.nfull + 1;
    };
    int tile = t0 + wave * MT;
    int v_loads = 0;                 // loads of the V tile issued after the current K tile
    if (tile < t1) issue_k(tile);

    // ---- the structs' slots; the P buffers' high halves (the wait for the query rows also covers the
    // tables and the first K tile: all are needed now)
    {
        if (tid < N_QJOBS) lds_put<uint4v>(job_slot(tid), job0);
        if (nthr < N_QJOBS)                                   // (uniform) small work-groups only
            for (int j = tid + nthr; j < N_QJOBS; j += nthr) lds_put<uint4v>(job_slot(j), job_load(j));
#pragma unroll
        for (int i = 0; i < PBUF_BYTES; i += 1024)
            if (i + 1024 <= PBUF_BYTES || lane * 16 < PBUF_BYTES - i) lds_put<uint4v>(pbuf + i + lane * 16, (uint4v){0, 0, 0, 0});
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // this wave's table chunks and its first K tile
    if (tile < t1) v_loads = issue_v(tile);
    __syncthreads();

    const float c2 = a.scale * 1.44269504088896340736f;      // scores are kept in log2 units
    constexpr bool two = TWO;
    const uint32_t rep = ((uint32_t)lane & 31u) * 4u;          // this lane's replica of the 32-fold tables
    // QK^T operands: this lane's record and norm row; its A rows (4 lg' + h' with lg' = li >> 2: the queries of
    // head h' (+ 4 for the second MFMA) where lg' is this lane's own group, the all-zero head elsewhere)
    const uint32_t krow_l = kbuf + kph + (uint32_t)lane * krow;
    const uint32_t knrow_l = kbuf + tl.kt + knph + (uint32_t)lane * kn_st * 2;
    const uint32_t vn_l = kbuf + tl.kt + tl.knr + vnph + (uint32_t)lane * 2;
    const bool q_live = (li >> 2) == lg;
    const uint32_t qs_l = QS_OFF + (q_live ? (li & 3) : 4) * QSTRUCT;
    // PV operands: V table replica (the table sits at LDS address 0, so field bits OR-ed in never meet the
    // base; the 256-entry tables are not replicated), raw codes, P rows
    constexpr bool V_UNREP = VBW == 4;                        // also every nibble record (VBW 4 by construction)
    const uint32_t vbank = V_UNREP ? 0u : rep;
    constexpr int vshift = V_UNREP ? 2 : 7;
    const uint32_t vc = vph + (uint32_t)li * VBW;
    const uint32_t vbase = vbuf + (vc & ~3u) + (uint32_t)lg * 4 * vrow, v_sh = vc & 3u;
    const uint32_t p_wr = pbuf + (uint32_t)lane * 4;                             // + head * 256
    const uint32_t p_rd = pbuf + (uint32_t)(li & 7) * PROW + (uint32_t)lg * 16;    // + block * 64
    const uint32_t p_shift = (li & 8) ? 16u : 0u;              // rows 8..15 carry the odd dims: P in the high half

    float m_ref[8], l_part[8];      // per head: reference in log2 units (never below a score seen), this lane's share of the denominator
#pragma unroll
    for (int hh = 0; hh < 8; hh++) { m_ref[hh] = -INFINITY; l_part[hh] = 0.f; }
    float4v acc[4];                 // acc[jb][r] = out[head 4(lg & 1) + r][dim 8 li + 2 jb + (lg >> 1)]
#pragma unroll
    for (int e = 0; e < 4; e++) acc[e] = (float4v){0, 0, 0, 0};

    for (; tile < t1; tile += step_tiles) {
        const int nt = min(MT, t1 - tile);
        const bool more = tile + step_tiles < t1;
        wait_loads(v_loads);                                 // K records and norms of this tile are in LDS
        __builtin_amdgcn_wave_barrier();
        const uint32_t vraw = lds_at<uint16_t>(vn_l);

        // ---- scores of this lane's token, 8 heads, in log2 units ----------------------------------------
        float S[8];
#pragma unroll
        for (int hh = 0; hh < 8; hh++) S[hh] = 0.f;
        {
            // One pointer walks this lane's struct: A rows and parameters of the unit.  The codes of a
            // unit and its parameters are requested while the previous unit's table words are on their
            // way (every parameter row names the byte offset of the unit after it).
            uint32_t qp = qs_l;
            uint32_t np = knrow_l;
            uint32_t n16 = lds_at<uint16_t>(np);                           // norm of the current segment
            float4v D1 = {0, 0, 0, 0}, D2 = {0, 0, 0, 0};                  // sums over the segment's units: heads 0..3, 4..7
            auto segment_done = [&]() {
                const float n = bgtq_h2f((uint16_t)n16) * c2;
                np += 2;
                n16 = lds_at<uint16_t>(np);                                // (past the last segment: unused)
#pragma unroll
                for (int e = 0; e < 4; e++) S[e] = fmaf(n, D1[e], S[e]);
                D1 = (float4v){0, 0, 0, 0};
                if (two) {
#pragma unroll
                    for (int e = 0; e < 4; e++) S[4 + e] = fmaf(n, D2[e], S[4 + e]);
                    D2 = (float4v){0, 0, 0, 0};
                }
            };
            // Pair-table units, two at a time (their count is even): the table words and query rows of
            // both are requested before the first is used, and so are the codes and parameters of the
            // two units after them (every parameter row names the byte offset of the unit two on).
            uint4v paA = lds_at<uint4v>(qp + QS_PA), pbA = lds_at<uint4v>(qp + QS_PB);
            uint4v paB = lds_at<uint4v>(qp + 16 + QS_PA), pbB = lds_at<uint4v>(qp + 16 + QS_PB);
            uint32_t xa = krow_l + kfirst0, xb = krow_l + kfirst1;         // byte addresses of the units whose codes are read next
            uint32_t rA = lds_codes4(xa), rB = lds_codes4(xb);
            int u = 0;
            for (; u < n_pair; u += 2) {
                const uint32_t baseA = and_or_v(rep, pbA.z, pbA.y), baseB = and_or_v(rep, pbB.z, pbB.y);
                uint32_t a0 = __builtin_amdgcn_alignbit(rA, rA, paA.x), a1 = __builtin_amdgcn_alignbit(rA, rA, paA.y);
                uint32_t a2 = __builtin_amdgcn_alignbit(rA, rA, paA.z), a3 = __builtin_amdgcn_alignbit(rA, rA, paA.w);
                uint32_t b0 = __builtin_amdgcn_alignbit(rB, rB, paB.x), b1 = __builtin_amdgcn_alignbit(rB, rB, paB.y);
                uint32_t b2 = __builtin_amdgcn_alignbit(rB, rB, paB.z), b3 = __builtin_amdgcn_alignbit(rB, rB, paB.w);
                a0 = and_or_v(a0, pbA.x, baseA); a1 = and_or_v(a1, pbA.x, baseA);
                a2 = and_or_v(a2, pbA.x, baseA); a3 = and_or_v(a3, pbA.x, baseA);
                b0 = and_or_v(b0, pbB.x, baseB); b1 = and_or_v(b1, pbB.x, baseB);
                b2 = and_or_v(b2, pbB.x, baseB); b3 = and_or_v(b3, pbB.x, baseB);
                xa = krow_l + pbA.w;
                xb = krow_l + pbB.w;
                __builtin_amdgcn_sched_barrier(0);
                uint4v WA, WB;
                WA[0] = lds_at<uint32_t>(a0); WA[1] = lds_at<uint32_t>(a1);
                WA[2] = lds_at<uint32_t>(a2); WA[3] = lds_at<uint32_t>(a3);
                const half8 A1a = lds_at<half8>(qp);
                half8 A2a = A1a;
                if (two) A2a = lds_at<half8>(qp + QS_A2);
                WB[0] = lds_at<uint32_t>(b0); WB[1] = lds_at<uint32_t>(b1);
                WB[2] = lds_at<uint32_t>(b2); WB[3] = lds_at<uint32_t>(b3);
                const half8 A1b = lds_at<half8>(qp + 16);
                half8 A2b = A1b;
                if (two) A2b = lds_at<half8>(qp + 16 + QS_A2);
                rA = lds_codes4(xa);
                rB = lds_codes4(xb);
                paA = lds_at<uint4v>(qp + 32 + QS_PA);
                pbA = lds_at<uint4v>(qp + 32 + QS_PB);
                paB = lds_at<uint4v>(qp + 48 + QS_PA);
                pbB = lds_at<uint4v>(qp + 48 + QS_PB);
                __builtin_amdgcn_sched_barrier(0);
                const half8 BkA = __builtin_bit_cast(half8, WA);
                D1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(A1a, BkA, D1, 0, 0, 0);
                if (two) D2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(A2a, BkA, D2, 0, 0, 0);
                if ((kend >> u) & 1u) segment_done();
                const half8 BkB = __builtin_bit_cast(half8, WB);
                D1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(A1b, BkB, D1, 0, 0, 0);
                if (two) D2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(A2b, BkB, D2, 0, 0, 0);
                if ((kend >> (u + 1)) & 1u) segment_done();
                qp += 32;
            }
            // raw-byte units, one at a time: xa, xb are the addresses of the first two, pbA the first one's parameters
            uint2v r = {0, 0};
            uint4v pb = pbA;
            if (u < n_units) r = lds_codes8(xa);
            for (; u < n_units; u++) {
                // one byte and one table read per code
                uint4v W;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const uint32_t x = e < 2 ? r.x : r.y;
                    const uint32_t c0 = pb.y + ((x >> ((e & 1) * 16)) & 0xFF) * 2;
                    const uint32_t c1 = pb.y + ((x >> ((e & 1) * 16 + 8)) & 0xFF) * 2;
                    W[e] = (uint32_t)lds_at<uint16_t>(c0) | ((uint32_t)lds_at<uint16_t>(c1) << 16);
                }
                const half8 A1 = lds_at<half8>(qp);
                half8 A2 = A1;
                if (two) A2 = lds_at<half8>(qp + QS_A2);
                r = lds_codes8(xb);
                xb = krow_l + pb.w;
                pb = lds_at<uint4v>(qp + 16 + QS_PB);
                const half8 Bk = __builtin_bit_cast(half8, W);
                D1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(A1, Bk, D1, 0, 0, 0);
                if (two) D2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(A2, Bk, D2, 0, 0, 0);
                qp += 16;
                if ((kend >> u) & 1u) segment_done();
            }
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        int k_loads = 0;
        if (more) k_loads = issue_k(tile + step_tiles);      // all reads of the K buffer are done

        // ---- online softmax: lane = token ----------------------------------------------------
        const bool live = lane < nt;
        float d[8];
#pragma unroll
        for (int hh = 0; hh < 8; hh++) d[hh] = S[hh] - m_ref[hh];
        float mx = fmaxf(fmaxf(fmaxf(d[0], d[1]), fmaxf(d[2], d[3])), fmaxf(fmaxf(d[4], d[5]), fmaxf(d[6], d[7])));
        if (__builtin_amdgcn_ballot_w64(live && mx > 0.f)) {   // wave-uniform, rare after the first tiles
            float alpha[8], wm[8];
#pragma unroll
            for (int hh = 0; hh < 8; hh++) wm[hh] = live ? S[hh] : -INFINITY;
            wave_max8(wm);
#pragma unroll
            for (int hh = 0; hh < 8; hh++) {
                const float top = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wm[hh]), 63));
                const float m_new = top > m_ref[hh] ? top + REFRESH : m_ref[hh];
                alpha[hh] = (m_ref[hh] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_ref[hh] - m_new);
                l_part[hh] *= alpha[hh];
                m_ref[hh] = m_new;
                d[hh] = S[hh] - m_new;
            }
            // acc rows are heads 4(lg & 1) + r
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const uint32_t pick = (lg & 1) ? 0xFFFFFFFFu : 0u;     // (bitwise: keeps the factors in registers)
                const float al = __builtin_bit_cast(float, (__builtin_bit_cast(uint32_t, alpha[4 + r]) & pick) |
                                                           (__builtin_bit_cast(uint32_t, alpha[r]) & ~pick));
#pragma unroll
                for (int e = 0; e < 4; e++) acc[e][r] *= al;
            }
        }
        // P * v_norm, formed in fp32 and rounded to fp16 once, goes to LDS as [head][token]
        {
            const float vn = live ? bgtq_h2f((uint16_t)vraw) : 0.f;
#pragma unroll
            for (int hh = 0; hh < 8; hh++) {
                const float pe = live ? __builtin_amdgcn_exp2f(d[hh]) : 0.f;
                l_part[hh] += pe;
                lds_put<uint16_t>(p_wr + hh * PROW, bgtq_f2h(pe * vn));
            }
        }
        wait_loads(k_loads);                                 // the V records of this tile are in LDS
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();

        {
            // values.  The product runs over (token, dim parity) pairs: A row (head h, parity e')
            // holds P[h][t] in slot (t, e') and zero in slot (t, 1 - e'), B column c of accumulator jb
            // holds the table word of token t = dims (8c + 2jb, + 1) in slots (t, 0), (t, 1).
            // D[(h, e')][c] is then out[h][8c + 2jb + e'], a table word is an MFMA operand as it
            // comes, and the 8 head rows that would repeat rows 0..7 carry the odd dims instead.
            // Lane (c = li, lg) decodes unit c of tokens 4lg .. 4lg+3 of every 16-token block; raw
            // codes are fetched one block ahead.
            uint32_t vlo[4], vhi[4];
#pragma unroll
            for (int i = 0; i < 4; i++) lds_read2(vbase + (uint32_t)i * vrow, vlo[i], vhi[i]);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint4v pw = lds_at<uint4v>(p_rd + k * 64);
                uint4v W[4];                                  // [pair of the unit][token]
                // stage by stage, so that neighbouring instructions do not depend on each other
                uint32_t raw[4], ad[4][4];
#pragma unroll
                for (int i = 0; i < 4; i++) raw[i] = __builtin_amdgcn_alignbyte(vhi[i], vlo[i], v_sh);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int e = 0; e < 4; e++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int fp = e * 2 * VBW;
                        ad[e][i] = fp <= vshift ? raw[i] << (vshift - fp) : raw[i] >> (fp - vshift);
                    }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int e = 0; e < 4; e++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        constexpr uint32_t fmask = ((1u << (2 * VBW)) - 1u) << vshift;
                        ad[e][i] = and_or(ad[e][i], fmask, vbank);
                    }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int e = 0; e < 4; e++)
#pragma unroll
                    for (int i = 0; i < 4; i++) W[e][i] = lds_at<uint32_t>(ad[e][i]);
                __builtin_amdgcn_sched_barrier(0);
                if (k + 1 < 4) {
#pragma unroll
                    for (int i = 0; i < 4; i++) lds_read2(vbase + (uint32_t)((k + 1) * 16 + i) * vrow, vlo[i], vhi[i]);
                }
                uint4v Pa;
#pragma unroll
                for (int i = 0; i < 4; i++) Pa[i] = pw[i] << p_shift;
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int jb = 0; jb < 4; jb++)
                    acc[jb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, Pa),
                                                                     __builtin_bit_cast(half8, W[jb]), acc[jb], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();     // V buffer, P buffer and norm areas are rewritten from here on
        v_loads = more ? issue_v(tile + step_tiles) : 0;
    }

    // ---- merge the waves -------------------------------------------------------------
    // Every wave leaves its reference, denominator and unnormalised sums in its own tile buffers
    // (dead by now), in the order the merging threads read them: [m 8][l 8][head 8][li 16][lg >> 1][jb 4].
    // After one barrier thread t of the first gqa * 32 owns head t / 32 and the four dims
    // 8 li + (lg >> 1) + {0, 2, 4, 6} with (li, lg >> 1) = t % 32 and folds the waves in a fixed order.
    {
        float lt[8];
#pragma unroll
        for (int hh = 0; hh < 8; hh++) lt[hh] = l_part[hh];
        wave_sum8(lt);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (lane == 63) {
            lds_put<float4v>(kbuf, (float4v){m_ref[0], m_ref[1], m_ref[2], m_ref[3]});
            lds_put<float4v>(kbuf + 16, (float4v){m_ref[4], m_ref[5], m_ref[6], m_ref[7]});
            lds_put<float4v>(kbuf + 32, (float4v){lt[0], lt[1], lt[2], lt[3]});
            lds_put<float4v>(kbuf + 48, (float4v){lt[4], lt[5], lt[6], lt[7]});
        }
#pragma unroll
        for (int r = 0; r < 4; r++)
            lds_put<float4v>(kbuf + 64 + ((((lg & 1) * 4 + r) * 16 + li) * 2 + (lg >> 1)) * 16,
                             (float4v){acc[0][r], acc[1][r], acc[2][r], acc[3][r]});
    }
    __syncthreads();
    for (int i = tid; i < gqa * 32; i += nthr) {
        const int hq = i >> 5, idx = i & 31;
        float mw[MAX_WAVES], lw[MAX_WAVES];
        float4v ow[MAX_WAVES];
#pragma unroll
        for (int w = 0; w < MAX_WAVES; w++) {                 // all reads go out before the first is used
            const uint32_t wb = WAVES_OFF + (uint32_t)(min(w, nw - 1) * wave_bytes);
            mw[w] = lds_at<float>(wb + hq * 4);
            lw[w] = lds_at<float>(wb + 32 + hq * 4);
            ow[w] = lds_at<float4v>(wb + 64 + (hq * 32 + idx) * 16);
        }
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < MAX_WAVES; w++) if (w < nw) m = fmaxf(m, mw[w]);
        float den = 0.f;
        float4v num = {0, 0, 0, 0};
#pragma unroll
        for (int w = 0; w < MAX_WAVES; w++) {
            if (w < nw) {
                const float f = (mw[w] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mw[w] - m);
                den += f * lw[w];
                num += f * ow[w];
            }
        }
        const bool any = t1 > t0;
        const float inv = any ? 1.f / den : 0.f;
        const size_t row = ((size_t)b * a.n_kv * gqa + (size_t)h * gqa + hq) * a.n_splits + c;
        float* dst = a.part_out + row * D + (idx >> 1) * 8 + (idx & 1);
#pragma unroll
        for (int jb = 0; jb < 4; jb++) dst[2 * jb] = num[jb] * inv;
        if (idx == 0) a.part_lse[row] = any ? (m + log2f(den)) * 0.69314718055994530942f : -INFINITY;
    }
}

// LDS bytes of a work-group of nw waves
size_t mfma_smem_bytes(const TileLayout& tl, int nw) {
    return (size_t)WAVES_OFF + (size_t)nw * wave_lds_bytes(tl);
}

template <int VBW, int VST, bool TWO>
int launch_kernel(DecodeArgs a, hipStream_t st) {
    a.tl = tile_layout(a.k_row_width, VST, (int)a.kn_st);
    // no more waves than the longest partition has tiles
    const int tiles = (a.T + MT - 1) / MT;
    int nw = (tiles + a.n_splits - 1) / a.n_splits;
    nw = nw < 1 ? 1 : nw > MAX_WAVES ? MAX_WAVES : nw;
    while (nw > 1 && mfma_smem_bytes(a.tl, nw) > (size_t)LDS_LIMIT) nw--;
    const size_t smem = mfma_smem_bytes(a.tl, nw);
    if (smem > (size_t)LDS_LIMIT) return BGTQ_EUNSUPPORTED;
    a.nw = nw;
    a.wave_bytes = wave_lds_bytes(a.tl);
    a.per_tiles = tiles / a.n_splits;
    a.rem_tiles = tiles - a.per_tiles * a.n_splits;
    auto kern = decode_mfma_kernel<VBW, VST, TWO>;
    // 1: usable, -1: not usable.  Two threads racing through the first call both run the idempotent
    // set-up below and store the same value.
    static std::atomic<int> ready{0};
    if (ready.load(std::memory_order_acquire) == 0) {
        // the kernel uses offsets into its dynamic LDS block as LDS addresses: that holds only
        // while it has no static LDS in front of the dynamic block
        hipFuncAttributes fa;
        hipError_t e = hipFuncGetAttributes(&fa, (const void*)kern);
        if (e != hipSuccess) return (int)e;
        e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_LIMIT);
        if (e != hipSuccess) return (int)e;
        ready.store(fa.sharedSizeBytes == 0 ? 1 : -1, std::memory_order_release);
    }
    if (ready.load(std::memory_order_acquire) < 0) return BGTQ_EUNSUPPORTED;
    dim3 grid((unsigned)a.n_splits, (unsigned)a.n_kv, (unsigned)a.B);
    hipLaunchKernelGGL(kern, grid, dim3(nw * 64), smem, st, a);
    return bgtq_launch_status();
}

template <int VBW, int VST>
int launch(const DecodeArgs& a, hipStream_t st) {
    return a.gqa > 4 ? launch_kernel<VBW, VST, true>(a, st) : launch_kernel<VBW, VST, false>(a, st);
}

}  // namespace


int bgtq_launch_decode_mfma(const DecodeArgs& a, hipStream_t stream) {
    // layout requirements of the fast path; anything else takes the generic kernel
    if (a.gqa > 8 || !(a.scale > 0.f)) return BGTQ_EUNSUPPORTED;
    // the kernel forms its addresses from 32-bit factors: batch and head strides, and the bytes of one
    // (row, head) slice, must fit
    {
        const int64_t lim = (int64_t)1 << 32;
        const int64_t strides[] = {a.q_sb, a.q_sh, a.kp_sb, a.kp_sh, a.kn_sb, a.kn_sh, a.vp_sb, a.vp_sh, a.vn_sb, a.vn_sh};
        for (int64_t st : strides) if (st < 0 || st >= lim) return BGTQ_EUNSUPPORTED;
        const int64_t rows = (int64_t)a.T + MT;
        if (rows * a.kp_st >= lim || rows * a.vp_st >= lim || rows * a.kn_st * 2 >= lim) return BGTQ_EUNSUPPORTED;
    }
    if ((a.kp_st & 3) || (a.kp_sb & 3) || (a.kp_sh & 3) || ((uintptr_t)a.kp & 3)) return BGTQ_EUNSUPPORTED;
    if ((a.vp_st & 3) || (a.vp_sb & 3) || (a.vp_sh & 3) || ((uintptr_t)a.vp & 3)) return BGTQ_EUNSUPPORTED;
    if (a.kp_st != a.k_row_width) return BGTQ_EUNSUPPORTED;   // K records contiguous
    if (a.k_row_width < 4 || a.k_row_width > 128) return BGTQ_EUNSUPPORTED;
    if (a.vn_st != 1 || a.kn_st < 1 || a.kn_st > MAX_KN) return BGTQ_EUNSUPPORTED;
    if ((a.q_sb & 1) || (a.q_sh & 1) || ((uintptr_t)a.q & 3)) return BGTQ_EUNSUPPORTED;
    if (a.v_layout == BGTQ_V_NIBBLE && a.v_row_width != 64) return BGTQ_EUNSUPPORTED;
    // a bit-packed V record of 128 dims is 16 bytes per bit of code width, a nibble record 64
    // V records follow each other directly, or 4 bytes apart where the record width itself
    // (32 or 64 bytes) would put the rows of a tile on the same LDS banks
    const int64_t pad = a.vp_st - a.v_row_width;
    switch (a.v_row_width) {
    case 16: return pad == 0 ? launch<1, 16>(a, stream) : BGTQ_EUNSUPPORTED;
    case 32: return pad == 0 ? launch<2, 32>(a, stream) : pad == 4 ? launch<2, 36>(a, stream) : BGTQ_EUNSUPPORTED;
    case 48: return pad == 0 ? launch<3, 48>(a, stream) : BGTQ_EUNSUPPORTED;
    case 64: return pad == 0 ? launch<4, 64>(a, stream) : pad == 4 ? launch<4, 68>(a, stream) : BGTQ_EUNSUPPORTED;
    default: return BGTQ_EUNSUPPORTED;
    }
}
