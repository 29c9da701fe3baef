// Decode attention over packed K and V records (gfx950): the bandwidth kernel.
//
// One work-group of up to 16 waves owns one partition of one (batch row, KV head).  The
// 64-token tiles of a (batch row, KV head) are dealt to the partitions as evenly as whole
// tiles allow and round-robin to the waves of a partition; every wave walks its tiles with
// a private online softmax and the waves are merged through LDS at the end.
//
// Data movement.  A tile of packed records is one contiguous byte range of the cache.  It
// goes from HBM straight into LDS with global_load_lds_dwordx4 (aligned 16-byte pieces, the
// 16-byte phase of the source is kept) into the wave's own K buffer as soon as the previous
// tile is done with it, V likewise, and the fp16 norms travel the same way.  The set-up
// barrier waits for the tables and query rows only; a wave waits for its own tile.
//
// What bounds the kernel is instruction issue (a wave issues at most one instruction per ten
// clocks or so, a SIMD one per three to four over its waves, whatever the class), not HBM:
// it is written around the number of instructions per tile.
//
// QK^T   lane = token.  The K record is walked step by step; a step is a run of up to 8 units
//        (8 consecutive codes each) of one segment, and there is one straight-line body per
//        (code width, unit count): the run's bytes are read as aligned dwords, one byte funnel
//        per dword brings them to bit 0, and from there every field position is a constant:
//        {shift, and-or, 4-byte table read} per code pair.  Tables of at most 64 entries are
//        replicated 32 times (entry stride 128 bytes): LDS serves the 32 lanes of a half-wave
//        together and the replicas put them on 32 different banks.  1- and 2-bit codes go four
//        at a time through 8-byte entries of unreplicated tables (16 and 256 entries).
//        One MFMA per unit: B = dequantised K (one token per lane), A = the unit's rotated
//        queries, zero outside the lane's own lane group ("block diagonal"), so every lane
//        receives the scores of its own token for all heads: v_mfma_f32_32x32x16_f16 for up
//        to 8 heads (lanes 0..31 and 32..63 are the two diagonal blocks), v_mfma_f32_16x16x32_f16
//        for up to 4.  The A rows are read from LDS once per unit (16 bytes a lane, immediate
//        offsets).  The units of a step accumulate in the MFMA and the step's sum is scaled by
//        the token's fp16 norm of that segment in fp32.
// Softmax lane = token, exponentials relative to a per-head wave-uniform reference that is kept
//        above every score seen so far and only moved when a score exceeds it.
// PV     P * v_norm goes through LDS once into the A layout of the value product, which runs
//        over (token, dim parity) pairs so that a V table word is an MFMA operand as it comes.
// Merge  every wave leaves its reference, denominator and sums in its own (then dead) tile
//        buffers; one thread per (wave, head) works out the factors, one per (head, output)
//        folds the waves.
#include <atomic>
#include <type_traits>

#include "bgtq_decode.h"
#include "bgtq_lds.h"

namespace {

constexpr int D = BGTQ_D;
constexpr int MT = 64;             // tokens per wave tile
constexpr int MAX_UNITS = BGTQ_MAX_UNITS;
constexpr int MAX_WAVES = 16;          // four per SIMD: the register budget of a wave is 128
constexpr int MAX_KN = 8;          // norm columns per token row
constexpr int LDS_LIMIT = 160 * 1024;
constexpr float REFRESH = 4.0f;    // log2 headroom put above the largest score when the reference is refreshed

typedef float float16v __attribute__((ext_vector_type(16)));

// ---- LDS layout (bytes) -----------------------------------------------------------
// [ V pair table | K tables of the record layout in use | query rows | per wave:
//   K tile + K norms + V norms, V tile, P ]
constexpr int VTAB_BYTES = BGTQ_VLUT_BYTES;
constexpr int KTAB_BYTES = BGTQ_LUT_IMAGE_BYTES;
constexpr int QS_OFF = VTAB_BYTES + KTAB_BYTES;
// Query rows: one struct per head and one of zeros (for the lanes outside a unit's lane group), a
// 16-byte slot per unit.  An odd number of slots per struct puts the structs a lane group reads
// together on different banks.
constexpr int QSTRUCT = (MAX_UNITS + 1) * 16;
constexpr int PROW = MT * 4 + 32;                                // bytes from one head pair's P row to the next: rows land 8 banks apart
constexpr int PBUF_BYTES = 4 * PROW;                             // P of a tile: [head pair][token], a dword holds heads 2j (low half) and 2j + 1
constexpr int MERGE_BYTES = 64 + 8 * 32 * 16;                    // what a wave leaves for the merge: m, l, 8 heads x 128 floats

__host__ __device__ constexpr int waves_off(int heads) { return QS_OFF + (heads + 1) * QSTRUCT; }
__host__ __device__ inline TileLayout tile_layout(int krow, int vrow, int kn_st) {
    TileLayout t;
    t.kt = (MT * krow + 32 + 15) & ~15;
    if (t.kt < PBUF_BYTES) t.kt = PBUF_BYTES;       // P of a tile takes the place of its K records
    t.vt = (MT * vrow + 32 + 15) & ~15;
    t.knr = (MT * kn_st * 2 + 16 + 15) & ~15;
    t.vnr = MT * 2 + 16;
    t.kbuf = t.kt + t.knr + t.vnr;
    return t;
}
__host__ __device__ inline int wave_lds_bytes(const TileLayout& t, bool p_over_k) {
    const int tiles = t.kbuf + t.vt + (p_over_k ? 0 : PBUF_BYTES);
    return tiles > MERGE_BYTES ? tiles : MERGE_BYTES;
}

static_assert(offsetof(bgtq_head_plan, lut_image) % 16 == 0 && offsetof(bgtq_head_plan, vlut_image) % 16 == 0 &&
              BGTQ_LUT_IMAGE_BYTES % 16 == 0 && BGTQ_VLUT_BYTES % 16 == 0, "plan tables are copied 16 bytes at a time");

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

// ---- score accumulators: the MFMA that fits the number of query heads ------------------------
// HEADS 4: v_mfma_f32_16x16x32_f16, lane (li, lg) of 4 lane groups: token 16 lg + li, A row li is
//          head li & 3 where li >> 2 == lg and zero elsewhere; d[r] = score of head r.
// HEADS 8: v_mfma_f32_32x32x16_f16, lane (m, hf) of 2 halves: token 32 hf + m, A row m is head
//          4 (m >> 3) + (m & 3) where (m >> 2) & 1 == hf and zero elsewhere; d[r] = score of head r
//          for r < 8 (rows of heads 8..15 are zero).
// An accumulator lives inside one segment: its first MFMA takes a literal zero as C.
template <int HEADS> struct ScoreAcc;
template <> struct ScoreAcc<4> {
    float4v d;
    __device__ __forceinline__ void mma0(const half8& a, const half8& b) { d = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, (float4v){0, 0, 0, 0}, 0, 0, 0); }
    __device__ __forceinline__ void mma(const half8& a, const half8& b) { d = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, d, 0, 0, 0); }
    __device__ __forceinline__ float get(int r) const { return d[r]; }
    static __device__ __forceinline__ int head_of_lane(int lane) { const int li = lane & 15, lg = lane >> 4; return (li >> 2) == lg ? (li & 3) : -1; }
};
template <> struct ScoreAcc<8> {
    float16v d;
    __device__ __forceinline__ void mma0(const half8& a, const half8& b) {
        const float16v z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        d = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, z, 0, 0, 0);
    }
    __device__ __forceinline__ void mma(const half8& a, const half8& b) { d = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, d, 0, 0, 0); }
    __device__ __forceinline__ float get(int r) const { return d[r]; }
    static __device__ __forceinline__ int head_of_lane(int lane) {
        const int m = lane & 31, hf = lane >> 5;
        const int hd = 4 * (m >> 3) + (m & 3);
        return (((m >> 2) & 1) == hf && hd < 8) ? hd : -1;
    }
};

// ---- unit decoders ----------------------------------------------------------------------------
// Code paths of a segment (word 0 of its LDS parameters, bits 0..3)
enum { PATH_B1 = BGTQ_PATH_B1, PATH_B2 = BGTQ_PATH_B2, PATH_B3 = BGTQ_PATH_B3, PATH_BYTE = BGTQ_PATH_BYTE, PATH_RAW = BGTQ_PATH_RAW };

// raw-byte units: one byte and one 2-byte table read per code
__device__ __forceinline__ uint4v raw_unit_words(uint32_t xp, uint32_t tb) {
    const uint2v r = lds_codes8(xp);
    uint4v w;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const uint32_t x = e < 2 ? r.x : r.y;
        const uint32_t c0 = tb + ((x >> ((e & 1) * 16)) & 0xFF) * 2;
        const uint32_t c1 = tb + ((x >> ((e & 1) * 16 + 8)) & 0xFF) * 2;
        w[e] = (uint32_t)lds_at<uint16_t>(c0) | ((uint32_t)lds_at<uint16_t>(c1) << 16);
    }
    return w;
}

// A run of NU units of W-bit codes read through pair tables (W = 3 bit-packed, 4: nibbles) or through
// tables of four codes an entry (W = 1, 2 bit-packed), as straight-line code.  The run starts m bytes behind the 4-byte aligned LDS address a0 of this lane's
// record; its bytes are read as aligned dwords and brought to bit 0 by one byte funnel each, after
// which every field position is a constant: a field reaches its table-index position (bit SH up)
// with one shift, or one bit funnel where it straddles two dwords.  A rows come from qa + 16 * unit.
// The run's sums, scaled by the token's norm n of the segment, are added to S.
template <int W, int HEADS, int NU>
__device__ __forceinline__ void step_pairs(float (&S)[8], float n, uint32_t a0, uint32_t m, uint32_t tab, uint32_t rep, uint32_t qa) {
    constexpr int SH = W == 4 ? 2 : 7;                     // 256-entry tables are not replicated
    constexpr uint32_t MASK = ((1u << (2 * W)) - 1u) << SH;
    constexpr int ND = (NU * W + 3) / 4;
    // (bit-packed codes of 1..3 bits: the table sits at a fixed place of the table area; nibble tables are one per
    // segment and their address comes with the step)
    constexpr uint32_t FIXED = VTAB_BYTES + (W == 1 ? BGTQ_LUT_K1Q : W == 2 ? BGTQ_LUT_K2Q : BGTQ_LUT_K3);
    static_assert((VTAB_BYTES + BGTQ_LUT_K1Q) % 128 == 0 && (VTAB_BYTES + BGTQ_LUT_K2Q) % 2048 == 0, "index bits are OR-ed into the table address");
    const uint32_t tb = W == 4 ? tab : W == 3 ? (rep | FIXED) : FIXED;
    uint32_t r[ND + 1], e[ND];
#pragma unroll
    for (int i = 0; i <= ND; i++) r[i] = lds_at<uint32_t>(a0 + 4 * i);      // (the last one may lie past the run: inside the tile buffer's slack)
#pragma unroll
    for (int i = 0; i < ND; i++) e[i] = __builtin_amdgcn_alignbyte(r[i + 1], r[i], m);
    ScoreAcc<HEADS> acc;
    half8 a[NU];
    uint4v w[NU];
#pragma unroll
    for (int k = 0; k < NU; k++) {
        if constexpr (W <= 2) {
            // 1- and 2-bit codes: four codes index an 8-byte entry of an unreplicated table (16 entries on 16
            // bank pairs; 256 entries): two reads a unit instead of four
            constexpr uint32_t QMASK = ((1u << (4 * W)) - 1u) << 3;
            uint32_t ad[2];
#pragma unroll
            for (int p = 0; p < 2; p++) {
                const int pos = 8 * W * k + 4 * W * p, i = pos >> 5, b = pos & 31;     // (a field of 4 or 8 bits never straddles two dwords)
                const uint32_t x = b > 3 ? e[i] >> (b - 3) : b < 3 ? e[i] << (3 - b) : e[i];
                ad[p] = and_or(x, QMASK, tb);
            }
#pragma unroll
            for (int p = 0; p < 2; p++) {
                const uint2v r = lds_at<uint2v>(ad[p]);
                w[k][2 * p] = r.x;
                w[k][2 * p + 1] = r.y;
            }
        } else {
            uint32_t ad[4];
#pragma unroll
            for (int p = 0; p < 4; p++) {
                const int pos = 8 * W * k + 2 * W * p, i = pos >> 5, b = pos & 31;
                uint32_t x;
                if (b + 2 * W > 32) x = __builtin_amdgcn_alignbit(e[i + 1 < ND ? i + 1 : i], e[i], b - SH);
                else if (b > SH) x = e[i] >> (b - SH);
                else if (b < SH) x = e[i] << (SH - b);
                else x = e[i];
                ad[p] = and_or(x, MASK, tb);
            }
#pragma unroll
            for (int p = 0; p < 4; p++) w[k][p] = lds_at<uint32_t>(ad[p]);
        }
        a[k] = lds_at<half8>(qa + 16 * k);
        // the MFMA of the unit before this one goes out while this unit's table words are on their way
        if (k == 1) acc.mma0(a[0], __builtin_bit_cast(half8, w[0]));
        if (k > 1) acc.mma(a[k - 1], __builtin_bit_cast(half8, w[k - 1]));
    }
    if (NU == 1) acc.mma0(a[0], __builtin_bit_cast(half8, w[0]));
    else acc.mma(a[NU - 1], __builtin_bit_cast(half8, w[NU - 1]));
#pragma unroll
    for (int e8 = 0; e8 < HEADS; e8++) S[e8] = fmaf(n, acc.get(e8), S[e8]);
}

// A run of NU units of 5-bit codes stored one per byte: two bytes that follow each other index the
// 1024-entry pair table (entry address = byte 0 << 2 | byte 1 << 7), which sits at a fixed place of
// the table area and is not replicated.
template <int HEADS, int NU>
__device__ __forceinline__ void step_raw5(float (&S)[8], float n, uint32_t a0, uint32_t m, uint32_t qa) {
    constexpr uint32_t TAB = VTAB_BYTES + BGTQ_LUT_K5P;
    constexpr int ND = 2 * NU;
    uint32_t r[ND + 1], e[ND];
#pragma unroll
    for (int i = 0; i <= ND; i++) r[i] = lds_at<uint32_t>(a0 + 4 * i);
#pragma unroll
    for (int i = 0; i < ND; i++) e[i] = __builtin_amdgcn_alignbyte(r[i + 1], r[i], m);
    ScoreAcc<HEADS> acc;
    half8 a[NU];
    uint4v w[NU];
#pragma unroll
    for (int k = 0; k < NU; k++) {
        uint32_t ad[4];
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const uint32_t x = e[2 * k + i];
            ad[2 * i] = and_or(x >> 1, 0xF80u, (x << 2) & 0x7Cu);
            ad[2 * i + 1] = and_or(x >> 17, 0xF80u, (x >> 14) & 0x7Cu);
        }
#pragma unroll
        for (int p = 0; p < 4; p++) w[k][p] = lds_at<uint32_t>(ad[p] + TAB);
        a[k] = lds_at<half8>(qa + 16 * k);
        if (k == 1) acc.mma0(a[0], __builtin_bit_cast(half8, w[0]));
        if (k > 1) acc.mma(a[k - 1], __builtin_bit_cast(half8, w[k - 1]));
    }
    if (NU == 1) acc.mma0(a[0], __builtin_bit_cast(half8, w[0]));
    else acc.mma(a[NU - 1], __builtin_bit_cast(half8, w[NU - 1]));
#pragma unroll
    for (int e8 = 0; e8 < HEADS; e8++) S[e8] = fmaf(n, acc.get(e8), S[e8]);
}

// A run of nu units of one byte per code: one 2-byte table read per code.
template <int HEADS>
__device__ __forceinline__ void step_raw(float (&S)[8], float n, uint32_t xp, int nu, uint32_t tb, uint32_t qa) {
    ScoreAcc<HEADS> acc;
    {
        const uint4v w = raw_unit_words(xp, tb);
        const half8 a = lds_at<half8>(qa);
        acc.mma0(a, __builtin_bit_cast(half8, w));
    }
    for (int j = 1; j < nu; j++) {
        xp += 8;
        qa += 16;
        const uint4v w = raw_unit_words(xp, tb);
        const half8 a = lds_at<half8>(qa);
        acc.mma(a, __builtin_bit_cast(half8, w));
    }
#pragma unroll
    for (int e = 0; e < HEADS; e++) S[e] = fmaf(n, acc.get(e), S[e]);
}

// HEADS: query heads per KV head the MFMA layout serves (4 or 8)
// VBW: bits per V code; VST: bytes from one V record to the next (the record itself is
// 16 * VBW bytes; a padded stride keeps the rows of a tile on different LDS banks)
template <int HEADS, int VBW, int VST>
__global__ __launch_bounds__(MAX_WAVES * 64) void decode_seg_kernel(DecodeArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nw = a.nw, nthr = nw * 64;                 // waves launched; the first nwt of them own tiles and tile buffers,
    const int nwt = a.nw_tiles;                          // the others help with the set-up and the merge of short partitions
    const int c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const bgtq_head_plan& P = a.plans[h];
    const int gqa = a.gqa;
    const int li = lane & 15, lg = lane >> 4;           // MFMA row/col index, lane group (value product)
    const int kl = a.k_layout;
    const bool vnib = a.v_layout == BGTQ_V_NIBBLE;
    constexpr int WAVES_OFF = waves_off(HEADS);

    // ---- this partition's tiles: the tiles of the row are dealt to the partitions as evenly as
    // whole tiles allow (partition sizes differ by at most one tile)
    int T = a.T, per = a.per_tiles, rem = a.rem_tiles;        // (the launcher divides when every row has T records)
    if (a.seq_lens) {
        T = min(max(a.seq_lens[b], 0), a.T);                  // a length beyond the capacity the launcher checked reads nothing past it
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
    auto at_bh = [&](int64_t sb, int64_t sh, int elem) -> uint64_t {
        return ((uint64_t)(uint32_t)b * (uint32_t)sb + (uint64_t)(uint32_t)h * (uint32_t)sh) * (uint32_t)elem;
    };
    const uint16_t* q_src = (const uint16_t*)((const uint8_t*)a.q + ((uint64_t)(uint32_t)b * (uint32_t)a.q_sb + (uint64_t)(uint32_t)(h * a.gqa_all + a.head0) * (uint32_t)a.q_sh) * 2u);

    // ---- first requests.  The loads of the set-up are written as instructions of their own, so that a
    // wait can leave the loads issued behind it in flight (the compiler would wait for all of them).
    // Lane s < BGTQ_MAX_WALK of every wave keeps the words of step s of the record walk (read back with
    // v_readlane; the steps past the last are zero in the plan, word 1 of a step in use is never zero).
    uint4v seg_w = {0, 0, 0, 0};
    {   // (every lane loads, so that no lane keeps an older value: the lanes behind the table repeat its last step)
        const uint32_t* src = &P.swalk[kl][min(lane, BGTQ_MAX_WALK - 1)][0];
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(seg_w) : "v"(src) : "memory");
    }
    // Set-up jobs: job j < (HEADS + 1) * MAX_UNITS fills one 16-byte query slot (head j / MAX_UNITS, the
    // last struct is the zero row) from the plan's unit map: a slot holds the unit's up to 8 query values,
    // zero where the unit has no dim.  The first N_QJOBS threads take one job each.
    constexpr int N_QJOBS = (HEADS + 1) * MAX_UNITS;
    auto job_slot = [&](int j) -> uint32_t { const int jh = j / MAX_UNITS; return QS_OFF + jh * QSTRUCT + (j - jh * MAX_UNITS) * 16; };
    auto job_mask = [&](uint4v w, int len) -> uint4v {
#pragma unroll
        for (int pp = 0; pp < 4; pp++) w[pp] &= (2 * pp < len ? 0xFFFFu : 0u) | (2 * pp + 1 < len ? 0xFFFF0000u : 0u);
        return w;
    };
    const bool job_wave = wave * 64 < N_QJOBS;               // (uniform)
    uint32_t job_dsc = 0;
    if (job_wave) {                                           // (every lane of the wave loads)
        const uint32_t* src = &P.sunit[kl][tid % MAX_UNITS];
        asm volatile("global_load_dword %0, %1, off" : "=v"(job_dsc) : "v"(src) : "memory");
    }
    const uint32_t voff = (uint32_t)lane * 16;

    // ---- per-wave buffers and streaming sources: 16-byte aligned bases and phases (constant per tile) ----
    const int wave_bytes = a.wave_bytes;
    const uint32_t kbuf = WAVES_OFF + wave * wave_bytes;                       // K records, K norms, V norms
    const uint32_t vbuf = kbuf + tl.kbuf;                                     // V records
    const bool p_over_k = a.p_over_k != 0;                                    // P * v_norm of the tile: over its K records (read by then), or behind the V tile
    const uint32_t pbuf = p_over_k ? kbuf : vbuf + tl.vt;
    const uint8_t* kp_base = a.kp + at_bh(a.kp_sb, a.kp_sh, 1);
    const uint8_t* vp_base = a.vp + at_bh(a.vp_sb, a.vp_sh, 1);
    const uint8_t* kn_base = (const uint8_t*)a.kn + at_bh(a.kn_sb, a.kn_sh, 2);
    const uint8_t* vn_base = (const uint8_t*)a.vn + at_bh(a.vn_sb, a.vn_sh, 2);
    // (every slice on a 16-byte boundary, the usual case: the phases are zero and the launcher has worked
    // out how a whole tile of each range is cut into 1 KB loads)
    uint32_t kph = 0, vph = 0, knph = 0, vnph = 0;
    DmaShape full_k, full_kn, full_vn, full_v;
    if (a.aligned16) {
        full_k = DmaShape{a.nfull[0], a.last[0]};
        full_kn = DmaShape{a.nfull[1], a.last[1]};
        full_vn = DmaShape{a.nfull[2], a.last[2]};
        full_v = DmaShape{a.nfull[3], a.last[3]};
    } else {
        kph = (uint32_t)((uintptr_t)kp_base & 15), vph = (uint32_t)((uintptr_t)vp_base & 15);
        knph = (uint32_t)((uintptr_t)kn_base & 15), vnph = (uint32_t)((uintptr_t)vn_base & 15);
        full_k = dma_shape_uniform((int)kph + MT * krow), full_kn = dma_shape_uniform((int)knph + MT * kn_st * 2);
        full_vn = dma_shape_uniform((int)vnph + MT * 2), full_v = dma_shape_uniform((int)vph + MT * vrow);
    }
    auto tail_of = [&](const uint8_t* base, uint32_t lds, const DmaShape& d) -> DmaTail {
        return DmaTail{base + d.nfull * 1024, lds + (uint32_t)d.nfull * 1024u, d.last};
    };
    const uint8_t *k_al = kp_base - kph, *kn_al = kn_base - knph, *vn_al = vn_base - vnph, *v_al = vp_base - vph;
    const uint32_t knbuf = kbuf + tl.kt, vnbuf = knbuf + tl.knr;
    const DmaTail tail_k = tail_of(k_al, kbuf, full_k), tail_kn = tail_of(kn_al, knbuf, full_kn);
    const DmaTail tail_vn = tail_of(vn_al, vnbuf, full_vn), tail_v = tail_of(v_al, vbuf, full_v);
    const int step_tiles = nwt * MT;
    const uint32_t first = (uint32_t)(t0 + wave * MT);          // (a (row, head) slice is below 4 GB: checked by the launcher)
    // a lane's byte offset from the aligned base of each range, for the wave's current tile
    uint32_t voff_k = voff + first * (uint32_t)krow, voff_kn = voff + first * (uint32_t)(kn_st * 2);
    uint32_t voff_vn = voff + first * 2u, voff_v = voff + first * (uint32_t)vrow;
    const int k_step = step_tiles * krow, kn_step = step_tiles * kn_st * 2, vn_step = step_tiles * 2, v_step = step_tiles * vrow;
    auto issue_k = [&](int tile) -> int {
        const int nt = min(MT, t1 - tile);
        int n_loads;
        if (nt == MT) {
            dma_chunks(voff_k, k_al, kbuf, full_k.nfull);
            if (full_kn.nfull) dma_chunks(voff_kn, kn_al, knbuf, full_kn.nfull);
            dma_tails(voff_k, tail_k, voff_kn, tail_kn, voff_vn, tail_vn);
            n_loads = full_k.nfull + full_kn.nfull + 3;
        } else {
            const DmaShape sk = dma_shape_uniform((int)kph + nt * krow), sn = dma_shape_uniform((int)knph + nt * kn_st * 2);
            const DmaShape sv = dma_shape_uniform((int)vnph + nt * 2);
            dma_chunks(voff_k, k_al, kbuf, sk.nfull);
            dma_chunks(voff_kn, kn_al, knbuf, sn.nfull);
            dma_tails(voff_k, tail_of(k_al, kbuf, sk), voff_kn, tail_of(kn_al, knbuf, sn), voff_vn, tail_of(vn_al, vnbuf, sv));
            n_loads = sk.nfull + sn.nfull + 3;
        }
        voff_k += k_step;
        voff_kn += kn_step;
        voff_vn += vn_step;
        return n_loads;
    };
    auto issue_v = [&](int tile) -> int {
        const int nt = min(MT, t1 - tile);
        int n_loads;
        if (nt == MT) {
            dma_chunks(voff_v, v_al, vbuf, full_v.nfull);
            dma_tail(voff_v, tail_v);
            n_loads = full_v.nfull + 1;
        } else {
            const DmaShape sv = dma_shape_uniform((int)vph + nt * vrow);
            dma_chunks(voff_v, v_al, vbuf, sv.nfull);
            dma_tail(voff_v, tail_of(v_al, vbuf, sv));
            n_loads = sv.nfull + 1;
        }
        voff_v += v_step;
        return n_loads;
    };
    // ---- tables by DMA: V table image at LDS offset 0, the K image of the record layout behind it (all of
    // both: what a plan does not use costs a few loads that the L2 serves, knowing it would cost a round trip);
    // the 1 KB chunks are dealt round-robin to the waves from the last one down (the first ones have the
    // query slots to fill)
    int tab_loads = 0;
    {
        // (chunk cc of the table area lies at LDS offset 1024 cc whichever image it belongs to: the V image
        // takes the first BGTQ_VLUT_BYTES of the area whole, and both images are copied whole)
        constexpr int VCH = BGTQ_VLUT_BYTES / 1024, NCH = VCH + (BGTQ_LUT_IMAGE_BYTES + 1023) / 1024;
        constexpr int LAST_PIECES = (BGTQ_LUT_IMAGE_BYTES - (NCH - VCH - 1) * 1024) / 16;
        static_assert(BGTQ_VLUT_BYTES % 1024 == 0 && VTAB_BYTES == BGTQ_VLUT_BYTES && LAST_PIECES >= 1 && LAST_PIECES <= 64, "");
        const uint8_t* vimg = (const uint8_t*)P.vlut_image[vnib ? 1 : 0];
        const uint8_t* kimg_m = (const uint8_t*)P.lut_image[kl] - VCH * 1024;
        for (int cc = nw - 1 - wave; cc < NCH; cc += nw) {
            const uint8_t* src = (cc < VCH ? vimg : kimg_m) + cc * 1024;
            const uint64_t lanes = cc == NCH - 1 ? (LAST_PIECES >= 64 ? ~0ull : (1ull << LAST_PIECES) - 1ull) : ~0ull;
            dma16(voff, src, (uint32_t)cc * 1024u, lanes);
            tab_loads++;
        }
    }

    // the query words of this thread's job: requested as soon as the unit's dims are known
    uint4v job_w = {0, 0, 0, 0};
    int job_len = 0;
    if (job_wave) {
        wait_loads(tab_loads);
        asm volatile("" : "+v"(job_dsc) :: "memory");
        const int jh = tid / MAX_UNITS, d0 = (int)(job_dsc & 0xFF);
        job_len = (tid < N_QJOBS && jh < gqa && jh < HEADS) ? (int)(job_dsc >> 8) : 0;
        {   // every lane loads (a lane without a job reads the first head's row and masks everything out)
            const uint32_t* row = (const uint32_t*)(q_src + (job_len > 0 ? jh : 0) * a.q_sh + d0);     // d0 is even
            const int last = (D - d0) / 2 - 1;                                        // (a unit's words past the row's end repeat its last one: masked out below)
            const uint32_t *r1 = row + min(1, last), *r2 = row + min(2, last), *r3 = row + min(3, last);
            asm volatile("global_load_dword %0, %4, off\n\tglobal_load_dword %1, %5, off\n\t"
                         "global_load_dword %2, %6, off\n\tglobal_load_dword %3, %7, off"
                         : "=&v"(job_w[0]), "=&v"(job_w[1]), "=&v"(job_w[2]), "=&v"(job_w[3]) : "v"(row), "v"(r1), "v"(r2), "v"(r3) : "memory");
        }
    }

    // ---- the K records and norms of the wave's first tile.  The barrier below does not wait for them: a wave
    // waits for its own tile where it uses it (the V records of a tile are requested when its K records are there)
    int tile = wave < nwt ? t0 + wave * MT : t1;
    int k_loads = 0;
    if (tile < t1) k_loads = issue_k(tile);
    bool fresh = true;                                     // (the wave has no sums yet)

    // ---- the set-up slots.  The wait covers the walk words, the wave's table chunks and query words
    wait_loads(k_loads);
    asm volatile("" : "+v"(seg_w) :: "memory");
    const uint32_t seg_w0 = seg_w[0], seg_w1 = seg_w[1], seg_w2 = seg_w[2];
    const int n_walk = __builtin_popcountll(__builtin_amdgcn_ballot_w64(lane < BGTQ_MAX_WALK && seg_w1 != 0));
    if (job_wave) {
        asm volatile("" : "+v"(job_w[0]), "+v"(job_w[1]), "+v"(job_w[2]), "+v"(job_w[3]) :: "memory");
        if (tid < N_QJOBS) lds_put<uint4v>(job_slot(tid), job_mask(job_w, job_len));
    }
    if (nthr < N_QJOBS)                                   // (uniform) small work-groups only: the other jobs, with plain loads
        for (int j = tid + nthr; j < N_QJOBS; j += nthr) {
            const int jh = j / MAX_UNITS;
            const uint32_t dsc = P.sunit[kl][j - jh * MAX_UNITS];
            const int d0 = (int)(dsc & 0xFF), len = (jh < gqa && jh < HEADS) ? (int)(dsc >> 8) : 0;
            uint4v w = {0, 0, 0, 0};
            if (len > 0) {
                const uint32_t* row = (const uint32_t*)(q_src + jh * a.q_sh + d0);
#pragma unroll
                for (int pp = 0; pp < 4; pp++) w[pp] = row[min(pp, (D - d0) / 2 - 1)];
            }
            lds_put<uint4v>(job_slot(j), job_mask(w, len));
        }
    __syncthreads();

    const float c2 = a.scale * 1.44269504088896340736f;      // scores are kept in log2 units
    const uint32_t rep = ((uint32_t)lane & 31u) * 4u;          // this lane's replica of the 32-fold tables
    // QK^T operands: this lane's record and norm row, its A rows (a head's struct or the zero struct)
    const uint32_t krow_l = kbuf + kph + (uint32_t)lane * krow;
    const uint32_t knrow_l = kbuf + tl.kt + knph + (uint32_t)lane * kn_st * 2;
    const uint32_t vn_l = kbuf + tl.kt + tl.knr + vnph + (uint32_t)lane * 2;
    const int q_head = ScoreAcc<HEADS>::head_of_lane(lane);
    const uint32_t qs_l = QS_OFF + (q_head >= 0 ? q_head : HEADS) * QSTRUCT;
    // PV operands: V table replica (the table sits at LDS address 0, so field bits OR-ed in never meet the
    // base; the 256-entry tables are not replicated), raw codes, P rows
    // V table replica (the table sits at LDS address 0, so field bits OR-ed in never meet the base; the
    // 256-entry tables are not replicated)
    constexpr bool V_UNREP = VBW == 4;                        // also every nibble record (VBW 4 by construction)
    constexpr int VWIN = V_UNREP ? 0 : 8;                     // replicated tables: codes fetched with the byte in front of them
    const uint32_t vbank = V_UNREP ? 0u : rep;
    constexpr int vshift = V_UNREP ? 2 : 7;
    const int vc = (int)vph + li * VBW - (V_UNREP ? 0 : 1);
    const uint32_t vbase = vbuf + (uint32_t)(vc & ~3) + (uint32_t)lg * 4 * vrow, v_sh = (uint32_t)vc & 3u;
    const uint32_t p_wr = pbuf + (uint32_t)lane * 4;                                   // + head pair * PROW
    const uint32_t p_rd = pbuf + (uint32_t)((li & 7) >> 1) * PROW + (uint32_t)lg * 16;   // + block * 64
    // A row (head h = li & 7, dim parity e = li >> 3) takes its head's half of the P dword into the half of
    // parity e and zero into the other: a byte permute per dword
    const uint32_t p_sel = (li & 8) ? ((li & 1) ? 0x03020C0Cu : 0x01000C0Cu) : ((li & 1) ? 0x0C0C0302u : 0x0C0C0100u);

    float m_ref[8], l_part[8];      // per head: reference in log2 units (never below a score seen), this lane's share of the denominator
#pragma unroll
    for (int hh = 0; hh < 8; hh++) { m_ref[hh] = -INFINITY; l_part[hh] = 0.f; }
    float4v acc[4];                 // acc[jb][r] = out[head 4(lg & 1) + r][dim 8 li + 2 jb + (lg >> 1)]
#pragma unroll
    for (int e = 0; e < 4; e++) acc[e] = (float4v){0, 0, 0, 0};

    for (; tile < t1; tile += step_tiles) {
        const int nt = min(MT, t1 - tile);
        const bool more = tile + step_tiles < t1;
        // Streaming order behind the first tile: the V tile is requested when the K tile has arrived and
        // the K tile of the wave's next tile when the V tile has, so every wait is for all loads in flight.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // K records and norms of this tile are in LDS
        __builtin_amdgcn_wave_barrier();
        issue_v(tile);                                       // (the V buffer's last readers were the products of the previous tile)
        const uint32_t vraw = lds_at<uint16_t>(vn_l);

        // ---- scores of this lane's token, HEADS heads, in log2 units ----------------------------------
        float S[8];
#pragma unroll
        for (int hh = 0; hh < 8; hh++) S[hh] = 0.f;
        {
            for (int s = 0; s < n_walk; s++) {
                const uint32_t w0 = __builtin_amdgcn_readlane(seg_w0, s), w2 = __builtin_amdgcn_readlane(seg_w2, s);
                const uint32_t n16 = lds_at<uint16_t>(knrow_l + ((w2 >> 8) & 0xFFu));
                const uint32_t a0 = krow_l + (w2 & 0xFFu), qa = qs_l + (w2 >> 16);
                const float n = bgtq_h2f((uint16_t)n16);
#define BGTQ_STEP(W, NU) case (W - 1) * 8 + NU - 1: step_pairs<W, HEADS, NU>(S, n, a0, w0, W == 4 ? __builtin_amdgcn_readlane(seg_w1, s) : 0u, rep, qa); break;
#define BGTQ_STEPS(W) BGTQ_STEP(W, 1) BGTQ_STEP(W, 2) BGTQ_STEP(W, 3) BGTQ_STEP(W, 4) BGTQ_STEP(W, 5) BGTQ_STEP(W, 6) BGTQ_STEP(W, 7) BGTQ_STEP(W, 8)
                switch (w0 >> 2) {
                BGTQ_STEPS(1) BGTQ_STEPS(2) BGTQ_STEPS(3) BGTQ_STEPS(4)
                case BGTQ_STEP_RAW5 + 0: step_raw5<HEADS, 1>(S, n, a0, w0, qa); break;
                case BGTQ_STEP_RAW5 + 1: step_raw5<HEADS, 2>(S, n, a0, w0, qa); break;
                case BGTQ_STEP_RAW5 + 2: step_raw5<HEADS, 3>(S, n, a0, w0, qa); break;
                case BGTQ_STEP_RAW5 + 3: step_raw5<HEADS, 4>(S, n, a0, w0, qa); break;
                case BGTQ_STEP_RAW5 + 4: step_raw5<HEADS, 5>(S, n, a0, w0, qa); break;
                case BGTQ_STEP_RAW5 + 5: step_raw5<HEADS, 6>(S, n, a0, w0, qa); break;
                case BGTQ_STEP_RAW5 + 6: step_raw5<HEADS, 7>(S, n, a0, w0, qa); break;
                case BGTQ_STEP_RAW5 + 7: step_raw5<HEADS, 8>(S, n, a0, w0, qa); break;
                default: step_raw<HEADS>(S, n, a0 + (w0 & 3u), (int)(w0 >> 2) - BGTQ_STEP_RAW + 1, __builtin_amdgcn_readlane(seg_w1, s), qa); break;
                }
#undef BGTQ_STEPS
#undef BGTQ_STEP
            }
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();

        // ---- online softmax: lane = token ----------------------------------------------------
        // FULL: every lane holds a token (all tiles but a row's last); FRESH: the wave's first tile (no
        // sums to rescale yet).  Both are wave-uniform and known before the tile: four copies of the code.
        auto softmax = [&](auto full_c, auto fresh_c) {
            constexpr bool FULL = decltype(full_c)::value, FRESH = decltype(fresh_c)::value;
            const bool live = FULL || lane < nt;
            float d[8];
#pragma unroll
            for (int hh = 0; hh < 8; hh++) d[hh] = __builtin_fmaf(S[hh], c2, -m_ref[hh]);      // S is in natural units, the reference in log2 units
            bool refresh = FRESH;
            if (!FRESH) {
                const float mx = fmaxf(fmaxf(fmaxf(d[0], d[1]), fmaxf(d[2], d[3])), fmaxf(fmaxf(d[4], d[5]), fmaxf(d[6], d[7])));
                refresh = __builtin_amdgcn_ballot_w64(live && mx > 0.f) != 0;       // wave-uniform, rare after the first tiles
            }
            if (refresh) {
                float wm[8];
#pragma unroll
                for (int hh = 0; hh < 8; hh++) wm[hh] = live ? S[hh] : -INFINITY;
                wave_max8(wm);
                float alpha[8];
#pragma unroll
                for (int hh = 0; hh < 8; hh++) {
                    const float top = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wm[hh]), 63));
                    const float top2 = top * c2;
                    if (FRESH) {
                        m_ref[hh] = top2 + REFRESH;
                    } else {
                        const float m_new = top2 > m_ref[hh] ? top2 + REFRESH : m_ref[hh];
                        alpha[hh] = __builtin_amdgcn_exp2f(m_ref[hh] - m_new);
                        l_part[hh] *= alpha[hh];
                        m_ref[hh] = m_new;
                    }
                    d[hh] = __builtin_fmaf(S[hh], c2, -m_ref[hh]);
                }
                if (!FRESH) {
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
            }
            // P * v_norm, formed in fp32 and rounded to fp16 once, goes to LDS as [head pair][token]
            const float vn = live ? bgtq_h2f((uint16_t)vraw) : 0.f;
#pragma unroll
            for (int hh = 0; hh < 8; hh += 2) {
                const float pe0 = live ? __builtin_amdgcn_exp2f(d[hh]) : 0.f;
                const float pe1 = live ? __builtin_amdgcn_exp2f(d[hh + 1]) : 0.f;
                l_part[hh] += pe0;
                l_part[hh + 1] += pe1;
                const half2v pk = {(_Float16)(pe0 * vn), (_Float16)(pe1 * vn)};
                lds_put<uint32_t>(p_wr + (hh >> 1) * PROW, __builtin_bit_cast(uint32_t, pk));
            }
        };
        if (nt == MT) { if (fresh) softmax(std::true_type{}, std::true_type{}); else softmax(std::true_type{}, std::false_type{}); }
        else          { if (fresh) softmax(std::false_type{}, std::true_type{}); else softmax(std::false_type{}, std::false_type{}); }
        fresh = false;
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");   // the V records of this tile are in LDS, P is written
        __builtin_amdgcn_wave_barrier();
        if (more && !p_over_k) issue_k(tile + step_tiles);   // all reads of the K buffer and of the norms are done

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
                uint32_t raw[4];
#pragma unroll
                for (int i = 0; i < 4; i++) raw[i] = __builtin_amdgcn_alignbyte(vhi[i], vlo[i], v_sh);
                __builtin_amdgcn_sched_barrier(0);
                uint32_t ad[4][4];
#pragma unroll
                for (int e = 0; e < 4; e++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        constexpr uint32_t fmask = ((1u << (2 * VBW)) - 1u) << vshift;
                        const int fp = VWIN + e * 2 * VBW;
                        ad[e][i] = and_or(fp <= vshift ? raw[i] << (vshift - fp) : raw[i] >> (fp - vshift), fmask, vbank);
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
                for (int i = 0; i < 4; i++) Pa[i] = __builtin_amdgcn_perm(pw[i], pw[i], p_sel);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int jb = 0; jb < 4; jb++)
                    acc[jb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, Pa),
                                                                     __builtin_bit_cast(half8, W[jb]), acc[jb], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();     // V buffer and P buffer are rewritten from here on
        if (more && p_over_k) issue_k(tile + step_tiles);
    }

    // ---- merge the waves -------------------------------------------------------------
    // Every wave leaves its reference, denominator and unnormalised sums in its own tile buffers
    // (dead by now), in the order the merging threads read them: [m 8][l 8][head 8][li 16][lg >> 1][jb 4].
    // After one barrier thread t of the first gqa * 32 owns head t / 32 and the four dims
    // 8 li + (lg >> 1) + {0, 2, 4, 6} with (li, lg >> 1) = t % 32 and folds the waves in a fixed order.
    if (wave < nwt) {
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
    // The fold runs in two short steps so that every wave takes part.  Step 1, one thread per (wave, head):
    // the head's reference over all waves, this wave's factor 2^(m_wave - m) and that factor times the
    // wave's denominator, left in LDS where the query rows were.  Step 2, one thread per (head, output):
    // the 16 scaled sums, the denominator, one store.
    constexpr int FW = (MAX_WAVES + 3) & ~3;                 // factors per head, padded to whole 16-byte reads
    constexpr uint32_t F_OFF = QS_OFF, FL_OFF = QS_OFF + 8 * FW * 4, M_OFF = QS_OFF + 16 * FW * 4;
    static_assert((HEADS + 1) * QSTRUCT >= 16 * FW * 4 + 32, "the fold's factors take the place of the query rows");
    auto wave_base = [&](int w) -> uint32_t { return WAVES_OFF + (uint32_t)(min(w, nwt - 1) * wave_bytes); };
    for (int i = tid; i < 8 * FW; i += nthr) {
        const int hh = i & 7, w = i >> 3;
        float m = -INFINITY;
#pragma unroll
        for (int x = 0; x < MAX_WAVES; x++) m = fmaxf(m, lds_at<float>(wave_base(x) + hh * 4));     // (waves past the last repeat it)
        const float mine = lds_at<float>(wave_base(w) + hh * 4), l = lds_at<float>(wave_base(w) + 32 + hh * 4);
        const float f = (w < nwt && mine != -INFINITY) ? __builtin_amdgcn_exp2f(mine - m) : 0.f;
        lds_put<float>(F_OFF + (hh * FW + w) * 4, f);
        lds_put<float>(FL_OFF + (hh * FW + w) * 4, f * l);
        if (w == 0) lds_put<float>(M_OFF + hh * 4, m);
    }
    __syncthreads();
    // (the sums of at most 4 waves where no more own tiles: short partitions)
    auto fold = [&](auto nwf_c) {
        constexpr int NWF = decltype(nwf_c)::value;
        for (int i = tid; i < gqa * 128; i += nthr) {
            const int hq = i >> 7, e = i & 127;                    // e = (li * 2 + (lg >> 1)) * 4 + jb
            float4v f4[NWF / 4], fl4[NWF / 4];
#pragma unroll
            for (int x = 0; x < NWF / 4; x++) {
                f4[x] = lds_at<float4v>(F_OFF + (hq * FW + 4 * x) * 4);
                fl4[x] = lds_at<float4v>(FL_OFF + (hq * FW + 4 * x) * 4);
            }
            float o[NWF];
#pragma unroll
            for (int w = 0; w < NWF; w++) o[w] = lds_at<float>(wave_base(w) + 64 + (hq * 128 + e) * 4);
            float num = 0.f, den = 0.f;
#pragma unroll
            for (int w = 0; w < NWF; w++) {                       // (a wave past the last has factor 0)
                num = fmaf(f4[w >> 2][w & 3], o[w], num);
                den += fl4[w >> 2][w & 3];
            }
            const bool any = t1 > t0;
            const float inv = any ? 1.f / den : 0.f;
            const size_t row = ((size_t)b * a.n_kv * a.gqa_all + (size_t)h * a.gqa_all + a.head0 + hq) * a.n_splits + c;
            const int x = e >> 2;
            a.part_out[row * D + (x >> 1) * 8 + (e & 3) * 2 + (x & 1)] = num * inv;
            if (e == 0) a.part_lse[row] = any ? (lds_at<float>(M_OFF + hq * 4) + log2f(den)) * 0.69314718055994530942f : -INFINITY;
        }
    };
    if (nwt <= 4) fold(std::integral_constant<int, 4>{}); else fold(std::integral_constant<int, FW>{});
}

template <int HEADS>
size_t seg_smem_bytes(const TileLayout& tl, int nw, bool p_over_k) {
    return (size_t)waves_off(HEADS) + (size_t)nw * wave_lds_bytes(tl, p_over_k);
}

template <int HEADS, int VBW, int VST>
int launch_kernel(DecodeArgs a, hipStream_t st) {
    a.tl = tile_layout(a.k_row_width, VST, (int)a.kn_st);
    // no more waves than the longest partition has tiles
    const int tiles = (a.T + MT - 1) / MT;
    int nw = (tiles + a.n_splits - 1) / a.n_splits;
    nw = nw < 1 ? 1 : nw > MAX_WAVES ? MAX_WAVES : nw;
    // P of a tile has a buffer of its own where that leaves room for the waves wanted, else it
    // goes over the tile's K records and the next K tile is requested a phase later
    const bool over = seg_smem_bytes<HEADS>(a.tl, nw, false) > (size_t)LDS_LIMIT;
    while (nw > 1 && seg_smem_bytes<HEADS>(a.tl, nw, over) > (size_t)LDS_LIMIT) nw--;
    const size_t smem = seg_smem_bytes<HEADS>(a.tl, nw, over);
    if (smem > (size_t)LDS_LIMIT) return BGTQ_EUNSUPPORTED;
    // short partitions: more waves than own tiles share the table copies, the query slots and the merge
    a.nw_tiles = nw;
    a.nw = nw < 8 ? 8 : nw;
    a.p_over_k = over ? 1 : 0;
    a.wave_bytes = wave_lds_bytes(a.tl, over);
    {
        // slices that all start on 16-byte boundaries: the cut of a whole tile into 1 KB loads is the same everywhere
        const int64_t al[] = {(int64_t)(uintptr_t)a.kp, a.kp_sb, a.kp_sh, (int64_t)(uintptr_t)a.kn, 2 * a.kn_sb, 2 * a.kn_sh,
                              (int64_t)(uintptr_t)a.vp, a.vp_sb, a.vp_sh, (int64_t)(uintptr_t)a.vn, 2 * a.vn_sb, 2 * a.vn_sh};
        a.aligned16 = 1;
        for (int64_t v : al) if (v & 15) a.aligned16 = 0;
        const int bytes[4] = {MT * a.k_row_width, MT * (int)a.kn_st * 2, MT * 2, MT * VST};
        for (int r = 0; r < 4; r++) {
            const int nfull = ((bytes[r] + 1023) >> 10) - 1, pieces = (bytes[r] - nfull * 1024 + 15) >> 4;
            a.nfull[r] = nfull;
            a.last[r] = pieces >= 64 ? ~0ull : ((1ull << pieces) - 1ull);
        }
    }
    a.per_tiles = tiles / a.n_splits;
    a.rem_tiles = tiles - a.per_tiles * a.n_splits;
    auto kern = decode_seg_kernel<HEADS, VBW, VST>;
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
    hipLaunchKernelGGL(kern, grid, dim3(a.nw * 64), smem, st, a);
    return bgtq_launch_status();
}

template <int VBW, int VST>
int launch(const DecodeArgs& a, hipStream_t st) {
    return a.gqa > 4 ? launch_kernel<8, VBW, VST>(a, st) : launch_kernel<4, VBW, VST>(a, st);
}

}  // namespace


static int launch_group(const DecodeArgs& a, hipStream_t stream);

int bgtq_launch_decode_seg(const DecodeArgs& all, hipStream_t stream) {
    // one launch takes up to 8 query heads per KV head; 9..16 go as two launches over halves of the
    // heads (the records are streamed twice, which still beats the generic kernel several times over)
    if (all.gqa > 16) return BGTQ_EUNSUPPORTED;
    const int n_groups = all.gqa > 8 ? 2 : 1, first = (all.gqa + n_groups - 1) / n_groups;
    for (int g = 0; g < n_groups; g++) {
        DecodeArgs a = all;
        a.gqa_all = all.gqa;
        a.head0 = g * first;
        a.gqa = g == 0 ? first : all.gqa - first;
        const int rc = launch_group(a, stream);
        if (rc != BGTQ_OK) return rc;            // a refusal comes from the first group, before any launch
    }
    return BGTQ_OK;
}

static int launch_group(const DecodeArgs& a, hipStream_t stream) {
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
