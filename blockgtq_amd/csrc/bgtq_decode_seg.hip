// Decode attention over packed K and V records (gfx950): the bandwidth kernel.
//
// One work-group of up to 12 waves owns one partition of one (batch row, KV head).  The
// 64-token tiles of a (batch row, KV head) are dealt to the partitions as evenly as whole
// tiles allow and round-robin to the waves of a partition; every wave walks its tiles with
// a private online softmax and the waves are merged through LDS at the end.
//
// Data movement.  A tile of packed records is one contiguous byte range of the cache.  It
// goes from HBM straight into LDS with global_load_lds_dwordx4 (aligned 16-byte pieces, the
// 16-byte phase of the source is kept) into the wave's own K buffer as soon as QK^T of the
// previous tile has read it, V likewise after PV, and the fp16 norms travel the same way.
//
// What bounds the kernel is the LDS pipe (one wave instruction per two clocks per CU at
// best) and then vector-ALU issue, not HBM: every table lookup is an LDS read.  The kernel
// is therefore written around the number of LDS instructions per tile:
//
// QK^T   lane = token.  The K record is walked segment by segment (a segment is a run of dims
//        of one code width, so field positions are compile-time constants inside a segment's
//        loop and nothing but the segment's table address and byte offset is read per
//        segment).  A "unit" is 8 consecutive codes: one aligned 8-byte read and a byte funnel
//        shift bring the unit's bytes into a register, four {shift, and-or, 4-byte table read}
//        triples turn it into the eight fp16 operands of one MFMA k-group.  Tables of at most
//        64 entries are replicated 32 times (entry stride 128 bytes): LDS serves the 32 lanes
//        of a half-wave together and the replicas put them on 32 different banks.
//        One MFMA per unit: B = dequantised K (one token per lane), A = the unit's rotated
//        queries, zero outside the lane's own lane group ("block diagonal"), so every lane
//        receives the scores of its own token for all heads: v_mfma_f32_32x32x16_f16 for up
//        to 8 heads (lanes 0..31 and 32..63 are the two diagonal blocks), v_mfma_f32_16x16x32_f16
//        for up to 4.  The A rows are read from LDS once per unit (16 bytes a lane).  The
//        units of a segment accumulate in the MFMA and the segment's sum is scaled by the
//        token's fp16 norm of that segment in fp32.
// Softmax lane = token, exponentials relative to a per-head wave-uniform reference that is kept
//        above every score seen so far and only moved when a score exceeds it.
// PV     P * v_norm goes through LDS once into the A layout of the value product, which runs
//        over (token, dim parity) pairs so that a V table word is an MFMA operand as it comes.
// Merge  every wave leaves its reference, denominator and sums in its own (then dead) tile
//        buffers; after one barrier the first 32 * gqa threads fold the waves.
#include <atomic>

#include "bgtq_decode.h"
#include "bgtq_lds.h"

namespace {

constexpr int D = BGTQ_D;
constexpr int MT = 64;             // tokens per wave tile
constexpr int MAX_UNITS = BGTQ_MAX_UNITS;
constexpr int MAX_WAVES = 12;
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
__host__ __device__ constexpr int kimg_bytes(int k_layout) { return k_layout == BGTQ_K_MIXED ? BGTQ_LUTM_KEND : BGTQ_LUT_KEND; }
__host__ __device__ constexpr int vlut_bytes(int vbw, bool nibble) {
    return (nibble || vbw == 4) ? 1024 : (1 << (2 * vbw)) * 128;
}

__host__ __device__ inline TileLayout tile_layout(int krow, int vrow, int kn_st) {
    TileLayout t;
    t.kt = (MT * krow + 32 + 15) & ~15;
    t.vt = (MT * vrow + 32 + 15) & ~15;
    t.knr = (MT * kn_st * 2 + 16 + 15) & ~15;
    t.vnr = MT * 2 + 16;
    t.kbuf = t.kt + t.knr + t.vnr;
    return t;
}
__host__ __device__ inline int wave_lds_bytes(const TileLayout& t) {
    const int tiles = t.kbuf + t.vt + PBUF_BYTES;
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

// bytes of one unit in the record
template <int PATH> __host__ __device__ constexpr int unit_bytes() { return PATH <= 3 ? PATH : PATH == PATH_BYTE ? 4 : 8; }

// The unit's bytes as one register.  Bit-packed units of 1..3 bytes are fetched with the byte in
// front of them, so that the unit sits at bits 8..31 and every field reaches its table-index
// position (bit 7 up) with a right shift; byte-pair units are fetched as they lie.
template <int PATH>
__device__ __forceinline__ uint32_t fetch_unit(uint32_t xp) {
    const uint32_t x = PATH <= 3 ? xp - 1u : xp;
    uint32_t lo, hi;
    lds_read2(x & ~3u, lo, hi);
    return __builtin_amdgcn_alignbyte(hi, lo, x);
}
// the four pair-table words of the unit in register r
template <int PATH>
__device__ __forceinline__ uint4v unit_words(uint32_t r, uint32_t tb, uint32_t mask) {
    uint32_t ad[4];
#pragma unroll
    for (int p = 0; p < 4; p++) {
        if (PATH <= 3) {
            ad[p] = and_or(r >> (1 + 2 * PATH * p), mask, tb);           // index to bits 7.., replica in tb
        } else {
            ad[p] = and_or(p == 0 ? r << 2 : r >> (8 * p - 2), mask, tb);  // byte p -> bits 2..9
        }
    }
    uint4v w;
#pragma unroll
    for (int p = 0; p < 4; p++) w[p] = lds_at<uint32_t>(ad[p]);
    return w;
}
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

// All units of one segment: nu >= 1 units of PATH starting at LDS byte address xp of this lane's record,
// A rows from qp (advanced by qstep a unit: 16 for the lanes that hold a head's rows, 0 for the lanes
// that read the zero row).  Units go two at a time: the table words and query rows of both are in
// flight together, and so are the codes of the two after them.  The segment's sums, scaled by the
// token's norm n of the segment, are added to S.
template <int PATH, int HEADS>
__device__ __forceinline__ void run_segment(float (&S)[8], float n, uint32_t xp, int nu, uint32_t tb, uint32_t& qp, uint32_t qstep) {
    constexpr int UB = unit_bytes<PATH>();
    ScoreAcc<HEADS> acc;
    if (PATH == PATH_RAW) {
        {
            const uint4v w = raw_unit_words(xp, tb);
            const half8 a = lds_at<half8>(qp);
            acc.mma0(a, __builtin_bit_cast(half8, w));
        }
        for (int j = 1; j < nu; j++) {
            xp += UB;
            qp += qstep;
            const uint4v w = raw_unit_words(xp, tb);
            const half8 a = lds_at<half8>(qp);
            acc.mma(a, __builtin_bit_cast(half8, w));
        }
        qp += qstep;
    } else {
        constexpr uint32_t mask = PATH == 1 ? 0x3u << 7 : PATH == 2 ? 0xFu << 7 : PATH == 3 ? 0x3Fu << 7 : 0xFFu << 2;
        uint32_t r0 = fetch_unit<PATH>(xp), r1 = fetch_unit<PATH>(xp + UB);
        int left = nu;
        {   // the first unit, or the first two when the count is even: what is left is a whole number of pairs
            const uint4v w0 = unit_words<PATH>(r0, tb, mask);
            const half8 a0 = lds_at<half8>(qp);
            if (nu & 1) {
                xp += UB;
                qp += qstep;
                r0 = r1;
                r1 = fetch_unit<PATH>(xp + UB);
                acc.mma0(a0, __builtin_bit_cast(half8, w0));
                left -= 1;
            } else {
                const uint4v w1 = unit_words<PATH>(r1, tb, mask);
                const half8 a1 = lds_at<half8>(qp + qstep);
                xp += 2 * UB;
                qp += 2 * qstep;
                r0 = fetch_unit<PATH>(xp);
                r1 = fetch_unit<PATH>(xp + UB);
                acc.mma0(a0, __builtin_bit_cast(half8, w0));
                acc.mma(a1, __builtin_bit_cast(half8, w1));
                left -= 2;
            }
        }
        for (; left > 0; left -= 2) {
            const uint4v w0 = unit_words<PATH>(r0, tb, mask);
            const half8 a0 = lds_at<half8>(qp);
            const uint4v w1 = unit_words<PATH>(r1, tb, mask);
            const half8 a1 = lds_at<half8>(qp + qstep);
            xp += 2 * UB;
            qp += 2 * qstep;
            r0 = fetch_unit<PATH>(xp);              // (past the segment's last unit: inside the tile buffer's slack, unused)
            r1 = fetch_unit<PATH>(xp + UB);
            acc.mma(a0, __builtin_bit_cast(half8, w0));
            acc.mma(a1, __builtin_bit_cast(half8, w1));
        }
    }
#pragma unroll
    for (int e = 0; e < HEADS; e++) S[e] = fmaf(n, acc.get(e), S[e]);
}

// A segment of exactly N units as straight-line code: all codes are requested first, then all table
// words and query rows, then the MFMAs (two LDS round trips, no loop, no unit counter).  1-bit units
// are one byte each, so one fetch serves three of them.
template <int PATH, int HEADS, int N>
__device__ __forceinline__ void seg_fixed(float (&S)[8], float n, uint32_t xp, uint32_t tb, uint32_t& qp, uint32_t qstep) {
    constexpr int UB = unit_bytes<PATH>();
    ScoreAcc<HEADS> acc;
    half8 a[N];
    uint4v w[N];
    if (PATH == PATH_RAW) {
        uint2v r[N];
#pragma unroll
        for (int i = 0; i < N; i++) r[i] = lds_codes8(xp + i * UB);
        uint32_t ad[N][8];
#pragma unroll
        for (int i = 0; i < N; i++)
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const uint32_t x = e < 4 ? r[i].x : r[i].y;
                ad[i][e] = and_or((e & 3) == 0 ? x << 1 : x >> ((e & 3) * 8 - 1), 0xFFu << 1, tb);    // byte e -> bits 1..8
            }
        uint32_t h16[N][8];
#pragma unroll
        for (int i = 0; i < N; i++) {
#pragma unroll
            for (int e = 0; e < 8; e++) h16[i][e] = lds_at<uint16_t>(ad[i][e]);
            a[i] = lds_at<half8>(qp + i * qstep);
        }
#pragma unroll
        for (int i = 0; i < N; i++)
#pragma unroll
            for (int e = 0; e < 4; e++) w[i][e] = h16[i][2 * e] | (h16[i][2 * e + 1] << 16);
    } else {
        constexpr uint32_t mask = PATH == 1 ? 0x3u << 7 : PATH == 2 ? 0xFu << 7 : PATH == 3 ? 0x3Fu << 7 : 0xFFu << 2;
        uint32_t r[N];
#pragma unroll
        for (int i = 0; i < N; i++) {
            if (PATH == PATH_B1) { if (i % 3 == 0) r[i] = fetch_unit<PATH>(xp + i); }
            else r[i] = fetch_unit<PATH>(xp + i * UB);
        }
#pragma unroll
        for (int i = 0; i < N; i++) {
            uint32_t ad[4];
#pragma unroll
            for (int p = 0; p < 4; p++) {
                if (PATH == PATH_B1) ad[p] = and_or(r[i - i % 3] >> (1 + 2 * p + 8 * (i % 3)), mask, tb);
                else if (PATH <= 3) ad[p] = and_or(r[i] >> (1 + 2 * PATH * p), mask, tb);          // index to bits 7.., replica in tb
                else ad[p] = and_or(p == 0 ? r[i] << 2 : r[i] >> (8 * p - 2), mask, tb);            // byte p -> bits 2..9
            }
#pragma unroll
            for (int p = 0; p < 4; p++) w[i][p] = lds_at<uint32_t>(ad[p]);
            a[i] = lds_at<half8>(qp + i * qstep);
            // the MFMA of the unit before this one goes out while this unit's table words are on their way
            if (i == 1) acc.mma0(a[0], __builtin_bit_cast(half8, w[0]));
            if (i > 1) acc.mma(a[i - 1], __builtin_bit_cast(half8, w[i - 1]));
        }
        if (N == 1) acc.mma0(a[0], __builtin_bit_cast(half8, w[0]));
        else acc.mma(a[N - 1], __builtin_bit_cast(half8, w[N - 1]));
    }
    if (PATH == PATH_RAW) {
        acc.mma0(a[0], __builtin_bit_cast(half8, w[0]));
#pragma unroll
        for (int i = 1; i < N; i++) acc.mma(a[i], __builtin_bit_cast(half8, w[i]));
    }
    qp += N * qstep;
#pragma unroll
    for (int e = 0; e < HEADS; e++) S[e] = fmaf(n, acc.get(e), S[e]);
}

// A segment of nu units: straight-line code for the usual sizes, the loop for long segments.
template <int PATH, int HEADS>
__device__ __forceinline__ void segment(float (&S)[8], float n, uint32_t xp, int nu, uint32_t tb, uint32_t& qp, uint32_t qstep) {
    switch (nu) {
    case 1: seg_fixed<PATH, HEADS, 1>(S, n, xp, tb, qp, qstep); break;
    case 2: seg_fixed<PATH, HEADS, 2>(S, n, xp, tb, qp, qstep); break;
    case 3: seg_fixed<PATH, HEADS, 3>(S, n, xp, tb, qp, qstep); break;
    case 4: if (PATH != PATH_RAW) { seg_fixed<PATH, HEADS, PATH != PATH_RAW ? 4 : 1>(S, n, xp, tb, qp, qstep); break; }
    default: run_segment<PATH, HEADS>(S, n, xp, nu, tb, qp, qstep); break;
    }
}

// HEADS: query heads per KV head the MFMA layout serves (4 or 8)
// VBW: bits per V code; VST: bytes from one V record to the next (the record itself is
// 16 * VBW bytes; a padded stride keeps the rows of a tile on different LDS banks)
template <int HEADS, int VBW, int VST>
__global__ __launch_bounds__(MAX_WAVES * 64) void decode_seg_kernel(DecodeArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nw = a.nw, nthr = nw * 64;
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
    const int n_seg = min(P.n_seg, BGTQ_MAX_SEGMENTS);

    // ---- set-up jobs: job j < (HEADS + 1) * MAX_UNITS fills one 16-byte query slot (head j / MAX_UNITS, the
    // last struct is the zero row) from the plan's unit map.  The loads of a thread's first job go out
    // here, the LDS slots are written once the streaming loads have been issued.
    constexpr int N_QJOBS = (HEADS + 1) * MAX_UNITS;
    auto job_load = [&](int j, uint32_t& slot) -> uint4v {
        uint4v w = {0, 0, 0, 0};
        const int jh = j / MAX_UNITS, ju = j - jh * MAX_UNITS;
        slot = QS_OFF + jh * QSTRUCT + ju * 16;
        const uint32_t dsc = P.sunit[kl][ju];
        const int d0 = (int)(dsc & 0xFF), len = (int)(dsc >> 8);
        if (jh < gqa && jh < HEADS && len > 0) {
            const uint32_t* row = (const uint32_t*)(q_src + jh * a.q_sh + d0);        // d0 is even
#pragma unroll
            for (int pp = 0; pp < 4; pp++)
                w[pp] = row[min(pp, (D - d0) / 2 - 1)] &
                        ((2 * pp < len ? 0xFFFFu : 0u) | (2 * pp + 1 < len ? 0xFFFF0000u : 0u));
        }
        return w;
    };
    uint4v job0 = {0, 0, 0, 0};
    uint32_t job0_slot = 0;
    if (tid < N_QJOBS) job0 = job_load(tid, job0_slot);
    // segment words: lane s of every wave keeps the two words of segment s (read back with v_readlane)
    uint32_t seg_w0 = 0, seg_w1 = 0;
    if (lane < n_seg) {
        seg_w0 = P.sseg[kl][lane][0];
        seg_w1 = P.sseg[kl][lane][1];
    }

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
    const DmaShape full_k = dma_shape_uniform((int)kph + MT * krow), full_kn = dma_shape_uniform((int)knph + MT * kn_st * 2);
    const DmaShape full_vn = dma_shape_uniform((int)vnph + MT * 2), full_v = dma_shape_uniform((int)vph + MT * vrow);
    const int step_tiles = nw * MT;
    const uint32_t first = (uint32_t)(t0 + wave * MT);          // (a (row, head) slice is below 4 GB: checked by the launcher)
    const uint8_t* k_src = kp_base - kph + first * (uint32_t)krow;
    const uint8_t* kn_src = kn_base - knph + first * (uint32_t)(kn_st * 2);
    const uint8_t* vn_src = vn_base - vnph + first * 2u;
    const uint8_t* v_src = vp_base - vph + first * (uint32_t)vrow;
    const int k_step = step_tiles * krow, kn_step = step_tiles * kn_st * 2, vn_step = step_tiles * 2, v_step = step_tiles * vrow;
    auto issue_k = [&](int tile) -> int {
        const int nt = min(MT, t1 - tile);
        DmaShape sk = full_k, sn = full_kn, sv = full_vn;
        if (nt < MT) {
            sk = dma_shape_uniform((int)kph + nt * krow);
            sn = dma_shape_uniform((int)knph + nt * kn_st * 2);
            sv = dma_shape_uniform((int)vnph + nt * 2);
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
        if (nt < MT) sv = dma_shape_uniform((int)vph + nt * vrow);
        dma_region<5>(v_src, vbuf, sv, voff);
        v_src += v_step;
        return sv.nfull + 1;
    };
    int tile = t0 + wave * MT;
    if (tile < t1) { issue_k(tile); issue_v(tile); }        // the wave's first tile: K and V travel together
    bool v_issued = true;

    // ---- the set-up slots (the wait for the query rows also covers the
    // tables and the first K tile: all are needed now)
    {
        if (tid < N_QJOBS) lds_put<uint4v>(job0_slot, job0);
        if (nthr < N_QJOBS)                                   // (uniform) small work-groups only
            for (int j = tid + nthr; j < N_QJOBS; j += nthr) {
                uint32_t slot = 0;
                const uint4v w = job_load(j, slot);
                lds_put<uint4v>(slot, w);
            }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // this wave's table chunks and its first K tile
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
        // Streaming order: the V tile is requested when the K tile has arrived and the K tile of the
        // wave's next tile when the V tile has, so every wait is for all loads in flight.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // K records and norms of this tile are in LDS
        __builtin_amdgcn_wave_barrier();
        if (!v_issued) issue_v(tile);                        // (the V buffer's last readers were the products of the previous tile)
        v_issued = false;
        const uint32_t vraw = lds_at<uint16_t>(vn_l);

        // ---- scores of this lane's token, HEADS heads, in log2 units ----------------------------------
        float S[8];
#pragma unroll
        for (int hh = 0; hh < 8; hh++) S[hh] = 0.f;
        {
            uint32_t qp = qs_l;
            const uint32_t qstep = q_head >= 0 ? 16u : 0u;
            for (int s = 0; s < n_seg; s++) {
                const uint32_t n16 = lds_at<uint16_t>(knrow_l + 2 * s);
                const uint32_t w0 = __builtin_amdgcn_readlane(seg_w0, s), tab = __builtin_amdgcn_readlane(seg_w1, s);
                const int path = (int)(w0 & 15u), nu = (int)((w0 >> 4) & 255u);
                const uint32_t xp = krow_l + (w0 >> 12);
                const float n = bgtq_h2f((uint16_t)n16) * c2;
                switch (path) {
                case PATH_B1: segment<PATH_B1, HEADS>(S, n, xp, nu, tab | rep, qp, qstep); break;
                case PATH_B2: segment<PATH_B2, HEADS>(S, n, xp, nu, tab | rep, qp, qstep); break;
                case PATH_B3: segment<PATH_B3, HEADS>(S, n, xp, nu, tab | rep, qp, qstep); break;
                case PATH_BYTE: segment<PATH_BYTE, HEADS>(S, n, xp, nu, tab, qp, qstep); break;
                default: segment<PATH_RAW, HEADS>(S, n, xp, nu, tab, qp, qstep); break;
                }
            }
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();

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
            for (int hh = 0; hh < 8; hh += 2) {
                const float pe0 = live ? __builtin_amdgcn_exp2f(d[hh]) : 0.f;
                const float pe1 = live ? __builtin_amdgcn_exp2f(d[hh + 1]) : 0.f;
                l_part[hh] += pe0;
                l_part[hh + 1] += pe1;
                const half2v pk = {(_Float16)(pe0 * vn), (_Float16)(pe1 * vn)};
                lds_put<uint32_t>(p_wr + (hh >> 1) * PROW, __builtin_bit_cast(uint32_t, pk));
            }
        }
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");   // the V records of this tile are in LDS, P is written
        __builtin_amdgcn_wave_barrier();
        if (more) issue_k(tile + step_tiles);                // all reads of the K buffer and of the norms are done

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
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();     // V buffer and P buffer are rewritten from here on
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
        const size_t row = ((size_t)b * a.n_kv * a.gqa_all + (size_t)h * a.gqa_all + a.head0 + hq) * a.n_splits + c;
        float* dst = a.part_out + row * D + (idx >> 1) * 8 + (idx & 1);
#pragma unroll
        for (int jb = 0; jb < 4; jb++) dst[2 * jb] = num[jb] * inv;
        if (idx == 0) a.part_lse[row] = any ? (m + log2f(den)) * 0.69314718055994530942f : -INFINITY;
    }
}

template <int HEADS>
size_t seg_smem_bytes(const TileLayout& tl, int nw) {
    return (size_t)waves_off(HEADS) + (size_t)nw * wave_lds_bytes(tl);
}

template <int HEADS, int VBW, int VST>
int launch_kernel(DecodeArgs a, hipStream_t st) {
    a.tl = tile_layout(a.k_row_width, VST, (int)a.kn_st);
    // no more waves than the longest partition has tiles
    const int tiles = (a.T + MT - 1) / MT;
    int nw = (tiles + a.n_splits - 1) / a.n_splits;
    nw = nw < 1 ? 1 : nw > MAX_WAVES ? MAX_WAVES : nw;
    while (nw > 1 && seg_smem_bytes<HEADS>(a.tl, nw) > (size_t)LDS_LIMIT) nw--;
    const size_t smem = seg_smem_bytes<HEADS>(a.tl, nw);
    if (smem > (size_t)LDS_LIMIT) return BGTQ_EUNSUPPORTED;
    a.nw = nw;
    a.wave_bytes = wave_lds_bytes(a.tl);
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
    hipLaunchKernelGGL(kern, grid, dim3(nw * 64), smem, st, a);
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
