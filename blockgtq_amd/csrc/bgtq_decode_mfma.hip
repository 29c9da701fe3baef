// MFMA decode attention over bit-packed K and V records (gfx950).
//
// One work-group of up to 12 waves (3 per SIMD, as many as the tile buffers leave
// room for in LDS) owns one partition of one (batch row, KV head); every wave
// walks its own 64-token tiles with a private online softmax and the results
// are merged through LDS at the end.
//
// Data movement.  A tile of packed records is one contiguous byte range of the
// cache.  It goes from HBM straight into LDS with global_load_lds_dwordx4
// (aligned 16-byte pieces, the 16-byte phase of the source is kept), into the
// wave's K buffer as soon as QK^T of the previous tile has read it (BGTQ_KB = 2
// keeps two buffers and fetches a whole tile ahead: not faster, and the LDS is
// better spent on a third wave per SIMD), V likewise after PV.  The raw
// fp16 norms of the tile travel the same way.  Nothing on the streaming path
// passes through vector registers.
//
// Dequantisation is table driven.  A "unit" is 8 consecutive codes of one
// token (bw bytes of the record).  For every bit width <= 4 the plan carries a
// pair table that the work-group copies into LDS: entry (c0 | c1 << bw) holds
// the two fp16 centroids of a code pair, replicated across LDS banks so that
// lanes with different indices do not collide (32 copies, 8 for the 256-entry
// 4-bit table).
// A unit costs one raw read, four {bit-field extract, shift-add, table read}
// triples and yields the eight fp16 operands of one MFMA k-group.
//
// QK^T:  v_mfma_f32_16x16x32_f16, A = dequantised K (row = token, lane group g
//        supplies unit g of step m; field width and table come from the step
//        table per lane group), B = rotated queries stored per unit in LDS (zero
//        on padding dims), D[token][head].  Every step starts from a zero
//        accumulator and is scaled by the fp16 group norm of its token rows in
//        fp32.  With more than 8 query heads a step holds units of one segment.
//        With at most 8, columns 8..15 repeat heads 0..7 and a step may hold two
//        segments: the first one's query units are non-zero only in columns 0..7,
//        the second one's only in columns 8..15, each half is scaled by its own
//        segment's norm and the halves are added once per tile.
// PV:    the D layout of two 16-token blocks is exactly the A layout of a
//        K=32 step (row = head, lane group g holds 8 tokens), so P never leaves
//        its lane; B = dequantised V where lane (j, g) decodes unit j of its 8
//        tokens and hands dim 8j+e to MFMA e.  The V norm is folded into P in
//        fp32 before P is rounded to fp16.
// Softmax: exponentials are taken relative to a per-head reference that is kept
//        above every score seen so far.  It is only moved (to the new maximum
//        plus a headroom of 4 in log2 units) when a score of the tile exceeds it;
//        otherwise the tile needs no cross-lane traffic at all.
#include <atomic>

#include "bgtq_decode.h"

namespace {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) uint8_t* lds_ptr_t;

constexpr int D = BGTQ_D;
#ifndef BGTQ_MT
#define BGTQ_MT 64
#endif
#ifndef BGTQ_MAX_WAVES
#define BGTQ_MAX_WAVES 12
#endif
#ifndef BGTQ_KB
#define BGTQ_KB 1
#endif
constexpr int MT = BGTQ_MT;        // tokens per wave tile = MT / 16 MFMA row blocks
constexpr int NBLK = MT / 16;
constexpr int MAX_STEPS = BGTQ_MAX_STEPS;
constexpr int MAX_WAVES = BGTQ_MAX_WAVES;
constexpr int KB = BGTQ_KB;         // K tile buffers per wave: 2 = fetched a whole tile ahead, 1 = refilled right after QK^T
constexpr int MAX_KN = 8;          // norm columns per token row the staging area can hold
constexpr int LDS_LIMIT = 160 * 1024;
constexpr int MERGE_STRIDE = BGTQ_D + 8;   // most floats from one row of a wave's result to the next in the merge area
constexpr float REFRESH = 4.0f;    // log2 headroom put above the largest score when the reference is refreshed

// ---- LDS layout (bytes) -----------------------------------------------------------
// LDS starts with the V pair table (8 KB reserved, so that an entry address is the table
// offset OR-ed with field and bank bits), then a copy of the plan's K tables (kimg bytes:
// lut_image up to BGTQ_LUT_V, or lut_image_mixed up to BGTQ_LUTM_V for the mixed K layout).
constexpr int QROW = 400;                      // one head: zero unit + up to 24 units x 16 B
constexpr int VTAB_BYTES = 8192;
__host__ __device__ constexpr int kimg_bytes(int k_layout) { return k_layout == BGTQ_K_MIXED ? BGTQ_LUTM_V : BGTQ_LUT_V; }
__host__ __device__ constexpr int vlut_bytes(int vbw) { return vbw == 4 ? 256 * 32 : (1 << (2 * vbw)) * 128; }
__host__ __device__ constexpr int steptab_off(int kimg) { return VTAB_BYTES + kimg; }   // [step][column half][lane group] x 32 B
__host__ __device__ constexpr int qpad_off(int kimg) { return steptab_off(kimg) + MAX_STEPS * 8 * 32; }
__host__ __device__ constexpr int waves_off(int kimg) { return qpad_off(kimg) + 16 * QROW; }
constexpr int WAVE_NORM_BYTES = BGTQ_MAX_SEGMENTS * MT * 2 + MT * 4;   // fp16 K norms [seg][token], fp32 V norms
constexpr int INIT_SCRATCH = MAX_STEPS * 8 * 32 + 256 + 16 * D * 2;

struct TileLayout {
    int kt, vt, knr, vnr, kbuf;    // bytes of the K, V, K-norm, V-norm areas; K + both norm areas
};
__host__ __device__ inline TileLayout tile_layout(int krow, int vrow, int kn_st) {
    TileLayout t;
    t.kt = (MT * krow + 32 + 15) & ~15;
    t.vt = (MT * vrow + 32 + 15) & ~15;
    t.knr = (MT * kn_st * 2 + 16 + 16 + 15) & ~15;     // phase + the 8-column over-read of the last row
    t.vnr = MT * 2 + 16;
    t.kbuf = t.kt + t.knr + t.vnr;
    return t;
}

// (a & mask) | c in one instruction; the mask travels in a scalar register
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t c) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(c));
    return r;
}

// Read through an absolute LDS address.  Going through the `smem` symbol instead
// costs one extra add per access (the symbol's address is only known at link time).
template <class T>
__device__ __forceinline__ T lds_at(uint32_t addr) {
    return *(const __attribute__((address_space(3))) T*)(uintptr_t)addr;
}

// 16 bytes per lane from sbase + voff into LDS at lds_addr + lane * 16, for the lanes
// set in `lanes`.  The execution mask is switched inside the block, so the copy needs
// no divergent branch around it.
__device__ __forceinline__ void dma16(uint32_t voff, const uint8_t* sbase, uint32_t lds_addr, uint64_t lanes) {
    uint64_t saved;
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %4\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, %0\n"
                 : "=&s"(saved) : "v"(voff), "s"(sbase), "s"(lds_addr), "s"(lanes) : "memory", "m0");
}

// Same for all 64 lanes of a 1 KB chunk at a compile-time distance from sbase / lds_addr:
// the instruction offset moves the global and the LDS address together.
template <int OFF>
__device__ __forceinline__ void dma_chunk(uint32_t voff, const uint8_t* sbase, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3\n"
                 :: "v"(voff), "s"(sbase), "s"(lds_addr), "n"(OFF) : "memory", "m0");
}

// How a byte range [src_al, src_al + total) is cut into 1 KB load instructions: every
// chunk but the last runs with all lanes, the last one with the lanes whose aligned
// 16-byte piece still starts inside the range.  Pieces are aligned, so a piece that holds
// at least one wanted byte never crosses into a page the range itself does not touch.
struct DmaShape {
    int nfull;          // chunks before the last
    uint64_t last;      // lanes of the last chunk
};
__device__ __forceinline__ int dma_count(int total) { return (total + 1023) >> 10; }
__device__ __forceinline__ DmaShape dma_shape(int total, uint32_t voff) {
    DmaShape d;
    d.nfull = dma_count(total) - 1;
    d.last = __builtin_amdgcn_ballot_w64((int)voff < total - d.nfull * 1024);
    return d;
}

// Issues the nfull + 1 loads of a range of at most NCH chunks.
template <int NCH>
__device__ __forceinline__ void dma_region(const uint8_t* src_al, uint32_t lds_addr, const DmaShape& d, uint32_t voff) {
#pragma unroll
    for (int c = 0; c + 1 < NCH; c++)
        if (c < d.nfull) {
            if ((c & 3) == 0) dma_chunk<0>(voff, src_al + (c >> 2) * 4096, lds_addr + (c >> 2) * 4096);
            if ((c & 3) == 1) dma_chunk<1024>(voff, src_al + (c >> 2) * 4096, lds_addr + (c >> 2) * 4096);
            if ((c & 3) == 2) dma_chunk<2048>(voff, src_al + (c >> 2) * 4096, lds_addr + (c >> 2) * 4096);
            if ((c & 3) == 3) dma_chunk<3072>(voff, src_al + (c >> 2) * 4096, lds_addr + (c >> 2) * 4096);
        }
    dma16(voff, src_al + d.nfull * 1024, lds_addr + d.nfull * 1024, d.last);
}

// Waits until at most n of the loads issued so far are still in flight.
__device__ __forceinline__ void wait_loads(int n) {
#define BGTQ_WAIT_CASE(k) case k: asm volatile("s_waitcnt vmcnt(" #k ")" ::: "memory"); break;
    switch (n) {
    BGTQ_WAIT_CASE(0) BGTQ_WAIT_CASE(1) BGTQ_WAIT_CASE(2) BGTQ_WAIT_CASE(3) BGTQ_WAIT_CASE(4) BGTQ_WAIT_CASE(5)
    BGTQ_WAIT_CASE(6) BGTQ_WAIT_CASE(7) BGTQ_WAIT_CASE(8) BGTQ_WAIT_CASE(9) BGTQ_WAIT_CASE(10) BGTQ_WAIT_CASE(11)
    BGTQ_WAIT_CASE(12) BGTQ_WAIT_CASE(13) BGTQ_WAIT_CASE(14) BGTQ_WAIT_CASE(15) BGTQ_WAIT_CASE(16) BGTQ_WAIT_CASE(17)
    BGTQ_WAIT_CASE(18) BGTQ_WAIT_CASE(19) BGTQ_WAIT_CASE(20) BGTQ_WAIT_CASE(21) BGTQ_WAIT_CASE(22) BGTQ_WAIT_CASE(23)
    BGTQ_WAIT_CASE(24) BGTQ_WAIT_CASE(25) BGTQ_WAIT_CASE(26) BGTQ_WAIT_CASE(27) BGTQ_WAIT_CASE(28) BGTQ_WAIT_CASE(29)
    BGTQ_WAIT_CASE(30) BGTQ_WAIT_CASE(31) BGTQ_WAIT_CASE(32) BGTQ_WAIT_CASE(33) BGTQ_WAIT_CASE(34) BGTQ_WAIT_CASE(35)
    default: asm volatile("s_waitcnt vmcnt(36)" ::: "memory"); break;
    }
#undef BGTQ_WAIT_CASE
}

// One step of raw byte codes (bw 5..8): one table read per code.
__device__ __forceinline__ void k_raw_step(float4v (&S)[NBLK], uint32_t st, uint32_t qrow, uint32_t kbase,
                                           uint32_t kstride, uint32_t nrm) {
    const uint4v e0 = lds_at<uint4v>(st), e1 = lds_at<uint4v>(st + 16);
    const half8 Q = lds_at<half8>(qrow + e1.w);
    const uint32_t oa = kbase + e0.x;
#pragma unroll
    for (int k = 0; k < NBLK; k++) {
        const uint32_t ad = oa + k * kstride;
        const uint32_t lo = lds_at<uint32_t>(ad), hi = lds_at<uint32_t>(ad + 4), hi2 = lds_at<uint32_t>(ad + 8);
        const uint32_t r0 = __builtin_amdgcn_alignbyte(hi, lo, e0.y);
        const uint32_t r1 = __builtin_amdgcn_alignbyte(hi2, hi, e0.y);
        half8 A;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const uint32_t r = e < 4 ? r0 : r1;
            const uint32_t byte = (r >> ((e & 3) * 8)) & 0xFF;
            A[e] = __builtin_bit_cast(_Float16, lds_at<uint16_t>(e0.z + byte * 2));
        }
        const float4v d = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, Q, (float4v){0, 0, 0, 0}, 0, 0, 0);
        const half4v n4 = lds_at<half4v>(nrm + e1.z + k * 32);
#pragma unroll
        for (int r = 0; r < 4; r++) S[k][r] = fmaf((float)n4[r], d[r], S[k][r]);
    }
}

#ifdef BGTQ_TRACE
__device__ unsigned long long* g_trace;
#define TRACE(slot)                                                                              \
    do {                                                                                         \
        if (lane == 0 && (slot) < 64 && g_trace)                                                 \
            g_trace[(((size_t)(blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) * 16 + wave) * 64 + (slot)] = \
                __builtin_readcyclecounter();                                                    \
    } while (0)
#else
#define TRACE(slot) do {} while (0)
#endif
#ifdef BGTQ_TRACE
#define TRACE_WALL(slot)                                                                         \
    do {                                                                                         \
        if (lane == 0 && g_trace)                                                                \
            g_trace[(((size_t)(blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) * 16 + wave) * 64 + (slot)] = \
                __builtin_amdgcn_s_memrealtime();                                                \
    } while (0)
#else
#define TRACE_WALL(slot) do {} while (0)
#endif

// VBW: bits per V code; VST: bytes from one V record to the next (the record itself is
// 16 * VBW bytes; a padded stride keeps the rows of a tile on different LDS banks)
// DENSE: at most 8 query heads per KV head (the two-segment step schedule, and a PV product
// that uses the eight spare head rows of the MFMA instead of transposing V)
template <int VBW, int VST, bool DENSE>
__global__ __launch_bounds__(MAX_WAVES * 64) void decode_mfma_kernel(DecodeArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nw = blockDim.x >> 6, nthr = blockDim.x;
    const int c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const bgtq_head_plan& P = a.plans[h];
    const int gqa = a.gqa;
    const int li = lane & 15, lg = lane >> 4;           // MFMA row/col index, lane group

    const int T = a.seq_lens ? a.seq_lens[b] : a.T;
    int chunk = (T + a.n_splits - 1) / a.n_splits;
    chunk = (chunk + MT - 1) / MT * MT;
    const int t0 = min(c * chunk, T), t1 = min(t0 + chunk, T);
    TRACE(0);
    TRACE_WALL(6);

    // ---- LDS carve-up --------------------------------------------------------
    const int krow = a.k_row_width;
    constexpr int vrow = VST;
    const int kn_st = (int)a.kn_st;
    const TileLayout tl = tile_layout(krow, vrow, kn_st);
    const bool kmix = a.k_layout == BGTQ_K_MIXED, vnib = a.v_layout == BGTQ_V_NIBBLE;
    const int kimg = kimg_bytes(a.k_layout);             // LDS offset of the V table
    uint4* steptab = (uint4*)(smem + steptab_off(kimg));
    uint8_t* qpad = smem + qpad_off(kimg);
    const uint32_t smem_lds = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
    // ---- pair tables first: their addresses need nothing but the plan, and they are the last
    // thing the set-up waits for.  V table of the value layout in use at LDS offset 0, K tables
    // of the record layout in use behind it; the chunks of both are dealt round-robin to the waves.
    {
        const uint32_t voff0 = (uint32_t)lane * 16;
        const uint8_t* vimg = vnib ? (const uint8_t*)P.lut_image_mixed + BGTQ_LUTM_V
                                   : (const uint8_t*)P.lut_image + BGTQ_LUT_V;
        const uint8_t* kimg_src = (const uint8_t*)(kmix ? P.lut_image_mixed : P.lut_image);
        constexpr int vch = (vlut_bytes(VBW) + 1023) >> 10;
        const int kch = (kimg + 1023) >> 10;
        for (int cc = wave; cc < vch + kch; cc += nw) {
            const bool isv = cc < vch;
            const int o = (isv ? cc : cc - vch) * 1024;
            const int left = (isv ? vlut_bytes(VBW) : kimg) - o;
            dma16(voff0, (isv ? vimg : kimg_src) + o,
                  __builtin_amdgcn_readfirstlane(smem_lds + (isv ? 0 : VTAB_BYTES) + o),
                  __builtin_amdgcn_ballot_w64((int)voff0 < left));
        }
    }
    const uint32_t kbufs_off = waves_off(kimg);                                   // [KB][nw] K + norm buffers
    const uint32_t vbuf_off = kbufs_off + KB * nw * tl.kbuf + wave * tl.vt;        // [nw] V buffers
    const uint32_t norm_off = kbufs_off + nw * (KB * tl.kbuf + tl.vt) + wave * WAVE_NORM_BYTES;
    uint8_t* kn_h = smem + norm_off;                                 // fp16 [segment][token]
    float* vn_f = (float*)(kn_h + BGTQ_MAX_SEGMENTS * MT * 2);       // fp32 [token]
    uint8_t* scratch = smem + kbufs_off + nw * tl.kbuf;              // everything past the first K buffers is idle during init

    // ---- streaming sources: 16-byte aligned bases and phases (constant per tile) ----
    const uint8_t* kp_base = a.kp + b * a.kp_sb + h * a.kp_sh;
    const uint8_t* vp_base = a.vp + b * a.vp_sb + h * a.vp_sh;
    const uint8_t* kn_base = (const uint8_t*)(a.kn + b * a.kn_sb + h * a.kn_sh);
    const uint8_t* vn_base = (const uint8_t*)(a.vn + b * a.vn_sb + h * a.vn_sh);
    const uint32_t kph = (uint32_t)((uintptr_t)kp_base & 15), vph = (uint32_t)((uintptr_t)vp_base & 15);
    const uint32_t knph = (uint32_t)((uintptr_t)kn_base & 15), vnph = (uint32_t)((uintptr_t)vn_base & 15);
    const uint32_t voff = (uint32_t)lane * 16;
    // K records and both norm arrays of a tile go to K buffer `which`; returns the loads issued.
    // The shapes of a full tile are the same for every tile of the partition.
    const DmaShape full_k = dma_shape((int)kph + MT * krow, voff), full_kn = dma_shape((int)knph + MT * kn_st * 2, voff);
    const DmaShape full_vn = dma_shape((int)vnph + MT * 2, voff), full_v = dma_shape((int)vph + MT * vrow, voff);
    auto issue_k = [&](int tile, int which) -> int {
        const int nt = min(MT, t1 - tile);
        const uint32_t buf = smem_lds + kbufs_off + (which * nw + wave) * tl.kbuf;
        DmaShape sk = full_k, sn = full_kn, sv = full_vn;
        if (nt < MT) {
            sk = dma_shape((int)kph + nt * krow, voff);
            sn = dma_shape((int)knph + nt * kn_st * 2, voff);
            sv = dma_shape((int)vnph + nt * 2, voff);
        }
        dma_region<9>(kp_base - kph + (int64_t)tile * krow, buf, sk, voff);
        dma_region<2>(kn_base - knph + (int64_t)tile * kn_st * 2, buf + tl.kt, sn, voff);
        dma_region<1>(vn_base - vnph + (int64_t)tile * 2, buf + tl.kt + tl.knr, sv, voff);
        return sk.nfull + sn.nfull + sv.nfull + 3;
    };
    auto issue_v = [&](int tile) -> int {
        const int nt = min(MT, t1 - tile);
        DmaShape sv = full_v;
        if (nt < MT) sv = dma_shape((int)vph + nt * vrow, voff);
        dma_region<5>(vp_base - vph + (int64_t)tile * vrow, smem_lds + vbuf_off, sv, voff);
        return sv.nfull + 1;
    };
    const int step_tiles = nw * MT;
    int tile = t0 + wave * MT;
    int v_loads = 0;                 // loads of the V tile issued after the current K tile

    // ---- init: step parameters, query units, tables --------------------------------------
    // Everything a work-group needs comes in by DMA.  The pair tables were requested at the top of
    // the kernel; here follow the small things the set-up code reads (step table, query-unit map,
    // rotated queries) into a scratch area and then the first K and V tiles.  Loads of one wave
    // land in issue order, so the set-up can run while the first tiles are still on their way.
    //
    // Step table per (step, column half, lane group).  Query groups of at most 8 heads use the
    // plan's two-segment schedule (the halves differ); larger groups need all 16 columns for
    // heads and run the one-segment schedule with both halves alike.
    constexpr bool dense = DENSE;
    uint32_t* st_raw = (uint32_t*)scratch;                // step table as stored in the plan
    int* qu_s = (int*)(scratch + MAX_STEPS * 8 * 32);     // qunit_dim[32], qunit_len[32]
    uint16_t* q_s = (uint16_t*)(scratch + MAX_STEPS * 8 * 32 + 256);   // [16][128] rotated queries
    const uint32_t scratch_lds = smem_lds + (uint32_t)(scratch - smem);
    const uint8_t* st_src = dense ? (const uint8_t*)(kmix ? &P.steptab_dense_mixed[0][0][0][0] : &P.steptab_dense[0][0][0][0])
                                  : (const uint8_t*)(kmix ? &P.steptab_mixed[0][0][0] : &P.steptab[0][0][0]);
    const uint8_t* qu_src = (const uint8_t*)(kmix ? P.qunit_dim_mixed : P.qunit_dim);   // qunit_len follows qunit_dim
    const uint8_t* q_src = (const uint8_t*)(a.q + b * a.q_sb + (int64_t)h * gqa * a.q_sh);
    const bool q_dma = ((((uintptr_t)q_src) | (uintptr_t)(a.q_sh * 2)) & 15) == 0;   // rows on 16-byte boundaries
    for (int j = nw - 1 - wave; j < 8; j += nw) {         // 3 KB step table, 256 B unit map, 4 x 4 query rows (dealt from the last wave down: the first waves carry one table chunk more)
        if (j < 3) {
            const uint32_t i = (uint32_t)j * 64 + lane;                          // 16-byte piece of the LDS copy
            const uint32_t m = i >> 4, g = (i >> 1) & 3, part = i & 1;           // piece = (step, half, group, part)
            dma16(dense ? i * 16 : ((m * 4 + g) * 2 + part) * 16, st_src, scratch_lds + j * 1024, ~0ull);
        } else if (j == 3) {
            dma16(voff, qu_src, scratch_lds + MAX_STEPS * 8 * 32, 0xFFFFull);
        } else if (q_dma) {
            const int row = (j - 4) * 4 + (lane >> 4);
            const int src = dense ? (row & 7) : row;                             // columns 8..15 repeat heads 0..7
            const uint64_t ok = __builtin_amdgcn_ballot_w64(src < gqa);
            if (src >= gqa) ((uint4*)q_s)[row * 16 + (lane & 15)] = uint4{0, 0, 0, 0};
            if (ok) {
                dma16((uint32_t)(src * (int)a.q_sh * 2 + (lane & 15) * 16), q_src,
                      scratch_lds + MAX_STEPS * 8 * 32 + 256 + (j - 4) * 1024, ok);
            }
        }
    }
    // first tiles; the V tile only if its buffer does not lie under the scratch area
    const bool v_early = KB == 2 && (size_t)nw * tl.kbuf >= (size_t)INIT_SCRATCH;
    int k0_loads = 0;
    if (tile < t1) {
        k0_loads = issue_k(tile, 0);
        if (v_early) v_loads = issue_v(tile);
    }
    TRACE(1);
    if (!q_dma)                                           // odd query strides: through registers
        for (int i = tid; i < 16 * D / 2; i += nthr) {
            int hq = i / (D / 2), d2 = i - hq * (D / 2);
            const int src = dense ? (hq & 7) : hq;
            uint32_t v = 0;
            if (src < gqa) v = *(const uint32_t*)(a.q + b * a.q_sb + (h * gqa + src) * a.q_sh + d2 * 2);
            ((uint32_t*)q_s)[i] = v;
        }
    const int n_steps = min(dense ? (kmix ? P.n_steps_dense_mixed : P.n_steps_dense)
                                  : (kmix ? P.n_steps_mixed : P.n_steps), MAX_STEPS);
    const int n_packed = min(dense ? (kmix ? P.n_packed_steps_dense_mixed : P.n_packed_steps_dense)
                                   : (kmix ? P.n_packed_steps_mixed : P.n_packed_steps), n_steps);   // raw-byte steps come last
    wait_loads(k0_loads + v_loads);                        // this wave's table chunks and small loads have landed
    __syncthreads();
    TRACE(2);
    for (int i = tid; i < n_steps * 8; i += nthr) {        // the row offset depends on the cache's alignment
        const uint32_t* r = st_raw + i * 8;
        const uint32_t o = kph + r[0];
        steptab[i * 2] = (uint4){o & ~3u, o & 3u, r[2] + smem_lds + VTAB_BYTES, r[3]};     // table as an absolute LDS address
        steptab[i * 2 + 1] = (uint4){r[4], r[5], r[6] * MT / 64, r[7]};   // norm rows are MT tokens long here
    }
    // query units, zero padded: one thread per 16-byte unit (two LDS round trips in all: the unit
    // map, then the four words of the row, which start on an even dim)
    for (int i = tid; i < 16 * (QROW / 16); i += nthr) {
        const int hd = i / (QROW / 16), uid = i - hd * (QROW / 16);
        const int d0 = qu_s[uid], len = qu_s[32 + uid];
        const uint32_t* row = (const uint32_t*)(q_s + hd * D + d0);
        uint32_t w[4];
#pragma unroll
        for (int pp = 0; pp < 4; pp++) w[pp] = row[min(pp, (D - d0) / 2 - 1)];
#pragma unroll
        for (int pp = 0; pp < 4; pp++) {
            const uint32_t keep = (2 * pp < len ? 0xFFFFu : 0u) | (2 * pp + 1 < len ? 0xFFFF0000u : 0u);
            w[pp] &= keep;
        }
        ((uint4*)qpad)[i] = uint4{w[0], w[1], w[2], w[3]};
    }
    __syncthreads();                                        // scratch is dead from here
    if (tile < t1 && !v_early) v_loads = issue_v(tile);
    TRACE(4);
#ifdef BGTQ_TRACE
    int trace_j = 0;
#endif

    const float c2 = a.scale * 1.44269504088896340736f;      // logits go through exp2
    const uint32_t lane4 = (uint32_t)lane * 4;
    // V table replica of this lane.  The table sits at the very start of LDS (this kernel has
    // no static LDS, the launcher checks that), so field bits OR-ed in never meet the base.
    const uint32_t vbank = smem_lds + (VBW == 4 ? (lane4 & 28u) : (lane4 & 124u));
    constexpr int vshift = VBW == 4 ? 5 : 7;
    const uint32_t rowoff = (uint32_t)li * krow;
    const uint32_t kstride = 16u * krow;
    const uint32_t vc = vph + (uint32_t)li * VBW;
    const uint32_t vbase = smem_lds + vbuf_off + (vc & ~3u) + (uint32_t)lg * 4 * vrow, v_sh = vc & 3u;
    const uint32_t stl = smem_lds + steptab_off(kimg) + (li >> 3) * 128 + lg * 32;   // absolute LDS addresses from here on
    const uint32_t qrow = smem_lds + qpad_off(kimg) + li * QROW;
    const uint32_t nrm = smem_lds + norm_off + lg * 8;
    const uint32_t vnf = smem_lds + norm_off + BGTQ_MAX_SEGMENTS * MT * 2;

    float m_ref = -INFINITY;        // reference of head li, in exp2 units; never below a score seen
    float l_part = 0.f;             // this lane's share of the softmax denominator
    constexpr int NACC = DENSE ? 4 : 8;         // output accumulators (16 x 16 each)
    float4v acc[NACC];
#pragma unroll
    for (int e = 0; e < NACC; e++) acc[e] = (float4v){0, 0, 0, 0};

    int which = 0;
    for (; tile < t1; tile += step_tiles, which ^= 1) {
        const int nt = min(MT, t1 - tile);
        const bool more = tile + step_tiles < t1;
        const uint32_t kbuf = kbufs_off + ((KB == 2 ? which : 0) * nw + wave) * tl.kbuf;
        TRACE(8 + trace_j * 8 + 0);
        wait_loads(v_loads);                                 // K records and norms of this tile are in LDS
        __builtin_amdgcn_wave_barrier();
        TRACE(8 + trace_j * 8 + 1);
        // ---- norms of the tile: lane = token; read raw, start the next K tile, then store
        //      them as fp16 [segment][token] and fp32 V norms -------------------------------------
        // All 8 columns are moved whatever the head's segment count: columns past the row end
        // read neighbouring bytes of the staging area, land in rows no step refers to, and the
        // copy stays free of branches.
        uint16_t nraw[BGTQ_MAX_SEGMENTS];
        {
            const uint32_t kraw = smem_lds + kbuf + tl.kt + knph + (uint32_t)lane * kn_st * 2;
#pragma unroll
            for (int s = 0; s < BGTQ_MAX_SEGMENTS; s++) nraw[s] = lds_at<uint16_t>(kraw + s * 2);
        }
        const uint16_t vraw = lds_at<uint16_t>(smem_lds + kbuf + tl.kt + tl.knr + vnph + lane * 2);
        int k_loads = 0;
        if (KB == 2 && more) k_loads = issue_k(tile + step_tiles, which ^ 1);
        if (MT == 64 || lane < MT) {
#pragma unroll
            for (int s = 0; s < BGTQ_MAX_SEGMENTS; s++) *(uint16_t*)(kn_h + (s * MT + lane) * 2) = nraw[s];
            vn_f[lane] = lane < nt ? bgtq_h2f(vraw) : 0.f;
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        TRACE(8 + trace_j * 8 + 2);

        // ---- scores ---------------------------------------------------------------
        float4v S[NBLK];
#pragma unroll
        for (int k = 0; k < NBLK; k++) S[k] = (float4v){0, 0, 0, 0};
        {
            // Software pipeline over the packed steps.  The iteration that multiplies step m
            // first forms the table addresses of step m+1 (from raw codes and parameters read
            // one iteration earlier), issues the MFMAs of step m, then fetches parameters and
            // raw codes of step m+2 together with the query unit and norms of step m+1, and
            // last the table words of step m+1.  Every LDS read is consumed one iteration
            // after it was issued and every register set is rewritten only after its last
            // reader has issued, so the loop carries no copies.  The small reads go first
            // because the counter of outstanding LDS reads saturates at 15: the next iteration
            // can then wait for them while most table reads are still in flight.
            const uint32_t kbase = smem_lds + kbuf + rowoff;
            const int last = n_packed - 1;
            uint4v e0, e1;                                  // parameters of the step whose addresses are formed next
            uint32_t xoff;                                  // raw-code offset of the step fetched next
            uint32_t rlo[NBLK], rhi[NBLK];                  // raw codes
            uint32_t ad[NBLK][4], qad, nad;                 // table, query-unit and norm addresses
            uint4v w[NBLK];                                 // table words = the MFMA A operands
            half8 Q;
            half4v n4[NBLK];
            auto params = [&](int m) {
                const uint32_t at = stl + (uint32_t)min(m, last) * 256;
                e0 = lds_at<uint4v>(at);
                e1 = lds_at<uint4v>(at + 16);
            };
            auto raw_offset = [&](int m) { return lds_at<uint32_t>(stl + (uint32_t)min(m, last) * 256); };
            auto raws = [&](uint32_t off) {
                const uint32_t oa = kbase + off;
#pragma unroll
                for (int k = 0; k < NBLK; k++) {
                    rlo[k] = lds_at<uint32_t>(oa + k * kstride);
                    rhi[k] = lds_at<uint32_t>(oa + k * kstride + 4);
                }
            };
            auto addresses = [&]() {                        // bit fields -> table addresses
                const uint32_t lb = (lane4 & e0.w) | e0.z;
                const uint32_t pw = e1.x, pw2 = pw * 2, pw3 = pw * 3, tsh = e1.y;
#pragma unroll
                for (int k = 0; k < NBLK; k++) {
                    const uint32_t raw = __builtin_amdgcn_alignbyte(rhi[k], rlo[k], e0.y);
                    ad[k][0] = (__builtin_amdgcn_ubfe(raw, 0, pw) << tsh) + lb;
                    ad[k][1] = (__builtin_amdgcn_ubfe(raw, pw, pw) << tsh) + lb;
                    ad[k][2] = (__builtin_amdgcn_ubfe(raw, pw2, pw) << tsh) + lb;
                    ad[k][3] = (__builtin_amdgcn_ubfe(raw, pw3, pw) << tsh) + lb;
                }
                qad = qrow + e1.w;
                nad = nrm + e1.z;
            };
            auto operands = [&]() {                         // query unit and norms of the segment
                Q = lds_at<half8>(qad);
#pragma unroll
                for (int k = 0; k < NBLK; k++) n4[k] = lds_at<half4v>(nad + k * 32);
            };
            auto tables = [&]() {                           // table words
#pragma unroll
                for (int k = 0; k < NBLK; k++)
                    w[k] = (uint4v){lds_at<uint32_t>(ad[k][0]), lds_at<uint32_t>(ad[k][1]),
                                   lds_at<uint32_t>(ad[k][2]), lds_at<uint32_t>(ad[k][3])};
            };
            // one MFMA per row block from a zero accumulator, scaled by the fp16 group norm of
            // its token rows in fp32
            auto multiply = [&]() {
                float4v d[NBLK];
#pragma unroll
                for (int k = 0; k < NBLK; k++)
                    d[k] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, w[k]), Q,
                                                                  (float4v){0, 0, 0, 0}, 0, 0, 0);
#pragma unroll
                for (int k = 0; k < NBLK; k++)
#pragma unroll
                    for (int r = 0; r < 4; r++) S[k][r] = fmaf((float)n4[k][r], d[k][r], S[k][r]);
            };
            if (n_packed > 0) {
                params(0);
                const uint32_t x1 = raw_offset(1);
                xoff = raw_offset(2);
                raws(e0.x);
                addresses();                                // step 0
                __builtin_amdgcn_sched_barrier(0);
                params(1);                                  // same order as in the loop, so that the
                raws(x1);                                   // wait at the loop head is the same on
                operands();                                 // both ways into it
                __builtin_amdgcn_sched_barrier(0);
                tables();
                for (int m = 0; m < last; m++) {
                    __builtin_amdgcn_sched_barrier(0);
                    addresses();                            // step m+1
                    __builtin_amdgcn_sched_barrier(0);
                    multiply();                             // step m
                    __builtin_amdgcn_sched_barrier(0);
                    params(m + 2);
                    raws(xoff);                             // step m+2
                    xoff = raw_offset(m + 3);
                    operands();                             // step m+1
                    __builtin_amdgcn_sched_barrier(0);
                    tables();                               // step m+1
                }
                __builtin_amdgcn_sched_barrier(0);
                multiply();
            }
            TRACE(8 + trace_j * 8 + 6);
            for (int m = n_packed; m < n_steps; m++) k_raw_step(S, stl + m * 256, qrow, kbase, kstride, nrm);
            if (dense) {
                // the two column halves hold the partial sums of different segments: add them, so
                // that column c and column c ^ 8 both carry the full score of head c & 7
#pragma unroll
                for (int k = 0; k < NBLK; k++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
{
                        // (through a scalar: bit-casting the vector element in place makes the
                        // compiler read element 0 of the vector for every r)
                        const float x = S[k][r];
                        const int rot = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x),
                                                                    0x128 /* row_ror:8 */, 0xf, 0xf, false);
                        S[k][r] = x + __builtin_bit_cast(float, rot);
                    }
            }
        }
        if (KB == 1 && more) k_loads = issue_k(tile + step_tiles, 0);   // all reads of the K buffer are done
        TRACE(8 + trace_j * 8 + 3);

        // ---- online softmax: lane (head li, group lg) holds tokens 16k + 4lg + r ------
        if (nt < MT) {
#pragma unroll
            for (int r = 0; r < 4 * NBLK; r++) {
                const int tk = (r >> 2) * 16 + lg * 4 + (r & 3);
                if (tk >= nt) S[r >> 2][r & 3] = -INFINITY;
            }
        }
        float mx = S[0][0];
#pragma unroll
        for (int r = 1; r < 4 * NBLK; r++) mx = fmaxf(mx, S[r >> 2][r & 3]);
        mx *= c2;
        if (__builtin_amdgcn_ballot_w64(mx > m_ref)) {    // wave-uniform, rare after the first tiles
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m_ref, mx + REFRESH);
            const float alpha = (m_ref == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_ref - m_new);
            // acc rows are heads 4lg+r, not this lane's head: fetch their factors
            float al[4];
#pragma unroll
            for (int r = 0; r < 4; r++) al[r] = __shfl(alpha, lg * 4 + r, 64);
#pragma unroll
            for (int e = 0; e < NACC; e++)
#pragma unroll
                for (int r = 0; r < 4; r++) acc[e][r] *= al[r];
            l_part *= alpha;
            m_ref = m_new;
        }
        TRACE(8 + trace_j * 8 + 4);
        wait_loads(k_loads);                                 // the V records of this tile are in LDS
        __builtin_amdgcn_wave_barrier();

        if constexpr (DENSE) {
            // values, at most 8 heads.  The product runs over (token, dim parity) pairs: A row
            // (head h, parity e') holds P[h][t] in slot (t, e') and zero in slot (t, 1 - e'), B
            // column c of accumulator jb holds the table word of token t = dims (8c + 2jb, + 1) in
            // slots (t, 0), (t, 1).  D[(h, e')][c] is then out[h][8c + 2jb + e'], a table word
            // is an MFMA operand as it comes, and the 8 head rows that would repeat rows 0..7
            // carry the odd dims instead.  Lane (c = li, lg) decodes unit c of tokens 4lg .. 4lg+3
            // of every 16-token block; raw codes are fetched one block ahead.
            const uint32_t pmask = (li & 8) ? 0xFFFF0000u : 0x0000FFFFu;
            uint32_t vlo[4], vhi[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                vlo[i] = lds_at<uint32_t>(vbase + (uint32_t)i * vrow);
                vhi[i] = lds_at<uint32_t>(vbase + (uint32_t)i * vrow + 4);
            }
#pragma unroll
            for (int k = 0; k < NBLK; k++) {
                const float4v vn4 = lds_at<float4v>(vnf + (k * 16 + lg * 4) * 4);
                uint4v W[4];                                  // [pair of the unit][token]
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t raw = __builtin_amdgcn_alignbyte(vhi[i], vlo[i], v_sh);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        constexpr uint32_t fmask = ((1u << (2 * VBW)) - 1u) << vshift;
                        const int fp = e * 2 * VBW;
                        const uint32_t sh = fp <= vshift ? raw << (vshift - fp) : raw >> (fp - vshift);
                        W[e][i] = lds_at<uint32_t>(and_or(sh, fmask, vbank));
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                if (k + 1 < NBLK) {
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int tk = (k + 1) * 16 + i;
                        vlo[i] = lds_at<uint32_t>(vbase + (uint32_t)tk * vrow);
                        vhi[i] = lds_at<uint32_t>(vbase + (uint32_t)tk * vrow + 4);
                    }
                }
                // P * v_norm is formed in fp32, rounded to fp16 once and kept in the half of
                // the word that belongs to this lane's parity
                uint4v Pa;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float pe = __builtin_amdgcn_exp2f(fmaf(S[k][i], c2, -m_ref));
                    l_part += pe;
                    const float x = pe * vn4[i];
                    const float2v xx = {x, x};
                    Pa[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(xx, half2v)) & pmask;
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int jb = 0; jb < 4; jb++)
                    acc[jb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, Pa),
                                                                     __builtin_bit_cast(half8, W[jb]), acc[jb], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
            // values: lane (j = li, group lg) decodes unit j of its 8 tokens per half tile.  Raw
            // codes are fetched one half ahead; the exponentials run while the table reads fly.
            uint32_t vlo[8], vhi[8];
#pragma unroll
            for (int r = 0; r < 8; r++) {
                const int tk = (r >> 2) * 16 + (r & 3);                       // + 4lg, folded into vbase
                vlo[r] = lds_at<uint32_t>(vbase + (uint32_t)tk * vrow);
                vhi[r] = lds_at<uint32_t>(vbase + (uint32_t)tk * vrow + 4);
            }
#pragma unroll
            for (int half = 0; half < NBLK / 2; half++) {
                const float4v vn_lo = lds_at<float4v>(vnf + (half * 32 + lg * 4) * 4);        // tokens 4lg .. 4lg+3
                const float4v vn_hi = lds_at<float4v>(vnf + (half * 32 + 16 + lg * 4) * 4);   // tokens 16+4lg ..
                uint32_t W[8][4];
#pragma unroll
                for (int r = 0; r < 8; r++) {
                    const uint32_t raw = __builtin_amdgcn_alignbyte(vhi[r], vlo[r], v_sh);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        // shift the pair field to its place in the table address, then one and-or
                        // merges the bank replica (the compiler would spend an and plus an add)
                        constexpr uint32_t fmask = ((1u << (2 * VBW)) - 1u) << vshift;
                        const int fp = e * 2 * VBW;
                        const uint32_t sh = fp <= vshift ? raw << (vshift - fp) : raw >> (fp - vshift);
                        W[r][e] = lds_at<uint32_t>(and_or(sh, fmask, vbank));
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                if (half + 1 < NBLK / 2) {
#pragma unroll
                    for (int r = 0; r < 8; r++) {
                        const int tk = (half + 1) * 32 + (r >> 2) * 16 + (r & 3);
                        vlo[r] = lds_at<uint32_t>(vbase + (uint32_t)tk * vrow);
                        vhi[r] = lds_at<uint32_t>(vbase + (uint32_t)tk * vrow + 4);
                    }
                }
                // P * v_norm is formed in fp32 and rounded to fp16 once
                half8 Pm;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int k = half * 2 + (e >> 1), r = (e & 1) * 2;
                    const float p0 = __builtin_amdgcn_exp2f(fmaf(S[k][r], c2, -m_ref));
                    const float p1 = __builtin_amdgcn_exp2f(fmaf(S[k][r + 1], c2, -m_ref));
                    l_part += p0 + p1;
                    const float4v vn4 = (e >> 1) ? vn_hi : vn_lo;
                    const float2v pv = {p0 * vn4[r], p1 * vn4[r + 1]};
                    const half2v ph = __builtin_convertvector(pv, half2v);
                    Pm[2 * e] = ph[0];
                    Pm[2 * e + 1] = ph[1];
                }
                __builtin_amdgcn_sched_barrier(0);
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
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();     // V buffer and norm areas are rewritten from here on
        v_loads = more ? issue_v(tile + step_tiles) : 0;
        TRACE(8 + trace_j * 8 + 5);
#ifdef BGTQ_TRACE
        trace_j++;
#endif
    }
    TRACE(60);

    // ---- merge the waves -------------------------------------------------------------
    float l_tot = l_part;
    l_tot += __shfl_xor(l_tot, 16, 64);
    l_tot += __shfl_xor(l_tot, 32, 64);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();                         // tables and tile buffers are dead from here
    // Dim d of a row sits at (d & 7) * 16 + (d >> 3); with that column order and a row stride of
    // MS floats the 64 lanes of every store below fall on 64 different banks.
    constexpr int MS = DENSE ? MERGE_STRIDE : MERGE_STRIDE - 4;
    float* mg_m = (float*)smem;              // [nw][16]
    float* mg_l = mg_m + nw * 16;            // [nw][16]
    float* mg_o = mg_l + nw * 16;            // [nw][16][MS]
    if (lane < 16) { mg_m[wave * 16 + lane] = m_ref; mg_l[wave * 16 + lane] = l_tot; }
    if constexpr (DENSE) {                   // acc[jb][r] = out[head 4(lg & 1) + r][dim 8li + 2jb + (lg >> 1)]
#pragma unroll
        for (int jb = 0; jb < 4; jb++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                mg_o[(wave * 16 + (lg & 1) * 4 + r) * MS + (2 * jb + (lg >> 1)) * 16 + li] = acc[jb][r];
    } else {                                 // acc[e][r] = out[head 4lg + r][dim 8li + e]
#pragma unroll
        for (int e = 0; e < 8; e++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                mg_o[(wave * 16 + lg * 4 + r) * MS + e * 16 + li] = acc[e][r];
    }
    __syncthreads();
    TRACE(61);
    for (int i = tid; i < gqa * D; i += nthr) {
        const int hq = i / D, d = i - hq * D;
        const int col = (d & 7) * 16 + (d >> 3);
        // all reads of a batch go out before the first is used (one LDS round trip per batch)
        float mw[MAX_WAVES], lw[MAX_WAVES], ow[MAX_WAVES];
#pragma unroll
        for (int w = 0; w < MAX_WAVES; w++) {
            const int ww = min(w, nw - 1);
            mw[w] = mg_m[ww * 16 + hq];
            lw[w] = mg_l[ww * 16 + hq];
            ow[w] = mg_o[(ww * 16 + hq) * MS + col];
        }
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < MAX_WAVES; w++) if (w < nw) m = fmaxf(m, mw[w]);
        float den = 0.f, num = 0.f;
#pragma unroll
        for (int w = 0; w < MAX_WAVES; w++) {
            if (w < nw) {
                const float f = (mw[w] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mw[w] - m);
                den += f * lw[w];
                num += f * ow[w];
            }
        }
        size_t row = ((size_t)b * a.n_kv * gqa + (size_t)h * gqa + hq) * a.n_splits + c;
        a.part_out[row * D + d] = (t1 > t0) ? num / den : 0.f;
        if (d == 0) a.part_lse[row] = (t1 > t0) ? (m + log2f(den)) * 0.69314718055994530942f : -INFINITY;
    }
    TRACE(62);
    TRACE_WALL(7);
}

// LDS bytes of a work-group of nw waves
size_t mfma_smem_bytes(int k_layout, int krow, int vrow, int kn_st, int nw) {
    const int woff = waves_off(kimg_bytes(k_layout));
    const TileLayout tl = tile_layout(krow, vrow, kn_st);
    size_t need = (size_t)woff + (size_t)nw * (KB * tl.kbuf + tl.vt + WAVE_NORM_BYTES);
    size_t scratch = (size_t)woff + (size_t)nw * tl.kbuf + INIT_SCRATCH;
    size_t merge = (size_t)nw * (32 + 16 * MERGE_STRIDE) * 4;
    size_t s = need > scratch ? need : scratch;
    return s > merge ? s : merge;
}

template <int VBW, int VST, bool DENSE>
int launch_kernel(const DecodeArgs& a, hipStream_t st) {
    // no more waves than the longest partition has tiles
    const int part = (a.T + a.n_splits - 1) / a.n_splits;
    int nw = (part + MT - 1) / MT;
    nw = nw < 1 ? 1 : nw > MAX_WAVES ? MAX_WAVES : nw;
    while (nw > 1 && mfma_smem_bytes(a.k_layout, a.k_row_width, VST, (int)a.kn_st, nw) > (size_t)LDS_LIMIT) nw--;
    const size_t smem = mfma_smem_bytes(a.k_layout, a.k_row_width, VST, (int)a.kn_st, nw);
    if (smem > (size_t)LDS_LIMIT) return BGTQ_EUNSUPPORTED;
    auto kern = decode_mfma_kernel<VBW, VST, DENSE>;
    // 1: usable, -1: not usable.  Two threads racing through the first call both run the idempotent
    // set-up below and store the same value.
    static std::atomic<int> ready{0};
    if (ready.load(std::memory_order_acquire) == 0) {
        // the kernel addresses its V table as "LDS offset 0": that holds only while it has
        // no static LDS in front of the dynamic block
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
    return a.gqa <= 8 ? launch_kernel<VBW, VST, true>(a, st) : launch_kernel<VBW, VST, false>(a, st);
}

}  // namespace

#ifdef BGTQ_TRACE
extern "C" int bgtq_debug_set_trace(void* buf) {
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(g_trace), &buf, sizeof(buf));
}
#endif

int bgtq_launch_decode_mfma(const DecodeArgs& a, hipStream_t stream) {
    // layout requirements of the fast path; anything else takes the generic kernel
    if (a.gqa > 16 || !(a.scale > 0.f)) return BGTQ_EUNSUPPORTED;
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
