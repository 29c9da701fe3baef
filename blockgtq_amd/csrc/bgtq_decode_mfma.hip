// MFMA decode attention over packed K and V records (gfx950).
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
// more often than none).  A unit costs one raw read, four {bit-field extract,
// shift-add, table read} triples and yields the eight fp16 operands of one MFMA
// k-group.
//
// QK^T:  v_mfma_f32_16x16x32_f16, A = dequantised K (row = token, lane group g
//        supplies unit g of step m; field width, table and norm column come from the
//        plan's step table per lane group), B = rotated queries per step, gathered
//        once per work-group into LDS (zero on padding dims).  Every table word is
//        multiplied by the fp16 norm of its own segment before the MFMA and enters it as
//        the rounded fp16 product plus its exact rounding error (a second MFMA), which
//        keeps the scores at fp32 accuracy; a step may therefore mix units of several
//        segments and the steps of a token block accumulate in the MFMA itself.
// PV:    the D layout of a 16-token block is the A layout of the value product
//        (row = head, lane group g holds 4 tokens), so P never leaves its lane.  With
//        at most 8 query heads the product runs over (token, dim parity) pairs and a
//        V table word is an MFMA operand as it comes; with 9..16 heads V words are
//        transposed with v_perm_b32.  The V norm is folded into P in fp32 before P is
//        rounded to fp16.
// Softmax: exponentials are taken relative to a per-head reference that is kept
//        above every score seen so far.  It is only moved (to the new maximum
//        plus a headroom of 4 in log2 units) when a score of the tile exceeds it;
//        otherwise the tile needs no cross-lane traffic at all.
#include <atomic>

#include "bgtq_decode.h"

namespace {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) uint8_t* lds_ptr_t;

constexpr int D = BGTQ_D;
constexpr int MT = 64;             // tokens per wave tile = 4 MFMA row blocks
constexpr int MAX_STEPS = BGTQ_MAX_STEPS;
constexpr int MAX_WAVES = 12;
constexpr int MAX_KN = 8;          // norm columns per token row
constexpr int LDS_LIMIT = 160 * 1024;
constexpr int MERGE_STRIDE = BGTQ_D + 8;   // most floats from one row of a wave's result to the next in the merge area
constexpr float REFRESH = 4.0f;    // log2 headroom put above the largest score when the reference is refreshed

// ---- LDS layout (bytes) -----------------------------------------------------------
// [ V pair table | K tables of the record layout in use | step table | query operands | per wave: K tile + K norms
//   + V norms, V tile, fp32 V norms ]
constexpr int VTAB_BYTES = BGTQ_VLUT_BYTES;
constexpr int KTAB_BYTES = BGTQ_LUT_IMAGE_BYTES;
constexpr int STEPTAB_OFF = VTAB_BYTES + KTAB_BYTES;            // [step][lane group] x 32 B
constexpr int QB_OFF = STEPTAB_OFF + MAX_STEPS * 4 * 32;        // [step][lane] x 16 B: the MFMA B operand
constexpr int WAVES_OFF = QB_OFF + MAX_STEPS * 1024;

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
constexpr int VNF_BYTES = MT * 4;      // fp32 V norms of the tile, per wave

// (a & mask) | c in one instruction; the mask travels in a scalar register
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t c) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(c));
    return r;
}
// Both halves of a table word times the fp16 in the low half of n, as an unevaluated sum of two
// fp16 pairs: hi is the rounded product and lo the rounding error (a fused multiply-add returns it
// exactly), so hi + lo is the 22-bit product itself.
__device__ __forceinline__ void scale_pair(uint32_t w, uint32_t n, uint32_t& hi, uint32_t& lo) {
    asm("v_pk_mul_f16 %0, %1, %2 op_sel_hi:[1,0]" : "=v"(hi) : "v"(w), "v"(n));
    asm("v_pk_fma_f16 %0, %1, %2, %3 op_sel_hi:[1,0,1] neg_lo:[0,0,1] neg_hi:[0,0,1]" : "=v"(lo) : "v"(w), "v"(n), "v"(hi));
}

// Read through an absolute LDS address (the kernel has no static LDS, so the dynamic block
// starts at LDS address 0 and offsets into it are addresses).
template <class T>
__device__ __forceinline__ T lds_at(uint32_t addr) {
    return *(const __attribute__((address_space(3))) T*)(uintptr_t)addr;
}
template <class T>
__device__ __forceinline__ void lds_put(uint32_t addr, T v) {
    *(__attribute__((address_space(3))) T*)(uintptr_t)addr = v;
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
__device__ __forceinline__ DmaShape dma_shape(int total, uint32_t voff) {
    DmaShape d;
    d.nfull = ((total + 1023) >> 10) - 1;
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
    default: asm volatile("s_waitcnt vmcnt(24)" ::: "memory"); break;
    }
#undef BGTQ_WAIT_CASE
}

static_assert(offsetof(bgtq_head_plan, steptab) % 16 == 0 && offsetof(bgtq_head_plan, lut_image) % 16 == 0 &&
              offsetof(bgtq_head_plan, vlut_image) % 16 == 0 && (sizeof(uint32_t) * MAX_STEPS * 4 * 8) % 16 == 0 &&
              BGTQ_LUT_IMAGE_BYTES % 16 == 0 && BGTQ_VLUT_BYTES % 16 == 0,
              "plan tables are copied 16 bytes at a time");

// VBW: bits per V code; VST: bytes from one V record to the next (the record itself is
// 16 * VBW bytes; a padded stride keeps the rows of a tile on different LDS banks)
// DENSE: at most 8 query heads per KV head (a PV product that uses the eight spare head
// rows of the MFMA instead of transposing V)
template <int VBW, int VST, bool DENSE>
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
    constexpr uint32_t smem_lds = 0;                     // no static LDS: checked by the launcher

    // ---- this partition's tiles: the tiles of the row are dealt to the partitions as evenly as
    // whole tiles allow (partition sizes differ by at most one tile)
    const int T = a.seq_lens ? a.seq_lens[b] : a.T;
    const int n_tiles = (T + MT - 1) / MT;
    const int per = n_tiles / a.n_splits, rem = n_tiles - per * a.n_splits;
    const int tile_lo = c * per + min(c, rem), tile_hi = tile_lo + per + (c < rem ? 1 : 0);
    const int t0 = tile_lo * MT, t1 = min(tile_hi * MT, T);

    // ---- query operand, part 1: which dims unit (step, lane group) covers -> this thread's 16 bytes
    // of the rotated queries.  Thread i builds B operand (step i / 64, lane i % 64): head = column.
    const int krow = a.k_row_width;
    constexpr int vrow = VST;
    const int kn_st = (int)a.kn_st;
    const TileLayout tl = a.tl;
    const uint16_t* q_src = a.q + b * a.q_sb + (int64_t)h * gqa * a.q_sh;
    // Wave w builds the operand of step w (and w + nw, ... when there are fewer waves than steps):
    // the four descriptors of a step are wave-uniform, so they arrive through the scalar cache and
    // do not queue behind the copies below.
    uint32_t qd[4] = {0, 0, 0, 0};
    if (wave < MAX_STEPS) {
#pragma unroll
        for (int g = 0; g < 4; g++) qd[g] = P.steptab[kl][wave][g][7];
    }
    const int n_steps = min(P.n_steps[kl], MAX_STEPS);
    const int n_packed = min(P.n_packed_steps[kl], n_steps);   // raw-byte steps come last
    auto load_q = [&](uint32_t dsc, uint32_t (&w)[4]) {
        const int col = DENSE ? (li & 7) : li;
        const int d0 = (int)(dsc & 0xFF), len = (int)(dsc >> 8);
#pragma unroll
        for (int pp = 0; pp < 4; pp++) w[pp] = 0;
        if (col < gqa && len > 0) {
            const uint32_t* row = (const uint32_t*)(q_src + col * a.q_sh + d0);      // d0 is even
#pragma unroll
            for (int pp = 0; pp < 4; pp++)
                w[pp] = row[min(pp, (D - d0) / 2 - 1)] &
                        ((2 * pp < len ? 0xFFFFu : 0u) | (2 * pp + 1 < len ? 0xFFFF0000u : 0u));
        }
    };

    // ---- tables by DMA: V table at LDS offset 0, K tables behind it, then the step table; the chunks
    // are dealt round-robin to the waves
    const uint32_t voff = (uint32_t)lane * 16;
    {
        const uint8_t* vimg = (const uint8_t*)P.vlut_image[vnib ? 1 : 0];
        const uint8_t* kimg_src = (const uint8_t*)P.lut_image[kl];
        const uint8_t* st_src = (const uint8_t*)&P.steptab[kl][0][0][0];
        const int vbytes = vlut_bytes(VBW, vnib), kbytes = kimg_bytes(kl);
        const int vch = (vbytes + 1023) >> 10, kch = (kbytes + 1023) >> 10;
        for (int cc = wave; cc < vch + kch + 1; cc += nw) {
            const uint8_t* src;
            uint32_t dst;
            int left;
            if (cc < vch) { src = vimg + cc * 1024; dst = cc * 1024; left = vbytes - cc * 1024; }
            else if (cc < vch + kch) { src = kimg_src + (cc - vch) * 1024; dst = VTAB_BYTES + (cc - vch) * 1024; left = kbytes - (cc - vch) * 1024; }
            else { src = st_src; dst = STEPTAB_OFF; left = MAX_STEPS * 4 * 32; }
            dma16(voff, src, __builtin_amdgcn_readfirstlane(smem_lds + dst), __builtin_amdgcn_ballot_w64((int)voff < left));
        }
    }

    // ---- per-wave buffers and streaming sources: 16-byte aligned bases and phases (constant per tile) ----
    const uint32_t kbuf = WAVES_OFF + wave * tl.kbuf;                          // K records, K norms, V norms
    const uint32_t vbuf = WAVES_OFF + nw * tl.kbuf + wave * (tl.vt + VNF_BYTES); // V records, then fp32 V norms
    const uint32_t vnf = vbuf + tl.vt;
    const uint8_t* kp_base = a.kp + b * a.kp_sb + h * a.kp_sh;
    const uint8_t* vp_base = a.vp + b * a.vp_sb + h * a.vp_sh;
    const uint8_t* kn_base = (const uint8_t*)(a.kn + b * a.kn_sb + h * a.kn_sh);
    const uint8_t* vn_base = (const uint8_t*)(a.vn + b * a.vn_sb + h * a.vn_sh);
    const uint32_t kph = (uint32_t)((uintptr_t)kp_base & 15), vph = (uint32_t)((uintptr_t)vp_base & 15);
    const uint32_t knph = (uint32_t)((uintptr_t)kn_base & 15), vnph = (uint32_t)((uintptr_t)vn_base & 15);
    // The shapes of a full tile are the same for every tile of the partition.
    const DmaShape full_k = dma_shape((int)kph + MT * krow, voff), full_kn = dma_shape((int)knph + MT * kn_st * 2, voff);
    const DmaShape full_vn = dma_shape((int)vnph + MT * 2, voff), full_v = dma_shape((int)vph + MT * vrow, voff);
    // K records and both norm arrays of a tile go to the K buffer; returns the loads issued.
    auto issue_k = [&](int tile) -> int {
        const int nt = min(MT, t1 - tile);
        DmaShape sk = full_k, sn = full_kn, sv = full_vn;
        if (nt < MT) {
            sk = dma_shape((int)kph + nt * krow, voff);
            sn = dma_shape((int)knph + nt * kn_st * 2, voff);
            sv = dma_shape((int)vnph + nt * 2, voff);
        }
        dma_region<9>(kp_base - kph + (int64_t)tile * krow, kbuf, sk, voff);
        dma_region<2>(kn_base - knph + (int64_t)tile * kn_st * 2, kbuf + tl.kt, sn, voff);
        dma_region<1>(vn_base - vnph + (int64_t)tile * 2, kbuf + tl.kt + tl.knr, sv, voff);
        return sk.nfull + sn.nfull + sv.nfull + 3;
    };
    auto issue_v = [&](int tile) -> int {
        const int nt = min(MT, t1 - tile);
        DmaShape sv = full_v;
        if (nt < MT) sv = dma_shape((int)vph + nt * vrow, voff);
        dma_region<5>(vp_base - vph + (int64_t)tile * vrow, vbuf, sv, voff);
        return sv.nfull + 1;
    };
    const int step_tiles = nw * MT;
    int tile = t0 + wave * MT;
    int v_loads = 0;                 // loads of the V tile issued after the current K tile
    if (tile < t1) issue_k(tile);

    // ---- query operand, part 2: rows of the rotated queries straight from memory, cut to the dims
    // of the unit (the wait for them also covers the tables and the first K tile: all are needed now)
    for (int m = wave; m < MAX_STEPS; m += nw) {
        uint32_t dsc;
        if (m == wave) dsc = lg == 0 ? qd[0] : lg == 1 ? qd[1] : lg == 2 ? qd[2] : qd[3];
        else dsc = P.steptab[kl][m][lg][7];
        uint32_t w[4];
        load_q(dsc, w);
        lds_put<uint4v>(QB_OFF + m * 1024 + lane * 16, (uint4v){w[0], w[1], w[2], w[3]});
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // waves without a step to build wait for their copies here
    if (tile < t1) v_loads = issue_v(tile);
    __syncthreads();

    const float c2 = a.scale * 1.44269504088896340736f;      // logits go through exp2
    const uint32_t lane4 = (uint32_t)lane * 4;
    // V table replica of this lane (the table sits at LDS address 0, so field bits OR-ed in never
    // meet the base); the 256-entry tables are not replicated
    constexpr bool V_UNREP = VBW == 4;                        // also every nibble record (VBW 4 by construction)
    const uint32_t vbank = V_UNREP ? 0u : (lane4 & 124u);
    constexpr int vshift = V_UNREP ? 2 : 7;
    const uint32_t kstride = 16u * krow;
    const uint32_t krow0 = kbuf + kph + (uint32_t)li * krow;                 // record of token li of block 0
    const uint32_t knrow0 = kbuf + tl.kt + knph + (uint32_t)li * kn_st * 2;  // its norm row
    const uint32_t vc = vph + (uint32_t)li * VBW;
    const uint32_t vbase = vbuf + (vc & ~3u) + (uint32_t)lg * 4 * vrow, v_sh = vc & 3u;
    const uint32_t stl = STEPTAB_OFF + lg * 32;
    const uint32_t qbl = QB_OFF + lane * 16;

    float m_ref = -INFINITY;        // reference of head li, in exp2 units; never below a score seen
    float l_part = 0.f;             // this lane's share of the softmax denominator
    constexpr int NACC = DENSE ? 4 : 8;         // output accumulators (16 x 16 each)
    float4v acc[NACC];
#pragma unroll
    for (int e = 0; e < NACC; e++) acc[e] = (float4v){0, 0, 0, 0};

    for (; tile < t1; tile += step_tiles) {
        const int nt = min(MT, t1 - tile);
        const bool more = tile + step_tiles < t1;
        wait_loads(v_loads);                                 // K records and norms of this tile are in LDS
        __builtin_amdgcn_wave_barrier();
        // fp32 V norms of the tile (lane = token), 0 past the end
        {
            const uint16_t vraw = lds_at<uint16_t>(kbuf + tl.kt + tl.knr + vnph + lane * 2);
            lds_put<float>(vnf + lane * 4, lane < nt ? bgtq_h2f(vraw) : 0.f);
        }

        // ---- scores ---------------------------------------------------------------
        float4v S[4];
#pragma unroll
        for (int k = 0; k < 4; k++) S[k] = (float4v){0, 0, 0, 0};
        {
            // Software pipeline over the packed steps.  The iteration that multiplies step m first
            // forms the table addresses of step m+1 (from raw codes and parameters read one
            // iteration earlier), multiplies step m, then fetches the parameters of step m+2, its raw
            // codes and norms (through offsets read one iteration earlier still) and last the table
            // words of step m+1.  Every LDS read is consumed one iteration after it was issued.
            const int last = n_packed - 1;
            uint4v e0, e1;                                  // parameters of the step whose addresses are formed next
            uint32_t xo, no;                                // record and norm offsets of the step fetched next
            uint32_t rlo[4], rhi[4], nrm[4], ncur[4];
            uint32_t ad[4][4];
            uint4v w[4];
            half8 Q;
            auto params = [&](int m) {
                const uint32_t at = stl + (uint32_t)min(m, last) * 128;
                e0 = lds_at<uint4v>(at);
                e1 = lds_at<uint4v>(at + 16);
            };
            auto offsets = [&](int m) {
                const uint32_t at = stl + (uint32_t)min(m, last) * 128;
                xo = lds_at<uint32_t>(at);
                no = lds_at<uint32_t>(at + 24);
            };
            auto raws = [&](uint32_t xoff, uint32_t noff) {
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const uint32_t at = krow0 + xoff + k * kstride;
                    rlo[k] = lds_at<uint32_t>(at);
                    rhi[k] = lds_at<uint32_t>(at + 4);
                    nrm[k] = lds_at<uint16_t>(knrow0 + noff + k * (32u * kn_st));
                }
            };
            auto addresses = [&]() {                        // bit fields -> table addresses
                const uint32_t lb = (lane4 & e0.w) + e0.z;
                const uint32_t pw = e1.x, pw2 = pw * 2, pw3 = pw * 3, tsh = e1.y;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const uint32_t raw = __builtin_amdgcn_alignbyte(rhi[k], rlo[k], e0.y);
                    ad[k][0] = (__builtin_amdgcn_ubfe(raw, 0, pw) << tsh) + lb;
                    ad[k][1] = (__builtin_amdgcn_ubfe(raw, pw, pw) << tsh) + lb;
                    ad[k][2] = (__builtin_amdgcn_ubfe(raw, pw2, pw) << tsh) + lb;
                    ad[k][3] = (__builtin_amdgcn_ubfe(raw, pw3, pw) << tsh) + lb;
                }
            };
            auto tables = [&](int m) {                      // table words and the query operand of step m
                Q = lds_at<half8>(qbl + (uint32_t)m * 1024);
#pragma unroll
                for (int k = 0; k < 4; k++)
                    w[k] = (uint4v){lds_at<uint32_t>(ad[k][0]), lds_at<uint32_t>(ad[k][1]),
                                   lds_at<uint32_t>(ad[k][2]), lds_at<uint32_t>(ad[k][3])};
            };
            auto multiply = [&]() {                         // table words times their segment's norm, then the MFMAs
                uint4v x[4], y[4];
#pragma unroll
                for (int k = 0; k < 4; k++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        uint32_t hi, lo;
                        scale_pair(w[k][i], ncur[k], hi, lo);
                        x[k][i] = hi;
                        y[k][i] = lo;
                    }
#pragma unroll
                for (int k = 0; k < 4; k++)
                    S[k] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, x[k]), Q, S[k], 0, 0, 0);
#pragma unroll
                for (int k = 0; k < 4; k++)
                    S[k] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, y[k]), Q, S[k], 0, 0, 0);
            };
            auto latch_norms = [&]() {
#pragma unroll
                for (int k = 0; k < 4; k++) ncur[k] = nrm[k];
            };
            if (n_packed > 0) {
                params(0);
                offsets(1);
                const uint32_t x1 = xo, n1 = no;
                offsets(2);
                raws(e0.x, e1.z);                           // step 0
                addresses();
                latch_norms();
                __builtin_amdgcn_sched_barrier(0);
                params(1);
                raws(x1, n1);                               // step 1
                __builtin_amdgcn_sched_barrier(0);
                tables(0);
                for (int m = 0; m < last; m++) {
                    __builtin_amdgcn_sched_barrier(0);
                    addresses();                            // step m+1
                    __builtin_amdgcn_sched_barrier(0);
                    multiply();                             // step m
                    latch_norms();                          // norms of step m+1
                    __builtin_amdgcn_sched_barrier(0);
                    params(m + 2);
                    raws(xo, no);                           // step m+2
                    offsets(m + 3);
                    __builtin_amdgcn_sched_barrier(0);
                    tables(m + 1);
                }
                __builtin_amdgcn_sched_barrier(0);
                multiply();
            }
            // raw-byte steps (codes of 5..8 bits): one table read per code
            for (int m = n_packed; m < n_steps; m++) {
                const uint4v f0 = lds_at<uint4v>(stl + m * 128), f1 = lds_at<uint4v>(stl + m * 128 + 16);
                const half8 Qr = lds_at<half8>(qbl + (uint32_t)m * 1024);
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const uint32_t at = krow0 + f0.x + k * kstride;
                    const uint32_t lo = lds_at<uint32_t>(at), hi = lds_at<uint32_t>(at + 4), hi2 = lds_at<uint32_t>(at + 8);
                    const uint32_t n16 = lds_at<uint16_t>(knrow0 + f1.z + k * (16u * kn_st * 2));
                    const uint32_t r0 = __builtin_amdgcn_alignbyte(hi, lo, f0.y);
                    const uint32_t r1 = __builtin_amdgcn_alignbyte(hi2, hi, f0.y);
                    uint4v x, y;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const uint32_t r = e < 2 ? r0 : r1;
                        const uint32_t b0 = (r >> ((e & 1) * 16)) & 0xFF, b1 = (r >> ((e & 1) * 16 + 8)) & 0xFF;
                        const uint32_t c0 = lds_at<uint16_t>(f0.z + b0 * 2), c1 = lds_at<uint16_t>(f0.z + b1 * 2);
                        uint32_t hi, lo;
                        scale_pair(c0 | (c1 << 16), n16, hi, lo);
                        x[e] = hi;
                        y[e] = lo;
                    }
                    S[k] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, x), Qr, S[k], 0, 0, 0);
                    S[k] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, y), Qr, S[k], 0, 0, 0);
                }
            }
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        int k_loads = 0;
        if (more) k_loads = issue_k(tile + step_tiles);      // all reads of the K buffer are done

        // ---- online softmax: lane (head li, group lg) holds tokens 16k + 4lg + r ------
        if (nt < MT) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int tk = (r >> 2) * 16 + lg * 4 + (r & 3);
                if (tk >= nt) S[r >> 2][r & 3] = -INFINITY;
            }
        }
        float mx = S[0][0];
#pragma unroll
        for (int r = 1; r < 16; r++) mx = fmaxf(mx, S[r >> 2][r & 3]);
        mx *= c2;
        if (__builtin_amdgcn_ballot_w64(mx > m_ref)) {    // wave-uniform, rare after the first tiles
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m_ref, mx + REFRESH);
            const float alpha = (m_ref == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_ref - m_new);
            // acc rows are columns 4lg+r (head (4lg + r) & 7 where columns 8..15 repeat heads 0..7), not
            // this lane's: fetch their factors
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
            for (int k = 0; k < 4; k++) {
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
                if (k + 1 < 4) {
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
            // values, 9..16 heads: lane (j = li, group lg) decodes unit j of its 8 tokens per half
            // tile.  Raw codes are fetched one half ahead; the exponentials run while the table
            // reads fly.
            uint32_t vlo[8], vhi[8];
#pragma unroll
            for (int r = 0; r < 8; r++) {
                const int tk = (r >> 2) * 16 + (r & 3);                       // + 4lg, folded into vbase
                vlo[r] = lds_at<uint32_t>(vbase + (uint32_t)tk * vrow);
                vhi[r] = lds_at<uint32_t>(vbase + (uint32_t)tk * vrow + 4);
            }
#pragma unroll
            for (int half = 0; half < 2; half++) {
                const float4v vn_lo = lds_at<float4v>(vnf + (half * 32 + lg * 4) * 4);        // tokens 4lg .. 4lg+3
                const float4v vn_hi = lds_at<float4v>(vnf + (half * 32 + 16 + lg * 4) * 4);   // tokens 16+4lg ..
                uint32_t W[8][4];
#pragma unroll
                for (int r = 0; r < 8; r++) {
                    const uint32_t raw = __builtin_amdgcn_alignbyte(vhi[r], vlo[r], v_sh);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        constexpr uint32_t fmask = ((1u << (2 * VBW)) - 1u) << vshift;
                        const int fp = e * 2 * VBW;
                        const uint32_t sh = fp <= vshift ? raw << (vshift - fp) : raw >> (fp - vshift);
                        W[r][e] = lds_at<uint32_t>(and_or(sh, fmask, vbank));
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                if (half + 1 < 2) {
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
    }

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
}

// LDS bytes of a work-group of nw waves
size_t mfma_smem_bytes(const TileLayout& tl, int nw) {
    size_t need = (size_t)WAVES_OFF + (size_t)nw * (tl.kbuf + tl.vt + VNF_BYTES);
    size_t merge = (size_t)nw * (32 + 16 * MERGE_STRIDE) * 4;
    return need > merge ? need : merge;
}

template <int VBW, int VST, bool DENSE>
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
    auto kern = decode_mfma_kernel<VBW, VST, DENSE>;
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
    return a.gqa <= 8 ? launch_kernel<VBW, VST, true>(a, st) : launch_kernel<VBW, VST, false>(a, st);
}

}  // namespace

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
