/*
 * bgtq.h - C ABI of the MI355X packed-KV decode path of Block-GTQ.
 *
 * One shared library (libbgtq.so, built from blockgtq_amd/csrc for gfx950)
 * exports the entry points below.  Every pointer is a plain device pointer
 * unless stated otherwise, every stride is in ELEMENTS of the pointed-to type,
 * `stream` is a hipStream_t passed as void*, and every function returns 0 on
 * success or a negative BGTQ_E* code / positive hipError_t.  Nothing in here
 * allocates or frees device memory and nothing throws.
 *
 * The reference has no FFI: its device code is Triton launched from Python.
 * Each entry point therefore cites the Python/Triton function whose launch it
 * replaces (paths relative to the reference checkout).
 */
#ifndef BGTQ_H
#define BGTQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BGTQ_HEAD_DIM      128   /* the only head width the kernels are built for */
#define BGTQ_MAX_SEGMENTS  8     /* distinct K bit widths per head */
#define BGTQ_MAX_CENTROIDS 256   /* 8-bit codebook */
#define BGTQ_LUT_BINS      256
#define BGTQ_MAX_GQA       16    /* query heads per KV head */
#define BGTQ_MAX_SPLITS    512   /* FlashDecoding partitions per (batch, KV head) */
#define BGTQ_STATIC_SCRATCH_BYTES (8u << 20)  /* partition results of bgtq_decode_attend_static */
#define BGTQ_ROT_COL       48    /* longest rotated segment that bgtq_head_plan.k_rot_cols holds */
#define BGTQ_MAX_WALK      12    /* steps of the decode kernel's walk over one K record, see bgtq_head_plan.swalk */
#define BGTQ_STEP_RAW      32    /* first step kind of raw-byte runs */
#define BGTQ_STEP_RAW5     40    /* first step kind of raw-byte runs of 5-bit codes, read in pairs through the table at BGTQ_LUT_K5P */
#define BGTQ_MAX_UNITS     24    /* 8-dim units of one K record, see bgtq_head_plan.kunit */
/* byte offsets inside bgtq_head_plan.lut_image[BGTQ_K_BITPACKED] (= offsets in the decode kernel's table area) */
/* (every pair table starts on a multiple of its own size in the kernel's table area, which puts the K image
 * at offset BGTQ_VLUT_BYTES: an entry address is then the table offset OR-ed with the entry's index bits) */
#define BGTQ_LUT_K3      0                       /* 64 entries  x 32 replicas */
#define BGTQ_LUT_K2      8192                    /* 16 entries  x 32 replicas */
#define BGTQ_LUT_K4      10240                   /* 256 entries, not replicated */
#define BGTQ_LUT_K1      11264                   /* 4 entries   x 32 replicas */
#define BGTQ_LUT_KRAW    11776                   /* 4 tables x 256 fp16       */
#define BGTQ_LUT_KEND    13824                   /* end of the K tables       */
/* the same for lut_image[BGTQ_K_MIXED]: up to 4 byte-indexed tables of 256 entries, then the raw tables */
#define BGTQ_LUTM_K0     0
#define BGTQ_LUTM_KRAW   4096
#define BGTQ_LUTM_KEND   6144
#define BGTQ_LUT_K5P     13824                   /* either image: 1024 entries (c0 | c1 << 5) for the 5-bit codebook, not
                                                  * replicated; present when n_walk[2 + layout] is non-zero */
#define BGTQ_LUT_K5PEND  17920
/* bit-packed image only, for the decode kernel: four codes per entry (index c0 | c1 << bw | c2 << 2 bw | c3 << 3 bw,
 * 8 bytes = their four fp16 centroids), not replicated: 16 entries of 1-bit codes (every entry on a bank pair of its
 * own) and 256 entries of 2-bit codes (on a multiple of its size in the kernel's table area) */
#define BGTQ_LUT_K1Q     17920
#define BGTQ_LUT_K2Q     18432
#define BGTQ_LUT_IMAGE_BYTES 20480               /* room for either K image */
/* how a segment's units are unpacked */
#define BGTQ_PATH_B1     1   /* bit-packed 1-bit codes: a unit is 1 byte, pair table of 4 entries x 32 replicas */
#define BGTQ_PATH_B2     2   /* bit-packed 2-bit codes: 2 bytes, 16 entries x 32 replicas */
#define BGTQ_PATH_B3     3   /* bit-packed 3-bit codes: 3 bytes, 64 entries x 32 replicas */
#define BGTQ_PATH_BYTE   4   /* a byte holds a code pair as nibbles: 4 bytes, 256-entry table indexed by the byte */
#define BGTQ_PATH_RAW    5   /* one byte per code: 8 bytes, 256 single fp16 entries */
#define BGTQ_VLUT_BYTES  8192                    /* a V pair table: 64 entries x 32 replicas at most */

/* error codes (negative); positive return values are hipError_t */
#define BGTQ_OK            0
#define BGTQ_EINVAL       -1     /* bad argument (null pointer, shape, stride, flag) */
#define BGTQ_EUNSUPPORTED -2     /* legal in the reference but not built here */
#define BGTQ_ELIMIT       -3     /* size beyond a documented maximum */

/* K record layouts (blockgtq/quantizer.py:34-102 and :1930-1951) */
#define BGTQ_K_BITPACKED   0     /* [1b|2b|3b|4b segments bit-packed|5..8b raw], raw group norms */
#define BGTQ_K_MIXED       1     /* [bw<=4 dims as nibbles | bw>=5 raw], corrected norms */
/* V record layouts (blockgtq/v_packing.py:17-28, blockgtq/quantizer.py:2096-2099) */
#define BGTQ_V_BITPACKED   0     /* v_bits per code, LSB first */
#define BGTQ_V_NIBBLE      1     /* 4 bits per code whatever v_bits is */
/* K scalar quantisation rule */
#define BGTQ_QUANT_LUT256  0     /* 256-bin table, blockgtq/quantizer.py:841-850 */
#define BGTQ_QUANT_EXACT   1     /* count of boundaries below y, blockgtq/block_gtq_pipeline.py:337-341 */

/*
 * Static per-(layer, KV head) plan.  Built once on the host from the
 * calibrated quantizer (blockgtq/quantizer.py:1024-1148 and :1478-1497) and
 * uploaded as an array of n_kv structs per layer.  All dim indices are in
 * "packed order": coordinates sorted by ascending bit width, the two
 * coordinates of a RoPE block adjacent (blockgtq/block_gtq_pipeline.py:161-177).
 */
typedef struct bgtq_head_plan {
    /* K segment table: one segment == one bit width == one norm group */
    int32_t  n_seg;                             /* 0..BGTQ_MAX_SEGMENTS */
    int32_t  n_zero_dims;                       /* leading dims that got 0 bits */
    int32_t  k_row_bytes;                       /* BGTQ_K_BITPACKED record length */
    int32_t  k_mixed_bytes;                     /* BGTQ_K_MIXED record length */
    int32_t  nopack_start;                      /* first dim with bw >= 5, HEAD_DIM if none */
    int32_t  nopack_len;
    int32_t  v_bits;                            /* 1..4 */
    int32_t  reserved0;
    int32_t  seg_bw[BGTQ_MAX_SEGMENTS];
    int32_t  seg_start[BGTQ_MAX_SEGMENTS];      /* first dim of the segment */
    int32_t  seg_len[BGTQ_MAX_SEGMENTS];        /* dims in the segment (even) */
    int32_t  seg_pack_off[BGTQ_MAX_SEGMENTS];   /* byte offset, BGTQ_K_BITPACKED */
    int32_t  seg_mixed_off[BGTQ_MAX_SEGMENTS];  /* byte offset, BGTQ_K_MIXED */
    int32_t  seg_identity[BGTQ_MAX_SEGMENTS];   /* 1: rotation block is the identity */
    /* K encode tables */
    int32_t  head_perm[BGTQ_HEAD_DIM];          /* packed dim -> original coordinate */
    int32_t  group_of[BGTQ_HEAD_DIM];           /* packed dim -> segment, -1 for 0-bit dims */
    float    lut_offset[BGTQ_HEAD_DIM];
    float    lut_inv_scale[BGTQ_HEAD_DIM];
    uint8_t  code_lut[BGTQ_MAX_SEGMENTS][BGTQ_LUT_BINS];
    float    k_centroids[BGTQ_MAX_SEGMENTS][BGTQ_MAX_CENTROIDS];
    float    k_boundaries[BGTQ_MAX_SEGMENTS][BGTQ_MAX_CENTROIDS]; /* 2^bw-1 valid, +inf after */
    uint16_t k_codebook_f16[BGTQ_MAX_SEGMENTS][BGTQ_MAX_CENTROIDS];
    float    k_rot_T[BGTQ_HEAD_DIM * BGTQ_HEAD_DIM];  /* y = xhat @ k_rot_T, block diagonal */
    /* the same rotation by columns, each cut down to its own diagonal block: k_rot_cols[j][i] =
     * k_rot_T[(start of j's segment + i) * 128 + j], 0 past the segment's end.  Filled (rot_compact[0] = 1)
     * when no rotated segment is longer than BGTQ_ROT_COL dims: the single-row append reads a dim's
     * column from here without knowing the segment table first */
    float    k_rot_cols[BGTQ_HEAD_DIM][BGTQ_ROT_COL];
    int32_t  rot_compact[4];                    /* [0]: k_rot_cols is filled; rest padding */
    /* what the K encoder's thread j needs, ready-made: as owner of packed dim j
     * enc_dim[j] = { segment of the dim (-1: a 0-bit dim), first dim of that segment, one past its
     * last, seg_identity | head_perm[j] << 8 }, and as writer of record byte j (one table per K layout)
     * enc_byte[l][j] = { mode | code width << 2 | skip << 6 | n << 8, first code }: mode 0 writes 0,
     * mode 1 the byte of the LSB-first stream that holds the n codes from `first code` on, less the
     * `skip` low bits that belong to the byte before, mode 2 the code itself */
    int32_t  enc_dim[BGTQ_HEAD_DIM][4];
    uint32_t enc_byte[2][BGTQ_HEAD_DIM][2];
    /* V tables */
    float    v_centroids[16];
    float    v_boundaries[16];                  /* 2^v_bits-1 valid, +inf after */
    uint16_t v_lut_f16[16];
    float    v_rot_T[BGTQ_HEAD_DIM * BGTQ_HEAD_DIM];  /* encode: y = vhat @ v_rot_T */
    float    v_rot[BGTQ_HEAD_DIM * BGTQ_HEAD_DIM];    /* decode: out = acc @ v_rot */
    /* v_rot_T once more, four rows interleaved: v_rot_T4[q][j][c] = v_rot_T[(4 q + c) * 128 + j], so that
     * the single-row append's thread j reads its column with 32 loads of 16 bytes that are contiguous
     * across the threads */
    float    v_rot_T4[BGTQ_HEAD_DIM / 4][BGTQ_HEAD_DIM][4];
    /* what the V encoder's thread j needs as writer of record byte j (one table per V layout), in the
     * format of enc_byte */
    uint32_t enc_vbyte[2][BGTQ_HEAD_DIM / 2][2];
    /*
     * Decode schedule of the K record for the MFMA attention kernel, one per K
     * layout (index BGTQ_K_BITPACKED / BGTQ_K_MIXED).  A "unit" is 8 consecutive
     * packed dims of one segment (zero padded at the segment's end); the kernel
     * walks the units in order, every lane decoding the unit of its own token,
     * accumulates the units of a segment in the MFMA and scales the segment's sum
     * by the token's norm of that segment.  Units of segments with codes of at most
     * 4 bits (two codes select one pair-table entry) come first, n_pair_units[l] of
     * them, an even number: an empty unit (kunit 0, parameters 0) is inserted where the
     * count would be odd; the others take one byte and one table read per code.
     * kprog[l][u] (32 bytes, read by every lane as it is):
     *   [0..3] pair units: right-rotation that brings code pair 0..3 of the unit (8
     *       codes, little-endian bit stream) to the bit position of the table's entry index
     *   [4] mask of the entry index at that position
     *   [5] byte offset of the segment's table from the start of the kernel's table
     *       area: BGTQ_VLUT_BYTES + offset inside lut_image[l]
     *   [6] bank-replica mask (lane * 4 & mask selects the replica; 0: not replicated)
     *   [7] byte offset in the record of the unit after the next (0 if there is none;
     *       units 0 and 1 start at kfirst[l][0..1])
     * kend[l]: bit u set = unit u is the last of its segment.
     * kunit[l][u] = first packed dim of unit u | number of real dims (1..8) << 8, units
     * numbered through the segments in order; 0 past the last unit.
     *
     * lut_image[l]: pair tables, entry (c0 | c1 << bw) = fp16 centroid pair (c0 in the
     * low half).  Bit-packed layout: bw 1..3 at BGTQ_LUT_K1/K2/K3 with every entry
     * replicated over 32 consecutive dwords (the 32 lanes of a half-wave then read 32
     * different LDS banks whatever their codes), bw 4 at BGTQ_LUT_K4 unreplicated
     * (fewer bank collisions than 8 or 16 replicas give); raw tables of 256 single fp16
     * entries (0 beyond 2^bw) at BGTQ_LUT_KRAW + (bw - 5) * 512.  Mixed layout: a pair of
     * codes is one byte, so the i-th packed segment has its own 256-entry table indexed by
     * that byte at BGTQ_LUTM_K0 + i * 1024 (0 where a nibble is not a code of the segment),
     * raw tables at BGTQ_LUTM_KRAW + (bw - 5) * 512.
     * vlut_image[v]: V pair table for V layout v (BGTQ_V_BITPACKED: entry (c0 | c1 <<
     * v_bits), 32 replicas for v_bits <= 3, unreplicated for 4; BGTQ_V_NIBBLE: 256
     * byte-indexed entries, unreplicated).
     */
    int32_t  n_units[2];
    int32_t  n_pair_units[2];
    uint32_t kend[2];
    uint32_t kfirst[2][2];
    uint32_t reserved1[2];
    uint32_t kprog[2][BGTQ_MAX_UNITS][8];
    uint32_t kunit[2][BGTQ_MAX_UNITS];
    /*
     * The same K record as the decode attention kernel walks it, step by step (one walk per K
     * layout).  A step is a run of 1..8 units (8 consecutive packed dims each, the last unit of a
     * segment may hold fewer) of one segment; a segment of more than 8 units is cut into several
     * steps that name the same norm column.  swalk[l][i] = {
     *   (byte offset of the run in the record & 3) | step kind << 2,
     *   byte offset of the segment's table in the kernel's table area (BGTQ_VLUT_BYTES + offset
     *   inside lut_image[l]),
     *   (byte offset of the run & ~3) | norm column * 2 << 8 | index of the run's first unit * 16 << 16,
     *   0 }
     * with step kind = (w - 1) * 8 + (units - 1) for codes read through pair tables (w = 1..3:
     * bit-packed codes of w bits; w = 4: a byte holds a code pair as nibbles, which is every
     * segment of up to 4 bits in BGTQ_K_MIXED), BGTQ_STEP_RAW5 + (units - 1) for 5-bit codes stored one
     * per byte and BGTQ_STEP_RAW + (units - 1) for wider codes stored one per byte.  n_walk[l] steps;
     * all zero past the last (the decode kernel counts the steps by their table word, which is never
     * zero for a step in use, and copies all BGTQ_LUT_IMAGE_BYTES of lut_image[l]).
     * sunit[l][u] = first packed dim of unit u | number of real dims (1..8) << 8, units numbered
     * through the segments in order with no empty units between them; 0 past the last unit.
     */
    uint32_t swalk[2][BGTQ_MAX_WALK][4];
    uint32_t n_walk[4];                         /* [l]: steps of layout l; [2 + l]: 1 when lut_image[l] holds the 5-bit pair table */
    uint32_t sunit[2][BGTQ_MAX_UNITS];
    uint32_t lut_image[2][BGTQ_LUT_IMAGE_BYTES / 4];
    uint32_t vlut_image[2][BGTQ_VLUT_BYTES / 4];
} bgtq_head_plan;

/* sizeof(bgtq_head_plan) as the library was compiled; the host mirror checks it. */
size_t bgtq_plan_sizeof(void);

/* Library/ABI version, bumped whenever a signature or the plan struct changes. */
int bgtq_abi_version(void);

/* Revision of the decode-attention kernels' memory access pattern (tile shapes, what
 * is staged through LDS, partition scheme).  Figures measured on one revision, such as
 * HBM traffic per launch, are only quoted while the library reports the same number.
 * No counterpart in the reference. */
int bgtq_decode_kernel_revision(void);

/* Human-readable text for a return code of this library (static storage). */
const char* bgtq_strerror(int code);

/*
 * K encode + pack, all KV heads of one layer in one launch, written straight
 * into the cache slots.
 * Replaces _compress_pack_kernel_v8_batched (blockgtq/quantizer.py:713-990)
 * as driven by compress_k_packed_batched (:2105-2172) for BGTQ_K_BITPACKED and
 * by compress_k_mixed_batched (:1844-1976, nibble repack + norm correction)
 * for BGTQ_K_MIXED, plus the slice-assign cache writes of
 * blockgtq/packed_kv_manager.py:138-180 / blockgtq/production_cache.py:174-201.
 *
 *   plans      n_kv structs (device)
 *   k          fp16 [B][n_kv][S][128], strides k_sb/k_sh/k_ss in halves, dim contiguous
 *   k_packed   u8   [B][n_kv][T][row],  strides in bytes; record written at token
 *              t_pos[b] + s (t_pos device int32[B]) or t_pos_scalar + s when t_pos is NULL;
 *              bytes beyond the head's own record up to k_row_width are zeroed
 *   k_norms    fp16 [B][n_kv][T][norm_width], strides in halves; entries beyond the
 *              head's own n_seg up to norm_width are zeroed
 *   max_T      token capacity of the cache tensors.  With a host position the call is
 *              refused (BGTQ_ELIMIT) when t_pos_scalar + S > max_T, before anything is
 *              launched; with device positions a record whose position falls outside
 *              [0, max_T) is dropped by the kernel, so an append past the end never
 *              writes outside the cache (the reference's slice assignment raises there,
 *              blockgtq/packed_kv_manager.py:172-178)
 */
int bgtq_encode_k(const bgtq_head_plan* plans,
                  const void* k, int64_t k_sb, int64_t k_sh, int64_t k_ss,
                  int B, int n_kv, int S,
                  void* k_packed, int64_t kp_sb, int64_t kp_sh, int64_t kp_st, int k_row_width,
                  void* k_norms, int64_t kn_sb, int64_t kn_sh, int64_t kn_st, int norm_width,
                  const int32_t* t_pos, int t_pos_scalar, int max_T,
                  int k_layout, int quant_mode, void* stream);

/*
 * V encode + pack, all KV heads in one launch, written into the cache slots.
 * Replaces _compress_v_pack_kernel_batched (blockgtq/quantizer.py:518-706) as
 * driven by compress_v_packed_batched (:1980-2029) for BGTQ_V_BITPACKED and by
 * compress_v_nibble4_batched (:2033-2101) for BGTQ_V_NIBBLE.
 *   v_norms    fp16 [B][n_kv][T], corrected norm ||v|| / ||centroids[codes]||
 */
int bgtq_encode_v(const bgtq_head_plan* plans,
                  const void* v, int64_t v_sb, int64_t v_sh, int64_t v_ss,
                  int B, int n_kv, int S,
                  void* v_packed, int64_t vp_sb, int64_t vp_sh, int64_t vp_st, int v_row_width,
                  void* v_norms, int64_t vn_sb, int64_t vn_sh, int64_t vn_st,
                  const int32_t* t_pos, int t_pos_scalar, int max_T,
                  int v_layout, void* stream);

/*
 * Unpacked K codes + raw group norms (no packing), one head.
 * Replaces _compress_only_kernel (blockgtq/kernels/quant_kernels.py:471-565)
 * behind BlockGTQQuantizer.compress (blockgtq/quantizer.py:1246-1296).
 *   k      fp16 [N][128] contiguous
 *   codes  u8   [N][128] in packed order
 *   norms  fp32 [N][norm_width] raw group norms (corrected when `corrected` != 0)
 */
int bgtq_compress_k_codes(const bgtq_head_plan* plan, const void* k, int64_t N,
                          void* codes, float* norms, int norm_width,
                          int corrected, int quant_mode, void* stream);

/* Unpacked V codes + fp16 corrected norms, one head
 * (PolarQuantGPU.quantize + _corrected_v_norms, blockgtq/quantizer.py:1510-1541). */
int bgtq_compress_v_codes(const bgtq_head_plan* plan, const void* v, int64_t N,
                          void* codes, void* norms_f16, void* stream);

/*
 * Query permute + rotate into the packed K space, all query heads of a layer.
 * Replaces BlockGTQQuantizer.rotate_q_for_packed_kernel
 * (blockgtq/quantizer.py:1160-1187), called once per KV head per step by
 * blockgtq/production_cache.py:240-245.
 *   q      fp16 [n_rows][n_q][128], strides q_sr/q_sh in halves
 *   q_rot  fp16 [n_rows][n_q][128], strides likewise; n_q = n_kv * gqa
 */
int bgtq_rotate_q(const bgtq_head_plan* plans,
                  const void* q, int64_t q_sr, int64_t q_sh,
                  void* q_rot, int64_t qr_sr, int64_t qr_sh,
                  int n_rows, int n_kv, int gqa, void* stream);

/*
 * Decode-step preparation in ONE launch: append-encode the new K and V tokens
 * into their cache slots (as bgtq_encode_k / bgtq_encode_v) and rotate the
 * queries (as bgtq_rotate_q).  Results are identical to the three separate
 * calls.  Covers what one layer of a decode step does before attention in
 * BlockGTQKVManager.append_and_attend (blockgtq/packed_kv_manager.py:269-330:
 * _compress_and_store K, V, then rotate_q_for_packed_kernel per KV head) and in
 * BlockGTQProductionCache.encode_and_attend (blockgtq/production_cache.py:207-245).
 * Arguments have the meaning they have in those three entry points; q has
 * B rows of n_kv * gqa heads.  q and q_rot may both be NULL: then only K and V
 * are appended, still in one launch (the caller's queries are rotated already,
 * e.g. by a q_proj with the rotation folded in, blockgtq/quantizer.py:1190-1243).
 */
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
                        void* q_rot, int64_t qr_sr, int64_t qr_sh, int gqa, void* stream);

/*
 * Kernel selection of bgtq_decode_attn (process-wide; meant for tests and
 * profiling): 0 = automatic (MFMA kernel when the layout allows it, otherwise
 * the layout-agnostic kernel), 1 = always the layout-agnostic kernel,
 * 2 = MFMA kernel only (BGTQ_EUNSUPPORTED if it cannot take the call).
 */
int bgtq_set_decode_path(int path);

/*
 * Which kernel the last bgtq_decode_attn of this process launched: 1 layout-agnostic,
 * 2 MFMA (0 before the first call).  The automatic
 * choice falls back silently; callers that depend on the fast path check here.
 * No counterpart in the reference.
 */
int bgtq_last_decode_path(void);

/* Bytes of fp32 scratch bgtq_decode_attn needs for (B, n_q, n_splits). */
size_t bgtq_workspace_bytes(int B, int n_q, int n_splits);

/* Partition count bgtq_decode_attn would pick for n_splits <= 0. */
int bgtq_default_splits(int B, int n_kv, int max_T);

/*
 * Fused unpack + dequant + split-T decode attention over the packed cache,
 * every (batch row, KV head, partition) in one launch.
 * Replaces _packed_decode_kernel (blockgtq/kernels/fused_packed_attention.py:153-894)
 * which the reference launches once per KV head from
 * fused_blockgtq_decode_attention (:1541-1843).
 *
 *   q_rot      fp16 [B][n_q][128] already permuted+rotated (bgtq_rotate_q)
 *   k_packed / k_norms / v_packed / v_norms as written by the encoders;
 *              k_row_width / v_row_width = record bytes per token the cache holds
 *              (the widest head's record), strides may be larger
 *   seq_lens   device int32[B] tokens visible per batch row, or NULL -> T for all
 *   n_splits   partitions per (b, kv head); the partitions tile [0, T_b) in
 *              order, how the boundaries are rounded is up to the kernel
 *   partial_out fp32 [B][n_q][n_splits][128]  (normalised, V still rotated)
 *   partial_lse fp32 [B][n_q][n_splits]       (natural log; -inf for an empty partition)
 */
int bgtq_decode_attn(const bgtq_head_plan* plans,
                     const void* q_rot, int64_t q_sb, int64_t q_sh,
                     const void* k_packed, int64_t kp_sb, int64_t kp_sh, int64_t kp_st, int k_row_width,
                     const void* k_norms, int64_t kn_sb, int64_t kn_sh, int64_t kn_st,
                     const void* v_packed, int64_t vp_sb, int64_t vp_sh, int64_t vp_st, int v_row_width,
                     const void* v_norms, int64_t vn_sb, int64_t vn_sh, int64_t vn_st,
                     const int32_t* seq_lens, int T,
                     int B, int n_kv, int gqa, int n_splits,
                     float* partial_out, float* partial_lse,
                     int k_layout, int v_layout, float scale, void* stream);

/*
 * Log-sum-exp merge of the partitions, optional extra partials (an fp16
 * sink/recent-window attention computed elsewhere), V un-rotation applied once
 * to the merged vector, fp16 store.
 * Replaces _split_t_merge_kernel (blockgtq/kernels/fused_packed_attention.py:60-103),
 * the per-partition `partial_out @ R` of :875-882 and the return_lse
 * logsumexp of :1856-1860.  Partitions whose lse is -inf are skipped.
 *
 *   partial_out, plans  16-byte aligned (read 16 bytes at a time; BGTQ_EINVAL otherwise);
 *              n_splits <= BGTQ_MAX_SPLITS (BGTQ_ELIMIT otherwise)
 *   extra_out  fp32 [B][n_q][n_extra][128] or NULL, in the ORIGINAL value space:
 *              added after the packed sum has been un-rotated (needs unrotate != 0)
 *   extra_lse  fp32 [B][n_q][n_extra] or NULL
 *   unrotate   != 0: multiply the merged vector by plans[h].v_rot
 *   out        fp16 [B][n_q][128], strides o_sb/o_sh in halves
 *   lse_out    fp32 [B][n_q] total log-sum-exp, or NULL
 */
int bgtq_lse_reduce(const bgtq_head_plan* plans,
                    const float* partial_out, const float* partial_lse, int n_splits,
                    const float* extra_out, const float* extra_lse, int n_extra,
                    int B, int n_kv, int gqa, int unrotate,
                    void* out, int64_t o_sb, int64_t o_sh,
                    float* lse_out, void* stream);

/*
 * Decode attention of one layer, partitions merged, without any allocation:
 * bgtq_decode_attn followed by bgtq_lse_reduce (no extra partials), with the
 * partition results kept in a fixed array inside the library instead of a
 * caller-provided workspace.  This entry point has no counterpart in the
 * reference; it is for callers that cannot allocate device memory or size a
 * workspace at call time: code under HIP graph capture, tight serving loops,
 * harnesses that forbid allocation.  It calls no allocating routine.
 *
 *   arguments  as for bgtq_decode_attn (inputs) and bgtq_lse_reduce (unrotate, out,
 *              o_sb, o_sh, lse_out); n_splits <= 0 picks bgtq_default_splits
 *   limit      bgtq_workspace_bytes(B, n_kv * gqa, n_splits) must not exceed
 *              BGTQ_STATIC_SCRATCH_BYTES (8 MiB; BGTQ_ELIMIT otherwise) - e.g.
 *              B * n_q * n_splits <= 16256
 * Every GPU the library runs on holds one such array until the process ends, and
 * every call on a GPU uses that GPU's array: calls that overlap on one GPU (two
 * streams, two threads) race and must be serialised by the caller.  Nothing in the
 * array has to start at zero: each call overwrites every entry it later reads.
 * The first call on a device asks the runtime for the array's address and sets kernel
 * attributes, which are not stream operations: make one eager call per device before
 * capturing this entry point into a HIP graph.
 */
int bgtq_decode_attend_static(const bgtq_head_plan* plans,
                              const void* q_rot, int64_t q_sb, int64_t q_sh,
                              const void* k_packed, int64_t kp_sb, int64_t kp_sh, int64_t kp_st, int k_row_width,
                              const void* k_norms, int64_t kn_sb, int64_t kn_sh, int64_t kn_st,
                              const void* v_packed, int64_t vp_sb, int64_t vp_sh, int64_t vp_st, int v_row_width,
                              const void* v_norms, int64_t vn_sb, int64_t vn_sh, int64_t vn_st,
                              const int32_t* seq_lens, int T,
                              int B, int n_kv, int gqa, int n_splits,
                              int k_layout, int v_layout, float scale, int unrotate,
                              void* out, int64_t o_sb, int64_t o_sh, float* lse_out, void* stream);

/*
 * Dense fp16 attention partial for the with-buffer setting: sink tokens and a
 * recent window are kept as plain fp16 K/V (post-RoPE, unrotated) next to the
 * packed cache.  The partial lives in the ORIGINAL value space and feeds
 * bgtq_lse_reduce as `extra`, which adds it after un-rotating the packed sum.
 * Takes the ORIGINAL queries (not bgtq_rotate_q's output).  The reference has
 * this three-region cache only in its unaccelerated path
 * (blockgtq/unaccelerated.py:163-244).
 *   q          fp16 [B][n_q][128], strides q_sb/q_sh in halves
 *   kbuf, vbuf fp16 [B][n_kv][W][128], common strides w_sb/w_sh/w_st in halves
 *   lens       device int32[B] valid rows (<= W) or NULL -> W; W <= 8192
 *   part_out   fp32 [B][n_q][128], part_lse fp32 [B][n_q] (-inf when no row is valid)
 */
int bgtq_window_attn(const void* q, int64_t q_sb, int64_t q_sh,
                     const void* kbuf, const void* vbuf,
                     int64_t w_sb, int64_t w_sh, int64_t w_st,
                     const int32_t* lens, int W,
                     int B, int n_kv, int gqa, float scale,
                     float* part_out, float* part_lse, void* stream);

/*
 * With-buffer append, one launch for the ring update of a decode step: for every
 * batch row the fp16 token in ring slot slot[b] leaves the window (it is copied to
 * old_k / old_v, from where the caller encodes it into the packed cache) and this
 * step's token takes its place.  One launch instead of the four indexed tensor
 * copies per layer that the same update costs otherwise.  The reference keeps
 * sink, quantised middle and fp16 tail in one growing fp16 cache and rewrites the
 * oldest tail block in place once the tail exceeds the window
 * (blockgtq/unaccelerated.py:204-240); here the tail is a ring of W slots.
 *   kbuf, vbuf    fp16 [B][n_kv][W][128], common strides w_sb/w_sh/w_st in halves
 *   new_k, new_v  fp16 [B][n_kv][128], common strides n_sb/n_sh in halves
 *   slot          device int32[B]; a slot outside [0, W) moves nothing for that row
 *   old_k, old_v  fp16 [B][n_kv][128] contiguous (zeros for rows that moved nothing)
 */
int bgtq_window_swap(void* kbuf, void* vbuf, int64_t w_sb, int64_t w_sh, int64_t w_st,
                     const void* new_k, const void* new_v, int64_t n_sb, int64_t n_sh,
                     const int32_t* slot, int W, int B, int n_kv,
                     void* old_k, void* old_v, void* stream);

/*
 * Packed records back to fp16 vectors, all KV heads of a layer in one launch:
 * the tile dequantisation of the reference's prompt-phase attention kernel
 * (blockgtq/kernels/fused_packed_attention.py:1876-2594, helpers :1384-1533)
 * as a pass of its own.  Causal attention of bgtq_rotate_q's queries over
 * k_out / v_out, followed by the V un-rotation, equals attention over the
 * packed cache.
 *   inputs     as for bgtq_decode_attn (same strides, layouts and row widths)
 *   k_out      fp16 [B][n_kv][T][128] in the packed-dim order and rotated space of
 *              the records: fp16(codebook[code] * group norm), 0 on 0-bit dims;
 *              strides ko_sb/ko_sh/ko_st in halves
 *   v_out      fp16 [B][n_kv][T][128] in rotated V space: fp16(centroid[code] * norm)
 */
int bgtq_dequant_kv(const bgtq_head_plan* plans,
                    const void* k_packed, int64_t kp_sb, int64_t kp_sh, int64_t kp_st, int k_row_width,
                    const void* k_norms, int64_t kn_sb, int64_t kn_sh, int64_t kn_st,
                    const void* v_packed, int64_t vp_sb, int64_t vp_sh, int64_t vp_st, int v_row_width,
                    const void* v_norms, int64_t vn_sb, int64_t vn_sh, int64_t vn_st,
                    int B, int n_kv, int T, int k_layout, int v_layout,
                    void* k_out, int64_t ko_sb, int64_t ko_sh, int64_t ko_st,
                    void* v_out, int64_t vo_sb, int64_t vo_sh, int64_t vo_st,
                    void* stream);

/*
 * Prompt-phase attention straight over the packed cache: S query tokens per
 * sequence attend to records [0, T), query token s seeing t <= q_pos_offset + s
 * when is_causal.  Every 64-token tile of records is dequantised once per block of
 * 256 query rows inside the kernel (same values as bgtq_dequant_kv writes), both
 * products run on matrix cores, the V un-rotation (when unrotate != 0) is applied
 * before the fp16 store; no fp16 K/V tensor of the layer exists.  Replaces
 * _packed_prefill_kernel as driven by fused_blockgtq_prefill_attention
 * (blockgtq/kernels/fused_packed_attention.py:1876-2594, :2597-2760), for all KV
 * heads of a layer in one launch.
 *   q_rot      fp16 [B][n_kv*gqa][S][128], already permuted + rotated
 *              (bgtq_rotate_q semantics), strides q_sb/q_sh/q_ss in halves, rows 16-byte aligned
 *   cache      as for bgtq_decode_attn (same strides, layouts and row widths)
 *   out        fp16 [B][n_kv*gqa][S][128], strides o_sb/o_sh/o_ss in halves
 * B == 0 or S == 0 returns BGTQ_OK with nothing written.  Returns BGTQ_EUNSUPPORTED,
 * with nothing launched, unless all of these hold: gqa <= 256, scale > 0, T > 0;
 * K rows follow each other (kp_st == k_row_width, 4..128, a multiple of 4; kp_sb, kp_sh
 * and the base multiples of 4); kn_st in 1..8; v_row_width one of 16, 32, 48, 64 (64 for
 * the nibble layout) with v_row_width <= vp_st <= v_row_width + 4 and vp_* and the base
 * multiples of 4; vn_st == 1; query strides multiples of 8 halves and a 16-byte base;
 * output strides multiples of 4 halves and an 8-byte base.  A caller whose cache does
 * not meet them copies the records into rows that do (a cache filled by bgtq_encode_append
 * into tensors allocated at bgtq_cache_row_bytes already does).
 */
int bgtq_prefill_attn(const bgtq_head_plan* plans,
                      const void* q_rot, int64_t q_sb, int64_t q_sh, int64_t q_ss,
                      const void* k_packed, int64_t kp_sb, int64_t kp_sh, int64_t kp_st, int k_row_width,
                      const void* k_norms, int64_t kn_sb, int64_t kn_sh, int64_t kn_st,
                      const void* v_packed, int64_t vp_sb, int64_t vp_sh, int64_t vp_st, int v_row_width,
                      const void* v_norms, int64_t vn_sb, int64_t vn_sh, int64_t vn_st,
                      int B, int n_kv, int gqa, int S, int T, int q_pos_offset, int is_causal,
                      int k_layout, int v_layout, float scale, int unrotate,
                      void* out, int64_t o_sb, int64_t o_sh, int64_t o_ss, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BGTQ_H */
