// Argument block shared by the decode attention kernels (internal).
#pragma once
#include "bgtq_common.h"

// LDS bytes of one wave's tile buffers in the MFMA kernel (filled in by its launcher)
struct TileLayout {
    int kt, vt, knr, vnr, kbuf;    // K, V, K-norm, V-norm areas; K + both norm areas
};

struct DecodeArgs {
    const bgtq_head_plan* plans;
    const uint16_t* q;  int64_t q_sb, q_sh;
    const uint8_t* kp;  int64_t kp_sb, kp_sh, kp_st;
    const uint16_t* kn; int64_t kn_sb, kn_sh, kn_st;
    const uint8_t* vp;  int64_t vp_sb, vp_sh, vp_st;
    const uint16_t* vn; int64_t vn_sb, vn_sh, vn_st;
    const int32_t* seq_lens; int T;
    int B, n_kv, gqa, n_splits;
    int gqa_all, head0;    // MFMA kernel: query heads per KV head in q and the partials, first head of this launch
    float* part_out; float* part_lse;
    int k_layout, v_layout;
    float scale;
    int k_row_width;       // widest K record over the heads (LDS sizing)
    int v_row_width;
    int nw;                // MFMA kernel: waves per work-group
    int nw_tiles;          // MFMA kernel: how many of them own tiles and tile buffers (the first ones)
    int p_over_k;          // MFMA kernel: the P tile lies over the K tile (no buffer of its own)
    TileLayout tl;
    int wave_bytes;        // MFMA kernel: LDS bytes of one wave's buffers
    // MFMA kernel: 1 when every (row, head) slice of the four cache tensors starts on a 16-byte boundary;
    // then a whole 64-token tile of the K records, K norms, V norms and V records is nfull[i] whole 1 KB
    // loads and one more for the lanes in last[i]
    int aligned16;
    int nfull[4];
    uint64_t last[4];
    int per_tiles, rem_tiles;   // MFMA kernel, equal row lengths: tiles per partition, partitions with one more
};

// Fast path: MFMA kernel for packed K and V records (bgtq_decode_seg.hip).
// Returns BGTQ_EUNSUPPORTED when the arguments do not meet its layout
// requirements, in which case the caller takes the layout-agnostic kernel.
int bgtq_launch_decode_seg(const DecodeArgs& a, hipStream_t stream);
