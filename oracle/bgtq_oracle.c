/*
 * bgtq_oracle.c - CPU restatement of the packed-KV path of Block-GTQ.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product (blockgtq_amd/) links,
 * loads or calls this file; it is the checker the GPU kernels are compared
 * against in tests/, in the smoke run and as the CPU baseline of bench.py.
 *
 * Every function states the arithmetic of one reference kernel in scalar C
 * with a FIXED evaluation order (sequential fused multiply-adds in ascending
 * dim order, IEEE sqrt and divide), so that "bit-exact" is well defined: the
 * reference itself rotates with a TF32 tensor-core dot whose rounding cannot
 * be reproduced off NVIDIA hardware (blockgtq/quantizer.py:187,377,838).
 *
 * Reference files followed (paths relative to the reference checkout):
 *   K encode        blockgtq/quantizer.py:800-857 (norms, rotate, 256-bin LUT)
 *   K exact rule    blockgtq/block_gtq_pipeline.py:337-341 (searchsorted)
 *   K bit packing   blockgtq/quantizer.py:861-990, sizes :34-102
 *   K mixed layout  blockgtq/quantizer.py:1930-1951, corrected norms :1956-1974
 *   V encode        blockgtq/quantizer.py:560-596
 *   V packing       blockgtq/v_packing.py:31-109, nibble blockgtq/quantizer.py:2096-2099
 *   Q rotation      blockgtq/quantizer.py:1160-1187
 *   decode          blockgtq/kernels/fused_packed_attention.py:257-294,770-894,
 *                   unpack rules :1010-1372, merge :60-103
 *
 * Parity unpinned: the reference ships no tests or golden vectors for this
 * path, and four things no independent check fixes: the Monte-Carlo Lloyd V
 * centroids for 3 bits and more (blockgtq/v_quantize_gpu.py:19-117), the tie
 * order of torch.argsort on equal bit widths (blockgtq/block_gtq_pipeline.py:163),
 * scipy's Lloyd-Max centroids to the last ulp, and the TF32 / fp16-tile
 * rounding of the reference's own kernels on NVIDIA hardware.  All four are
 * inputs (tables) to the functions below, not part of their arithmetic.
 *
 * Parity pins (tests/test_oracle.py, tests/test_host_plan.py): packers against an independent
 * LSB-first bitstream writer and against the reference's per-dim unpack rule
 * (blockgtq/v_packing.py:118-120); V codes against numpy.searchsorted; K codes
 * of an identity-rotation single-group head against plain scalar quantisation;
 * corrected norms against ||centroids[codes]|| * norm == ||x||; attention
 * against torch.nn.functional.scaled_dot_product_attention on dequantised
 * tensors and against split/merge invariance.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "../include/bgtq.h"

#define D BGTQ_HEAD_DIM

/* ---- IEEE binary16 <-> binary32, round to nearest even ------------------- */
static float h2f(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {                      /* subnormal half -> normal float */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static uint16_t f2h(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u)                       /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | (ax > 0x7F800000u ? 0x200u : 0u));
    if (ax >= 0x477FF000u)                       /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7C00u);
    if (ax < 0x33000001u)                        /* <= 2^-25 -> +-0 */
        return sign;
    int e = (int)(ax >> 23) - 127;
    uint32_t man = (ax & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
    int shift;                                   /* bits dropped from the significand */
    uint32_t hexp;
    if (e < -14) { shift = 13 + (-14 - e); hexp = 0; }
    else         { shift = 13;             hexp = (uint32_t)(e + 15); }
    uint32_t kept = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (kept & 1u))) kept++;
    /* kept carries the implicit bit for normals; adding the exponent field
       lets a mantissa overflow ripple into the exponent correctly */
    uint32_t out = (hexp == 0) ? kept : ((hexp - 1u) << 10) + kept;
    return (uint16_t)(sign | out);
}

void orc_f2h(const float* in, uint16_t* out, int64_t n)
{ for (int64_t i = 0; i < n; i++) out[i] = f2h(in[i]); }

void orc_h2f(const uint16_t* in, float* out, int64_t n)
{ for (int64_t i = 0; i < n; i++) out[i] = h2f(in[i]); }

size_t orc_plan_sizeof(void) { return sizeof(bgtq_head_plan); }

/* ---- K encode ------------------------------------------------------------ */
/* codes: N x 128 in packed order (0 for 0-bit dims); raw/corr norms: N x 8 fp32 */
void orc_encode_k(const bgtq_head_plan* p, const uint16_t* k, int64_t N, int quant_mode,
                  uint8_t* codes, float* raw_norms, float* corr_norms)
{
    for (int64_t r = 0; r < N; r++) {
        const uint16_t* row = k + r * D;
        float x[D], xh[D], y[D];
        uint8_t* c = codes + r * D;
        for (int j = 0; j < D; j++) x[j] = h2f(row[p->head_perm[j]]);
        memset(c, 0, D);
        for (int g = 0; g < BGTQ_MAX_SEGMENTS; g++) {
            raw_norms[r * BGTQ_MAX_SEGMENTS + g] = 0.f;
            corr_norms[r * BGTQ_MAX_SEGMENTS + g] = 0.f;
        }
        for (int g = 0; g < p->n_seg; g++) {
            int s = p->seg_start[g], e = s + p->seg_len[g];
            float ss = 0.f;
            for (int j = s; j < e; j++) ss = fmaf(x[j], x[j], ss);
            float n = sqrtf(ss + 1e-30f);
            float safe = n > 1e-10f ? n : 1.0f;
            for (int j = s; j < e; j++) xh[j] = x[j] / safe;
            for (int j = s; j < e; j++) {
                if (p->seg_identity[g]) {
                    y[j] = xh[j];
                } else {
                    float acc = 0.f;
                    for (int kk = s; kk < e; kk++)
                        acc = fmaf(xh[kk], p->k_rot_T[kk * D + j], acc);
                    y[j] = acc;
                }
            }
            float cs = 0.f;
            for (int j = s; j < e; j++) {
                int code;
                if (quant_mode == BGTQ_QUANT_EXACT) {
                    int nb = (1 << p->seg_bw[g]) - 1;
                    code = 0;
                    for (int b = 0; b < nb; b++) code += (p->k_boundaries[g][b] < y[j]);
                } else {
                    float t = (y[j] - p->lut_offset[j]) * p->lut_inv_scale[j];
                    t = fminf(fmaxf(t, 0.0f), (float)(BGTQ_LUT_BINS - 1));
                    code = p->code_lut[g][(int)t];
                }
                c[j] = (uint8_t)code;
                float cv = p->k_centroids[g][code];
                cs = fmaf(cv, cv, cs);
            }
            raw_norms[r * BGTQ_MAX_SEGMENTS + g] = n;
            corr_norms[r * BGTQ_MAX_SEGMENTS + g] = n / fmaxf(sqrtf(cs), 1e-10f);
        }
    }
}

/* LSB-first stream of `bw`-bit codes; codes past `len` contribute zero bits */
static uint8_t stream_byte(const uint8_t* codes, int len, int bw, int byte_idx)
{
    unsigned out = 0;
    for (int b = 0; b < 8; b++) {
        int bit = byte_idx * 8 + b;
        int ci = bit / bw;
        if (ci < len) out |= ((unsigned)(codes[ci] >> (bit % bw)) & 1u) << b;
    }
    return (uint8_t)out;
}

static int seg_bytes(int bw, int len)
{
    switch (bw) {
    case 1: return (len + 7) / 8;
    case 2: return (len + 3) / 4;
    case 3: return ((len + 7) / 8) * 3;
    case 4: return (len + 1) / 2;
    default: return len;
    }
}

/* BGTQ_K_BITPACKED record; `out` rows are `stride` bytes apart, the first
   `width` bytes of each are written (record, then zeros). */
void orc_pack_k_bits(const bgtq_head_plan* p, const uint8_t* codes, int64_t N,
                     uint8_t* out, int64_t stride, int width)
{
    for (int64_t r = 0; r < N; r++) {
        uint8_t* o = out + r * stride;
        memset(o, 0, (size_t)width);
        for (int g = 0; g < p->n_seg; g++) {
            int bw = p->seg_bw[g], len = p->seg_len[g];
            const uint8_t* c = codes + r * D + p->seg_start[g];
            uint8_t* dst = o + p->seg_pack_off[g];
            int nb = seg_bytes(bw, len);
            if (bw >= 5) {
                for (int i = 0; i < len; i++) dst[i] = c[i];
            } else {
                for (int i = 0; i < nb; i++) dst[i] = stream_byte(c, len, bw, i);
            }
        }
    }
}

/* BGTQ_K_MIXED record: nibbles for dims [n_zero, nopack_start), raw bytes after */
void orc_pack_k_mixed(const bgtq_head_plan* p, const uint8_t* codes, int64_t N,
                      uint8_t* out, int64_t stride, int width)
{
    int z = p->n_zero_dims;
    int nib = (p->nopack_start - z) / 2;
    for (int64_t r = 0; r < N; r++) {
        const uint8_t* c = codes + r * D;
        uint8_t* o = out + r * stride;
        memset(o, 0, (size_t)width);
        for (int i = 0; i < nib; i++)
            o[i] = (uint8_t)((c[z + 2 * i] & 0xF) | ((c[z + 2 * i + 1] & 0xF) << 4));
        for (int i = 0; i < p->nopack_len; i++) o[nib + i] = c[p->nopack_start + i];
    }
}

void orc_unpack_k_bits(const bgtq_head_plan* p, const uint8_t* packed, int64_t N,
                       int64_t stride, uint8_t* codes)
{
    for (int64_t r = 0; r < N; r++) {
        const uint8_t* o = packed + r * stride;
        uint8_t* c = codes + r * D;
        memset(c, 0, D);
        for (int g = 0; g < p->n_seg; g++) {
            int bw = p->seg_bw[g], len = p->seg_len[g], s = p->seg_start[g];
            const uint8_t* src = o + p->seg_pack_off[g];
            for (int i = 0; i < len; i++) {
                if (bw >= 5) { c[s + i] = src[i]; continue; }
                int bit = i * bw;
                unsigned w = src[bit >> 3] | ((unsigned)src[(bit >> 3) + ((bit & 7) + bw > 8)] << 8);
                c[s + i] = (uint8_t)((w >> (bit & 7)) & ((1u << bw) - 1u));
            }
        }
    }
}

void orc_unpack_k_mixed(const bgtq_head_plan* p, const uint8_t* packed, int64_t N,
                        int64_t stride, uint8_t* codes)
{
    int z = p->n_zero_dims;
    int nib = (p->nopack_start - z) / 2;
    for (int64_t r = 0; r < N; r++) {
        const uint8_t* o = packed + r * stride;
        uint8_t* c = codes + r * D;
        memset(c, 0, D);
        for (int i = 0; i < nib; i++) {
            c[z + 2 * i] = o[i] & 0xF;
            c[z + 2 * i + 1] = o[i] >> 4;
        }
        for (int i = 0; i < p->nopack_len; i++) c[p->nopack_start + i] = o[nib + i];
    }
}

/* ---- V encode ------------------------------------------------------------ */
void orc_encode_v(const bgtq_head_plan* p, const uint16_t* v, int64_t N,
                  uint8_t* codes, uint16_t* norms)
{
    int nb = (1 << p->v_bits) - 1;
    for (int64_t r = 0; r < N; r++) {
        float x[D], xh[D];
        float ss = 0.f;
        for (int j = 0; j < D; j++) { x[j] = h2f(v[r * D + j]); ss = fmaf(x[j], x[j], ss); }
        float n = sqrtf(ss + 1e-30f);
        float safe = n > 1e-8f ? n : 1.0f;
        for (int j = 0; j < D; j++) xh[j] = x[j] / safe;
        float cs = 0.f;
        for (int j = 0; j < D; j++) {
            float acc = 0.f;
            for (int kk = 0; kk < D; kk++) acc = fmaf(xh[kk], p->v_rot_T[kk * D + j], acc);
            int code = 0;
            for (int b = 0; b < nb; b++) code += (acc > p->v_boundaries[b]);
            codes[r * D + j] = (uint8_t)code;
            float cv = p->v_centroids[code];
            cs = fmaf(cv, cv, cs);
        }
        float cn = sqrtf(cs + 1e-20f);
        float safe_c = cn > 1e-10f ? cn : 1.0f;
        norms[r] = f2h(n / safe_c);
    }
}

void orc_pack_v(const uint8_t* codes, int64_t N, int v_bits, int nibble,
                uint8_t* out, int64_t stride)
{
    int bw = nibble ? 4 : v_bits;
    int nb = seg_bytes(bw, D);
    for (int64_t r = 0; r < N; r++)
        for (int i = 0; i < nb; i++)
            out[r * stride + i] = stream_byte(codes + r * D, D, bw, i);
}

void orc_unpack_v(const uint8_t* packed, int64_t N, int64_t stride, int v_bits, int nibble,
                  uint8_t* codes)
{
    int bw = nibble ? 4 : v_bits;
    for (int64_t r = 0; r < N; r++) {
        const uint8_t* src = packed + r * stride;
        for (int i = 0; i < D; i++) {
            int bit = i * bw;
            unsigned w = src[bit >> 3] | ((unsigned)src[(bit >> 3) + ((bit & 7) + bw > 8)] << 8);
            codes[r * D + i] = (uint8_t)((w >> (bit & 7)) & ((1u << bw) - 1u));
        }
    }
}

/* ---- Q permute + rotate -------------------------------------------------- */
void orc_rotate_q(const bgtq_head_plan* p, const uint16_t* q, int64_t N, uint16_t* q_rot)
{
    for (int64_t r = 0; r < N; r++) {
        float x[D];
        for (int j = 0; j < D; j++) x[j] = h2f(q[r * D + p->head_perm[j]]);
        for (int j = 0; j < D; j++) q_rot[r * D + j] = 0;
        for (int g = 0; g < p->n_seg; g++) {
            int s = p->seg_start[g], e = s + p->seg_len[g];
            for (int j = s; j < e; j++) {
                float acc;
                if (p->seg_identity[g]) {
                    acc = x[j];
                } else {
                    acc = 0.f;
                    for (int kk = s; kk < e; kk++) acc = fmaf(x[kk], p->k_rot_T[kk * D + j], acc);
                }
                q_rot[r * D + j] = f2h(acc);
            }
        }
    }
}

/* ---- decode attention ---------------------------------------------------- */
/*
 * One (batch row, KV head): `gqa` rotated queries against T packed tokens in
 * [t0, t1).  All accumulation in double.  out_rot (gqa x 128, V still in its
 * rotated space, normalised) and lse (natural log; -inf when t0 >= t1).
 */
void orc_decode_partial(const bgtq_head_plan* p, const uint16_t* q_rot, int gqa,
                        const uint8_t* k_packed, int64_t kp_stride,
                        const uint16_t* k_norms, int64_t kn_stride,
                        const uint8_t* v_packed, int64_t vp_stride,
                        const uint16_t* v_norms, int64_t vn_stride,
                        int64_t t0, int64_t t1, int k_layout, int v_layout, float scale,
                        double* out_rot, double* lse)
{
    int64_t T = t1 - t0;
    for (int h = 0; h < gqa; h++) {
        lse[h] = -INFINITY;
        for (int j = 0; j < D; j++) out_rot[h * D + j] = 0.0;
    }
    if (T <= 0) return;
    double* logit = (double*)malloc(sizeof(double) * (size_t)T * (size_t)gqa);
    uint8_t kc[D], vc[D];
    float qf[BGTQ_MAX_GQA][D];
    for (int h = 0; h < gqa; h++)
        for (int j = 0; j < D; j++) qf[h][j] = h2f(q_rot[h * D + j]);

    for (int64_t t = 0; t < T; t++) {
        const uint8_t* kp = k_packed + (t0 + t) * kp_stride;
        if (k_layout == BGTQ_K_MIXED) orc_unpack_k_mixed(p, kp, 1, 0, kc);
        else                          orc_unpack_k_bits(p, kp, 1, 0, kc);
        for (int h = 0; h < gqa; h++) {
            double acc = 0.0;
            for (int g = 0; g < p->n_seg; g++) {
                int s = p->seg_start[g], e = s + p->seg_len[g];
                double part = 0.0;
                for (int j = s; j < e; j++)
                    part += (double)qf[h][j] * (double)h2f(p->k_codebook_f16[g][kc[j]]);
                acc += part * (double)h2f(k_norms[(t0 + t) * kn_stride + g]);
            }
            logit[t * gqa + h] = acc * (double)scale;
        }
    }
    for (int h = 0; h < gqa; h++) {
        double m = -INFINITY;
        for (int64_t t = 0; t < T; t++) if (logit[t * gqa + h] > m) m = logit[t * gqa + h];
        double l = 0.0;
        for (int64_t t = 0; t < T; t++) {
            double w = exp(logit[t * gqa + h] - m);
            logit[t * gqa + h] = w;
            l += w;
        }
        lse[h] = m + log(l);
        for (int64_t t = 0; t < T; t++) logit[t * gqa + h] /= l;
    }
    for (int64_t t = 0; t < T; t++) {
        orc_unpack_v(v_packed + (t0 + t) * vp_stride, 1, 0, p->v_bits,
                     v_layout == BGTQ_V_NIBBLE, vc);
        double vn = (double)h2f(v_norms[(t0 + t) * vn_stride]);
        for (int j = 0; j < D; j++) {
            double val = (double)h2f(p->v_lut_f16[vc[j]]) * vn;
            for (int h = 0; h < gqa; h++) out_rot[h * D + j] += logit[t * gqa + h] * val;
        }
    }
    free(logit);
}

/* merge n partials (normalised vectors + lse), skipping lse == -inf */
void orc_merge(const double* parts, const double* lses, int n, double* out, double* lse_out)
{
    double m = -INFINITY;
    for (int i = 0; i < n; i++) if (lses[i] > m) m = lses[i];
    for (int j = 0; j < D; j++) out[j] = 0.0;
    if (m == -INFINITY) { *lse_out = -INFINITY; return; }
    double den = 0.0;
    for (int i = 0; i < n; i++) {
        if (lses[i] == -INFINITY) continue;
        double a = exp(lses[i] - m);
        den += a;
        for (int j = 0; j < D; j++) out[j] += a * parts[i * D + j];
    }
    for (int j = 0; j < D; j++) out[j] /= den;
    *lse_out = m + log(den);
}

/* out = vec @ v_rot (row vector times matrix), double accumulate */
void orc_unrotate_v(const bgtq_head_plan* p, const double* vec, double* out)
{
    for (int j = 0; j < D; j++) {
        double acc = 0.0;
        for (int k = 0; k < D; k++) acc += vec[k] * (double)p->v_rot[k * D + j];
        out[j] = acc;
    }
}

/*
 * Full decode attention for one (batch row, KV head): n_splits partitions of
 * [0, T) with chunk = ceil(T / n_splits), merged, un-rotated.  out: gqa x 128
 * float, lse: gqa float.
 */
void orc_decode_attn(const bgtq_head_plan* p, const uint16_t* q_rot, int gqa,
                     const uint8_t* k_packed, int64_t kp_stride,
                     const uint16_t* k_norms, int64_t kn_stride,
                     const uint8_t* v_packed, int64_t vp_stride,
                     const uint16_t* v_norms, int64_t vn_stride,
                     int64_t T, int n_splits, int k_layout, int v_layout, float scale,
                     int unrotate, float* out, float* lse)
{
    if (n_splits < 1) n_splits = 1;
    int64_t chunk = (T + n_splits - 1) / n_splits;
    double* parts = (double*)malloc(sizeof(double) * (size_t)n_splits * gqa * D);
    double* lses = (double*)malloc(sizeof(double) * (size_t)n_splits * gqa);
    for (int c = 0; c < n_splits; c++) {
        int64_t t0 = c * chunk, t1 = t0 + chunk;
        if (t1 > T) t1 = T;
        if (t0 > T) t0 = T;
        orc_decode_partial(p, q_rot, gqa, k_packed, kp_stride, k_norms, kn_stride,
                           v_packed, vp_stride, v_norms, vn_stride, t0, t1,
                           k_layout, v_layout, scale,
                           parts + (size_t)c * gqa * D, lses + (size_t)c * gqa);
    }
    double* hp = (double*)malloc(sizeof(double) * (size_t)n_splits * D);
    double* hl = (double*)malloc(sizeof(double) * (size_t)n_splits);
    for (int h = 0; h < gqa; h++) {
        for (int c = 0; c < n_splits; c++) {
            memcpy(hp + (size_t)c * D, parts + ((size_t)c * gqa + h) * D, sizeof(double) * D);
            hl[c] = lses[(size_t)c * gqa + h];
        }
        double merged[D], fin[D], l;
        orc_merge(hp, hl, n_splits, merged, &l);
        if (unrotate) orc_unrotate_v(p, merged, fin);
        else memcpy(fin, merged, sizeof(fin));
        for (int j = 0; j < D; j++) out[h * D + j] = (float)fin[j];
        lse[h] = (float)l;
    }
    free(parts); free(lses); free(hp); free(hl);
}

/* ---- dequantised tensors (for checks against library attention) ---------- */
/* K in packed (permuted + rotated) space: khat[t][j] = cb16[code] * norm16 */
void orc_dequant_k(const bgtq_head_plan* p, const uint8_t* codes, const uint16_t* norms,
                   int64_t kn_stride, int64_t N, float* khat)
{
    for (int64_t r = 0; r < N; r++) {
        for (int j = 0; j < D; j++) khat[r * D + j] = 0.f;
        for (int g = 0; g < p->n_seg; g++) {
            float n = h2f(norms[r * kn_stride + g]);
            for (int j = p->seg_start[g]; j < p->seg_start[g] + p->seg_len[g]; j++)
                khat[r * D + j] = h2f(p->k_codebook_f16[g][codes[r * D + j]]) * n;
        }
    }
}

/* V in rotated space: vhat[t][j] = vlut16[code] * norm16 */
void orc_dequant_v(const bgtq_head_plan* p, const uint8_t* codes, const uint16_t* norms,
                   int64_t N, float* vhat)
{
    for (int64_t r = 0; r < N; r++) {
        float n = h2f(norms[r]);
        for (int j = 0; j < D; j++) vhat[r * D + j] = h2f(p->v_lut_f16[codes[r * D + j]]) * n;
    }
}
