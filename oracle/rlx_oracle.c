/*
 * CPU oracle for the GGUF dequant-matmul / FakeQuantize path of MIT-RLX/rlx.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, the algorithm the
 * reference runs on its CPU backend.  It is the checker the HIP kernels are
 * compared against; nothing in the shipped library links or calls it.
 * Build: `make -C oracle` (gcc -O2 -ffp-contract=off -fno-fast-math), so no
 * multiply-add is ever fused and every rounding step matches the scalar Rust.
 *
 * Pinning status (which independent check pins each function):
 *   f16 -> f32            exhaustive 65536 values vs numpy.float16 (library routine)
 *   f32 -> f16 / bf16     RNE, vs numpy.float16 cast / closed-form bit rule
 *   Q8_0 / Q4_0 / Q4_K    the reference's own known-answer blocks
 *                         (rlx-gguf/src/lib.rs:1187-1264) + independent numpy
 *                         bit-field restatements on random bytes
 *   Q5_K                  reduces to the pinned Q4_K decoder when the fifth-bit plane is zero; a set bit adds exactly
 *                         16 * d * sc at the position the format fixes (closed form), random bytes vs numpy
 *   Q6_K / Q2_K / Q3_K / Q8_K  the reference's known-answer blocks (rlx-gguf/src/lib.rs:1266-1334) + one-hot
 *                         position probes against the closed-form index map of each format + numpy on random bytes;
 *                         Q6_K in both scale readings (block decoder unsigned, lib.rs:819-845; tensor decoder i8,
 *                         lib.rs:1070-1112)
 *   gguf_matmul_bt        reference tests rlx-cpu/src/gguf_matmul.rs:238-277 and
 *                         rlx-runtime/tests/dequant_matmul_gguf.rs:176-308
 *                         (layout idx = j*k + p), f64 dense matmul (textbook)
 *   rms_norm              closed forms (constant row -> +-gamma + beta up to eps, scale invariance, eps only on a zero row),
 *                         numpy f64 within a few ulp
 *   fused_swiglu          closed forms (gate 0 -> 0, large gate -> up * gate, silu(g) - silu(-g) = g), numpy f64 within
 *                         2 ulp; the last ulp follows the platform's expf like the reference's f32::exp (unpinned there)
 *   gguf_tied_lm_argmax   the reference's test (rlx-cpu/src/lm_head.rs:306-334: equals the argmax of gguf_matmul_bt's
 *                         logits) + constructed ties, NaN and all -inf rows against the loop's stated rule
 *   gguf_tied_lm_topk     the inputs of the reference's test (rlx-cpu/src/lm_head.rs:278-304) against a brute-force
 *                         stable sort of all scores (values pinned; the rows among the tied scores follow the
 *                         smaller-row rule stated here, the reference leaves their order to an unstable selection),
 *                         random rows of three schemes against the same brute force, cap = 1 against the argmax
 *   fake_quantize         closed forms (channel max -> code +-q_max, all-zero
 *                         channel, constructed ties, NaN), shapes/inputs of
 *                         rlx-mlx/tests/autodiff_fakequant_parity.rs:189-308
 *   philox4x32            Random123 known-answer vectors when run with the
 *                         standard multiplier; the reference's own multiplier
 *                         (rlx-ir/src/rng.rs:55) only changes that constant
 *   philox normal()       PARITY UNPINNED in the last ulp: the reference calls
 *                         Rust std ln/sqrt/cos (platform libm); no reference test
 *                         holds literal values (rlx-ir/src/rng.rs:149-205)
 *   encoders              not here: the reference has none (rlx-gguf is
 *                         decode-only), so there is nothing to restate
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define QK8_0 32
#define QK4_0 32
#define QK_K 256
#define K_SCALE_SIZE 12

/* scheme ids shared with include/rlx_mi355x.h (rlx-ir/src/quant.rs:39-79 order) */
enum { ORC_Q4K = 5, ORC_Q5K = 6, ORC_Q6K = 7, ORC_Q8K = 8, ORC_Q2K = 9, ORC_Q3K = 10, ORC_Q4_0 = 11, ORC_Q8_0 = 12 };

/* ---- half / bfloat16 -------------------------------------------------- */

/* half::f16::to_f32 as used by rlx-gguf/src/lib.rs:569-571: exact IEEE widening. */
float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while (!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* half::f16::from_f32 (rlx-driver/src/arena.rs:72-76): round-to-nearest-even, NaN kept quiet. */
uint16_t orc_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t exp = (x >> 23) & 0xFFu;
    uint32_t man = x & 0x7FFFFFu;
    if (exp == 255) {
        if (man) return (uint16_t)(sign | 0x7E00u | (man >> 13));
        return (uint16_t)(sign | 0x7C00u);
    }
    int e = (int)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u);
    if (e <= 0) {
        if (e < -10) return sign;
        man |= 0x800000u;
        int shift = 14 - e; /* 14..24 */
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1))) half_man++;
        return (uint16_t)(sign | half_man);
    }
    uint32_t half_man = man >> 13;
    uint32_t rem = man & 0x1FFFu;
    uint16_t out = (uint16_t)(sign | ((uint32_t)e << 10) | half_man);
    if (rem > 0x1000u || (rem == 0x1000u && (half_man & 1))) out++; /* carry may roll into exp/inf: correct */
    return out;
}

/* half::bf16::from_f32 (rlx-driver/src/arena.rs:78-83): RNE on the upper 16 bits. */
uint16_t orc_f32_to_bf16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x0040u);
    uint32_t round_bit = 0x8000u;
    if ((x & round_bit) && (x & (3u * round_bit - 1u))) return (uint16_t)((x >> 16) + 1);
    return (uint16_t)(x >> 16);
}

float orc_bf16_to_f32(uint16_t h) {
    uint32_t x = (uint32_t)h << 16;
    float f;
    memcpy(&f, &x, 4);
    return f;
}

/* ---- block geometry (rlx-ir/src/quant.rs:138-164, rlx-gguf/src/lib.rs:393-414) ---- */

int orc_block_elems(int scheme) {
    switch (scheme) {
    case ORC_Q4K:
    case ORC_Q5K:
    case ORC_Q6K:
    case ORC_Q8K:
    case ORC_Q2K:
    case ORC_Q3K: return QK_K;
    case ORC_Q4_0: return QK4_0;
    case ORC_Q8_0: return QK8_0;
    default: return 0;
    }
}

int orc_block_bytes(int scheme) {
    switch (scheme) {
    case ORC_Q4K: return 2 + 2 + K_SCALE_SIZE + QK_K / 2; /* 144 */
    case ORC_Q5K: return 2 + 2 + K_SCALE_SIZE + QK_K / 8 + QK_K / 2; /* 176 */
    case ORC_Q6K: return QK_K / 2 + QK_K / 4 + QK_K / 16 + 2;       /* 210 */
    case ORC_Q8K: return 4 + QK_K + (QK_K / 16) * 2;                /* 292 */
    case ORC_Q2K: return 2 + 2 + QK_K / 16 + QK_K / 4;              /* 84 */
    case ORC_Q3K: return 2 + K_SCALE_SIZE + QK_K / 8 + QK_K / 4;    /* 110 */
    case ORC_Q4_0: return 2 + QK4_0 / 2;                  /* 18 */
    case ORC_Q8_0: return 2 + QK8_0;                      /* 34 */
    default: return 0;
    }
}

/* bytes_for (rlx-gguf/src/lib.rs:393-399): -1 when n is not a multiple of the block. */
int64_t orc_bytes_for(int scheme, int64_t n) {
    int be = orc_block_elems(scheme);
    if (be == 0 || n % be != 0) return -1;
    return (n / be) * orc_block_bytes(scheme);
}

/* ---- block decoders ---------------------------------------------------- */

static float read_f16_le(const uint8_t *b) { return orc_f16_to_f32((uint16_t)(b[0] | (b[1] << 8))); }

/* rlx-gguf/src/lib.rs:574-581 */
void orc_dequant_q8_0_block(const uint8_t *block, float *out) {
    float d = read_f16_le(block);
    const uint8_t *qs = block + 2;
    for (int i = 0; i < QK8_0; i++) out[i] = d * (float)(int8_t)qs[i];
}

/* rlx-gguf/src/lib.rs:584-597: low nibbles -> first half, high nibbles -> second half. */
void orc_dequant_q4_0_block(const uint8_t *block, float *out) {
    float d = read_f16_le(block);
    const uint8_t *qs = block + 2;
    for (int j = 0; j < QK4_0 / 2; j++) {
        int v0 = (int)(qs[j] & 0x0F) - 8;
        out[j] = d * (float)v0;
    }
    for (int j = 0; j < QK4_0 / 2; j++) {
        int v1 = (int)(qs[j] >> 4) - 8;
        out[QK4_0 / 2 + j] = d * (float)v1;
    }
}

/* rlx-gguf/src/lib.rs:743-751 */
void orc_get_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *mn) {
    if (j < 4) {
        *sc = q[j] & 63;
        *mn = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4));
        *mn = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* rlx-gguf/src/lib.rs:754-780: four roundings per element, none fused. */
void orc_dequant_q4_k_block(const uint8_t *block, float *out) {
    float d = read_f16_le(block);
    float dmin = read_f16_le(block + 2);
    const uint8_t *scales = block + 4;
    const uint8_t *qs = block + 4 + K_SCALE_SIZE;
    int is = 0, oi = 0;
    for (int j = 0; j < 8; j += 2) {
        uint8_t sc0, m0, sc1, m1;
        orc_get_scale_min_k4(j, scales, &sc0, &m0);
        orc_get_scale_min_k4(j + 1, scales, &sc1, &m1);
        float d0 = d * (float)sc0;
        float m0f = dmin * (float)m0;
        float d1 = d * (float)sc1;
        float m1f = dmin * (float)m1;
        for (int l = 0; l < 32; l++) {
            uint8_t q = qs[is + l];
            float t = d0 * (float)(q & 0x0F);
            out[oi++] = t - m0f;
        }
        for (int l = 0; l < 32; l++) {
            uint8_t q = qs[is + l];
            float t = d1 * (float)(q >> 4);
            out[oi++] = t - m1f;
        }
        is += 32;
    }
}

/* rlx-gguf/src/lib.rs:783-816 */
void orc_dequant_q5_k_block(const uint8_t *block, float *out) {
    float d = read_f16_le(block);
    float dmin = read_f16_le(block + 2);
    const uint8_t *scales = block + 4;
    const uint8_t *qh = block + 4 + K_SCALE_SIZE;
    const uint8_t *qs = block + 4 + K_SCALE_SIZE + QK_K / 8;
    int is = 0, oi = 0;
    uint8_t u1 = 1, u2 = 2;
    for (int j = 0; j < 8; j += 2) {
        uint8_t sc0, m0, sc1, m1;
        orc_get_scale_min_k4(j, scales, &sc0, &m0);
        orc_get_scale_min_k4(j + 1, scales, &sc1, &m1);
        float d0 = d * (float)sc0;
        float m0f = dmin * (float)m0;
        float d1 = d * (float)sc1;
        float m1f = dmin * (float)m1;
        for (int l = 0; l < 32; l++) {
            uint8_t lo = qs[is + l] & 0x0F;
            uint8_t hi = (qh[l] & u1) ? 16 : 0;
            float t = d0 * (float)(uint8_t)(lo + hi);
            out[oi++] = t - m0f;
        }
        for (int l = 0; l < 32; l++) {
            uint8_t lo = qs[is + l] >> 4;
            uint8_t hi = (qh[l] & u2) ? 16 : 0;
            float t = d1 * (float)(uint8_t)(lo + hi);
            out[oi++] = t - m1f;
        }
        is += 32;
        u1 <<= 2;
        u2 <<= 2;
    }
}

/* rlx-gguf/src/lib.rs:819-845 (signed_scales = 0): the block decoder the matmul calls converts the sixteen scale bytes
 * as unsigned. rlx-gguf/src/lib.rs:1070-1112 (signed_scales = 1): the whole-tensor decoder reads them as i8. */
void orc_dequant_q6_k_block(const uint8_t *block, float *out, int signed_scales) {
    const int ql_len = QK_K / 2, qh_len = QK_K / 4, sc_len = QK_K / 16;
    const uint8_t *ql = block, *qh = block + ql_len, *sc = block + ql_len + qh_len;
    float d = read_f16_le(block + ql_len + qh_len + sc_len);
    for (int h = 0; h < 2; h++) {
        int dst_base = h * 128, ql_off = h * 64, qh_off_h = h * 32, sc_off = h * 8;
        for (int l = 0; l < 32; l++) {
            int is = l / 16;
            uint8_t qh_b = qh[qh_off_h + l];
            int32_t q1 = (int32_t)(uint8_t)((ql[ql_off + l] & 0x0F) | ((qh_b & 3) << 4)) - 32;
            int32_t q2 = (int32_t)(uint8_t)((ql[ql_off + l + 32] & 0x0F) | (((qh_b >> 2) & 3) << 4)) - 32;
            int32_t q3 = (int32_t)(uint8_t)((ql[ql_off + l] >> 4) | (((qh_b >> 4) & 3) << 4)) - 32;
            int32_t q4 = (int32_t)(uint8_t)((ql[ql_off + l + 32] >> 4) | (((qh_b >> 6) & 3) << 4)) - 32;
            float s1 = signed_scales ? (float)(int8_t)sc[sc_off + is] : (float)sc[sc_off + is];
            float s2 = signed_scales ? (float)(int8_t)sc[sc_off + is + 2] : (float)sc[sc_off + is + 2];
            float s3 = signed_scales ? (float)(int8_t)sc[sc_off + is + 4] : (float)sc[sc_off + is + 4];
            float s4 = signed_scales ? (float)(int8_t)sc[sc_off + is + 6] : (float)sc[sc_off + is + 6];
            float t1 = d * s1, t2 = d * s2, t3 = d * s3, t4 = d * s4;
            out[dst_base + l] = t1 * (float)q1;
            out[dst_base + l + 32] = t2 * (float)q2;
            out[dst_base + l + 64] = t3 * (float)q3;
            out[dst_base + l + 96] = t4 * (float)q4;
        }
    }
}

/* rlx-gguf/src/lib.rs:848-854 */
void orc_dequant_q8_k_block(const uint8_t *block, float *out) {
    float d;
    memcpy(&d, block, 4);
    const uint8_t *qs = block + 4;
    for (int i = 0; i < QK_K; i++) out[i] = d * (float)(int8_t)qs[i];
}

/* rlx-gguf/src/lib.rs:857-886 */
void orc_dequant_q2_k_block(const uint8_t *block, float *out) {
    float d = read_f16_le(block);
    float mn = read_f16_le(block + 2);
    const uint8_t *q = block + 4 + QK_K / 16;
    int is = 0, oi = 0;
    for (int n = 0; n < QK_K / 128; n++) {
        unsigned shift = 0;
        for (int j = 0; j < 4; j++) {
            uint8_t sc = block[4 + is];
            is++;
            float dl = d * (float)(sc & 0xF);
            float ml = mn * (float)(sc >> 4);
            for (int l = 0; l < 16; l++) {
                float t = dl * (float)((q[l] >> shift) & 3);
                out[oi++] = t - ml;
            }
            sc = block[4 + is];
            is++;
            dl = d * (float)(sc & 0xF);
            ml = mn * (float)(sc >> 4);
            for (int l = 0; l < 16; l++) {
                float t = dl * (float)((q[l + 16] >> shift) & 3);
                out[oi++] = t - ml;
            }
            shift += 2;
        }
        q += 32;
    }
}

/* rlx-gguf/src/lib.rs:889-930 */
void orc_dequant_q3_k_block(const uint8_t *block, float *out) {
    const uint32_t KMASK1 = 0x03030303u, KMASK2 = 0x0f0f0f0fu;
    float d_all = read_f16_le(block);
    const uint8_t *hm = block + 2 + K_SCALE_SIZE;
    const uint8_t *q = block + 2 + K_SCALE_SIZE + QK_K / 8;
    uint32_t aux[4];
    memcpy(&aux[0], block + 2, 4); /* little-endian host, as u32::from_le_bytes */
    memcpy(&aux[1], block + 6, 4);
    memcpy(&aux[2], block + 10, 4);
    uint32_t tmp = aux[2];
    aux[2] = ((aux[0] >> 4) & KMASK2) | (((tmp >> 4) & KMASK1) << 4);
    aux[3] = ((aux[1] >> 4) & KMASK2) | (((tmp >> 6) & KMASK1) << 4);
    aux[0] = (aux[0] & KMASK2) | ((tmp & KMASK1) << 4);
    aux[1] = (aux[1] & KMASK2) | (((tmp >> 2) & KMASK1) << 4);
    int8_t scales[16];
    memcpy(scales, aux, 16);
    int is = 0, oi = 0;
    uint8_t m = 1;
    for (int n = 0; n < QK_K / 128; n++) {
        unsigned shift = 0;
        for (int j = 0; j < 4; j++) {
            float dl = d_all * (float)(int8_t)(scales[is] - 32);
            is++;
            for (int l = 0; l < 16; l++) {
                int8_t h = (hm[l] & m) ? 0 : 4;
                out[oi++] = dl * (float)(int8_t)((int8_t)((q[l] >> shift) & 3) - h);
            }
            dl = d_all * (float)(int8_t)(scales[is] - 32);
            is++;
            for (int l = 0; l < 16; l++) {
                int8_t h = (hm[l + 16] & m) ? 0 : 4;
                out[oi++] = dl * (float)(int8_t)((int8_t)((q[l + 16] >> shift) & 3) - h);
            }
            shift += 2;
            m <<= 1;
        }
        q += 32;
    }
}

/* rlx-cpu/src/gguf_matmul.rs:25-37 */
static void dequant_block(int scheme, const uint8_t *block, float *out) {
    switch (scheme) {
    case ORC_Q4K: orc_dequant_q4_k_block(block, out); break;
    case ORC_Q5K: orc_dequant_q5_k_block(block, out); break;
    case ORC_Q6K: orc_dequant_q6_k_block(block, out, 0); break;
    case ORC_Q8K: orc_dequant_q8_k_block(block, out); break;
    case ORC_Q2K: orc_dequant_q2_k_block(block, out); break;
    case ORC_Q3K: orc_dequant_q3_k_block(block, out); break;
    case ORC_Q4_0: orc_dequant_q4_0_block(block, out); break;
    case ORC_Q8_0: orc_dequant_q8_0_block(block, out); break;
    default: break;
    }
}

/* Whole-tensor forms (rlx-gguf/src/lib.rs:600-633, 932-1145). Returns 0, or -1 on a bad size. */
int orc_dequant(int scheme, const uint8_t *bytes, int64_t nbytes, int64_t n, float *out) {
    int be = orc_block_elems(scheme), bb = orc_block_bytes(scheme);
    if (be == 0 || n % be != 0) return -1;
    int64_t nb = n / be;
    if (nbytes != nb * bb) return -1;
    float tmp[QK_K];
    for (int64_t i = 0; i < nb; i++) {
        if (scheme == ORC_Q6K) orc_dequant_q6_k_block(bytes + i * bb, tmp, 1); /* lib.rs:1070-1112 reads the scales as i8 */
        else dequant_block(scheme, bytes + i * bb, tmp);
        memcpy(out + i * be, tmp, (size_t)be * sizeof(float));
    }
    return 0;
}

/* The same, with the block decoders the matmul dispatches to (rlx-cpu/src/gguf_matmul.rs:25-37): differs from
 * orc_dequant only for Q6_K (scale bytes read as unsigned). */
int orc_dequant_matmul_blocks(int scheme, const uint8_t *bytes, int64_t nbytes, int64_t n, float *out) {
    int be = orc_block_elems(scheme), bb = orc_block_bytes(scheme);
    if (be == 0 || n % be != 0) return -1;
    int64_t nb = n / be;
    if (nbytes != nb * bb) return -1;
    float tmp[QK_K];
    for (int64_t i = 0; i < nb; i++) {
        dequant_block(scheme, bytes + i * bb, tmp);
        memcpy(out + i * be, tmp, (size_t)be * sizeof(float));
    }
    return 0;
}

/* ---- RmsNorm ------------------------------------------------------------ */

/* rlx-cpu/src/thunk.rs:8839-8869 */
void orc_rms_norm(const float *input, const float *gamma, const float *beta, float *output, int64_t rows, int64_t h, float eps) {
    float inv_h = 1.0f / (float)h;
    for (int64_t row = 0; row < rows; row++) {
        const float *in_row = input + row * h;
        float *out_row = output + row * h;
        float sumsq = 0.0f;
        for (int64_t i = 0; i < h; i++) {
            float sq = in_row[i] * in_row[i];
            sumsq += sq;
        }
        float mean = sumsq * inv_h;
        float inv_rms = 1.0f / sqrtf(mean + eps);
        for (int64_t i = 0; i < h; i++) {
            float t = in_row[i] * inv_rms;
            t = t * gamma[i];
            out_row[i] = t + beta[i];
        }
    }
}

/* ---- FusedSwiGLU -------------------------------------------------------- */

/* rlx-cpu/src/thunk.rs:10337-10366: input rows of 2 n values, output rows of n; up is the low half unless gate_first. */
void orc_fused_swiglu(const float *inp, float *out, int64_t n_half, int64_t total, int gate_first) {
    int64_t n = n_half, outer = total / n;
    for (int64_t o = 0; o < outer; o++) {
        const float *in_row = inp + o * 2 * n;
        float *out_row = out + o * n;
        for (int64_t i = 0; i < n; i++) {
            float up = gate_first ? in_row[n + i] : in_row[i];
            float gate = gate_first ? in_row[i] : in_row[n + i];
            float den = 1.0f + expf(-gate);
            float sg = gate / den;
            out_row[i] = up * sg;
        }
    }
}

/* ---- tied LM head ------------------------------------------------------ */

/* rlx-cpu/src/lm_head.rs:46-77: one row of the packed matrix against `hidden`, block by block, f32 accumulation. */
static float row_dot_gguf(const float *hidden, const uint8_t *w_bytes, int64_t row, int64_t n_embd, int scheme) {
    int64_t k = n_embd, row_start = row * k, row_end = row_start + k;
    int be = orc_block_elems(scheme), bb = orc_block_bytes(scheme);
    int64_t first_block = row_start / be, last_block = (row_end - 1) / be;
    float block_f32[QK_K];
    float dot = 0.0f;
    for (int64_t bi = first_block; bi <= last_block; bi++) {
        dequant_block(scheme, w_bytes + bi * bb, block_f32);
        int64_t idx0 = bi * be;
        for (int t = 0; t < be; t++) {
            int64_t idx = idx0 + t;
            if (idx < row_start || idx >= row_end) continue;
            float prod = hidden[idx - row_start] * block_f32[t];
            dot += prod;
        }
    }
    return dot;
}

/* rlx-cpu/src/lm_head.rs:223-248: first row with the largest dot; starts from (0, -inf), replaced only on `>`. */
int orc_gguf_tied_lm_argmax(const float *hidden, const uint8_t *w_bytes, int64_t w_nbytes, int64_t n_embd, int64_t n_vocab,
                            int scheme, uint32_t *best_idx, float *best_val) {
    int be = orc_block_elems(scheme), bb = orc_block_bytes(scheme);
    if (be == 0 || (n_embd * n_vocab) % be != 0 || w_nbytes != (n_embd * n_vocab) / be * bb) return -1;
    uint32_t bi = 0;
    float bv = -INFINITY;
    for (int64_t j = 0; j < n_vocab; j++) {
        float dot = row_dot_gguf(hidden, w_bytes, j, n_embd, scheme);
        if (dot > bv) {
            bv = dot;
            bi = (uint32_t)j;
        }
    }
    *best_idx = bi;
    *best_val = bv;
    return 0;
}

/* rlx-cpu/src/lm_head.rs:172-198 with topk_from_scores (:130-141): the cap largest (row, dot) pairs, largest first, cap
 * clamped to [1, n_vocab]. The reference's early exit (row_dot_gguf_early_exit, :79-128) only drops rows whose bound
 * says they cannot reach the current floor, so the answer is the top of the full score list; its order among equal
 * scores is whatever select_nth_unstable leaves, here the smaller row comes first. NaN scores are left out (the
 * reference's partial_cmp treats them as equal to anything). Returns the number of pairs written, or -1. */
int orc_gguf_tied_lm_topk(const float *hidden, const uint8_t *w_bytes, int64_t w_nbytes, int64_t n_embd, int64_t n_vocab,
                          int scheme, int cap, uint32_t *out_idx, float *out_val) {
    int be = orc_block_elems(scheme), bb = orc_block_bytes(scheme);
    if (be == 0 || (n_embd * n_vocab) % be != 0 || w_nbytes != (n_embd * n_vocab) / be * bb) return -1;
    if (cap > n_vocab) cap = (int)n_vocab;
    if (cap < 1) cap = 1;
    int have = 0;
    for (int64_t j = 0; j < n_vocab; j++) {
        float dot = row_dot_gguf(hidden, w_bytes, j, n_embd, scheme);
        if (dot != dot) continue;
        /* insertion into the sorted list: after every entry with a value >= dot (earlier rows win ties) */
        int pos = have;
        while (pos > 0 && out_val[pos - 1] < dot) pos--;
        if (pos >= cap) continue;
        int last = have < cap ? have : cap - 1;
        for (int i = last; i > pos; i--) {
            out_val[i] = out_val[i - 1];
            out_idx[i] = out_idx[i - 1];
        }
        out_val[pos] = dot;
        out_idx[pos] = (uint32_t)j;
        if (have < cap) have++;
    }
    return have;
}

/* ---- matmul ------------------------------------------------------------ */

/* rlx-cpu/src/gguf_matmul.rs:40-95, loop for loop: out zeroed, then for each block in
 * storage order, for each element t: j = idx / k, p = idx % k, out[mi*n+j] += x[mi*k+p]*w. */
int orc_gguf_matmul_bt(const float *x, const uint8_t *w_bytes, int64_t w_nbytes, float *out, int64_t m, int64_t k,
                       int64_t n, int scheme) {
    int be = orc_block_elems(scheme), bb = orc_block_bytes(scheme);
    if (be == 0) return -1;
    int64_t total = k * n;
    if (total % be != 0) return -1;
    int64_t num_blocks = total / be;
    if (w_nbytes != num_blocks * bb) return -1;
    for (int64_t i = 0; i < m * n; i++) out[i] = 0.0f;
    float blk[QK_K];
    if (m == 1) {
        for (int64_t bi = 0; bi < num_blocks; bi++) {
            dequant_block(scheme, w_bytes + bi * bb, blk);
            int64_t idx0 = bi * be;
            for (int t = 0; t < be; t++) {
                int64_t idx = idx0 + t;
                int64_t j = idx / k;
                int64_t p = idx % k;
                float prod = x[p] * blk[t];
                out[j] = out[j] + prod;
            }
        }
        return 0;
    }
    for (int64_t bi = 0; bi < num_blocks; bi++) {
        dequant_block(scheme, w_bytes + bi * bb, blk);
        int64_t idx0 = bi * be;
        for (int t = 0; t < be; t++) {
            int64_t idx = idx0 + t;
            int64_t j = idx / k;
            int64_t p = idx % k;
            float w_val = blk[t];
            for (int64_t mi = 0; mi < m; mi++) {
                float prod = x[mi * k + p] * w_val;
                out[mi * n + j] = out[mi * n + j] + prod;
            }
        }
    }
    return 0;
}

/* rlx-cpu/src/gguf_matmul.rs:101-139 with grouped_moe_sort_plan (:178-206) and grouped_moe_unpermute_out (:208-219):
 * rows are gathered per expert (stable order), each expert's slab multiplies its rows with orc_gguf_matmul_bt, and
 * the packed result is scattered back. expert_idx holds float-encoded indices; an index outside [0, num_experts)
 * returns -2 (the reference debug-asserts and then slices out of range). */
int orc_gguf_grouped_matmul_bt(const float *x, const uint8_t *w_bytes, int64_t w_nbytes, const float *expert_idx, float *out,
                               int64_t m, int64_t k, int64_t n, int64_t num_experts, int scheme) {
    int be = orc_block_elems(scheme), bb = orc_block_bytes(scheme);
    if (be == 0 || (k * n) % be != 0 || num_experts <= 0) return -1;
    int64_t slab_bytes = (k * n) / be * bb;
    if (w_nbytes != num_experts * slab_bytes) return -1;
    int64_t *counts = (int64_t *)calloc((size_t)num_experts, sizeof(int64_t));
    int64_t *offsets = (int64_t *)calloc((size_t)num_experts + 1, sizeof(int64_t));
    int64_t *write_idx = (int64_t *)calloc((size_t)num_experts, sizeof(int64_t));
    int64_t *original_pos = (int64_t *)calloc((size_t)(m > 0 ? m : 1), sizeof(int64_t));
    float *packed_in = (float *)malloc(sizeof(float) * (size_t)(m * k > 0 ? m * k : 1));
    float *packed_out = (float *)calloc((size_t)(m * n > 0 ? m * n : 1), sizeof(float));
    int rc = 0;
    for (int64_t i = 0; i < m; i++) {
        int64_t e = (int64_t)expert_idx[i];
        if (expert_idx[i] < 0.0f || e >= num_experts) { rc = -2; goto done; }
        counts[e] += 1;
    }
    for (int64_t e = 0; e < num_experts; e++) offsets[e + 1] = offsets[e] + counts[e];
    for (int64_t i = 0; i < m; i++) {
        int64_t e = (int64_t)expert_idx[i];
        int64_t dst_row = offsets[e] + write_idx[e];
        memcpy(packed_in + dst_row * k, x + i * k, sizeof(float) * (size_t)k);
        original_pos[dst_row] = i;
        write_idx[e] += 1;
    }
    for (int64_t e = 0; e < num_experts; e++) {
        int64_t count = offsets[e + 1] - offsets[e];
        if (count == 0) continue;
        int64_t in_start = offsets[e];
        rc = orc_gguf_matmul_bt(packed_in + in_start * k, w_bytes + e * slab_bytes, slab_bytes, packed_out + in_start * n, count, k,
                                n, scheme);
        if (rc != 0) goto done;
    }
    for (int64_t pi = 0; pi < m; pi++) {
        int64_t i = original_pos[pi];
        memcpy(out + i * n, packed_out + pi * n, sizeof(float) * (size_t)n);
    }
done:
    free(counts); free(offsets); free(write_idx); free(original_pos); free(packed_in); free(packed_out);
    return rc;
}

/* Error yardstick: same decoded weights, products and sums in f64. Rows [n0, n1) only. */
int orc_gguf_matmul_f64(const float *x, const uint8_t *w_bytes, int64_t w_nbytes, double *out, int64_t m, int64_t k,
                        int64_t n, int scheme, int64_t n0, int64_t n1) {
    int be = orc_block_elems(scheme), bb = orc_block_bytes(scheme);
    if (be == 0 || k % be != 0) return -1;
    if (w_nbytes != (k * n / be) * bb) return -1;
    int64_t bpr = k / be;
    float blk[QK_K];
    for (int64_t j = n0; j < n1; j++) {
        for (int64_t mi = 0; mi < m; mi++) out[mi * (n1 - n0) + (j - n0)] = 0.0;
        for (int64_t b = 0; b < bpr; b++) {
            dequant_block(scheme, w_bytes + (j * bpr + b) * bb, blk);
            for (int64_t mi = 0; mi < m; mi++) {
                double acc = 0.0;
                const float *xr = x + mi * k + b * be;
                for (int t = 0; t < be; t++) acc += (double)xr[t] * (double)blk[t];
                out[mi * (n1 - n0) + (j - n0)] += acc;
            }
        }
    }
    return 0;
}

/* ---- FakeQuantize (rlx-cpu/src/thunk.rs:11159-11253, 14163-14175) ------- */

enum { ORC_SCALE_PER_BATCH = 0, ORC_SCALE_EMA = 1, ORC_SCALE_FIXED = 2 };
enum { ORC_ROUND_HALF_AWAY = 0, ORC_ROUND_HALF_EVEN = 1 };

static float clampf(float v, float lo, float hi) {
    /* Rust f32::clamp: NaN passes through. */
    if (v < lo) return lo;
    if (v > hi) return hi;
    return v;
}

static float fmax_rust(float a, float b) {
    /* Rust f32::max: if one side is NaN the other is returned. */
    if (a != a) return b;
    if (b != b) return a;
    return a > b ? a : b;
}

/* x, out: len floats. codes (optional): len int8 integer codes q. state: chan_dim floats for
 * EMA (updated in place) / Fixed. scales_out (optional): chan_dim. Returns 0, -1 on bad bits. */
int orc_fake_quantize(const float *x, float *out, int8_t *codes, int64_t len, int64_t chan_dim, int64_t inner, int bits,
                      int scale_mode, float decay, float *state, int round_mode, float *scales_out) {
    float q_max;
    switch (bits) {
    case 8: q_max = 127.0f; break;
    case 4: q_max = 7.0f; break;
    case 2: q_max = 1.0f; break;
    default: return -1;
    }
    if (chan_dim < 1) chan_dim = 1;
    float *scale = scales_out;
    float local_scale[1];
    float *heap = NULL;
    if (!scale) {
        if (chan_dim == 1) scale = local_scale;
        else scale = heap = (float *)malloc((size_t)chan_dim * sizeof(float));
    }
    if (scale_mode == ORC_SCALE_PER_BATCH || scale_mode == ORC_SCALE_EMA) {
        float *max_abs = (float *)malloc((size_t)chan_dim * sizeof(float));
        for (int64_t c = 0; c < chan_dim; c++) max_abs[c] = 0.0f;
        for (int64_t i = 0; i < len; i++) {
            int64_t c = chan_dim == 1 ? 0 : (i / inner) % chan_dim;
            float a = fabsf(x[i]);
            if (a > max_abs[c]) max_abs[c] = a;
        }
        for (int64_t c = 0; c < chan_dim; c++) {
            float cur = fmax_rust(max_abs[c] / q_max, 1e-12f);
            if (scale_mode == ORC_SCALE_EMA) {
                float blended;
                if (state[c] <= 0.0f) {
                    blended = cur;
                } else {
                    float a = decay * state[c];
                    float b = (1.0f - decay) * cur;
                    blended = a + b;
                }
                state[c] = blended;
                scale[c] = blended;
            } else {
                scale[c] = cur;
            }
        }
        free(max_abs);
    } else {
        for (int64_t c = 0; c < chan_dim; c++) scale[c] = fmax_rust(state[c], 1e-12f);
    }
    for (int64_t i = 0; i < len; i++) {
        int64_t c = chan_dim == 1 ? 0 : (i / inner) % chan_dim;
        float s = scale[c];
        float r = x[i] / s;
        r = round_mode == ORC_ROUND_HALF_EVEN ? rintf(r) : roundf(r);
        float qv = clampf(r, -q_max, q_max);
        out[i] = qv * s;
        if (codes) codes[i] = (qv != qv) ? 0 : (int8_t)qv;
    }
    if (heap) free(heap);
    return 0;
}

/* ---- Philox4x32-10 (rlx-ir/src/rng.rs:43-143) ---------------------------- */

typedef struct {
    uint32_t seed[2];
    uint32_t counter[4];
    uint32_t buffer[4];
    uint32_t cursor;
    uint32_t m0; /* 0xD2561A75 in the reference (rng.rs:55); Random123's is 0xD2511F53 */
} orc_philox;

void orc_philox_init(orc_philox *p, uint64_t seed, uint32_t m0) {
    p->seed[0] = (uint32_t)(seed & 0xFFFFFFFFu);
    p->seed[1] = (uint32_t)(seed >> 32);
    memset(p->counter, 0, sizeof p->counter);
    memset(p->buffer, 0, sizeof p->buffer);
    p->cursor = 4;
    p->m0 = m0;
}

void orc_philox_set_counter(orc_philox *p, const uint32_t c[4]) {
    memcpy(p->counter, c, sizeof p->counter);
    p->cursor = 4;
}

static void philox_fill(orc_philox *p) {
    uint32_t s[4], key[2];
    memcpy(s, p->counter, sizeof s);
    key[0] = p->seed[0];
    key[1] = p->seed[1];
    for (int r = 0; r < 10; r++) {
        uint64_t p0 = (uint64_t)s[0] * (uint64_t)p->m0;
        uint64_t p1 = (uint64_t)s[2] * 0xCD9E8D57ull;
        uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0;
        uint32_t hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
        uint32_t n0 = hi1 ^ s[1] ^ key[0];
        uint32_t n2 = hi0 ^ s[3] ^ key[1];
        s[0] = n0;
        s[1] = lo1;
        s[2] = n2;
        s[3] = lo0;
        key[0] += 0x9E3779B9u;
        key[1] += 0xBB67AE85u;
    }
    memcpy(p->buffer, s, sizeof s);
    p->cursor = 0;
    if (++p->counter[0] == 0)
        if (++p->counter[1] == 0)
            if (++p->counter[2] == 0) ++p->counter[3];
}

uint32_t orc_philox_next_u32(orc_philox *p) {
    if (p->cursor >= 4) philox_fill(p);
    return p->buffer[p->cursor++];
}

float orc_philox_next_f32(orc_philox *p) {
    uint32_t bits = orc_philox_next_u32(p) >> 8;
    return (float)bits / (float)(1u << 24);
}

/* rng.rs:121-127. Uses this platform's f32 libm (logf/sqrtf/cosf): last-ulp parity unpinned. */
float orc_philox_normal(orc_philox *p) {
    float u1 = orc_philox_next_f32(p);
    if (u1 < 1.17549435e-38f) u1 = 1.17549435e-38f;
    float u2 = orc_philox_next_f32(p);
    float r = sqrtf(-2.0f * logf(u1));
    float theta = 2.0f * 3.14159274101257324f * u2;
    return r * cosf(theta);
}

void orc_philox_fill_u32(uint64_t seed, uint32_t m0, uint32_t *out, int64_t n) {
    orc_philox p;
    orc_philox_init(&p, seed, m0);
    for (int64_t i = 0; i < n; i++) out[i] = orc_philox_next_u32(&p);
}

void orc_philox_fill_uniform(uint64_t seed, float *out, int64_t n) {
    orc_philox p;
    orc_philox_init(&p, seed, 0xD2561A75u);
    for (int64_t i = 0; i < n; i++) out[i] = orc_philox_next_f32(&p);
}

void orc_philox_fill_normal(uint64_t seed, float *out, int64_t n) {
    orc_philox p;
    orc_philox_init(&p, seed, 0xD2561A75u);
    for (int64_t i = 0; i < n; i++) out[i] = orc_philox_normal(&p);
}

/* One Philox block for an explicit (counter, key): used by the known-answer test. */
void orc_philox_block(const uint32_t counter[4], const uint32_t key[2], uint32_t m0, uint32_t out[4]) {
    orc_philox p;
    orc_philox_init(&p, ((uint64_t)key[1] << 32) | key[0], m0);
    orc_philox_set_counter(&p, counter);
    philox_fill(&p);
    memcpy(out, p.buffer, sizeof p.buffer);
}
