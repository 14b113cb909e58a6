// Host-side format code: GGUF block geometry, the one-time repack into the device layout, the encoders that
// produce GGUF bytes from f32 (the reference has none: rlx-gguf is decode-only), and the reference's Philox stream.
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "common.hpp"

namespace rlx {

static inline uint16_t f32_to_f16_bits(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t exp = (x >> 23) & 0xFFu, man = x & 0x7FFFFFu;
    if (exp == 255) return (uint16_t)(sign | (man ? 0x7E00u | (man >> 13) : 0x7C00u));
    int e = (int)exp - 112;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u);
    if (e <= 0) {
        if (e < -10) return sign;
        man |= 0x800000u;
        int shift = 14 - e;
        uint32_t hm = man >> shift, rem = man & ((1u << shift) - 1), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (hm & 1))) hm++;
        return (uint16_t)(sign | hm);
    }
    uint32_t hm = man >> 13, rem = man & 0x1FFFu;
    uint16_t out = (uint16_t)(sign | ((uint32_t)e << 10) | hm);
    if (rem > 0x1000u || (rem == 0x1000u && (hm & 1))) out++;
    return out;
}

static inline float f16_bits_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, bits;
    if (exp == 0) {
        if (!man) bits = sign;
        else {
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(112 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) bits = sign | 0x7F800000u | (man << 13);
    else bits = sign | ((exp + 112) << 23) | (man << 13);
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

// ---- Q3_K fields ----------------------------------------------------------------------------------------

// Q3_K in the reference's field order (lib.rs:889-930): d, 12 scale bytes, 32 bytes of high-bit mask, 64 bytes of 2-bit
// codes. The value of element i is d * (scale[i / 16] - 32) * code(i) with code in [-4, 3]: at most 20 significant bits, so
// every product is exact in f32 in any order, and the super-block is the Q6_K super-block with codes code + 32 and signed
// scale bytes scale - 32. These two read the fields a Q6_K unit needs.
static void q3k_scales(const uint8_t *b, int scale[16]) {
    const uint8_t *s = b + 2;
    for (int j = 0; j < 4; j++) {
        scale[j] = (s[j] & 0xF) | ((s[8 + j] & 3) << 4);
        scale[4 + j] = (s[4 + j] & 0xF) | (((s[8 + j] >> 2) & 3) << 4);
        scale[8 + j] = (s[j] >> 4) | (((s[8 + j] >> 4) & 3) << 4);
        scale[12 + j] = (s[4 + j] >> 4) | (((s[8 + j] >> 6) & 3) << 4);
    }
}
static inline int q3k_code(const uint8_t *b, int i) {
    const uint8_t *hm = b + 14, *q = b + 46;
    const int h = i >> 7, pair = (i >> 5) & 3, l = i & 31;
    return ((q[32 * h + l] >> (2 * pair)) & 3) - ((hm[l] >> (4 * h + pair)) & 1 ? 0 : 4);
}

// ---- repack ---------------------------------------------------------------------------------------------

int repack_host(int scheme, uint32_t flags, const uint8_t *src, size_t nbytes, int64_t n, int64_t k, uint8_t *out) {
    Layout L = layout_of(scheme);
    // Q6_K scale bytes read as signed are stored XOR 0x80 (offset binary): the kernels subtract 128 from the byte
    const uint8_t q6_flip = (flags & RLX_QW_Q6K_SIGNED_SCALES) ? 0x80u : 0u;
    if (L.unit_k == 0 || L.block_elems == 0) {
        set_error("repack: scheme %d is not a claimed GGUF scheme (Q4_K=5, Q5_K=6, Q6_K=7, Q8_K=8, Q2_K=9, Q3_K=10, Q4_0=11, Q8_0=12)", scheme);
        return RLX_ERR_UNSUPPORTED;
    }
    if (n <= 0 || k <= 0 || k % L.block_elems != 0) {
        set_error("repack: k=%lld must be a positive multiple of the %d-element block (n=%lld)", (long long)k,
                  L.block_elems, (long long)n);
        return RLX_ERR_INVALID;
    }
    const int64_t bpr = k / L.block_elems;  // GGUF blocks per row
    if ((int64_t)nbytes != n * bpr * L.block_bytes) {
        set_error("repack: got %zu bytes, [%lld x %lld] needs %lld", nbytes, (long long)n, (long long)k,
                  (long long)(n * bpr * L.block_bytes));
        return RLX_ERR_INVALID;
    }
    WeightDims D = weight_dims(L, n, k);
    for (int64_t tile = 0; tile < D.row_tiles; tile++) {
        for (int64_t u = 0; u < D.units; u++) {
            uint8_t *unit = out + (tile * D.units + u) * L.unit_bytes;
            for (int l = 0; l < 64; l++) {
                const int nrow = l & 15, g = l >> 4;
                const int64_t r = tile * 16 + nrow;
                if (scheme == SCHEME_Q4_0 || scheme == SCHEME_Q8_0) {
                    for (int t = 0; t < 4; t++) {
                        const int64_t blk = u * 4 + t;
                        const bool live = r < n && blk < bpr;
                        const uint8_t *b = live ? src + (r * bpr + blk) * L.block_bytes : nullptr;
                        if (g == 0) {
                            uint16_t d = live ? (uint16_t)(b[0] | (b[1] << 8)) : 0;
                            memcpy(unit + L.quant_bytes + nrow * 8 + t * 2, &d, 2);
                        }
                        if (scheme == SCHEME_Q4_0) {
                            uint32_t word = 0;
                            for (int e = 0; e < 8; e++) {
                                int i = 8 * g + e;  // element inside the block: low nibbles first, then high nibbles
                                uint32_t q = live ? (i < 16 ? (b[2 + i] & 0xFu) : (uint32_t)(b[2 + i - 16] >> 4)) : 8u;
                                word |= q << (4 * nib_pos(e));
                            }
                            memcpy(unit + l * 16 + t * 4, &word, 4);
                        } else {
                            uint8_t *dst = unit + (t >> 1) * 1024 + l * 16 + (t & 1) * 8;
                            for (int e = 0; e < 8; e++) dst[e] = live ? (uint8_t)(b[2 + 8 * g + e] ^ 0x80u) : 0x80u;
                        }
                    }
                } else if (scheme == SCHEME_Q8K) {  // one super-block per unit: eight blocks of offset-binary bytes, f32 d
                    const bool live = r < n && u < bpr;
                    const uint8_t *b = live ? src + (r * bpr + u) * L.block_bytes : nullptr;
                    if (g == 0) {
                        if (live) memcpy(unit + 4096 + nrow * 4, b, 4);
                        else memset(unit + 4096 + nrow * 4, 0, 4);
                    }
                    for (int j = 0; j < 8; j++) {
                        uint8_t *dst = unit + (j >> 1) * 1024 + l * 16 + (j & 1) * 8;
                        for (int e = 0; e < 8; e++) dst[e] = live ? (uint8_t)(b[4 + 32 * j + 8 * g + e] ^ 0x80u) : 0x80u;
                    }
                } else if (scheme == SCHEME_Q2K) {  // one super-block per unit: 2-bit codes, 16 scale bytes, d and dmin
                    // the reference's field order (lib.rs:857-886): d, dmin, 16 scale bytes, 64 bytes of codes
                    const bool live = r < n && u < bpr;
                    const uint8_t *b = live ? src + (r * bpr + u) * L.block_bytes : nullptr;
                    if (g == 0) {
                        if (live) {
                            memcpy(unit + 1024 + nrow * 16, b + 4, 16);
                            memcpy(unit + 1280 + nrow * 4, b, 4);
                        } else {
                            memset(unit + 1024 + nrow * 16, 0, 16);
                            memset(unit + 1280 + nrow * 4, 0, 4);
                        }
                    }
                    uint32_t words[4] = {0, 0, 0, 0};
                    for (int j = 0; live && j < 8; j++)
                        for (int e = 0; e < 8; e++) {
                            const int i = 32 * j + 8 * g + e;  // element of the super-block
                            const int h = i >> 7, pair = (i >> 5) & 3, l5 = i & 31;
                            const uint32_t code = (uint32_t)(b[20 + 32 * h + l5] >> (2 * pair)) & 3u;
                            words[j >> 1] |= code << (16 * (e & 1) + 8 * (j & 1) + 2 * (e >> 1));
                        }
                    memcpy(unit + l * 16, words, 16);
                } else if (scheme == SCHEME_Q5K) {  // one super-block per unit: nibbles as Q4_K, fifth-bit words, 16 meta bytes
                    const bool live = r < n && u < bpr;
                    const uint8_t *b = live ? src + (r * bpr + u) * L.block_bytes : nullptr;
                    if (g == 0) {
                        if (live) memcpy(unit + 2560 + nrow * 16, b, 16);
                        else memset(unit + 2560 + nrow * 16, 0, 16);
                    }
                    uint32_t hb[2] = {0, 0};
                    for (int j = 0; j < 8; j++) {
                        uint32_t word = 0;
                        for (int e = 0; e < 8; e++) {
                            const int l5 = 8 * g + e;  // element of sub-block j
                            uint32_t nib = 0, bit = 0;
                            if (live) {
                                const uint8_t byte = b[48 + 32 * (j >> 1) + l5];
                                nib = (j & 1) ? (uint32_t)(byte >> 4) : (uint32_t)(byte & 0x0F);
                                bit = (uint32_t)(b[16 + l5] >> j) & 1u;
                            }
                            word |= nib << (4 * nib_pos(e));
                            hb[j >> 2] |= bit << ((q5k_hi_pos(e) + q5k_rot(j & 3)) & 31);
                        }
                        memcpy(unit + (j >> 2) * 1024 + l * 16 + (j & 3) * 4, &word, 4);
                    }
                    memcpy(unit + 2048 + l * 8, hb, 8);
                } else if (scheme == SCHEME_Q6K || scheme == SCHEME_Q3K) {
                    // one super-block per unit: low nibbles, high-bit words, scales, d. A Q3_K super-block is stored as the
                    // Q6_K super-block of the same values: codes + 32, scale bytes (scale - 32) XOR 0x80, the same d.
                    const bool live = r < n && u < bpr, q3 = scheme == SCHEME_Q3K;
                    const uint8_t *b = live ? src + (r * bpr + u) * L.block_bytes : nullptr;
                    if (g == 0) {
                        int sc3[16];
                        if (live && q3) q3k_scales(b, sc3);
                        for (int e = 0; e < 16; e++) {
                            const uint8_t byte = !live ? 0 : q3 ? (uint8_t)(int8_t)(sc3[e] - 32) : b[192 + e];
                            unit[3072 + nrow * 16 + e] = (uint8_t)(byte ^ (q3 ? 0x80u : q6_flip));
                        }
                        if (live) memcpy(unit + 3328 + nrow * 2, q3 ? b : b + 208, 2);
                        else memset(unit + 3328 + nrow * 2, 0, 2);
                    }
                    uint32_t hw[4] = {0, 0, 0, 0};
                    for (int j = 0; j < 8; j++) {
                        uint32_t word = 0;
                        for (int e = 0; e < 8; e++) {
                            const int i = 32 * j + 8 * g + e;  // element of the super-block
                            uint32_t code = 32;               // decodes to zero
                            if (live && q3) {
                                code = (uint32_t)(q3k_code(b, i) + 32);
                            } else if (live) {
                                const int h = i >> 7, quarter = (i >> 5) & 3, l5 = i & 31;
                                const uint8_t lowbyte = b[64 * h + 32 * (quarter & 1) + l5];
                                const uint32_t low = (quarter >> 1) ? (uint32_t)(lowbyte >> 4) : (uint32_t)(lowbyte & 0x0F);
                                const uint32_t high = (uint32_t)(b[128 + 32 * h + l5] >> (2 * quarter)) & 3u;
                                code = low | (high << 4);
                            }
                            word |= (code & 0xFu) << (4 * nib_pos(e));
                            hw[(j >> 2) * 2 + ((j & 3) >> 1)] |= (code >> 4) << ((q6k_hi_pos(e) + ((j & 1) ? 8 : 0)) & 31);
                        }
                        memcpy(unit + (j >> 2) * 1024 + l * 16 + (j & 3) * 4, &word, 4);
                    }
                    memcpy(unit + 2048 + l * 16, hw, 16);
                } else {  // Q4_K: one super-block per unit
                    const bool live = r < n && u < bpr;
                    const uint8_t *b = live ? src + (r * bpr + u) * L.block_bytes : nullptr;
                    if (g == 0) {
                        if (live) memcpy(unit + L.quant_bytes + nrow * 16, b, 16);
                        else memset(unit + L.quant_bytes + nrow * 16, 0, 16);
                    }
                    for (int j = 0; j < 8; j++) {
                        uint32_t word = 0;
                        for (int e = 0; e < 8; e++) {
                            int i = 8 * g + e;
                            uint32_t q = 0;
                            if (live) {
                                uint8_t byte = b[16 + 32 * (j >> 1) + i];
                                q = (j & 1) ? (uint32_t)(byte >> 4) : (byte & 0xFu);
                            }
                            word |= q << (4 * nib_pos(e));
                        }
                        memcpy(unit + (j >> 2) * 1024 + l * 16 + (j & 3) * 4, &word, 4);
                    }
                }
            }
        }
    }
    return RLX_OK;
}

// ---- encoders -------------------------------------------------------------------------------------------

// Q8_0 as llama.cpp quantize_row_q8_0_ref: d = amax/127, codes round(x / d) with d in f32, scale stored as f16.
static void quantize_q8_0(const float *x, int64_t n, uint8_t *out) {
    for (int64_t b = 0; b < n / 32; b++, x += 32, out += 34) {
        float amax = 0.f;
        for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(x[i]));
        float d = amax / 127.0f, id = d ? 1.0f / d : 0.0f;
        uint16_t h = f32_to_f16_bits(d);
        memcpy(out, &h, 2);
        for (int i = 0; i < 32; i++) out[2 + i] = (uint8_t)(int8_t)roundf(x[i] * id);
    }
}

// Q4_0 as llama.cpp quantize_row_q4_0_ref: d = max/-8 (max = signed value of largest magnitude), q = min(15, int(x/d + 8.5)).
static void quantize_q4_0(const float *x, int64_t n, uint8_t *out) {
    for (int64_t b = 0; b < n / 32; b++, x += 32, out += 18) {
        float amax = 0.f, mx = 0.f;
        for (int i = 0; i < 32; i++)
            if (fabsf(x[i]) > amax) { amax = fabsf(x[i]); mx = x[i]; }
        float d = mx / -8.0f, id = d ? 1.0f / d : 0.0f;
        uint16_t h = f32_to_f16_bits(d);
        memcpy(out, &h, 2);
        for (int j = 0; j < 16; j++) {
            int q0 = (int)(x[j] * id + 8.5f), q1 = (int)(x[16 + j] * id + 8.5f);
            q0 = q0 > 15 ? 15 : q0;
            q1 = q1 > 15 ? 15 : q1;
            out[2 + j] = (uint8_t)(q0 | (q1 << 4));
        }
    }
}

// Q4_K, simple deterministic variant (not llama.cpp's iterative make_qkx2_quants): per 32-element sub-block
// min = min(0, min x), scale = (max - min)/15; super-block d = max(scale)/63, dmin = max(-min)/63, both stored as
// f16 and read back before the 6-bit fields and nibbles are chosen, so decode(encode(x)) is consistent.
static void quantize_q4_k(const float *x, int64_t n, uint8_t *out) {
    for (int64_t sb = 0; sb < n / 256; sb++, x += 256, out += 144) {
        float scale[8], mn[8], max_scale = 0.f, max_min = 0.f;
        for (int j = 0; j < 8; j++) {
            float lo = 0.f, hi = x[32 * j];
            for (int i = 0; i < 32; i++) {
                lo = fminf(lo, x[32 * j + i]);
                hi = fmaxf(hi, x[32 * j + i]);
            }
            hi = fmaxf(hi, lo);
            scale[j] = (hi - lo) / 15.0f;
            mn[j] = -lo;
            max_scale = fmaxf(max_scale, scale[j]);
            max_min = fmaxf(max_min, mn[j]);
        }
        uint16_t hd = f32_to_f16_bits(max_scale / 63.0f), hm = f32_to_f16_bits(max_min / 63.0f);
        float d = f16_bits_to_f32(hd), dmin = f16_bits_to_f32(hm);
        uint8_t sc6[8], mn6[8];
        for (int j = 0; j < 8; j++) {
            int s = d > 0.f ? (int)roundf(scale[j] / d) : 0, m = dmin > 0.f ? (int)roundf(mn[j] / dmin) : 0;
            sc6[j] = (uint8_t)(s > 63 ? 63 : s);
            mn6[j] = (uint8_t)(m > 63 ? 63 : m);
        }
        memcpy(out, &hd, 2);
        memcpy(out + 2, &hm, 2);
        uint8_t *q = out + 4;
        for (int j = 0; j < 4; j++) {  // inverse of get_scale_min_k4 (rlx-gguf/src/lib.rs:743-751)
            q[j] = (uint8_t)((sc6[j] & 63) | ((sc6[j + 4] >> 4) << 6));
            q[j + 4] = (uint8_t)((mn6[j] & 63) | ((mn6[j + 4] >> 4) << 6));
            q[j + 8] = (uint8_t)((sc6[j + 4] & 0xF) | ((mn6[j + 4] & 0xF) << 4));
        }
        uint8_t *qs = out + 16;
        for (int p = 0; p < 4; p++) {
            for (int i = 0; i < 32; i++) {
                int code[2];
                for (int h = 0; h < 2; h++) {
                    int j = 2 * p + h;
                    float dj = d * (float)sc6[j], mj = dmin * (float)mn6[j];
                    int c = dj > 0.f ? (int)roundf((x[32 * j + i] + mj) / dj) : 0;
                    code[h] = c < 0 ? 0 : (c > 15 ? 15 : c);
                }
                qs[32 * p + i] = (uint8_t)(code[0] | (code[1] << 4));
            }
        }
    }
}

// ---- Philox4x32-10 (rlx-ir/src/rng.rs:43-143) ------------------------------------------------------------

struct Philox {
    uint32_t seed[2], counter[4], buffer[4];
    unsigned cursor;
    explicit Philox(uint64_t s) : seed{(uint32_t)s, (uint32_t)(s >> 32)}, counter{0, 0, 0, 0}, buffer{0, 0, 0, 0}, cursor(4) {}
    void refill() {
        uint32_t s[4] = {counter[0], counter[1], counter[2], counter[3]}, key[2] = {seed[0], seed[1]};
        for (int r = 0; r < 10; r++) {
            uint64_t p0 = (uint64_t)s[0] * 0xD2561A75ull, p1 = (uint64_t)s[2] * 0xCD9E8D57ull;
            uint32_t n0 = (uint32_t)(p1 >> 32) ^ s[1] ^ key[0], n2 = (uint32_t)(p0 >> 32) ^ s[3] ^ key[1];
            s[0] = n0; s[1] = (uint32_t)p1; s[2] = n2; s[3] = (uint32_t)p0;
            key[0] += 0x9E3779B9u;
            key[1] += 0xBB67AE85u;
        }
        memcpy(buffer, s, sizeof s);
        cursor = 0;
        if (++counter[0] == 0 && ++counter[1] == 0 && ++counter[2] == 0) ++counter[3];
    }
    uint32_t next_u32() {
        if (cursor >= 4) refill();
        return buffer[cursor++];
    }
    float next_f32() { return (float)(next_u32() >> 8) / 16777216.0f; }
    float normal() {
        float u1 = next_f32();
        if (u1 < 1.17549435e-38f) u1 = 1.17549435e-38f;
        float u2 = next_f32();
        float r = sqrtf(-2.0f * logf(u1));
        return r * cosf(2.0f * 3.14159274101257324f * u2);
    }
};

}  // namespace rlx

extern "C" {

int rlx_mi355x_block_elems(int scheme) { return rlx::layout_of(scheme).block_elems; }
int rlx_mi355x_block_bytes(int scheme) { return rlx::layout_of(scheme).block_bytes; }
int64_t rlx_mi355x_bytes_for(int scheme, int64_t n) {
    rlx::Layout L = rlx::layout_of(scheme);
    if (L.block_elems == 0 || n < 0 || n % L.block_elems != 0) return -1;
    return n / L.block_elems * L.block_bytes;
}

size_t rlx_mi355x_qweight_device_bytes_for(int scheme, int64_t n, int64_t k) {
    return (size_t)rlx::weight_dims(rlx::layout_of(scheme), n, k).bytes;
}

int rlx_mi355x_repack_host(int scheme, const void *gguf_bytes, size_t nbytes, int64_t n, int64_t k, void *out) {
    return rlx::repack_host(scheme, 0, (const uint8_t *)gguf_bytes, nbytes, n, k, (uint8_t *)out);
}
int rlx_mi355x_repack_host_ex(int scheme, uint32_t flags, const void *gguf_bytes, size_t nbytes, int64_t n, int64_t k, void *out) {
    return rlx::repack_host(scheme, flags, (const uint8_t *)gguf_bytes, nbytes, n, k, (uint8_t *)out);
}

int rlx_mi355x_quantize(int scheme, const float *src, int64_t n_elems, void *out) {
    rlx::Layout L = rlx::layout_of(scheme);
    if (L.block_elems == 0 || (scheme != rlx::SCHEME_Q4K && scheme != rlx::SCHEME_Q4_0 && scheme != rlx::SCHEME_Q8_0)) {
        rlx::set_error("quantize: scheme %d unsupported", scheme);
        return RLX_ERR_UNSUPPORTED;
    }
    if (n_elems < 0 || n_elems % L.block_elems != 0) {
        rlx::set_error("quantize: %lld elements is not a multiple of the %d-element block", (long long)n_elems, L.block_elems);
        return RLX_ERR_INVALID;
    }
    if (scheme == rlx::SCHEME_Q8_0) rlx::quantize_q8_0(src, n_elems, (uint8_t *)out);
    else if (scheme == rlx::SCHEME_Q4_0) rlx::quantize_q4_0(src, n_elems, (uint8_t *)out);
    else rlx::quantize_q4_k(src, n_elems, (uint8_t *)out);
    return RLX_OK;
}

void rlx_mi355x_philox_u32(uint64_t seed, uint32_t *out, int64_t n) {
    rlx::Philox p(seed);
    for (int64_t i = 0; i < n; i++) out[i] = p.next_u32();
}
void rlx_mi355x_philox_uniform(uint64_t seed, float *out, int64_t n) {
    rlx::Philox p(seed);
    for (int64_t i = 0; i < n; i++) out[i] = p.next_f32();
}
void rlx_mi355x_philox_normal(uint64_t seed, float *out, int64_t n) {
    rlx::Philox p(seed);
    for (int64_t i = 0; i < n; i++) out[i] = p.normal();
}

}  // extern "C"
