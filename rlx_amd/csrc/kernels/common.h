// Device-side helpers shared by every kernel: vector types, granule -> packed-half unpackers, MFMA wrappers.
// gfx950 only.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../layout.h"

namespace rlx {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

union Frag {  // one MFMA A/B operand: 8 halfs = 4 dwords
    half8_t h8;
    half2_t h2[4];
    uint32_t u[4];
    uint4_t u4;
};

__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
__device__ __forceinline__ uint32_t as_u32(half2_t h) { return __builtin_bit_cast(uint32_t, h); }
__device__ __forceinline__ float half_bits_to_float(uint32_t bits16) {
    return (float)__builtin_bit_cast(half_t, (uint16_t)bits16);  // exact IEEE widening (v_cvt_f32_f16)
}

// 0x6400 is 1024.0 in binary16 and its ulp is 1, so (0x6400 | v) is the half 1024 + v for 0 <= v < 1024.
constexpr uint32_t MAGIC = 0x64006400u;

// (a & mask) | magic in one VALU op (v_and_or_b32). gfx9 VOP3 encodings take no literal and at most one scalar
// operand, so with three compile-time constants the compiler emits v_and + v_or instead. The two empty asm
// statements only hide the constants from constant folding (mask in an SGPR, magic in a VGPR); the and/or itself
// stays ordinary code, so the compiler's MFMA hazard tracking sees every register it writes.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t magic) {
    asm("" : "+s"(mask));
    asm("" : "+v"(magic));
    return (a & mask) | magic;
}

// 4-bit granule word -> four half2 registers holding (q - OFF) for the 8 weights, fragment order.
// OFF = 8 for Q4_0 (signed codes), 0 for Q4_K. All results are exact integers.
template <int OFF>
__device__ __forceinline__ void unpack_q4(uint32_t w, Frag &f) {
    const half2_t sub_lo = {(half_t)(-(1024 + OFF)), (half_t)(-(1024 + OFF))};
    const half2_t mul_hi = {(half_t)0.0625f, (half_t)0.0625f};
    const half2_t sub_hi = {(half_t)(-(64 + OFF)), (half_t)(-(64 + OFF))};
    uint32_t w2 = w >> 8;
    half2_t a0 = as_half2(and_or(w, 0x000F000Fu, MAGIC));   // 1024 + q
    half2_t a1 = as_half2(and_or(w, 0x00F000F0u, MAGIC));   // 1024 + 16 q
    half2_t a2 = as_half2(and_or(w2, 0x000F000Fu, MAGIC));
    half2_t a3 = as_half2(and_or(w2, 0x00F000F0u, MAGIC));
    f.h2[0] = a0 + sub_lo;
    f.h2[1] = __builtin_elementwise_fma(a1, mul_hi, sub_hi);  // (1024+16q)/16 - 64 - OFF, single rounding of an exact value
    f.h2[2] = a2 + sub_lo;
    f.h2[3] = __builtin_elementwise_fma(a3, mul_hi, sub_hi);
}

// Q4_K granule word -> sc * q (exact integers <= 945) given sc as a half2 splat.
__device__ __forceinline__ void unpack_q4_scaled(uint32_t w, half2_t sc, Frag &f) {
    const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
    const half2_t k64 = {(half_t)64.0f, (half_t)64.0f};
    const half2_t r16 = {(half_t)0.0625f, (half_t)0.0625f};
    half2_t neg_lo = -(sc * k1024);  // exact: sc < 64
    half2_t neg_hi = -(sc * k64);
    half2_t sc16 = sc * r16;         // exact power-of-two scaling
    uint32_t w2 = w >> 8;
    half2_t a0 = as_half2(and_or(w, 0x000F000Fu, MAGIC));
    half2_t a1 = as_half2(and_or(w, 0x00F000F0u, MAGIC));
    half2_t a2 = as_half2(and_or(w2, 0x000F000Fu, MAGIC));
    half2_t a3 = as_half2(and_or(w2, 0x00F000F0u, MAGIC));
    f.h2[0] = __builtin_elementwise_fma(a0, sc, neg_lo);
    f.h2[1] = __builtin_elementwise_fma(a1, sc16, neg_hi);
    f.h2[2] = __builtin_elementwise_fma(a2, sc, neg_lo);
    f.h2[3] = __builtin_elementwise_fma(a3, sc16, neg_hi);
}

// Q5_K: the same two decoders with the fifth bits merged into the magic numbers first. hx is the half's high-bit word
// rotated right by q5k_rot(t) for code word t (see layout.h); sc * q <= 63 * 31 stays exact in binary16.
__device__ __forceinline__ void q5_magic(uint32_t w, uint32_t hx, uint32_t a[4]) {
    const uint32_t w2 = w >> 8, h1 = hx >> 1;
    a[0] = (hx & 0x00100010u) | and_or(w, 0x000F000Fu, MAGIC);   // 1024 + q
    a[1] = (hx & 0x01000100u) | and_or(w, 0x00F000F0u, MAGIC);   // 1024 + 16 q
    a[2] = (h1 & 0x00100010u) | and_or(w2, 0x000F000Fu, MAGIC);
    a[3] = (h1 & 0x01000100u) | and_or(w2, 0x00F000F0u, MAGIC);
}
__device__ __forceinline__ void unpack_q5(uint32_t w, uint32_t hx, Frag &f) {  // q, exact
    const half2_t sub_lo = {(half_t)(-1024.0f), (half_t)(-1024.0f)};
    const half2_t mul_hi = {(half_t)0.0625f, (half_t)0.0625f};
    const half2_t sub_hi = {(half_t)(-64.0f), (half_t)(-64.0f)};
    uint32_t a[4];
    q5_magic(w, hx, a);
    f.h2[0] = as_half2(a[0]) + sub_lo;
    f.h2[1] = __builtin_elementwise_fma(as_half2(a[1]), mul_hi, sub_hi);
    f.h2[2] = as_half2(a[2]) + sub_lo;
    f.h2[3] = __builtin_elementwise_fma(as_half2(a[3]), mul_hi, sub_hi);
}
__device__ __forceinline__ void unpack_q5_scaled(uint32_t w, uint32_t hx, half2_t sc, Frag &f) {  // sc * q, exact
    const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
    const half2_t k64 = {(half_t)64.0f, (half_t)64.0f};
    const half2_t r16 = {(half_t)0.0625f, (half_t)0.0625f};
    const half2_t neg_lo = -(sc * k1024), neg_hi = -(sc * k64), sc16 = sc * r16;
    uint32_t a[4];
    q5_magic(w, hx, a);
    f.h2[0] = __builtin_elementwise_fma(as_half2(a[0]), sc, neg_lo);
    f.h2[1] = __builtin_elementwise_fma(as_half2(a[1]), sc16, neg_hi);
    f.h2[2] = __builtin_elementwise_fma(as_half2(a[2]), sc, neg_lo);
    f.h2[3] = __builtin_elementwise_fma(as_half2(a[3]), sc16, neg_hi);
}

// Q8_0 granule (two words of offset-binary bytes) -> signed codes as halfs, fragment order.
__device__ __forceinline__ void unpack_q8(uint32_t w0, uint32_t w1, Frag &f) {
    const half2_t sub = {(half_t)(-1152.0f), (half_t)(-1152.0f)};  // 1024 + 128
    const uint32_t c64 = 0x64646464u;
    // v_perm_b32: selector byte 0..3 picks from the second source, 4..7 from the first.
    half2_t a0 = as_half2(__builtin_amdgcn_perm(c64, w0, 0x04010400u));  // bytes 0,1
    half2_t a1 = as_half2(__builtin_amdgcn_perm(c64, w0, 0x04030402u));  // bytes 2,3
    half2_t a2 = as_half2(__builtin_amdgcn_perm(c64, w1, 0x04010400u));
    half2_t a3 = as_half2(__builtin_amdgcn_perm(c64, w1, 0x04030402u));
    f.h2[0] = a0 + sub;
    f.h2[1] = a1 + sub;
    f.h2[2] = a2 + sub;
    f.h2[3] = a3 + sub;
}

// Q4_K: the eight 6-bit (scale, min) pairs of a super-block from its 12 packed bytes held in three words,
// all eight at once (rlx-gguf/src/lib.rs:743-751). Byte j%4 of sc[j/4] / mn[j/4] is the field of sub-block j.
__device__ __forceinline__ void q4k_scales(uint32_t s0, uint32_t s1, uint32_t s2, uint32_t sc[2], uint32_t mn[2]) {
    sc[0] = s0 & 0x3F3F3F3Fu;
    mn[0] = s1 & 0x3F3F3F3Fu;
    sc[1] = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);
    mn[1] = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
}

// Q6_K granule: code word w (eight low nibbles) and its high-bit word hx (the pair's word as stored for the even code
// word, rotated right by 8 for the odd one) -> sc * (q - 32) as halfs in fragment order, sc given as a half2 splat of an
// integer in [-128, 255] (the scale byte read as unsigned or as signed). (q - 32) is exact; the product is exact up to 2048
// and rounded to binary16 above (|.| <= 8160).
__device__ __forceinline__ void unpack_q6_scaled(uint32_t w, uint32_t hx, half2_t sc, Frag &f) {
    const half2_t off = {(half_t)(-1056.0f), (half_t)(-1056.0f)};   // 1024 + 32
    const half2_t r16 = {(half_t)0.0625f, (half_t)0.0625f};
    const half2_t m96 = {(half_t)(-96.0f), (half_t)(-96.0f)};        // (1024 + 16 q) / 16 - 96 = q - 32
    const half2_t sc16 = sc * r16, neg96 = sc * m96;                 // both exact: sc has 8 bits
    const uint32_t w2 = w >> 8, h2 = hx >> 2;
    const uint32_t a0 = (hx & 0x00300030u) | and_or(w, 0x000F000Fu, MAGIC);   // 1024 + q
    const uint32_t a1 = (hx & 0x03000300u) | and_or(w, 0x00F000F0u, MAGIC);   // 1024 + 16 q
    const uint32_t a2 = (h2 & 0x00300030u) | and_or(w2, 0x000F000Fu, MAGIC);
    const uint32_t a3 = (h2 & 0x03000300u) | and_or(w2, 0x00F000F0u, MAGIC);
    f.h2[0] = (as_half2(a0) + off) * sc;
    f.h2[1] = __builtin_elementwise_fma(as_half2(a1), sc16, neg96);
    f.h2[2] = (as_half2(a2) + off) * sc;
    f.h2[3] = __builtin_elementwise_fma(as_half2(a3), sc16, neg96);
}

// Q2_K: byte BYTE (0 / 1) of each 16-bit half of `w` holds four 2-bit codes at bits 0-1, 2-3, 4-5, 6-7; element pair i of
// the fragment is (low half, high half) at bits 2 i of that byte. ((w >> s) & 0x00030003) | magic is 1024 + q, and one fma
// with sc and -1024 sc turns it into sc * q (sc <= 15, q <= 3: exact integers, rounded once from an exact value).
template <int BYTE>
__device__ __forceinline__ void unpack_q2_scaled(uint32_t w, half2_t sc, Frag &f) {
    const half2_t m1024 = {(half_t)(-1024.0f), (half_t)(-1024.0f)};
    const half2_t nsc = sc * m1024;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t x = (8 * BYTE + 2 * i) ? (w >> (8 * BYTE + 2 * i)) : w;
        f.h2[i] = __builtin_elementwise_fma(as_half2(and_or(x, 0x00030003u, MAGIC)), sc, nsc);
    }
}

// half2 splat of the integer byte b (0..255), exact: bytes [b, 0x64, b, 0x64] = 1024 + b, minus 1024
__device__ __forceinline__ half2_t splat_ubyte_half(uint32_t b) {
    const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
    return as_half2(MAGIC | b | (b << 16)) - k1024;
}
// The same minus `bias` = splat of 1024 + off: the byte read as b - off (off = 128 undoes an offset-binary store).
__device__ __forceinline__ half2_t splat_ubyte_half(uint32_t b, half2_t bias) { return as_half2(MAGIC | b | (b << 16)) - bias; }
__device__ __forceinline__ half2_t ubyte_bias(int off) {
    const half_t v = (half_t)(float)(1024 + off);
    return half2_t{v, v};
}

__device__ __forceinline__ float ubyte_to_float(uint32_t w, int byte) { return (float)((w >> (8 * byte)) & 0xFFu); }

// D(16x16) += A(16x32) * B(32x16), halfs in, f32 accumulate. Lane l: A row / B column l & 15, k-slice 8*(l>>4)..+7;
// D column l & 15, rows 4*(l>>4)..+3.
__device__ __forceinline__ float4_t mfma16(const Frag &a, const Frag &b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a.h8, b.h8, c, 0, 0, 0);
}
// D(32x32) += A(32x16) * B(16x32). Lane l: A row / B column l & 31, k-slice 8*(l>>5)..+7;
// D column l & 31, rows 8*(i/4) + 4*(l>>5) + i%4 for register i.
__device__ __forceinline__ float16_t mfma32(const Frag &a, const Frag &b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a.h8, b.h8, c, 0, 0, 0);
}

}  // namespace rlx
