// Device layout of GGUF-packed weights in HBM. Shared by the host repacker and the kernels.
//
// A weight is a row-major [N, K] matrix packed in GGUF blocks along K (rlx-cpu/src/gguf_matmul.rs:15-20).
// The device layout keeps every bit of every block (same byte count per block) but regroups it into
// tiles of 16 rows x UNIT_K columns so that one 64-lane wavefront reads a tile with 16-byte loads and
// every 4-byte word it gets is one MFMA operand fragment:
//
//   lane l of the wave:  n = l & 15  (row inside the tile),  g = l >> 4  (which 8 of every 32 columns)
//   "granule" (n, blk, g) = the 8 weights of row n, 32-column block blk, columns 8g .. 8g+7
//
//   4-bit schemes: a granule is one 32-bit word; element e (0..7) sits in nibble NIB_POS[e] so that
//       (w      & 0x000F000F) -> elements 0,1      (w      & 0x00F000F0) -> elements 2,3 (times 16)
//       (w >> 8 & 0x000F000F) -> elements 4,5      (w >> 8 & 0x00F000F0) -> elements 6,7 (times 16)
//     i.e. two masks and one shift split a word into four packed-half pairs in fragment order.
//   Q8_0: a granule is 8 bytes, byte e = q_e XOR 0x80 (offset binary, so a byte permute builds 1024+u halfs).
//
// Tile ("unit") contents, in bytes:
//   Q4_0 : [0,1024)  lane slots: 16 B at 16*l = granules of blocks 4u+0..3        [1024,1152) f16 d[n][4]
//   Q8_0 : [0,2048)  two halves h: 16 B at 1024*h + 16*l = granules of blocks 4u+2h, 4u+2h+1
//          [2048,2176) f16 d[n][4]
//   Q4_K : [0,2048)  two halves h: 16 B at 1024*h + 16*l = granules of sub-blocks 4h+0..3 of super-block u
//          [2048,2304) per row n: 16 B = f16 d, f16 dmin, 12 scale bytes (verbatim from the GGUF block)
//   Q5_K : [0,2048)  the nibbles, as Q4_K          [2048,2560) the fifth bits: 8 B at 2048 + 8*l = words hb[h], one per half,
//                   serving the half's four code words t after a rotate right by Q5K_ROT[t] = {0, 2, 8, 10}: element e of the
//                   rotated word sits at bit Q5K_HI_POS[e] (elements 0,1 / 4,5 at mantissa bit 4 / 20 of 1024 + q, elements
//                   2,3 / 6,7 at bit 8 / 24 of 1024 + 16 q, elements 4-7 one bit higher and used after a shift by 1)
//          [2560,2816) per row n: 16 B = f16 d, f16 dmin, 12 scale bytes (verbatim, as Q4_K)
//   Q6_K : [0,2048)  low nibbles of the 6-bit codes, two halves h like Q4_K (word t of a slot = 32-column block 4h + t)
//          [2048,3072) the two high bits of every code: 16 B at 2048 + 16*l = words hw[2h + j], one per pair of code
//                   words (t = 2j, 2j + 1) of half h. In hw the field of element e of the even word sits at bit
//                   Q6K_HI_POS[e]; the odd word's fields sit 8 bits further (mod 32), so `hw` serves the even word as
//                   is and the odd word after a rotate by 8. The positions are those the f16 magic-number decode
//                   needs: elements 0,1 / 4,5 (value 1024 + q) take their high bits at mantissa bits 4-5 / 20-21,
//                   elements 2,3 / 6,7 (value 1024 + 16 q) at bits 8-9 / 24-25; elements 4-7 are stored 2 bits higher
//                   and used after a shift by 2, like their nibbles after a shift by 8.
//          [3072,3328) per row n: the 16 scale bytes verbatim          [3328,3360) f16 d[n]
//   Q8_K : [0,4096)  four quarters h: 16 B at 1024*h + 16*l = granules of 32-column blocks 2h, 2h+1 of super-block u, bytes
//                   XOR 0x80 as Q8_0          [4096,4160) f32 d[n] (the bsums of the GGUF block are not needed and not kept)
//   Q3_K : Q6_K units. A super-block's values d * (scale - 32) * code (code in [-4, 3]) are those of the Q6_K super-block
//          with 6-bit codes code + 32, scale bytes scale - 32 (stored XOR 0x80, read as byte - 128) and the same d.
//   Q2_K : [0,1024)  16 B at 16*l = the 2-bit codes of the lane slot's 8 columns in all eight 32-column blocks of
//                   super-block u: word w serves blocks 2w (low byte of each 16-bit half) and 2w + 1 (high byte); in a
//                   byte the codes of elements 2i (low half) / 2i + 1 (high half) sit at bits 2i
//          [1024,1280) per row n: the 16 scale bytes verbatim (low nibble scale, high nibble min of a 16-column sub-block)
//          [1280,1344) per row n: f16 d, f16 dmin
// Units are stored [row_tile][unit] with the unit index (K direction) fastest.
// N is padded to a multiple of 16 and K to a multiple of UNIT_K with zero-scale blocks.
#pragma once
#include <stdint.h>

#ifdef __HIPCC__
#define RLX_HD __host__ __device__
#else
#define RLX_HD
#endif

namespace rlx {

// Values of the reference's QuantScheme discriminants (rlx-ir/src/quant.rs:39-73).
enum Scheme : int {
    SCHEME_Q4K = 5, SCHEME_Q5K = 6, SCHEME_Q6K = 7, SCHEME_Q8K = 8, SCHEME_Q2K = 9, SCHEME_Q3K = 10,
    SCHEME_Q4_0 = 11, SCHEME_Q8_0 = 12
};

// Not a GGUF scheme: ready binary16 operand images of the prefill kernel (weights already multiplied by per-column
// scales, see rlx_wscale_* in kernels/dequant.hip). Never the scheme of a weight; names the prefill instantiation only.
constexpr int SCHEME_F16W = 100;

// fifth bit of element e inside a Q5_K high-bit word (after the rotate of its code word), and the rotates
RLX_HD constexpr int q5k_hi_pos(int e) { return e == 0 ? 4 : e == 1 ? 20 : e == 2 ? 8 : e == 3 ? 24 : e == 4 ? 5 : e == 5 ? 21 : e == 6 ? 9 : 25; }
RLX_HD constexpr int q5k_rot(int t) { return t == 0 ? 0 : t == 1 ? 2 : t == 2 ? 8 : 10; }
// low bit of the 2-bit high field of element e (even code word of a pair) inside a Q6_K high-bit word
RLX_HD constexpr int q6k_hi_pos(int e) { return e == 0 ? 4 : e == 1 ? 20 : e == 2 ? 8 : e == 3 ? 24 : e == 4 ? 6 : e == 5 ? 22 : e == 6 ? 10 : 26; }

constexpr int TILE_ROWS = 16;

struct Layout {
    int unit_k;        // columns per unit
    int unit_bytes;    // bytes per unit
    int quant_bytes;   // bytes of lane slots at the start of a unit
    int block_elems;   // GGUF block size
    int block_bytes;   // GGUF block bytes
};

RLX_HD constexpr Layout layout_of(int scheme) {
    return scheme == SCHEME_Q4_0   ? Layout{128, 1152, 1024, 32, 18}
           : scheme == SCHEME_Q8_0 ? Layout{128, 2176, 2048, 32, 34}
           : scheme == SCHEME_Q4K  ? Layout{256, 2304, 2048, 256, 144}
           : scheme == SCHEME_Q5K  ? Layout{256, 2816, 2560, 256, 176}
           : scheme == SCHEME_Q6K  ? Layout{256, 3360, 3072, 256, 210}
           : scheme == SCHEME_Q8K  ? Layout{256, 4160, 4096, 256, 292}
           : scheme == SCHEME_Q2K  ? Layout{256, 1344, 1024, 256, 84}
           : scheme == SCHEME_Q3K  ? Layout{256, 3360, 3072, 256, 110}  // rewritten as Q6_K units
                                   : Layout{0, 0, 0, 0, 0};
}

// The scheme whose kernels read a scheme's device units. A Q3_K super-block (3-bit codes in [-4, 3], 6-bit scales minus 32,
// one d) is rewritten at upload, exactly, as the Q6_K super-block of the same values with signed scale bytes.
RLX_HD constexpr int kernel_scheme(int scheme) { return scheme == SCHEME_Q3K ? SCHEME_Q6K : scheme; }
// What a scheme's prefill kernel needs next to the activation image: 0 nothing, 1 the sums of every 32-column block
// (Q4_K / Q5_K: the dmin term), 2 the sums of every 16-column sub-block (Q2_K).
RLX_HD constexpr int act_sums_kind(int scheme) { return (scheme == SCHEME_Q4K || scheme == SCHEME_Q5K) ? 1 : scheme == SCHEME_Q2K ? 2 : 0; }

// nibble position of fragment element e inside a granule word
RLX_HD constexpr int nib_pos(int e) { return ((e & 1) << 2) | (e >> 1); }

struct WeightDims {
    int64_t n, k;        // logical
    int64_t row_tiles;   // ceil(n / 16)
    int64_t units;       // ceil(k / unit_k)
    int64_t n_pad, k_pad;
    int64_t bytes;       // device bytes
};

RLX_HD inline WeightDims weight_dims(const Layout &L, int64_t n, int64_t k) {
    WeightDims d{};
    d.n = n;
    d.k = k;
    if (L.unit_k == 0) return d;
    d.row_tiles = (n + TILE_ROWS - 1) / TILE_ROWS;
    d.units = (k + L.unit_k - 1) / L.unit_k;
    d.n_pad = d.row_tiles * TILE_ROWS;
    d.k_pad = d.units * L.unit_k;
    d.bytes = d.row_tiles * d.units * (int64_t)L.unit_bytes;
    return d;
}
RLX_HD inline WeightDims weight_dims(int scheme, int64_t n, int64_t k) { return weight_dims(layout_of(scheme), n, k); }

}  // namespace rlx
