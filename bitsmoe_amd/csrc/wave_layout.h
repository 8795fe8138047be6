// The wave64-native ("prepared") payload layout and its in-register decode.
//
// The reference layout stores bit PLANES: one 32-bit word holds one bit of 32 neighbouring
// columns.  That is hostile to MFMA, whose operands want, per lane, 8 consecutive
// contraction indices of one output index.  Matrix sets are therefore re-laid out ONCE
// (bitsmoe_matset_prepare) into blocks with the same size and the same per-(slab, tile)
// word offsets as the reference payload, but ordered for a wave:
//
//   block (slab of 64 rows, tile of 128 columns), bit-width w, 256*w words.
//   lane l = 16*kg + n of a wavefront owns, for each 16-wide block `nb` of OUTPUT indices,
//   the codes of a run of contraction indices, stored as w-bit FIELDS (not planes):
//
//   role 0 (gate / up: contraction over rows, outputs are columns; nb = 0..7)
//     output column 16*nb + n, rows 16*kg + e, e = 0..15              (16 codes)
//   role 1 (down: contraction over columns, outputs are rows; nb = 0..3)
//     output row 16*nb + n, columns 32*m + 8*kg + e', m = 0..3, e' = 0..7   (32 codes)
//
//   Role 1: a run of 16 codes with index x = 0..15 sits in a word, precisely:
//     2-bit fields:  field LSB at  (x & ~1) + 16*(x & 1)
//     4-bit fields:  8 codes per word, field LSB at 4*(x'/2) + 16*(x' & 1), x' = x % 8
//     3-bit codes :  whole 3-bit fields, five PAIRS of neighbouring codes per word: pair P = 16*nb + 4*m + e'/2
//                    of the lane (0..63) sits in word P/5 of the lane's thirteen, its two fields at bits
//                    1 + 3*(P%5) and 17 + 3*(P%5) (832 words per block instead of 768)
//   so that ONE rotate and ONE and-or turn a word into a packed pair of 16-bit floats
//   (2^w + code) for two neighbouring contraction indices: the pair lives 16 bits apart.
//
//   Role 0 staggers the fields so that most rotates disappear.  The MFMA operand of one k-step
//   is four registers i = 0..3 (contraction indices 2i, 2i+1 of the lane's run of eight).  The
//   field of register i sits 2i bits (4-bit codes: 4*(i%2) bits) BELOW the place where it would
//   read as 2^w + code in an f16 mantissa, so the four registers of a k-step come out of the
//   same word with four different masks and no rotate, as 2^w + code / f_i with
//   f_i = 4^i (2- and 3-bit) or 16^(i%2) (4-bit).  The other k-step (4-bit: the registers 2, 3)
//   sits 8 bits further up: one rotate by 8 serves its four (two) registers.  The factor f_i
//   is a power of two and moves exactly into the other operand's scale (stagger_factor).
//     2/3-bit fields: field LSB at (10 - w - 2i + 16*(x&1) + 8*ks) mod 32, x = 8*ks + 2i + (x&1)
//     4-bit fields  : field LSB at (6 - 4*(i%2) + 16*(x'&1) + 8*(i/2)) mod 32, x' = 2i + (x'&1)
//     3-bit, bit 2  : (9 - 2i + 16*(x&1) + 8*upper + ks) mod 32 of a separate word shared by
//                     lanes n and n+8 (upper = n/8): one rotate by 8*upper + ks
//   (a field may wrap around bit 31).  Role 0 operands are f16 (a bf16 mantissa is too short).
//
// Word order inside a block (every lane reads one contiguous run):
//   role 0: the four wavefronts of a workgroup own the column-block PAIRS nbp = nb/2, so
//           the words of one pair are contiguous over the 64 lanes:
//           w=2: word[idx2(nb, l)]   idx2 = ((nb/2)*64 + l)*2 + nb%2
//           w=4: word[idx2(nb, l)*2 + j]
//           w=3: low word[idx2(nb, l)], high word[512 + hi_index0(kg, n, nb)]
//   role 1: w=2: word[(l*4 + nb)*2 + h]           w=4: word[(l*4 + nb)*4 + m]
//           w=3: word j of lane l at (j/4)*256 + l*4 + j%4 for j < 12 (three 16-byte loads per lane), word 12 at 768 + l
//
// Decoded operand value is (2^w + code); the true level is code - 2^(w-1), so every dot
// product carries the constant 1.5 * 2^w times the sum of the other operand, which the
// kernels remove with one extra MFMA against a constant operand.
#pragma once

#include <cstdint>

#include "common.h"

namespace bitsmoe {

constexpr int ROLE_GATE_UP = 0;
constexpr int ROLE_DOWN = 1;
constexpr int SLAB_ROWS = 64;
constexpr int GU_SLABS = 8;   // slabs (64 rows each) one gate/up workgroup contracts over

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

// position of the field LSB for index x (0..15) of a run of 16 two-bit fields
__host__ __device__ inline int pos2(int x) { return (x & ~1) + 16 * (x & 1); }
// index x' (0..7) of a run of 8 four-bit fields
__host__ __device__ inline int pos4(int x) { return 4 * (x >> 1) + 16 * (x & 1); }
// index y (0..31) of a run of 32 single bits (role 1) / (0..15) + 8*upper (role 0)
__host__ __device__ inline int pos1(int y) { return (y >> 1) + 16 * (y & 1); }

// role 1, 3-bit: words of one (slab, tile) block, the place of word j (0..12) of lane l, the low-half bit offset of
// slot sl (0..4) of a word, and the words of a block of either role and width
constexpr int R1W3_BLOCK_WORDS = 13 * 64;
__host__ __device__ inline int r1w3_word_index(int l, int j) { return j < 12 ? (j >> 2) * 256 + l * 4 + (j & 3) : 768 + l; }
__host__ __device__ inline int r1w3_slot_pos(int sl) { return 1 + 3 * sl; }
__host__ __device__ inline int block_words(int role, int w) { return (role == 1 && w == 3) ? R1W3_BLOCK_WORDS : 256 * w; }

// role 0 (staggered): field LSB of code x (0..15) of a run in a two-bit field word, w = 2 or 3
__host__ __device__ inline int pos2s(int w, int x) {
    const int p = x >> 1;
    return (10 - w - 2 * (p & 3) + 16 * (x & 1) + 8 * (p >> 2)) & 31;
}
// role 0 (staggered): field LSB of code x' (0..7) of a four-bit field word
__host__ __device__ inline int pos4s(int x) {
    const int i = x >> 1;
    return (6 - 4 * (i & 1) + 16 * (x & 1) + 8 * (i >> 1)) & 31;
}
// role 0 (staggered): bit 2 of code x (0..15) of the run of lane n (upper = n / 8)
__host__ __device__ inline int pos1s(int x, int upper) {
    const int p = x >> 1;
    return (9 - 2 * (p & 3) + 16 * (x & 1) + 8 * upper + (p >> 2)) & 31;
}
// role 0: the decoded value of row k of a w-bit slab is 2^w + code / stagger_factor(w, k)
__host__ __device__ inline int stagger_factor(int w, int k) {
    return w == 4 ? (((k >> 1) & 1) ? 16 : 1) : 1 << (2 * ((k & 7) >> 1));
}

// role 0: word index of column block nb for lane l (two-bit field words)
__host__ __device__ inline int idx2_role0(int nb, int l) { return ((nb >> 1) * 64 + l) * 2 + (nb & 1); }
// role 0, 3-bit: word index (inside the 256-word high region) shared by lanes n and n+8
__host__ __device__ inline int hi_index0(int kg, int n, int nb) {
    return ((nb >> 1) * 32 + kg * 8 + (n & 7)) * 2 + (nb & 1);
}

template <bool BF16>
struct FloatFmt {
    static constexpr int MANT = BF16 ? 7 : 10;
    static constexpr int BIAS = BF16 ? 127 : 15;
};

// Per bit-width constants of the packed-pair decode.
template <int W, bool BF16>
struct Codec {
    static constexpr int POS = FloatFmt<BF16>::MANT - W;                              // field LSB in each half
    static constexpr uint32_t MAGIC = (uint32_t)((FloatFmt<BF16>::BIAS + W) << FloatFmt<BF16>::MANT) * 0x10001u;  // 2^W
    static constexpr uint32_t FMASK_2BIT = (3u << POS) * 0x10001u;
    static constexpr uint32_t FMASK_4BIT = (15u << POS) * 0x10001u;
    static constexpr uint32_t FMASK_HIBIT = (1u << (POS + 2)) * 0x10001u;                  // bit 2 of a 3-bit code
    // 1.5 * 2^W: exponent BIAS + W, top mantissa bit set
    static constexpr uint32_t CORR =
        (uint32_t)(((FloatFmt<BF16>::BIAS + W) << FloatFmt<BF16>::MANT) | (1 << (FloatFmt<BF16>::MANT - 1))) * 0x10001u;
};

__device__ inline uint32_t rotr32(uint32_t x, int s) { return __builtin_amdgcn_alignbit(x, x, (uint32_t)(s & 31)); }
__device__ inline uint32_t rotl32(uint32_t x, int s) { return rotr32(x, 32 - (s & 31)); }

// Pointers that come out of a table in memory are generic; the hot kernels cast them to the
// global address space so that loads become global_load / s_load instead of flat_load.
template <class T>
using gptr = const T __attribute__((address_space(1)))*;
template <class T>
__device__ inline gptr<T> as_global(const T* p) { return (gptr<T>)p; }
typedef const u32x4 __attribute__((address_space(1)))* gptr_u32x4;

// (x & mask) | magic as ONE v_and_or_b32: gfx9 VALU encodings take a single scalar/literal
// operand, so the mask is kept in a vector register and the magic in a scalar one.
__device__ inline uint32_t vreg(uint32_t c) {
    asm("" : "+v"(c));
    return c;
}

// Four packed registers (8 values = one MFMA k-step) from two-bit fields: `first` is the
// run index of the first of the 8 codes (0 or 8).
template <int W, bool BF16>
__device__ inline u32x4 decode_fields2(uint32_t z, int first) {
    using C = Codec<W, BF16>;
    u32x4 r;
    const uint32_t m = vreg(C::FMASK_2BIT);
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = (rotr32(z, first + 2 * i - C::POS) & m) | C::MAGIC;
    return r;
}

template <bool BF16>
__device__ inline u32x4 decode_fields4(uint32_t z) {
    using C = Codec<4, BF16>;
    u32x4 r;
    const uint32_t m = vreg(C::FMASK_4BIT);
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = (rotr32(z, 4 * i - C::POS) & m) | C::MAGIC;
    return r;
}

// 3-bit: two-bit fields from `z`, third bit from `hi`; `hi_first` = position of the bit of
// the first of the 8 codes inside `hi` (pos1 of its run index, plus 8 for an upper lane).
template <bool BF16>
__device__ inline u32x4 decode_fields3(uint32_t z, int first, uint32_t hi, int hi_first) {
    using C = Codec<3, BF16>;
    u32x4 r;
    const uint32_t m = vreg(C::FMASK_2BIT), mh = vreg(C::FMASK_HIBIT);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t lo = (rotr32(z, first + 2 * i - C::POS) & m) | C::MAGIC;
        r[i] = (rotr32(hi, hi_first + i - (C::POS + 2)) & mh) | lo;
    }
    return r;
}

// role 1, 3-bit: the four registers of k-step m of row block nb from the lane's thirteen words (indices fold to
// constants where nb and m are unrolled).  One rotate (none for the slot that already sits in place) and one and-or each.
template <bool BF16>
__device__ __forceinline__ u32x4 decode_r1w3(const uint32_t (&w)[16], int nb, int m) {
    using C = Codec<3, BF16>;
    const uint32_t mask = vreg((7u << C::POS) * 0x10001u);
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int P = 16 * nb + 4 * m + i;
        r[i] = (rotr32(w[P / 5], r1w3_slot_pos(P % 5) - C::POS) & mask) | C::MAGIC;
    }
    return r;
}

// ---- role 0 (staggered fields, f16 operands) ----
// The k-step's four registers from a two-bit field word (W = 2 or 3), ks = 0 or 1.
template <int W>
__device__ inline u32x4 decode0_lo(uint32_t z, int ks) {
    const uint32_t zz = ks ? rotr32(z, 8) : z;
    const uint32_t magic = vreg(Codec<W, false>::MAGIC);
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = (zz & ((3u << (10 - W - 2 * i)) * 0x10001u)) | magic;
    return r;
}
__device__ inline u32x4 decode0_fields4(uint32_t z) {
    const uint32_t zz = rotr32(z, 8);
    const uint32_t magic = vreg(Codec<4, false>::MAGIC);
    const uint32_t m0 = (15u << 6) * 0x10001u, m1 = (15u << 2) * 0x10001u;
    u32x4 r = {(z & m0) | magic, (z & m1) | magic, (zz & m0) | magic, (zz & m1) | magic};
    return r;
}
__device__ inline u32x4 decode0_fields3(uint32_t z, int ks, uint32_t hi, int upper) {
    u32x4 r = decode0_lo<3>(z, ks);
    const uint32_t hh = rotr32(hi, 8 * upper + ks);
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = (hh & ((1u << (9 - 2 * i)) * 0x10001u)) | r[i];
    return r;
}
// The same decode with the eight field masks held in scalar registers by the caller
// (masks3_role0): gfx950's three-operand and-or takes no literal, and with literal masks the
// compiler falls back to two ands and an or3 per register; with scalar masks it is one and-or
// for the two low bits and one for the high bit.
struct Masks3 {
    uint32_t lo[4], hi[4];
};
__device__ __forceinline__ Masks3 masks3_role0() {
    Masks3 m;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        m.lo[i] = (3u << (7 - 2 * i)) * 0x10001u;
        m.hi[i] = (1u << (9 - 2 * i)) * 0x10001u;
        asm volatile("" : "+s"(m.lo[i]));      // opaque: stays a scalar register, not a literal
        asm volatile("" : "+s"(m.hi[i]));
    }
    return m;
}
__device__ __forceinline__ u32x4 decode0_fields3(uint32_t z, int ks, uint32_t hi, int upper, const Masks3& m) {
    const uint32_t zz = ks ? rotr32(z, 8) : z;
    const uint32_t hh = rotr32(hi, 8 * upper + ks);
    const uint32_t magic = vreg(Codec<3, false>::MAGIC);
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        // (written out: from the C expression the compiler selects and + and + or3)
        uint32_t low, both;
        asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(low) : "v"(zz), "s"(m.lo[i]), "v"(magic));
        asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(both) : "v"(hh), "s"(m.hi[i]), "v"(low));
        r[i] = both;
    }
    return r;
}
// What has to be subtracted from the decoded registers to leave (code - 2^(W-1)) / f_i:
// 2^W + 2^(W-1) / f_i as a packed f16 pair per register (mantissa 512 / f_i).
template <int W>
__device__ inline u32x4 offset0_regs() {
    constexpr uint32_t magic = Codec<W, false>::MAGIC;
    if constexpr (W == 4)
        return u32x4{magic | 512u * 0x10001u, magic | 32u * 0x10001u, magic | 512u * 0x10001u, magic | 32u * 0x10001u};
    else
        return u32x4{magic | 512u * 0x10001u, magic | 128u * 0x10001u, magic | 32u * 0x10001u, magic | 8u * 0x10001u};
}

// Packed f16 arithmetic on two values in one 32-bit register.
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
__device__ inline uint32_t pk_add_f16(uint32_t a, uint32_t b) {
    const h2 r = __builtin_bit_cast(h2, a) + __builtin_bit_cast(h2, b);
    return __builtin_bit_cast(uint32_t, r);
}
__device__ inline uint32_t pk_mul_f16(uint32_t a, uint32_t b) {
    const h2 r = __builtin_bit_cast(h2, a) * __builtin_bit_cast(h2, b);
    return __builtin_bit_cast(uint32_t, r);
}

template <bool BF16>
__device__ inline f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
    if constexpr (BF16)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// fp32 -> 16-bit operand type, round to nearest even
template <bool BF16>
__device__ inline uint16_t to_operand(float v) {
    // native conversions (v_cvt_pk_bf16_f32 / v_cvt_f16_f32), round to nearest even
    if constexpr (BF16) {
        return __builtin_bit_cast(uint16_t, (__bf16)v);
    } else {
        return __builtin_bit_cast(uint16_t, (_Float16)v);
    }
}

// z = silu(g) * u as a 16-bit MFMA operand: the product rounded to fp32, THEN to 16 bits -- the two steps of the
// reference's __float2half(silu(g) * u) (the tensor-core down kernel's operand, bitsmoe/algorithms/cpp/mlp_forward.cu).
// Left to itself the compiler folds product and conversion into one instruction with a single rounding wherever it sees
// both side by side (and a two-step conversion elsewhere in the same kernel), so that an element of z differed by one
// f16 unit now and then, and not alike from one variant of a kernel to the next.  The empty statement keeps the fp32
// product a value of its own.
template <bool BF16 = false>
__device__ __forceinline__ uint16_t z_operand(float g, float u) {
    float p = silu_f32(g) * u;
    asm("" : "+v"(p));
    return to_operand<BF16>(p);
}

}  // namespace bitsmoe
