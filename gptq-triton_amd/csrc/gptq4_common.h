// Shared device helpers for the gfx950 4-bit GPTQ kernels.
//
// Weight decode (README.md:93 of the reference, `w = (w - z - 1) * s`):
//   W[k,n] = fp16( float(q - (z + 1)) * float(s) )
// is produced here entirely in packed fp16 with ONE rounding:
//   (w & 0x000F000F) | 0x64006400  is the fp16 pair (1024 + q_t, 1024 + q_{t+4});
//   adding -(1024 + z + 1) is exact (small integers), the multiply by s rounds once.
// For the odd nibbles the mask 0x00F000F0 gives 1024 + 16*q; fma(v, 1/16, -(64+z+1))
// is again an exact small integer.  One 32-bit word therefore decodes to four fp16
// pairs holding rows (0,4) (1,5) (2,6) (3,7) of its 8-row block - "pair order".
// Matrix-core B operands are consumed in pair order; the activation operand is put
// in the same order (pair_order_a) so the sum over k is unchanged.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef _Float16 half_t;
typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef float f16_t __attribute__((ext_vector_type(16)));

__device__ __forceinline__ h2_t as_h2(uint32_t u) { return __builtin_bit_cast(h2_t, u); }
__device__ __forceinline__ uint32_t as_u32(h2_t h) { return __builtin_bit_cast(uint32_t, h); }

// 2*IW rows of 64 output columns in the register layout of the 32x32 MFMA result - word i of lane (l32 = lane % 32,
// lhi = lane / 32) holds columns 2*l32 and 2*l32 + 1 of row 8*(i/4) + 4*lhi + i%4 - are turned through 8*IW*32 bytes
// of LDS that belong to this wave into rows of 128 bytes and stored 16 bytes per lane: 8 lanes per row, 8 rows per
// instruction, a quarter of the instructions.  A CU hands a 4-byte-per-lane store to the L2 as 64-byte requests
// (16 lanes each); the 128 x 256 outputs of a tile went out as 1024 of them per wave, all at the end of the kernel,
// and the chip waited for them: 16 MiB of outputs cost 7 - 9 us that way, about 3 us like this.
// row_ptr(j, r): where the 64 halves of row r = 8*j + lane/8 of the block go (j is a constant after unrolling), or
// nullptr for a row that is not stored.
template <int IW, typename RowPtr>
__device__ __forceinline__ void store_block_rows(uint32_t *tr, const uint32_t (&w)[IW], int lane, RowPtr row_ptr) {
    const int l32 = lane & 31, lhi = lane >> 5;
#pragma unroll
    for (int i = 0; i < IW; ++i) tr[(8 * (i >> 2) + 4 * lhi + (i & 3)) * 32 + l32] = w[i];
    // (the wave's own LDS writes and reads are carried out in order: no barrier)
#pragma unroll
    for (int j = 0; j < IW / 4; ++j) {
        const int rr = 8 * j + (lane >> 3);
        const uint4 v = *reinterpret_cast<const uint4 *>(tr + rr * 32 + 4 * (lane & 7));
        half_t *const dst = row_ptr(j, rr);
        if (dst != nullptr) *reinterpret_cast<uint4 *>(dst + 8 * (lane & 7)) = v;
    }
}

// Per-column decode constants (both halves of each pair hold the same value).
struct ColDecode {
    h2_t neg_lo;  // -(1024 + z + 1)
    h2_t neg_hi;  // -(64 + z + 1)
    h2_t scale;   // s
};

// Built with integer ops only.  fp16 bit patterns: for v in [1024, 2048) the pattern
// is 0x6400 + (v - 1024), so -(1025 + z) is 0xE401 + z; for v in [64, 128) it is
// 0x5400 + 16 * (v - 64), so -(65 + z) is 0xD410 + 16 * z.  `scale_bits` holds the
// fp16 scale in its low 16 bits.
__device__ __forceinline__ ColDecode make_col_decode(uint32_t stored_zero, uint32_t scale_bits) {
    ColDecode c;
    c.neg_lo = as_h2((0xE401u + stored_zero) * 0x10001u);
    c.neg_hi = as_h2((0xD410u + (stored_zero << 4)) * 0x10001u);
    c.scale = as_h2((scale_bits & 0xFFFFu) * 0x10001u);
    return c;
}

// (a & mask) | orv in one VALU op.  v_and_or_b32 is VOP3 and gfx950 lets a VOP3 read a
// single scalar operand and no literal, so the mask travels in an SGPR and the fp16
// magic 0x64006400 in a VGPR; written as asm because the compiler emits v_and + v_or.
__device__ __forceinline__ uint32_t and_or_b32(uint32_t a, uint32_t mask, uint32_t orv) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(orv));
    return r;
}

// Decode one packed word into 4 fp16 pairs in pair order: out[j] = (row j, row j+4).
__device__ __forceinline__ void decode_word(uint32_t w, const ColDecode &c, h2_t out[4]) {
    const h2_t sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
    const uint32_t magic = 0x64006400u;
    const uint32_t w8 = w >> 8;
    const h2_t lo0 = as_h2(and_or_b32(w, 0x000F000Fu, magic));
    const h2_t hi0 = as_h2(and_or_b32(w, 0x00F000F0u, magic));
    const h2_t lo1 = as_h2(and_or_b32(w8, 0x000F000Fu, magic));
    const h2_t hi1 = as_h2(and_or_b32(w8, 0x00F000F0u, magic));
    out[0] = (lo0 + c.neg_lo) * c.scale;
    out[1] = __builtin_elementwise_fma(hi0, sixteenth, c.neg_hi) * c.scale;
    out[2] = (lo1 + c.neg_lo) * c.scale;
    out[3] = __builtin_elementwise_fma(hi1, sixteenth, c.neg_hi) * c.scale;
}

__device__ __forceinline__ h8_t decode_word_h8(uint32_t w, const ColDecode &c) {
    h2_t p[4];
    decode_word(w, c, p);
    h8_t r = {p[0].x, p[0].y, p[1].x, p[1].y, p[2].x, p[2].y, p[3].x, p[3].y};
    return r;
}

// Natural-order variant for the tiled kernel, whose activation operand arrives in LDS
// straight from memory and cannot be put in pair order on the way.  A byte permute puts
// byte j of the word (nibbles 2j, 2j+1) into both halves; the mask 0x00F0000F then leaves
// 1024 + q_{2j} in the low half and 1024 + 16 * q_{2j+1} in the high half, and one packed
// fma with the per-half constants (1, 1/16) and (-(1025 + z), -(65 + z)) gives the exact
// integers q - (z + 1) in both.  16 VALU ops per word instead of 13, but none per
// activation fragment.
struct ColDecodeNat {
    h2_t neg;    // (-(1024 + z + 1), -(64 + z + 1))
    h2_t scale;  // (s, s)
};

__device__ __forceinline__ ColDecodeNat make_col_decode_nat(uint32_t stored_zero, uint32_t scale_bits) {
    ColDecodeNat c;
    c.neg = as_h2((0xE401u + stored_zero) | ((0xD410u + (stored_zero << 4)) << 16));
    c.scale = as_h2((scale_bits & 0xFFFFu) * 0x10001u);
    return c;
}

// out = rows 0..7 of the word's 8-row block, in order.
__device__ __forceinline__ h8_t decode_word_natural(uint32_t w, const ColDecodeNat &c) {
    const h2_t unit = {(half_t)1.0f, (half_t)0.0625f};
    const uint32_t magic = 0x64006400u;
    h2_t p[4];
    p[0] = as_h2(and_or_b32(__builtin_amdgcn_perm(w, w, 0x0c000c00u), 0x00F0000Fu, magic));
    p[1] = as_h2(and_or_b32(__builtin_amdgcn_perm(w, w, 0x0c010c01u), 0x00F0000Fu, magic));
    p[2] = as_h2(and_or_b32(__builtin_amdgcn_perm(w, w, 0x0c020c02u), 0x00F0000Fu, magic));
    p[3] = as_h2(and_or_b32(__builtin_amdgcn_perm(w, w, 0x0c030c03u), 0x00F0000Fu, magic));
#pragma unroll
    for (int j = 0; j < 4; ++j) p[j] = __builtin_elementwise_fma(p[j], unit, c.neg) * c.scale;
    h8_t r = {p[0].x, p[0].y, p[1].x, p[1].y, p[2].x, p[2].y, p[3].x, p[3].y};
    return r;
}

// 8 consecutive activations a0..a7 (natural order, as a uint4) -> pair order
// (a0,a4,a1,a5,a2,a6,a3,a7).
__device__ __forceinline__ h8_t pair_order_a(uint4 v) {
    union {
        uint32_t u[4];
        h8_t h;
    } r;
    r.u[0] = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);  // (a0, a4)
    r.u[1] = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);  // (a1, a5)
    r.u[2] = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);  // (a2, a6)
    r.u[3] = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);  // (a3, a7)
    return r.h;
}

__device__ __forceinline__ uint4 pair_order_u4(uint4 v) {
    uint4 r;
    r.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
    r.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
    r.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
    r.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
    return r;
}

// x * sigmoid(x) with the hardware reciprocal (1 ulp) instead of an IEEE division: the result
// is rounded to fp16 right after.
__device__ __forceinline__ float silu_f32(float x) { return x * __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

// Epilogue selectors shared by the small-M and the tiled kernels.
enum { EPI_PLAIN = 0, EPI_SILU_MUL = 1, EPI_ROPE = 2 };

struct RopeArgs {
    const int32_t *position_ids;  // [B*S]
    const float *cos_table;       // [max_pos, 64]
    const float *sin_table;
    half_t *q;
    half_t *k;
    half_t *v;
    int S;
    int H;
    int kv_capacity;
    int kv_offset;
    int max_pos;  // rows of the tables; positions are clamped into [0, max_pos)
    uint32_t s_magic;  // floor(2^32 / S) + 1 when umulhi(row, s_magic) == row / S for every row < M, else 0
};

// row -> (sequence, token within it)
__device__ __forceinline__ void split_row(const RopeArgs &r, int row, int &b, int &s) {
    if (r.S == 1) {
        b = row;
        s = 0;
        return;
    }
    b = r.s_magic ? (int)__umulhi((unsigned)row, r.s_magic) : row / r.S;
    s = row - b * r.S;
}
