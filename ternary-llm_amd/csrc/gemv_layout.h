// Bit-level layout of the MFMA decode GEMV, shared by the device kernel and a host unit test.
//
// Idea. A ternary weight w in {-1,0,+1} is turned into the 2-bit code c = w + 1 in {0,1,2}
// (bit1 = "positive", bit0 = "not non-zero"), and the code is left IN PLACE inside a 32-bit
// word so that, after one AND with a constant, it sits in the low mantissa bits of an fp16
// half whose exponent field is zero. Such a half is an fp16 subnormal of value c * 2^(p-24),
// p being the bit offset of the code inside the half. Two weights (one per half) cost one
// VALU AND; no per-bit expansion is needed. The activation that meets the weight in the MFMA is
// pre-multiplied by 2^-p, and the constant "+1" of the code is removed by subtracting the
// MFMA result of an all-zero weight row (codes all 1) computed with the same instructions.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define TLLM_HD __host__ __device__ __forceinline__
#else
#define TLLM_HD inline
#endif

namespace tllm {

constexpr int kChunkCols = 128;    // one scale group = the 16 bytes per plane one lane loads
constexpr int kMfmaPerTile = 16;   // 16 MFMAs of K=32 consume the 64 lanes x 128 weights of a tile

// A 32-bit mask word holds 32 weights. Its even-numbered and odd-numbered weights are handled as two
// "interleaved words" z = 0, 1; inside one, weight number f = 0..15 (bit 2f + z of the mask word)
// owns the 2-bit field at bits (2f+1, 2f). Eight ANDs per interleaved word cut out eight operand
// dwords m = 0..7, each holding one field in its low half and one in its high half, at bit offset
// code_shift(m) inside the half. Fields 0..5 and 9..13 are taken in place; the others come from the
// word rotated right by 6, which also brings field 0 into the high half and field 8 into the low one.
//
// Offsets 0 is never used: measured on gfx950, v_mfma_f32_16x16x32_f16 truncates products whose
// subnormal operand has its significant bits at offset 0 (relative error up to 5e-6 per product);
// offset 2 shows about 1e-7 and offsets 4..10 stay below fp32 rounding noise (1e-8). Offset 10 puts
// the code in the lowest exponent bits: 0x0400 = 2^-14 and 0x0800 = 2^-13 continue the subnormal
// line c * 2^(10-24).
TLLM_HD constexpr int code_shift(int m) {
    return m == 0 ? 10 : m == 1 ? 2 : m == 2 ? 4 : m == 3 ? 6 : m == 4 ? 8 : m == 5 ? 10 : m == 6 ? 6 : 8;
}
// Operand dword m and half (0 = low) that carry field f of an interleaved word.
TLLM_HD constexpr int field_dword(int f) { return f & 7; }
TLLM_HD constexpr int field_half(int f) { return (f & 7) == 0 ? 1 - (f >> 3) : f >> 3; }

// 32 weights of one row -> 16 operand dwords out[8*z + m]. Sign bits under clear nz bits are
// ignored (pos = nz & sg). Cost: 5 operations to interleave the planes, 2 rotates and 16 ANDs.
TLLM_HD void decode_word(uint32_t nz, uint32_t sg, uint32_t out[16]) {
    const uint32_t pos = nz & sg;
    // 2-bit code per weight, in place: bit 2f+1 = positive, bit 2f = not non-zero
    uint32_t q[2];
#if defined(__HIP_DEVICE_COMPILE__)
    // one three-input bit operation each: (a & c) | (~b & ~c), c = 0xAAAAAAAA
    q[0] = __builtin_amdgcn_bitop3_b32(pos << 1, nz, 0xAAAAAAAAu, 0xB1);
    q[1] = __builtin_amdgcn_bitop3_b32(pos, nz >> 1, 0xAAAAAAAAu, 0xB1);
    // keep the interleaved words materialised: otherwise the optimiser distributes the field
    // masks over them and spends two operations per operand dword instead of one
    asm volatile("" : "+v"(q[0]), "+v"(q[1]));
#else
    q[0] = ((pos << 1) & 0xAAAAAAAAu) | (~nz & 0x55555555u);
    q[1] = (pos & 0xAAAAAAAAu) | (~(nz >> 1) & 0x55555555u);
#endif
#pragma unroll
    for (int z = 0; z < 2; z++) {
        const uint32_t rot = (q[z] >> 6) | (q[z] << 26);
        out[8 * z + 0] = rot & 0x0C000C00u;   // fields 8 (low half) and 0 (high half)
        out[8 * z + 1] = q[z] & 0x000C000Cu;  // fields 1, 9
        out[8 * z + 2] = q[z] & 0x00300030u;  // fields 2, 10
        out[8 * z + 3] = q[z] & 0x00C000C0u;  // fields 3, 11
        out[8 * z + 4] = q[z] & 0x03000300u;  // fields 4, 12
        out[8 * z + 5] = q[z] & 0x0C000C00u;  // fields 5, 13
        out[8 * z + 6] = rot & 0x00C000C0u;   // fields 6, 14
        out[8 * z + 7] = rot & 0x03000300u;   // fields 7, 15
    }
}

// Where column cc (0..127) of a 128-column chunk (= one scale group) meets the MFMAs: MFMA index
// t (0..15), element e (0..7) of the 8-half operand, and the code shift p of that element.
// MFMA t = 4*word + 2*z + h consumes out[8*z + 4*h .. 8*z + 4*h + 3] of that word's decode.
struct OperandSlot {
    int t, e, p;
};
TLLM_HD OperandSlot chunk_slot(int cc) {
    const int bit = cc & 31;
    const int word = (cc >> 5) & 3;
    const int z = bit & 1;
    const int field = bit >> 1;  // 0..15
    const int m = field_dword(field);
    const int h = m >> 2;
    OperandSlot s;
    s.t = 4 * word + 2 * z + h;
    s.e = 2 * (m & 3) + field_half(field);
    s.p = code_shift(m);
    return s;
}

// Index (in halfs) of operand element (t, chunk, e) inside the activation image of one slice of
// `chunks` 128-column chunks: the 16 bytes of one (t, chunk) are contiguous, chunks are adjacent.
TLLM_HD int image_index(int t, int chunk, int e, int chunks) { return (t * chunks + chunk) * 8 + e; }

}  // namespace tllm
