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

constexpr int kSliceCols = 512;   // columns whose activations one wave keeps in registers
constexpr int kSliceWords = kSliceCols / 32;
constexpr int kIterRows = 16;     // rows one MFMA tile covers
constexpr int kMfmaPerSlice = 16; // 16 MFMAs of K=32 consume 16 rows x 512 columns

// Bit offset (inside an fp16 half) of the code of field slot m = 0..7. Only offsets >= 4 are used:
// measured on gfx950, v_mfma_f32_16x16x32_f16 truncates products whose subnormal operand has its
// significant bits at offsets 0..2 (relative error up to 5e-6 per product at offset 0, 1e-6 at 2),
// while offsets 4..10 stay below fp32 rounding noise (1e-8). Offset 10 puts the code in the lowest
// exponent bits: 0x0400 = 2^-14 and 0x0800 = 2^-13 continue the subnormal line c * 2^(10-24).
TLLM_HD constexpr int code_shift(int m) {
    return m == 0 ? 4 : m == 1 ? 6 : m == 2 ? 4 : m == 3 ? 6 : m == 4 ? 8 : m == 5 ? 10 : m == 6 ? 6 : 8;
}

// 32 weights of one row -> 16 operand dwords. out[8*z + m] holds, in its low and high half, the
// codes of the weights at bit (2*m + z) and bit (16 + 2*m + z) of the word, each shifted left by
// code_shift(m) inside its half. Sign bits under clear nz bits are ignored (pos = nz & sg).
// Cost: 7 operations to interleave the planes, 4 shifts and 16 ANDs per 32 weights.
TLLM_HD void decode_word(uint32_t nz, uint32_t sg, uint32_t out[16]) {
    const uint32_t pos = nz & sg;
    const uint32_t nzn = ~nz;
    // 2-bit code per weight, in place: bit 2i+1 = positive, bit 2i = not non-zero
    uint32_t q[2];
    q[0] = ((pos << 1) & 0xAAAAAAAAu) | (nzn & 0x55555555u);  // weights at even bits
    q[1] = (pos & 0xAAAAAAAAu) | ((nzn >> 1) & 0x55555555u);  // weights at odd bits
#if defined(__HIP_DEVICE_COMPILE__)
    // keep the interleaved words materialised: otherwise the optimiser distributes the field
    // masks over the OR and spends two operations per operand dword instead of one
    asm volatile("" : "+v"(q[0]), "+v"(q[1]));
#endif
#pragma unroll
    for (int z = 0; z < 2; z++) {
        const uint32_t up = q[z] << 4;    // fields 0,1 (and 8,9 in the high half) move to offsets 4,6
        const uint32_t down = q[z] >> 6;  // fields 6,7 (and 14,15) move to offsets 6,8
        out[8 * z + 0] = up & 0x00300030u;
        out[8 * z + 1] = up & 0x00C000C0u;
        out[8 * z + 2] = q[z] & 0x00300030u;
        out[8 * z + 3] = q[z] & 0x00C000C0u;
        out[8 * z + 4] = q[z] & 0x03000300u;
        out[8 * z + 5] = q[z] & 0x0C000C00u;
        out[8 * z + 6] = down & 0x00C000C0u;
        out[8 * z + 7] = down & 0x03000300u;
    }
}

// Where a slice-local column c (0..511) meets the MFMA: lane quarter q (which 128-column group of
// the slice), MFMA index t (0..15), element e (0..7) of the 8-half operand, and the code shift p.
// MFMA t = 4*word + 2*z + h consumes out[8*z + 4*h .. 8*z + 4*h + 3] of that word's decode.
struct OperandSlot {
    int q, t, e, p;
};
TLLM_HD OperandSlot column_slot(int c) {
    const int bit = c & 31;
    const int word = (c >> 5) & 3;
    const int z = bit & 1;
    const int field = bit >> 1;  // 0..15
    const int half = field >> 3;
    const int m = field & 7;
    const int h = m >> 2;
    OperandSlot s;
    s.q = c >> 7;
    s.t = 4 * word + 2 * z + h;
    s.e = 2 * (m & 3) + half;
    s.p = code_shift(m);
    return s;
}

// Index (in halfs) of operand element (t, q, e) inside the 512-half image of one slice.
TLLM_HD int image_index(int t, int q, int e) { return (t * 4 + q) * 8 + e; }

}  // namespace tllm
