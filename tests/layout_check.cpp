// Host check of the MFMA-GEMV bit layout (ternary-llm_amd/csrc/gemv_layout.h): for random mask
// words, every slice column's 2-bit code must sit where column_slot() says the activation image
// puts that column, shifted by the slot's p, and nowhere else. Emulates one slice product in
// double precision and compares it with the plain ternary dot product.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "gemv_layout.h"

using namespace tllm;

int main() {
    std::mt19937 rng(12345);
    int bad = 0;
    for (int trial = 0; trial < 200; trial++) {
        // one lane quarter's 128 weights = 4 words per plane; do all 4 quarters of a 512-column slice
        uint32_t nz[16], sg[16];
        for (int i = 0; i < 16; i++) { nz[i] = rng(); sg[i] = rng(); }
        if (trial == 0) for (int i = 0; i < 16; i++) nz[i] = 0;            // all-zero row
        if (trial == 1) for (int i = 0; i < 16; i++) { nz[i] = ~0u; sg[i] = ~0u; }
        if (trial == 2) for (int i = 0; i < 16; i++) { nz[i] = ~0u; sg[i] = 0; }
        std::vector<double> x(512);
        for (auto &v : x) v = (double)((int)(rng() % 2001) - 1000);
        // image[q][t][e] as the kernel builds it, with the 2^-p factor kept symbolic (double)
        double img[4][16][8];
        int seen[4][16][8] = {};
        int used[512] = {};
        for (int c = 0; c < 512; c++) {
            const int q = c / 128;
            OperandSlot s = chunk_slot(c % 128);
            if (s.t < 0 || s.t > 15 || s.e < 0 || s.e > 7 || s.p < 2 || s.p > 10) bad++;
            if (seen[q][s.t][s.e]++) bad++;                                  // must be a bijection
            img[q][s.t][s.e] = std::ldexp(x[c], -s.p);
            const int idx = image_index(s.t, q, s.e, 4);
            if (idx < 0 || idx >= 512 || used[idx]++) bad++;                 // image slots are a bijection too
            if (image_index(s.t, q, s.e, 16) != (s.t * 16 + q) * 8 + s.e) bad++;
        }
        for (int q = 0; q < 4; q++) {
            double mfma_sum = 0.0, plain = 0.0, bias = 0.0;
            for (int w = 0; w < 4; w++) {
                uint32_t o[16], oz[16];
                decode_word(nz[4 * q + w], sg[4 * q + w], o);
                decode_word(0, 0xFFFFFFFFu, oz);
                for (int z = 0; z < 2; z++)
                    for (int h = 0; h < 2; h++) {
                        int t = 4 * w + 2 * z + h;
                        for (int e = 0; e < 8; e++) {
                            uint32_t d = o[8 * z + 4 * h + e / 2], dz = oz[8 * z + 4 * h + e / 2];
                            uint32_t half = (e & 1) ? d >> 16 : d & 0xFFFFu;
                            uint32_t halfz = (e & 1) ? dz >> 16 : dz & 0xFFFFu;
                            if (half >= 0x0C00u) bad++;  // only exponent field 0..2 with zero mantissa, or a subnormal
                            // fp16 value of the half: subnormal => bits * 2^-24 (also right for 0x400 and 0x800)
                            mfma_sum += std::ldexp((double)half, -24) * img[q][t][e];
                            bias += std::ldexp((double)halfz, -24) * img[q][t][e];
                        }
                    }
                for (int b = 0; b < 32; b++) {
                    int wv = ((nz[4 * q + w] >> b) & 1) ? (((sg[4 * q + w] >> b) & 1) ? 1 : -1) : 0;
                    plain += wv * x[128 * q + 32 * w + b];
                }
            }
            double got = std::ldexp(mfma_sum - bias, 24);
            if (std::fabs(got - plain) > 1e-6) { bad++; if (bad < 10) std::printf("trial %d q %d got %f want %f\n", trial, q, got, plain); }
        }
    }
    std::printf("bad=%d\n", bad);
    return bad ? 1 : 0;
}
