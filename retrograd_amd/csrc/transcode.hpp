// GGUF block types with no kernel of their own that Q8_0 can hold exactly, rewritten as Q8_0 rows when a model
// is loaded (host code). Every value of these types is its block's f16 scale times a small integer, with no
// rounding on the way (reference crates/rir-core/src/quant.rs: ScaleNibble :236-245, ScaleNibbleHigh :258-270,
// LutNibble :297-306, decode_q3_k :351-396), so the f16 scale and the integer as an int8 code decode to the same
// f32 under Q8_0's rule d * q (:228-234):
//
//   Q4_0    d * (q - 8),  q a nibble          -> code q - 8   in [-8, 7]
//   Q5_0    d * (q - 16), q five bits         -> code q - 16  in [-16, 15]
//   IQ4_NL  d * table[q]                      -> code table[q] in [-127, 113]
//   Q3_K    (d * (sc - 32)) * (q - 4 or q), sc six bits, q two: both products are exact in f32 (11 + 6 + 3 bits), the
//           code (sc - 32) * (q - [0|4]) lies in [-124, 128]; a 32-wide block that holds a 128 is stored with -d
//           and negated codes, which then lie in [-128, 124].
//
// The tensors cost 8.5 bits per weight in device memory afterwards instead of 4.5 / 5.5 / 3.4, and run on the
// Q8_0 kernels. Q4_1, Q5_1 (d * q + m), Q2_K (a min term per 16) and IQ4_XS (codes up to 31 * 127) have no such
// form: they stay as stored and go through the per-element decoder.
#pragma once

#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <vector>

namespace retro {

enum : int { GT_Q4_0 = 2, GT_Q5_0 = 6, GT_Q8_0 = 8, GT_Q3_K = 11, GT_IQ4_NL = 20 };

inline bool q8_0_holds(int type) { return type == GT_Q4_0 || type == GT_Q5_0 || type == GT_IQ4_NL || type == GT_Q3_K; }

// `n` elements (whole blocks of `type`) from src as n / 32 Q8_0 blocks (34 bytes each) into dst.
inline void to_q8_0(int type, const uint8_t * src, size_t n, uint8_t * dst) {
    static const int8_t table[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
    if (type == GT_Q4_0 || type == GT_IQ4_NL || type == GT_Q5_0) {
        const size_t nb = type == GT_Q5_0 ? 22 : 18, head = type == GT_Q5_0 ? 6 : 2;
        for (size_t b = 0; b < n / 32; ++b) {
            const uint8_t * blk = src + b * nb;
            uint8_t * out = dst + b * 34;
            out[0] = blk[0];
            out[1] = blk[1];
            uint32_t qh = 0;
            if (type == GT_Q5_0) std::memcpy(&qh, blk + 2, 4);
            for (int j = 0; j < 16; ++j) {
                const uint8_t q = blk[head + j];
                int lo = q & 0x0f, hi = q >> 4;
                if (type == GT_Q4_0) { lo -= 8; hi -= 8; }
                else if (type == GT_IQ4_NL) { lo = table[lo]; hi = table[hi]; }
                else { lo = (lo | (int)(((qh >> j) & 1) << 4)) - 16; hi = (hi | (int)(((qh >> (j + 16)) & 1) << 4)) - 16; }
                out[2 + j] = (uint8_t)(int8_t)lo;
                out[2 + j + 16] = (uint8_t)(int8_t)hi;
            }
        }
        return;
    }
    if (type != GT_Q3_K) throw std::runtime_error("this type has no exact Q8_0 form");
    for (size_t b = 0; b < n / 256; ++b) {
        const uint8_t * blk = src + b * 110;          // hmask[32] | qs[64] | scales[12] | d
        const uint8_t * hm = blk, * qs = blk + 32, * sc = blk + 96;
        int code[256];
        for (int e = 0; e < 256; ++e) {
            const int i = e >> 4;                      // scale i: four bits from scales[i % 8], two from scales[8 + i % 4]
            const int s = ((sc[i % 8] >> (4 * (i / 8))) & 15) | (((sc[8 + i % 4] >> (2 * (i / 4))) & 3) << 4);
            const int q = (qs[(e >> 7) * 32 + (e & 31)] >> (2 * ((e >> 5) & 3))) & 3;
            const int high = (hm[e & 31] >> (e >> 5)) & 1;
            code[e] = (s - 32) * (q - (high ? 0 : 4));
        }
        for (int k = 0; k < 8; ++k) {
            uint8_t * out = dst + (b * 8 + (size_t)k) * 34;
            bool flip = false;
            for (int j = 0; j < 32; ++j) flip = flip || code[32 * k + j] == 128;
            out[0] = blk[108];
            out[1] = (uint8_t)(blk[109] ^ (flip ? 0x80 : 0x00));
            for (int j = 0; j < 32; ++j) out[2 + j] = (uint8_t)(int8_t)(flip ? -code[32 * k + j] : code[32 * k + j]);
        }
    }
}

}  // namespace retro
