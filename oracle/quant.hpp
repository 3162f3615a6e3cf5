// TEST INFRASTRUCTURE - CPU oracle, never linked into or called by the product.
//
// Decoders for the GGUF block formats the decode step reads, restated from the
// reference's portable dequantisation oracle (crates/rir-core/src/quant.rs),
// which the reference proves bit-equal to ggml's to_float on identical bytes
// (tests/rir_quant_oracle.rs:67-103). Block geometry from
// crates/rir-core/src/quant_table.rs (Q8_0 32 el / 34 B, MXFP4 32 el / 17 B,
// Q4_K 256 el / 144 B, Q5_K 256 el / 176 B, Q6_K 256 el / 210 B; Q4_0 and
// IQ4_NL 32 / 18, Q4_1 32 / 20, Q5_0 32 / 22, Q5_1 32 / 24, Q2_K 256 / 84,
// Q3_K 256 / 110, IQ4_XS 256 / 136).
//
// Pinned by: tests/test_oracle_quant.py (known answers of quant.rs:534-581,
// exhaustive f16 against numpy, brute-force Q4_K addressing against
// generated/rir/mul_mat_vec_q4_K/cpu.rs:52-120 semantics; Q5_K and Q6_K each
// against an independent restatement of the loops quant.rs:418-464 spell out,
// single codes placed on single elements, and Q5_K's reduction to Q4_K when
// its fifth bits are clear).
#pragma once

#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>

namespace oracle {

// ggml type ids as stored in a GGUF tensor table.
enum ggml_type_id : uint32_t {
    T_F32 = 0, T_F16 = 1, T_Q4_0 = 2, T_Q4_1 = 3, T_Q5_0 = 6, T_Q5_1 = 7, T_Q8_0 = 8, T_Q2_K = 10, T_Q3_K = 11,
    T_Q4_K = 12, T_Q5_K = 13, T_Q6_K = 14, T_IQ4_NL = 20, T_IQ4_XS = 23, T_BF16 = 30, T_MXFP4 = 39,
};

struct block_geom { uint32_t elements; uint32_t bytes; };

inline block_geom geom_of(uint32_t type) {
    switch (type) {
        case T_F32:   return {1, 4};
        case T_F16:   return {1, 2};
        case T_BF16:  return {1, 2};
        case T_Q8_0:  return {32, 34};
        case T_Q4_0:  return {32, 18};
        case T_Q4_1:  return {32, 20};
        case T_Q5_0:  return {32, 22};
        case T_Q5_1:  return {32, 24};
        case T_IQ4_NL: return {32, 18};
        case T_Q2_K:  return {256, 84};
        case T_Q3_K:  return {256, 110};
        case T_IQ4_XS: return {256, 136};
        case T_MXFP4: return {32, 17};
        case T_Q4_K:  return {256, 144};
        case T_Q5_K:  return {256, 176};
        case T_Q6_K:  return {256, 210};
        default: throw std::runtime_error("oracle: unsupported ggml type " + std::to_string(type));
    }
}

inline size_t row_bytes(uint32_t type, size_t n) {
    const block_geom g = geom_of(type);
    if (n % g.elements != 0) throw std::runtime_error("oracle: row is not block aligned");
    return n / g.elements * g.bytes;
}

// IEEE binary16 -> binary32, exact incl. subnormals (quant.rs:82-103).
inline float half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h >> 15) << 31;
    const uint32_t e = (h >> 10) & 0x1f;
    const uint32_t m = h & 0x3ff;
    uint32_t bits;
    if (e == 0) {
        if (m == 0) {
            bits = sign;
        } else {
            // value = m * 2^-24: normalise the mantissa.
            int shift = 0;
            uint32_t mm = m;
            while ((mm & 0x400) == 0) { mm <<= 1; ++shift; }
            bits = sign | ((uint32_t)(113 - shift) << 23) | ((mm & 0x3ff) << 13);
        }
    } else if (e == 31) {
        bits = sign | 0x7f800000u | (m << 13);
    } else {
        bits = sign | ((e + 112) << 23) | (m << 13);
    }
    float out;
    std::memcpy(&out, &bits, 4);
    return out;
}

// binary64 -> binary16, round to nearest even in ONE rounding (what Python's
// struct.pack("<e", x) does on a double; a float argument widens exactly, so
// this is also the binary32 -> binary16 conversion). Overflow goes to infinity.
inline uint16_t double_to_half(double v) {
    const uint16_t sign = std::signbit(v) ? 0x8000 : 0;
    if (std::isnan(v)) return (uint16_t)(sign | 0x7e00);
    double a = std::fabs(v);
    if (std::isinf(a)) return (uint16_t)(sign | 0x7c00);
    if (a == 0.0) return sign;
    int e;
    std::frexp(a, &e);              // a = f * 2^e, f in [0.5, 1)  ->  floor(log2 a) = e - 1
    int exp2 = e - 1;
    if (exp2 < -14) exp2 = -14;     // subnormal halves share the quantum 2^-24
    const double quantum = std::ldexp(1.0, exp2 - 10);
    double q = std::nearbyint(a / quantum);   // exact division; ties to even
    if (q == 0.0) return sign;
    if (q >= 2048.0) { q = 1024.0; ++exp2; }  // mantissa carry
    if (exp2 > 15) return (uint16_t)(sign | 0x7c00);
    const uint32_t qi = (uint32_t)q;
    if (qi < 1024) return (uint16_t)(sign | qi);                       // subnormal
    return (uint16_t)(sign | ((uint32_t)(exp2 + 15) << 10) | (qi - 1024));
}

inline uint16_t float_to_half(float f) { return double_to_half((double)f); }

inline float bf16_to_float(uint16_t h) {
    const uint32_t bits = (uint32_t)h << 16;
    float out;
    std::memcpy(&out, &bits, 4);
    return out;
}

// E8M0 exponent byte scaled by 1/2 (quant.rs:107-115): 2^(x-128), the two
// smallest landing in binary32 subnormals.
inline float e8m0_half(uint8_t x) {
    uint32_t bits;
    if (x == 0) bits = 0x00200000u;
    else if (x == 1) bits = 0x00400000u;
    else bits = ((uint32_t)x - 1) << 23;
    float out;
    std::memcpy(&out, &bits, 4);
    return out;
}

inline uint16_t rd16(const uint8_t * p) { return (uint16_t)(p[0] | (p[1] << 8)); }

// 6-bit (scale, min) of sub-block j from the 12 packed bytes (quant.rs:119-128).
inline void q4k_scale_min(int j, const uint8_t * q, uint8_t & sc, uint8_t & mn) {
    if (j < 4) {
        sc = q[j] & 63;
        mn = q[j + 4] & 63;
    } else {
        sc = (uint8_t)((q[j + 4] & 0x0f) | ((q[j - 4] >> 6) << 4));
        mn = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

// quant.rs:56-58: the non-linear code book of IQ4_NL and IQ4_XS
static const int8_t k_iq4nl[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
static const int8_t k_fp4_doubled[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};

// Decode n elements (whole blocks) of `type` from src into out.
inline void decode_row(uint32_t type, const uint8_t * src, size_t n, float * out) {
    switch (type) {
        case T_F32:
            std::memcpy(out, src, n * 4);
            return;
        case T_F16:
            for (size_t i = 0; i < n; ++i) out[i] = half_to_float(rd16(src + 2 * i));
            return;
        case T_BF16:
            for (size_t i = 0; i < n; ++i) out[i] = bf16_to_float(rd16(src + 2 * i));
            return;
        case T_Q8_0:  // quant.rs:228-234: d (f16) then 32 signed bytes
            for (size_t b = 0; b < n / 32; ++b) {
                const uint8_t * blk = src + b * 34;
                const float d = half_to_float(rd16(blk));
                for (int j = 0; j < 32; ++j) out[b * 32 + j] = d * (float)(int8_t)blk[2 + j];
            }
            return;
        case T_Q4_0:  // quant.rs:236-245: d (f16) | 16 bytes; low nibbles are the first half; value = d * (q - 8)
        case T_IQ4_NL:  // quant.rs:297-306: the same block with the nibble looked up in the code book
            for (size_t b = 0; b < n / 32; ++b) {
                const uint8_t * blk = src + b * 18;
                const float d = half_to_float(rd16(blk));
                for (int j = 0; j < 16; ++j) {
                    const uint8_t q = blk[2 + j];
                    if (type == T_Q4_0) {
                        out[b * 32 + j]      = d * (float)((int)(q & 0x0f) - 8);
                        out[b * 32 + j + 16] = d * (float)((int)(q >> 4) - 8);
                    } else {
                        out[b * 32 + j]      = d * (float)k_iq4nl[q & 0x0f];
                        out[b * 32 + j + 16] = d * (float)k_iq4nl[q >> 4];
                    }
                }
            }
            return;
        case T_Q4_1:  // quant.rs:247-256: d, m (f16) | 16 bytes; value = d * q + m
            for (size_t b = 0; b < n / 32; ++b) {
                const uint8_t * blk = src + b * 20;
                const float d = half_to_float(rd16(blk)), m = half_to_float(rd16(blk + 2));
                for (int j = 0; j < 16; ++j) {
                    const uint8_t q = blk[4 + j];
                    out[b * 32 + j]      = d * (float)(q & 0x0f) + m;
                    out[b * 32 + j + 16] = d * (float)(q >> 4) + m;
                }
            }
            return;
        case T_Q5_0:  // quant.rs:258-270: d (f16) | qh (u32) | 16 bytes; fifth bit j of qh for the first half, j + 16 for the second
            for (size_t b = 0; b < n / 32; ++b) {
                const uint8_t * blk = src + b * 22;
                const float d = half_to_float(rd16(blk));
                const uint32_t qh = (uint32_t)blk[2] | ((uint32_t)blk[3] << 8) | ((uint32_t)blk[4] << 16) | ((uint32_t)blk[5] << 24);
                for (int j = 0; j < 16; ++j) {
                    const uint8_t q = blk[6 + j];
                    const uint32_t h0 = ((qh >> j) << 4) & 0x10, h1 = (qh >> (j + 12)) & 0x10;
                    out[b * 32 + j]      = d * (float)((int)((q & 0x0f) | h0) - 16);
                    out[b * 32 + j + 16] = d * (float)((int)((q >> 4) | h1) - 16);
                }
            }
            return;
        case T_Q5_1:  // quant.rs:272-284: d, m (f16) | qh (u32) | 16 bytes; value = d * q5 + m
            for (size_t b = 0; b < n / 32; ++b) {
                const uint8_t * blk = src + b * 24;
                const float d = half_to_float(rd16(blk)), m = half_to_float(rd16(blk + 2));
                const uint32_t qh = (uint32_t)blk[4] | ((uint32_t)blk[5] << 8) | ((uint32_t)blk[6] << 16) | ((uint32_t)blk[7] << 24);
                for (int j = 0; j < 16; ++j) {
                    const uint8_t q = blk[8 + j];
                    const uint32_t h0 = ((qh >> j) << 4) & 0x10, h1 = (qh >> (j + 12)) & 0x10;
                    out[b * 32 + j]      = d * (float)((q & 0x0f) | h0) + m;
                    out[b * 32 + j + 16] = d * (float)((q >> 4) | h1) + m;
                }
            }
            return;
        case T_Q2_K:  // quant.rs:327-349: scales[16] | qs[64] | d, dmin (f16); sixteen sub-blocks of 16
            for (size_t b = 0; b < n / 256; ++b) {
                const uint8_t * blk = src + b * 84;
                const float d = half_to_float(rd16(blk + 80)), dmin = half_to_float(rd16(blk + 82));
                float * y = out + b * 256;
                int o = 0, is = 0;
                for (int n0 = 0; n0 < 256; n0 += 128) {
                    const uint8_t * q = blk + 16 + n0 / 4;
                    for (int j = 0; j < 4; ++j) {
                        for (int half = 0; half < 2; ++half) {
                            const uint8_t sc = blk[is++];
                            const float dl = d * (float)(sc & 0x0f), ml = dmin * (float)(sc >> 4);
                            for (int l = 0; l < 16; ++l) y[o++] = dl * (float)((q[l + 16 * half] >> (2 * j)) & 3) - ml;
                        }
                    }
                }
            }
            return;
        case T_Q3_K:  // quant.rs:351-396: hmask[32] | qs[64] | scales[12] | d (f16); sixteen 6-bit scales split 4 + 2 bits
            for (size_t b = 0; b < n / 256; ++b) {
                const uint8_t * blk = src + b * 110;
                const float d_all = half_to_float(rd16(blk + 108));
                uint32_t aux[4] = {0, 0, 0, 0};
                for (int i = 0; i < 3; ++i)
                    aux[i] = (uint32_t)blk[96 + 4 * i] | ((uint32_t)blk[97 + 4 * i] << 8) | ((uint32_t)blk[98 + 4 * i] << 16) | ((uint32_t)blk[99 + 4 * i] << 24);
                const uint32_t kmask1 = 0x03030303u, kmask2 = 0x0f0f0f0fu, tmp = aux[2];
                aux[2] = ((aux[0] >> 4) & kmask2) | (((tmp >> 4) & kmask1) << 4);
                aux[3] = ((aux[1] >> 4) & kmask2) | (((tmp >> 6) & kmask1) << 4);
                aux[0] = (aux[0] & kmask2) | ((tmp & kmask1) << 4);
                aux[1] = (aux[1] & kmask2) | (((tmp >> 2) & kmask1) << 4);
                int8_t scales[16];
                for (int i = 0; i < 4; ++i)
                    for (int j = 0; j < 4; ++j) scales[4 * i + j] = (int8_t)((aux[i] >> (8 * j)) & 0xff);
                float * y = out + b * 256;
                int o = 0, is = 0;
                uint8_t m = 1;
                for (int n0 = 0; n0 < 256; n0 += 128) {
                    const uint8_t * q = blk + 32 + n0 / 4;
                    for (int j = 0; j < 4; ++j) {
                        for (int half = 0; half < 2; ++half) {
                            const float dl = d_all * (float)((int)scales[is++] - 32);
                            for (int l = 0; l < 16; ++l) {
                                const int idx = l + 16 * half;
                                const int qv = (q[idx] >> (2 * j)) & 3;
                                y[o++] = dl * (float)(qv - ((blk[idx] & m) ? 0 : 4));
                            }
                        }
                        m = (uint8_t)(m << 1);
                    }
                }
            }
            return;
        case T_IQ4_XS:  // quant.rs:465-480: d (f16) | scales_h (u16) | scales_l[4] | qs[128]; eight sub-blocks of 32
            for (size_t b = 0; b < n / 256; ++b) {
                const uint8_t * blk = src + b * 136;
                const float d = half_to_float(rd16(blk));
                const uint32_t scales_h = rd16(blk + 2);
                for (int ib = 0; ib < 8; ++ib) {
                    const int ls = ((blk[4 + ib / 2] >> (4 * (ib % 2))) & 0x0f) | (int)(((scales_h >> (2 * ib)) & 3) << 4);
                    const float dl = d * (float)(ls - 32);
                    const uint8_t * qs = blk + 8 + 16 * ib;
                    for (int j = 0; j < 16; ++j) {
                        out[b * 256 + 32 * ib + j]      = dl * (float)k_iq4nl[qs[j] & 0x0f];
                        out[b * 256 + 32 * ib + j + 16] = dl * (float)k_iq4nl[qs[j] >> 4];
                    }
                }
            }
            return;
        case T_MXFP4:  // quant.rs:286-295: e8m0 byte, low nibbles first half
            for (size_t b = 0; b < n / 32; ++b) {
                const uint8_t * blk = src + b * 17;
                const float d = e8m0_half(blk[0]);
                for (int j = 0; j < 16; ++j) {
                    const uint8_t q = blk[1 + j];
                    out[b * 32 + j]      = d * (float)k_fp4_doubled[q & 0x0f];
                    out[b * 32 + j + 16] = d * (float)k_fp4_doubled[q >> 4];
                }
            }
            return;
        case T_Q4_K:  // quant.rs:399-416: d, dmin | scales[12] | qs[128]
            for (size_t b = 0; b < n / 256; ++b) {
                const uint8_t * blk = src + b * 144;
                const float d = half_to_float(rd16(blk));
                const float dmin = half_to_float(rd16(blk + 2));
                const uint8_t * scales = blk + 4;
                const uint8_t * qs = blk + 16;
                float * y = out + b * 256;
                for (int pair = 0; pair < 4; ++pair) {   // 64 elements per pair of sub-blocks
                    uint8_t sc1, m1, sc2, m2;
                    q4k_scale_min(2 * pair, scales, sc1, m1);
                    q4k_scale_min(2 * pair + 1, scales, sc2, m2);
                    const float d1 = d * (float)sc1, mm1 = dmin * (float)m1;
                    const float d2 = d * (float)sc2, mm2 = dmin * (float)m2;
                    const uint8_t * q = qs + 32 * pair;
                    for (int l = 0; l < 32; ++l) {
                        y[64 * pair + l]      = d1 * (float)(q[l] & 0x0f) - mm1;
                        y[64 * pair + 32 + l] = d2 * (float)(q[l] >> 4) - mm2;
                    }
                }
            }
            return;
        case T_Q5_K:  // quant.rs:418-442: d, dmin | scales[12] | qh[32] | qs[128]
            // As Q4_K with a fifth bit: element l of sub-block s takes bit s of qh[l] as 16.
            for (size_t b = 0; b < n / 256; ++b) {
                const uint8_t * blk = src + b * 176;
                const float d = half_to_float(rd16(blk));
                const float dmin = half_to_float(rd16(blk + 2));
                const uint8_t * scales = blk + 4;
                const uint8_t * qh = blk + 16;
                const uint8_t * qs = blk + 48;
                float * y = out + b * 256;
                for (int pair = 0; pair < 4; ++pair) {
                    uint8_t sc1, m1, sc2, m2;
                    q4k_scale_min(2 * pair, scales, sc1, m1);
                    q4k_scale_min(2 * pair + 1, scales, sc2, m2);
                    const float d1 = d * (float)sc1, mm1 = dmin * (float)m1;
                    const float d2 = d * (float)sc2, mm2 = dmin * (float)m2;
                    const uint8_t * q = qs + 32 * pair;
                    for (int l = 0; l < 32; ++l) {
                        const int h1 = (qh[l] >> (2 * pair)) & 1 ? 16 : 0, h2 = (qh[l] >> (2 * pair + 1)) & 1 ? 16 : 0;
                        y[64 * pair + l]      = d1 * (float)((q[l] & 0x0f) + h1) - mm1;
                        y[64 * pair + 32 + l] = d2 * (float)((q[l] >> 4) + h2) - mm2;
                    }
                }
            }
            return;
        case T_Q6_K:  // quant.rs:444-464: ql[128] | qh[64] | scales[16] (i8) | d (f16)
            // Element e of a block: half = e / 128, group g = (e % 128) / 32, l = e % 32. Its low four bits
            // are a nibble of ql[64 half + l + 32 (g & 1)] (the high nibble for g >= 2), its top two bits
            // are bits 2g, 2g + 1 of qh[32 half + l]; the code is that six-bit number minus 32, the scale
            // is scales[8 half + 2 g + l / 16], and the value is (d * scale) * code.
            for (size_t b = 0; b < n / 256; ++b) {
                const uint8_t * blk = src + b * 210;
                const float d = half_to_float(rd16(blk + 208));
                for (int e = 0; e < 256; ++e) {
                    const int half = e >> 7, g = (e & 127) >> 5, l = e & 31;
                    const uint8_t lo = blk[64 * half + l + 32 * (g & 1)];
                    const int nib = g >= 2 ? (lo >> 4) : (lo & 0x0f);
                    const int top = (blk[128 + 32 * half + l] >> (2 * g)) & 3;
                    const int code = (nib | (top << 4)) - 32;
                    const float scale = (float)(int8_t)blk[192 + 8 * half + 2 * g + (l >> 4)];
                    out[b * 256 + e] = (d * scale) * (float)code;
                }
            }
            return;
        default:
            throw std::runtime_error("oracle: unsupported ggml type " + std::to_string(type));
    }
}

// ggml's quantize_row_q8_0_ref as the fixture generator restates it
// (scripts/gen-tiny-fixture.py:173-197): d = amax/127 stored as f16, the
// codes use the *unrounded* d, round half away from zero, clamp to 127.
inline void quantize_q8_0(const float * x, size_t n, uint8_t * dst) {
    for (size_t b = 0; b < n / 32; ++b) {
        const float * v = x + b * 32;
        double amax = 0.0;
        for (int j = 0; j < 32; ++j) amax = std::fmax(amax, std::fabs((double)v[j]));
        const double d = amax / 127.0;
        const double inv = d != 0.0 ? 1.0 / d : 0.0;
        const uint16_t h = double_to_half(d);
        uint8_t * blk = dst + b * 34;
        blk[0] = (uint8_t)(h & 0xff);
        blk[1] = (uint8_t)(h >> 8);
        for (int j = 0; j < 32; ++j) {
            const double scaled = (double)v[j] * inv;
            double code = std::floor(std::fabs(scaled) + 0.5);
            if (code > 127.0) code = 127.0;
            blk[2 + j] = (uint8_t)(int8_t)(scaled >= 0.0 ? code : -code);
        }
    }
}

}  // namespace oracle
