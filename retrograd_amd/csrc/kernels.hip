// gfx950 (CDNA4, wave64) kernels of the batched decode step.
//
// Data layouts (all chosen for this hardware, none inherited from GGUF beyond
// the bits of each quantised block):
//
//  * Weight tiles. A quantised matrix [N][K] (K % 256 == 0, N % 16 == 0) is cut
//    into tiles of 16 rows x 256 columns. A tile stores first one 16-byte
//    header per row, then the quantised payload ordered so that lane l of a
//    wave reads 16 contiguous bytes at offset l*16 of each 1 KiB load:
//      Q4_K  2304 B = 16 x (d, dmin, 12 bytes of re-encoded scales) + 2 loads;  lane (r = l%16,
//            g = l/16) of load h holds, as 4 dwords, the 8 nibbles of
//            elements 32*(4h+j) + 8g .. +8 of row r, j = 0..3. Inside a dword
//            the nibbles are ordered e0 e2 e4 e6 | e1 e3 e5 e7 so that masking
//            with 0x000F000F / 0x00F000F0 yields f16 pairs in natural order.
//      Q8_0  4352 B = 16 x scales[8] (f16) + 4 loads; lane (r, g) of load q
//            holds elements 32*(2q)+8g..+8 and 32*(2q+1)+8g..+8 of row r.
//      Q5_K  2816 B = the Q4_K tile of the low nibbles + 512 B of fifth bits (k_repack_q4k<true>).
//      Q6_K  3360 B = scales, d, a plane of low nibbles and a plane of top bit pairs (k_repack_q6k).
//    The byte count equals the GGUF byte count of the same matrix.
//
//  * KV pages. A page holds 32 positions of one sequence for one kv head:
//      K: [dims/32][token half (2)][g (4)][token (16)][8 halves]   - the A operand
//         of a 16x16x32 MFMA (row = token, k = 8 dims) is one 16-byte load/lane
//      V: [dims/16][g (4)][dim (16)][8 halves] holding, for k-slot (g, i), the
//         token 4g+i (i < 4) or 16+4g+(i-4) (i >= 4): exactly the tokens whose
//         scores lane group g owns after the QK^T MFMAs, so P feeds the PV MFMA
//         without any cross-lane movement.
//
// MFMA operand convention used throughout (v_mfma_f32_16x16x32_f16): lane l
// supplies row/column l%16 and k-slots (l/16, 0..7) of both operands; the
// result holds rows 4*(l/16)+i, column l%16. Both operands always use the same
// (lane group, slot) for the same logical k, so the hardware's internal k
// order never matters.
#include <mutex>
#include <cstdlib>
#include "dev_common.hpp"

namespace rk {

BlockGeom geom_of(int type) {
    switch (type) {
        case WT_F32:   return {1, 4};
        case WT_F16:   return {1, 2};
        case WT_BF16:  return {1, 2};
        case WT_Q8_0:  return {32, 34};
        case WT_MXFP4: return {32, 17};
        case WT_Q4_K:  return {256, 144};
        case WT_Q5_K:  return {256, 176};
        case WT_Q6_K:  return {256, 210};
        case WT_Q4_1:  return {32, 20};
        case WT_Q5_1:  return {32, 24};
        case WT_Q2_K:  return {256, 84};
        case WT_IQ4_XS: return {256, 136};
        default: throw std::runtime_error("unsupported tensor type " + std::to_string(type));
    }
}

size_t row_bytes(int type, int64_t k) {
    const BlockGeom g = geom_of(type);
    if (k % g.elements != 0) throw std::runtime_error("row length is not a whole number of blocks");
    return (size_t)(k / g.elements) * g.bytes;
}

bool can_pack(int type, int64_t K, int64_t N) {
    return (type == WT_Q4_K || type == WT_Q8_0 || type == WT_Q6_K || type == WT_Q5_K) && K % 256 == 0 && N % 16 == 0 && K > 0 && N > 0;
}

// ---------------------------------------------------------------------------
// small device helpers

// One element of a raw GGUF row, decoded exactly as the stored blocks define
// it (two roundings for d*q - m, no contraction).
__device__ float decode_elem(int type, const uint8_t * row, int k) {
    switch (type) {
        case WT_F32: return ((const float *)row)[k];
        case WT_F16: return h2f(((const uint16_t *)row)[k]);
        case WT_BF16: return __uint_as_float((uint32_t)((const uint16_t *)row)[k] << 16);
        case WT_Q8_0: {
            const uint8_t * b = row + (size_t)(k >> 5) * 34;
            const float d = h2f(*(const uint16_t *)b);
            return __fmul_rn(d, (float)(int8_t)b[2 + (k & 31)]);
        }
        case WT_MXFP4: {
            const uint8_t * b = row + (size_t)(k >> 5) * 17;
            const int e = k & 31;
            const uint8_t byte = b[1 + (e & 15)];
            const int code = e < 16 ? (byte & 0x0f) : (byte >> 4);
            const int mag = code & 7;
            // doubled E2M1 magnitudes 0 1 2 3 4 6 8 12
            const int dv = mag < 4 ? mag : (mag == 4 ? 4 : (mag == 5 ? 6 : (mag == 6 ? 8 : 12)));
            const uint8_t x = b[0];
            const uint32_t bits = x == 0 ? 0x00200000u : (x == 1 ? 0x00400000u : ((uint32_t)x - 1) << 23);
            const float d = __uint_as_float(bits);
            return __fmul_rn(d, (float)((code & 8) ? -dv : dv));
        }
        case WT_Q4_K:
        case WT_Q5_K: {
            // Q5_K: d, dmin | scales[12] | qh[32] | qs[128] - a Q4_K block with a fifth bit, bit (e / 32) of qh[e % 32]
            const bool five = type == WT_Q5_K;
            const uint8_t * b = row + (size_t)(k >> 8) * (five ? 176 : 144);
            const int e = k & 255;
            const int j = e >> 5;
            const uint8_t * sc = b + 4;
            int s, m;
            if (j < 4) {
                s = sc[j] & 63;
                m = sc[j + 4] & 63;
            } else {
                s = (sc[j + 4] & 0x0f) | ((sc[j - 4] >> 6) << 4);
                m = (sc[j + 4] >> 4) | ((sc[j] >> 6) << 4);
            }
            const uint8_t byte = b[(five ? 48 : 16) + (e >> 6) * 32 + (e & 31)];
            int q = (e & 32) ? (byte >> 4) : (byte & 0x0f);
            if (five) q += ((b[16 + (e & 31)] >> j) & 1) << 4;
            const float d = h2f(*(const uint16_t *)b);
            const float dmin = h2f(*(const uint16_t *)(b + 2));
            return __fsub_rn(__fmul_rn(__fmul_rn(d, (float)s), (float)q), __fmul_rn(dmin, (float)m));
        }
        case WT_Q6_K: {
            // ql[128] | qh[64] | scales[16] (i8) | d (f16): element e has half = e / 128, group g = (e % 128) / 32,
            // l = e % 32; low bits from a nibble of ql[64 half + l + 32 (g & 1)] (high nibble for g >= 2),
            // top two bits from qh[32 half + l] >> 2g; value = (d * scale[8 half + 2 g + l / 16]) * (code - 32)
            const uint8_t * b = row + (size_t)(k >> 8) * 210;
            const int e = k & 255;
            const int half = e >> 7, g = (e & 127) >> 5, l = e & 31;
            const uint8_t lo = b[64 * half + l + 32 * (g & 1)];
            const int nib = g >= 2 ? (lo >> 4) : (lo & 0x0f);
            const int top = (b[128 + 32 * half + l] >> (2 * g)) & 3;
            const float d = h2f((uint16_t)(b[208] | (b[209] << 8)));
            const float scale = (float)(int8_t)b[192 + 8 * half + 2 * g + (l >> 4)];
            return __fmul_rn(__fmul_rn(d, scale), (float)((nib | (top << 4)) - 32));
        }
        case WT_Q4_1:
        case WT_Q5_1: {
            // d, m (f16) | [qh (u32)] | 16 bytes: element e is a nibble of byte e % 16 (the high one for e >= 16), with
            // bit e of qh on top for Q5_1; value = d * q + m
            const bool five = type == WT_Q5_1;
            const uint8_t * b = row + (size_t)(k >> 5) * (five ? 24 : 20);
            const int e = k & 31;
            const uint8_t byte = b[(five ? 8 : 4) + (e & 15)];
            int q = e < 16 ? (byte & 0x0f) : (byte >> 4);
            if (five) q |= ((b[4 + (e >> 3)] >> (e & 7)) & 1) << 4;
            const float d = h2f(*(const uint16_t *)b), m = h2f(*(const uint16_t *)(b + 2));
            return __fadd_rn(__fmul_rn(d, (float)q), m);
        }
        case WT_Q2_K: {
            // scales[16] | qs[64] | d, dmin (f16): element e reads two bits of qs[32 (e / 128) + e % 32] at 2 ((e / 32) % 4),
            // its sub-block's byte scales[e / 16] holds the scale (low nibble) and the min (high)
            const uint8_t * b = row + (size_t)(k >> 8) * 84;
            const int e = k & 255;
            const int q = (b[16 + (e >> 7) * 32 + (e & 31)] >> (2 * ((e >> 5) & 3))) & 3;
            const uint8_t sc = b[e >> 4];
            const float d = h2f((uint16_t)(b[80] | (b[81] << 8))), dmin = h2f((uint16_t)(b[82] | (b[83] << 8)));
            return __fsub_rn(__fmul_rn(__fmul_rn(d, (float)(sc & 0x0f)), (float)q), __fmul_rn(dmin, (float)(sc >> 4)));
        }
        case WT_IQ4_XS: {
            // d (f16) | scales_h (u16) | scales_l[4] | qs[128]: sub-block ib = e / 32 has the six-bit scale
            // (scales_l nibble ib) | (scales_h bits 2 ib, 2 ib + 1) << 4, minus 32; its codes index the IQ4_NL table
            const int8_t table[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
            const uint8_t * b = row + (size_t)(k >> 8) * 136;
            const int e = k & 255, ib = e >> 5;
            const uint8_t byte = b[8 + 16 * ib + (e & 15)];
            const int code = (e & 16) ? (byte >> 4) : (byte & 0x0f);
            const int sh = b[2] | (b[3] << 8);
            const int ls = ((b[4 + (ib >> 1)] >> (4 * (ib & 1))) & 0x0f) | (((sh >> (2 * ib)) & 3) << 4);
            const float d = h2f((uint16_t)(b[0] | (b[1] << 8)));
            return __fmul_rn(__fmul_rn(d, (float)(ls - 32)), (float)table[code]);
        }
        default: return 0.0f;
    }
}

// Writes up to 32 consecutive activations of one token (k0 a multiple of 32) as
// f16 hi/lo pairs and, for a whole block, the sum of the stored values as hi + lo
// halves. Only the values themselves: rows of a width that is no multiple of 32
// have no quantised consumer.
__device__ __forceinline__ void store_act_block(const float * v, int count, const Act & out, int tok, int k0) {
    float sum = 0.0f;
    for (int i = 0; i < count; ++i) {
        const __half h = sat_half(v[i]);
        const __half l = __float2half_rn(fminf(fmaxf(v[i], -65504.0f), 65504.0f) - __half2float(h));
        out.x[act_at(tok, k0 + i, 0, out.K)] = h;
        out.x[act_at(tok, k0 + i, 1, out.K)] = l;
        sum += __half2float(h) + __half2float(l);
    }
    if (out.sums && count == 32) {
        const __half a = sat_half(sum);
        out.sums[act_sum_at(tok, k0 >> 5, 0, out.K)] = a;
        out.sums[act_sum_at(tok, k0 >> 5, 1, out.K)] = __float2half_rn(sum - __half2float(a));
    }
}

// Host-side check of what a producer is asked to write.
static void check_act_out(const Act & out, int K, const char * what, int n_rows) {
    if (out.qc && ((out.quant != AQ_Q8_K && out.quant != AQ_Q8_0) || !out.qx || !out.qd || (out.quant == AQ_Q8_K && !out.qbs) || n_rows > GEMV_MAX_T))
        throw std::runtime_error(std::string(what) + ": the integer code buffers go with a Q8_K or Q8_0 conversion of at most "
                                 + std::to_string(GEMV_MAX_T) + " rows");
    if (out.K != K) throw std::runtime_error(std::string(what) + ": activation width does not match");
    if (!out.x && !out.qx) throw std::runtime_error(std::string(what) + ": no activation buffer to write");
    if (out.qx) {
        if (out.quant != AQ_Q8_0 && out.quant != AQ_Q8_K)
            throw std::runtime_error(std::string(what) + ": unknown activation conversion");
        if (K % out.quant != 0)
            throw std::runtime_error(std::string(what) + ": the row width is no multiple of the conversion's block");
    }
}

// ---------------------------------------------------------------------------
// plain streaming kernels: the yardstick for memory counters and bandwidth

__global__ __launch_bounds__(256) void k_stream_copy(const u4 * __restrict__ src, u4 * __restrict__ dst, size_t n) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) dst[i] = src[i];
}

__global__ __launch_bounds__(256) void k_stream_read(const u4 * __restrict__ src, u4 * __restrict__ sink, size_t n) {
    u4 acc = {0, 0, 0, 0};
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const u4 v = src[i];
        acc.x ^= v.x; acc.y ^= v.y; acc.z ^= v.z; acc.w ^= v.w;
    }
    // data-dependent and practically never true: keeps the loads alive without a store stream
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[blockIdx.x] = acc;
}

void stream_copy(hipStream_t s, const void * src, void * dst, size_t bytes, int read_only) {
    const size_t n = bytes / 16;
    if (n == 0) return;
    const unsigned blocks = (unsigned)std::min<size_t>((n + 255) / 256, 256 * 16);
    if (read_only) hipLaunchKernelGGL(k_stream_read, dim3(blocks), dim3(256), 0, s, (const u4 *)src, (u4 *)dst, n);
    else hipLaunchKernelGGL(k_stream_copy, dim3(blocks), dim3(256), 0, s, (const u4 *)src, (u4 *)dst, n);
    check_launch("stream_copy");
}

// ---------------------------------------------------------------------------
// weight repacking (runs once per tensor at load)

// FIVE: Q5_K. The tile is the Q4_K tile of the low nibbles followed by 512 bytes of fifth bits, one dword per
// k-half and lane: for k-step j the bits of the lane's elements 0 and 4 at 2j and 2j + 1, of 2 and 6 at 8 + 2j.., of
// 1 and 5 at 16 + 2j.., of 3 and 7 at 24 + 2j.. - one shift puts them above the nibbles the Q4_K decode isolates.
template <bool FIVE>
__global__ void k_repack_q4k(const uint8_t * __restrict__ raw, uint8_t * __restrict__ dst, int nsb, int n_tiles) {
    // one thread per output dword: 576 (704) dwords per (tile, super-block)
    constexpr int DW = FIVE ? 704 : 576, BLK = FIVE ? 176 : 144, QS = FIVE ? 48 : 16;
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t total = (size_t)n_tiles * nsb * DW;
    if (gid >= total) return;
    const int w = (int)(gid % DW);
    const size_t ts = gid / DW;
    const int sb = (int)(ts % nsb);
    const size_t rt = ts / nsb;
    uint32_t out;
    if (w < 64) {                       // headers: row r, dword j
        const int r = w >> 2, j = w & 3;
        const uint8_t * blk = raw + ((rt * 16 + r) * nsb + sb) * BLK;
        if (j == 0) {
            out = *(const uint32_t *)blk;          // d, dmin
        } else {
            // the 6-bit scales and mins, re-encoded one per byte (see q4k_scales)
            const uint8_t * q = blk + 4;
            out = 0;
            for (int i = 0; i < 4; ++i) {
                const uint32_t sc_lo = q[i] & 63, mn_lo = q[i + 4] & 63;
                const uint32_t sc_hi = (q[i + 8] & 0x0f) | ((q[i] >> 6) << 4);
                const uint32_t mn_hi = (q[i + 8] >> 4) | ((q[i + 4] >> 6) << 4);
                const uint32_t low = j == 1 ? sc_lo : (j == 2 ? sc_hi : mn_lo);
                const uint32_t top = (mn_hi >> (2 * (j - 1))) & 3;
                out |= (low | (top << 6)) << (8 * i);
            }
        }
    } else if (FIVE && w >= 576) {
        const int v = w - 576;
        const int h = v >> 6, lane = v & 63;
        const int r = lane & 15, g = lane >> 4;
        const uint8_t * blk = raw + ((rt * 16 + r) * nsb + sb) * BLK;
        const int place[8] = {0, 16, 8, 24, 1, 17, 9, 25};      // element i of the lane's eight, at k-step 0
        out = 0;
        for (int j = 0; j < 4; ++j)
            for (int i = 0; i < 8; ++i)
                out |= (uint32_t)((blk[16 + 8 * g + i] >> (4 * h + j)) & 1) << (place[i] + 2 * j);
    } else {
        const int v = w - 64;           // 0..511
        const int h = v >> 8;           // load
        const int lane = (v >> 2) & 63;
        const int j = v & 3;
        const int r = lane & 15, g = lane >> 4;
        const uint8_t * blk = raw + ((rt * 16 + r) * nsb + sb) * BLK;
        const int s = 4 * h + j;        // sub-block
        uint32_t nib[8];
        for (int i = 0; i < 8; ++i) {
            const int e = 32 * s + 8 * g + i;
            const uint8_t byte = blk[QS + (e >> 6) * 32 + (e & 31)];
            nib[i] = (e & 32) ? (byte >> 4) : (byte & 0x0f);
        }
        out = nib[0] | (nib[2] << 4) | (nib[4] << 8) | (nib[6] << 12)
            | (nib[1] << 16) | (nib[3] << 20) | (nib[5] << 24) | (nib[7] << 28);
    }
    *(uint32_t *)(dst + ts * (DW * 4) + (size_t)w * 4) = out;
}

__global__ void k_repack_q8_0(const uint8_t * __restrict__ raw, uint8_t * __restrict__ dst, int nsb, int n_tiles) {
    // 1088 dwords per (tile, group of 8 blocks): 64 header + 1024 payload
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t total = (size_t)n_tiles * nsb * 1088;
    if (gid >= total) return;
    const int w = (int)(gid % 1088);
    const size_t ts = gid / 1088;
    const int sb = (int)(ts % nsb);
    const size_t rt = ts / nsb;
    uint32_t out;
    if (w < 64) {                       // row r, scales 2j and 2j+1
        const int r = w >> 2, j = w & 3;
        const uint8_t * row = raw + (rt * 16 + r) * (size_t)nsb * 272 + (size_t)sb * 272;
        const uint32_t a = *(const uint16_t *)(row + (2 * j) * 34);
        const uint32_t b = *(const uint16_t *)(row + (2 * j + 1) * 34);
        out = a | (b << 16);
    } else {
        const int v = w - 64;           // 0..1023
        const int q = v >> 8;           // load 0..3
        const int lane = (v >> 2) & 63;
        const int j = v & 3;            // dword within the 16 bytes
        const int r = lane & 15, g = lane >> 4;
        const int blk = 2 * q + (j >> 1);
        const int e0 = 8 * g + 4 * (j & 1);
        const uint8_t * p = raw + (rt * 16 + r) * (size_t)nsb * 272 + (size_t)sb * 272 + (size_t)blk * 34 + 2 + e0;
        out = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
    }
    *(uint32_t *)(dst + ts * 4352 + (size_t)w * 4) = out;
}

// Q6_K: 16 rows x one super-block = 3360 bytes, the size of the 16 raw blocks:
//   [0, 256)      the sixteen i8 scales of row r at 16 r
//   [256, 288)    d (f16) of row r at 256 + 2 r
//   [288, 2336)   low nibbles: for k-half h, lane = 16 g + r, k-step j one dword at 288 + 1024 h + 16 lane + 4 j with
//                 the eight codes c0..c7 of elements 128 h + 32 j + 8 g + i: c(2p) in bits 4p.., c(2p+1) in bits 16 + 4p..
//   [2336, 3360)  top two bits: one dword per two k-steps at 2336 + 512 h + 8 lane + 4 m. K-step 2m: c(2p) in bits
//                 4 + 2p.., c(2p+1) in bits 20 + 2p..; k-step 2m + 1: the same places rotated left by eight.
// so that (low >> 4p) & 0x000F000F and (top >> 2p) & 0x00300030 line a pair of codes up in the two halves of a dword.
__device__ __forceinline__ uint32_t q6k_code(const uint8_t * blk, int e) {
    const int half = e >> 7, g = (e & 127) >> 5, l = e & 31;
    const uint8_t lo = blk[64 * half + l + 32 * (g & 1)];
    const uint32_t nib = g >= 2 ? (lo >> 4) : (lo & 0x0f);
    const uint32_t top = (blk[128 + 32 * half + l] >> (2 * g)) & 3;
    return nib | (top << 4);
}

__global__ void k_repack_q6k(const uint8_t * __restrict__ raw, uint8_t * __restrict__ dst, int nsb, int n_tiles) {
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t total = (size_t)n_tiles * nsb * 840;
    if (gid >= total) return;
    const int w = (int)(gid % 840);
    const size_t ts = gid / 840;
    const int sb = (int)(ts % nsb);
    const size_t rt = ts / nsb;
    auto block_of = [&](int r) { return raw + ((rt * 16 + r) * nsb + sb) * 210; };
    uint32_t out = 0;
    if (w < 64) {
        const uint8_t * b = block_of(w >> 2) + 192 + 4 * (w & 3);
        out = (uint32_t)b[0] | ((uint32_t)b[1] << 8) | ((uint32_t)b[2] << 16) | ((uint32_t)b[3] << 24);
    } else if (w < 72) {
        const uint8_t * b0 = block_of(2 * (w - 64)) + 208, * b1 = block_of(2 * (w - 64) + 1) + 208;
        out = (uint32_t)b0[0] | ((uint32_t)b0[1] << 8) | ((uint32_t)b1[0] << 16) | ((uint32_t)b1[1] << 24);
    } else if (w < 584) {
        const int v = w - 72;
        const int h = v >> 8, lane = (v >> 2) & 63, j = v & 3;
        const uint8_t * b = block_of(lane & 15);
        const int e0 = 128 * h + 32 * j + 8 * (lane >> 4);
        for (int p = 0; p < 4; ++p) {
            out |= (q6k_code(b, e0 + 2 * p) & 15) << (4 * p);
            out |= (q6k_code(b, e0 + 2 * p + 1) & 15) << (16 + 4 * p);
        }
    } else {
        const int v = w - 584;
        const int h = v >> 7, lane = (v >> 1) & 63, m = v & 1;
        const uint8_t * b = block_of(lane & 15);
        const int e0 = 128 * h + 64 * m + 8 * (lane >> 4);
        for (int p = 0; p < 4; ++p) {
            out |= (q6k_code(b, e0 + 2 * p) >> 4) << (4 + 2 * p);
            out |= (q6k_code(b, e0 + 2 * p + 1) >> 4) << (20 + 2 * p);
            out |= (q6k_code(b, e0 + 32 + 2 * p) >> 4) << (12 + 2 * p);
            out |= (q6k_code(b, e0 + 32 + 2 * p + 1) >> 4) << ((28 + 2 * p) & 31);
        }
    }
    *(uint32_t *)(dst + ts * 3360 + (size_t)w * 4) = out;
}

void repack(hipStream_t s, int type, const uint8_t * raw, uint8_t * packed, int K, int N) {
    if (!can_pack(type, K, N)) throw std::runtime_error("repack: shape or type has no tile layout");
    const int nsb = K / 256, n_tiles = N / 16;
    const size_t per = type == WT_Q4_K ? 576 : (type == WT_Q5_K ? 704 : (type == WT_Q6_K ? 840 : 1088));     // dwords per tile and super-block
    const size_t total = (size_t)n_tiles * nsb * per;
    if ((total + 255) / 256 > 0x7fffffffu) throw std::runtime_error("repack: the matrix is too large for one launch");
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (type == WT_Q4_K) hipLaunchKernelGGL(k_repack_q4k<false>, dim3(blocks), dim3(256), 0, s, raw, packed, nsb, n_tiles);
    else if (type == WT_Q5_K) hipLaunchKernelGGL(k_repack_q4k<true>, dim3(blocks), dim3(256), 0, s, raw, packed, nsb, n_tiles);
    else if (type == WT_Q6_K) hipLaunchKernelGGL(k_repack_q6k, dim3(blocks), dim3(256), 0, s, raw, packed, nsb, n_tiles);
    else hipLaunchKernelGGL(k_repack_q8_0, dim3(blocks), dim3(256), 0, s, raw, packed, nsb, n_tiles);
    check_launch("repack");
}

// ---------------------------------------------------------------------------
// matmul over tiled quantised weights (MFMA)


template <int NT>
__device__ __forceinline__ void mm_finish(const MMArgs & a, f4 (&acc)[NT], int rt, int tbase, int nt,
                                          int wk, int wr, float * lds) {
    const int lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    if (a.ksplit > 1) {
        // lds[(wk-1)][wr][tile*4+i][lane]
        const int rows_per_wg = 4 / a.ksplit;
        if (wk > 0) {
            float * dst = lds + ((size_t)((wk - 1) * rows_per_wg + wr) * NT * 4) * 64;
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) dst[(t * 4 + i) * 64 + lane] = acc[t][i];
        }
        __syncthreads();
        if (wk > 0) return;
        for (int k = 1; k < a.ksplit; ++k) {
            const float * src = lds + ((size_t)((k - 1) * rows_per_wg + wr) * NT * 4) * 64;
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[t][i] += src[(t * 4 + i) * 64 + lane];
        }
    }
    if (rt >= a.n_row_tiles) return;
    const int n = rt * 16 + r;
    const float bias = a.bias ? a.bias[n] : 0.0f;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        if (t >= nt) break;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int tok = tbase + t * 16 + 4 * g + i;
            if (tok < a.T) {
                float * p = a.y + (size_t)tok * a.ldy + a.col0 + n;
                const float v = acc[t][i] + bias;
                *p = a.mode == MM_ADD ? *p + v : v;
            }
        }
    }
}

template <int NT>
__global__ __launch_bounds__(256) void k_mm_q4k(MMArgs a) {
    extern __shared__ float lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int wr = wave / a.ksplit, wk = wave % a.ksplit;
    const int rt = blockIdx.x * (4 / a.ksplit) + wr;
    const int tbase = blockIdx.y * 64;
    const int nt = min(NT, (a.T - tbase + 15) >> 4);
    const int nsb = a.K >> 8;

    f4 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = (f4){0.f, 0.f, 0.f, 0.f};

    // activation row of this lane for every token tile (clamped: rows past T
    // are computed on the last row and never stored)
    const __half * xt[NT];
    const __half * st[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        xt[t] = a.x + (size_t)blockIdx.y * act_chunk_halves(a.K) + t * 512 + lane * 8;
        st[t] = a.sums + (size_t)blockIdx.y * act_sum_chunk_halves(a.K) + t * 512 + lane * 8;
    }

    if (rt < a.n_row_tiles) {
        for (int sb = wk; sb < nsb; sb += a.ksplit) {
            const uint8_t * tile = a.w + ((size_t)rt * nsb + sb) * 2304;
            const u4 hdr = *(const u4 *)(tile + r * 16);
            const u4 q0 = *(const u4 *)(tile + 256 + lane * 16);
            const u4 q1 = *(const u4 *)(tile + 1280 + lane * 16);
            const float d = h2f((uint16_t)(hdr.x & 0xffff));
            const float dmin = h2f((uint16_t)(hdr.x >> 16));
            const Q4KScales s4 = q4k_scales(hdr);
            uint32_t sc[8], mn[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                sc[j] = (s4.sc[j >> 2] >> (8 * (j & 3))) & 0xff;
                mn[j] = (s4.mn[j >> 2] >> (8 * (j & 3))) & 0xff;
            }
            f4 accq[NT], accm[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                accq[t] = (f4){0.f, 0.f, 0.f, 0.f};
                accm[t] = (f4){0.f, 0.f, 0.f, 0.f};
            }
            // min term: sum_s m[r][s] * xsum[t][s], k-slots (g=0: hi sums, g=1: lo sums)
            {
                h8 mB;
#pragma unroll
                for (int i = 0; i < 8; ++i) mB[i] = g < 2 ? (_Float16)(float)mn[i] : (_Float16)0.0f;
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const h8 sA = load_h8(st[t] + (size_t)sb * 2048);
                    accm[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(sA, mB, accm[t], 0, 0, 0);
                }
            }
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const uint32_t wq = s < 4 ? q0[s & 3] : q1[s & 3];
                const _Float16 sch = (_Float16)(float)sc[s];
                const h2 k1 = {sch, sch};
                const h2 c1 = k1 * (_Float16)(-1024.0f);        // exact: sc <= 63
                const h2 k2 = k1 * (_Float16)(0.0625f);         // exact
                const h2 c2 = k1 * (_Float16)(-64.0f);          // exact
                const uint32_t w8 = wq >> 8;
                const h2 u0 = __builtin_bit_cast(h2, (wq & 0x000F000Fu) | 0x64006400u);   // 1024 + e0, e1
                const h2 u1 = __builtin_bit_cast(h2, (wq & 0x00F000F0u) | 0x64006400u);   // 1024 + 16*(e2, e3)
                const h2 u2 = __builtin_bit_cast(h2, (w8 & 0x000F000Fu) | 0x64006400u);
                const h2 u3 = __builtin_bit_cast(h2, (w8 & 0x00F000F0u) | 0x64006400u);
                // fused multiply-add: (1024 + e) * sc - 1024 * sc == sc * e exactly (<= 945)
                const h2 a0 = __builtin_elementwise_fma(u0, k1, c1);
                const h2 a1 = __builtin_elementwise_fma(u1, k2, c2);
                const h2 a2 = __builtin_elementwise_fma(u2, k1, c1);
                const h2 a3 = __builtin_elementwise_fma(u3, k2, c2);
                const h8 B = {a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const h8 A = load_h8(xt[t] + (size_t)((sb * 8 + s) * 2) * 2048);
                    const h8 Al = load_h8(xt[t] + (size_t)((sb * 8 + s) * 2 + 1) * 2048);
                    accq[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B, accq[t], 0, 0, 0);
                    accq[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Al, B, accq[t], 0, 0, 0);
                }
            }
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    acc[t][i] = fmaf(-dmin, accm[t][i], fmaf(d, accq[t][i], acc[t][i]));
        }
    }
    mm_finish<NT>(a, acc, rt, tbase, nt, wk, wr, lds);
}

template <int NT>
__global__ __launch_bounds__(256) void k_mm_q8_0(MMArgs a) {
    extern __shared__ float lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15;
    const int wr = wave / a.ksplit, wk = wave % a.ksplit;
    const int rt = blockIdx.x * (4 / a.ksplit) + wr;
    const int tbase = blockIdx.y * 64;
    const int nt = min(NT, (a.T - tbase + 15) >> 4);
    const int nsb = a.K >> 8;

    f4 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = (f4){0.f, 0.f, 0.f, 0.f};
    const __half * xt[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) xt[t] = a.x + (size_t)blockIdx.y * act_chunk_halves(a.K) + t * 512 + lane * 8;
    const h2 bias1152 = {(_Float16)(-1152.0f), (_Float16)(-1152.0f)};

    if (rt < a.n_row_tiles) {
        for (int sb = wk; sb < nsb; sb += a.ksplit) {
            const uint8_t * tile = a.w + ((size_t)rt * nsb + sb) * 4352;
            const u4 hdr = *(const u4 *)(tile + r * 16);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const u4 d4 = *(const u4 *)(tile + 256 + q * 1024 + lane * 16);
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int s = 2 * q + half;
                    const uint32_t sw = hdr[s >> 1];
                    const float d = h2f((uint16_t)((s & 1) ? (sw >> 16) : (sw & 0xffff)));
                    // bytes are two's complement; flipping the sign bit gives q + 128 in
                    // 0..255, and 0x6400 | b is the f16 1024 + b: subtract 1152 for q.
                    const uint32_t w0 = d4[2 * half] ^ 0x80808080u;
                    const uint32_t w1 = d4[2 * half + 1] ^ 0x80808080u;
                    const h2 u0 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w0, 0x04010400u));
                    const h2 u1 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w0, 0x04030402u));
                    const h2 u2 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w1, 0x04010400u));
                    const h2 u3 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w1, 0x04030402u));
                    const h2 a0 = u0 + bias1152, a1 = u1 + bias1152, a2 = u2 + bias1152, a3 = u3 + bias1152;
                    const h8 B = {a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
#pragma unroll
                    for (int t = 0; t < NT; ++t) {
                        const h8 A = load_h8(xt[t] + (size_t)((sb * 8 + s) * 2) * 2048);
                        const h8 Al = load_h8(xt[t] + (size_t)((sb * 8 + s) * 2 + 1) * 2048);
                        f4 part = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B, (f4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                        part = __builtin_amdgcn_mfma_f32_16x16x32_f16(Al, B, part, 0, 0, 0);
#pragma unroll
                        for (int i = 0; i < 4; ++i) acc[t][i] = fmaf(d, part[i], acc[t][i]);
                    }
                }
            }
        }
    }
    mm_finish<NT>(a, acc, rt, tbase, nt, wk, wr, lds);
}

// The operand of a product with a weight of storage type round_as under ggml's arithmetic (WT_F32: as it is).
__device__ __forceinline__ float generic_operand(float hi, float lo, int round_as) {
    // F16 weights multiply the activations rounded to f16 (the hi half is that rounding), BF16 weights those
    // rounded to bf16
    if (round_as == WT_F16) return hi;
    float xv = hi + lo;
    if (round_as == WT_BF16) {
        uint32_t u = __float_as_uint(xv);
        u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
        xv = __uint_as_float(u);
    }
    return xv;
}

// Any type, any shape: one wave per output feature and group of eight tokens, raw GGUF rows.
__global__ __launch_bounds__(256) void k_mm_generic(int type, const uint8_t * __restrict__ raw, size_t rb,
                                                    const __half * __restrict__ x, int K, int N, int T,
                                                    float * y, int ldy, int col0, int mode, const float * bias,
                                                    int round_as) {
    const int lane = threadIdx.x & 63;
    const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (n >= N) return;
    const uint8_t * row = raw + (size_t)n * rb;
    const int t0 = blockIdx.y * 8;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (K % 8 == 0) {
        // eight consecutive k per lane: the activations of a token are 16 contiguous bytes per half
        for (int k = lane * 8; k < K; k += 512) {
            float w[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) w[i] = decode_elem(type, row, k + i);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int t = min(t0 + j, T - 1);
                const h8 hi = load_h8(x + act_at(t, k, 0, K)), lo = load_h8(x + act_at(t, k, 1, K));
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[j] = fmaf(w[i], generic_operand((float)hi[i], (float)lo[i], round_as), acc[j]);
            }
        }
    } else {
        for (int k = lane; k < K; k += 64) {
            const float w = decode_elem(type, row, k);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int t = min(t0 + j, T - 1);
                acc[j] = fmaf(w, generic_operand(__half2float(x[act_at(t, k, 0, K)]), __half2float(x[act_at(t, k, 1, K)]), round_as), acc[j]);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float v = wave_sum(acc[j]);
        if (lane == 0 && t0 + j < T) {
            float * p = y + (size_t)(t0 + j) * ldy + col0 + n;
            const float o = v + (bias ? bias[n] : 0.0f);
            *p = mode == MM_ADD ? *p + o : o;
        }
    }
}

// F32 rows (the expert router; unquantised heads) for more than a few tokens. The generic kernel gives a wave one
// output feature and eight tokens, so the activations - eight times the bytes of a weight row - are read once per
// feature, and its k-chunks of 512 follow one another. Here a workgroup owns EW features and eight tokens, its four
// waves take the k-chunks in turn (all loads of a launch are in flight at once for K <= 2048), every wave keeps its
// chunk's activations in registers for the EW features, and the waves' sums meet in LDS in wave order.
template <int EW>
__global__ __launch_bounds__(256) void k_mm_f32_rows(const float * __restrict__ wm, const __half * __restrict__ x, int K, int N, int T,
                                                     float * y, int ldy, int col0, int mode, const float * bias) {
    __shared__ float part[4][EW][8];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = blockIdx.x * EW;
    const int t0 = blockIdx.y * 8;
    float acc[EW][8];
#pragma unroll
    for (int e = 0; e < EW; ++e)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[e][j] = 0.0f;
    for (int k = wave * 512 + lane * 8; k < K; k += 2048) {
        float xv[8][8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int t = min(t0 + j, T - 1);
            const h8 hi = load_h8(x + act_at(t, k, 0, K)), lo = load_h8(x + act_at(t, k, 1, K));
#pragma unroll
            for (int i = 0; i < 8; ++i) xv[j][i] = (float)hi[i] + (float)lo[i];
        }
#pragma unroll
        for (int e = 0; e < EW; ++e) {
            if (n0 + e < N) {
                const f4 wa = *(const f4 *)(wm + (size_t)(n0 + e) * K + k), wb = *(const f4 *)(wm + (size_t)(n0 + e) * K + k + 4);
                const float w[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
#pragma unroll
                for (int j = 0; j < 8; ++j)
#pragma unroll
                    for (int i = 0; i < 8; ++i) acc[e][j] = fmaf(w[i], xv[j][i], acc[e][j]);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < EW; ++e) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float v = wave_sum(acc[e][j]);
            if (lane == 0) part[wave][e][j] = v;
        }
    }
    __syncthreads();
    if (threadIdx.x < EW * 8) {
        const int e = threadIdx.x >> 3, j = threadIdx.x & 7;
        if (n0 + e < N && t0 + j < T) {
            const float v = ((part[0][e][j] + part[1][e][j]) + part[2][e][j]) + part[3][e][j];
            float * p = y + (size_t)(t0 + j) * ldy + col0 + n0 + e;
            const float o = v + (bias ? bias[n0 + e] : 0.0f);
            *p = mode == MM_ADD ? *p + o : o;
        }
    }
}

void matmul_generic(hipStream_t s, const Weight & w, const Act & x, int T, float * y, int ldy, int col0,
                    int mode, const float * bias) {
    if (!w.raw) throw std::runtime_error("matmul_generic: the weight has no raw layout");
    if (x.K != w.K) throw std::runtime_error("matmul: activation width does not match the weight");
    if (T <= 0) return;
    const Act xo = x.operand(w.type);
    if (!xo.x) throw std::runtime_error("matmul: the activations were not prepared for this weight type");
    if (w.type == WT_F32 && w.K % 8 == 0 && ((uintptr_t)w.raw & 15) == 0 && T > 8) {
        // several token groups (a step of few tokens keeps the generic kernel's feature per wave for the parallelism)
        constexpr int EW = 4;
        hipLaunchKernelGGL(k_mm_f32_rows<EW>, dim3((w.N + EW - 1) / EW, (T + 7) / 8), dim3(256), 0, s, (const float *)w.raw,
                           xo.x, w.K, w.N, T, y, ldy, col0, mode, bias);
        check_launch("matmul_generic");
        return;
    }
    hipLaunchKernelGGL(k_mm_generic, dim3((w.N + 3) / 4, (T + 7) / 8), dim3(256), 0, s, w.type, w.raw, row_bytes(w.type, w.K),
                       xo.x, w.K, w.N, T, y, ldy, col0, mode, bias, xo.faithful ? w.type : WT_F32);
    check_launch("matmul_generic");
}

template <int NT>
static void launch_mm(hipStream_t s, int type, const MMArgs & a, dim3 grid, size_t lds) {
    if (type == WT_Q4_K) hipLaunchKernelGGL(k_mm_q4k<NT>, grid, dim3(256), lds, s, a);
    else hipLaunchKernelGGL(k_mm_q8_0<NT>, grid, dim3(256), lds, s, a);
}

__global__ __launch_bounds__(256) void k_reduce_slices(Slices sl, int T, float * y, int ldy, int col0, int mode) {
    const size_t gid = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (gid >= (size_t)T * sl.N) return;
    const int t = (int)(gid / sl.N), c = (int)(gid % sl.N);
    f4 v = {0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < sl.n; ++k) v += *(const f4 *)(sl.data + (size_t)k * sl.stride + gid);
    float * p = y + (size_t)t * ldy + col0 + c;
#pragma unroll
    for (int i = 0; i < 4; ++i) p[i] = mode == MM_ADD ? p[i] + v[i] : v[i];
}

void reduce_slices(hipStream_t s, const Slices & sl, int T, float * y, int ldy, int col0, int mode) {
    if (sl.n <= 0 || T <= 0) return;
    if (sl.N % 4 != 0) throw std::runtime_error("reduce_slices: the row width must be a multiple of 4");
    const size_t n = (size_t)T * sl.N / 4;
    hipLaunchKernelGGL(k_reduce_slices, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, sl, T, y, ldy, col0, mode);
    check_launch("reduce_slices");
}

static Slices matmul_impl(hipStream_t s, const Weight & w, const Act & x, int T, float * y, int ldy, int col0,
                          int mode, const float * bias, void * ws, bool may_slice);

void matmul(hipStream_t s, const Weight & w, const Act & x, int T, float * y, int ldy, int col0,
            int mode, const float * bias, void * ws) {
    const Slices sl = matmul_impl(s, w, x, T, y, ldy, col0, mode, bias, ws, true);
    reduce_slices(s, sl, T, y, ldy, col0, mode);
}

Slices matmul_deferred(hipStream_t s, const Weight & w, const Act & x, int T, float * y, int ldy, int col0,
                       int mode, const float * bias, void * ws) {
    return matmul_impl(s, w, x, T, y, ldy, col0, mode, bias, ws, true);
}

static Slices matmul_impl(hipStream_t s, const Weight & w, const Act & x, int T, float * y, int ldy, int col0,
                          int mode, const float * bias, void * ws, bool may_slice) {
    if (T <= 0) return Slices();
    if (!w.packed) {
        matmul_generic(s, w, x, T, y, ldy, col0, mode, bias);
        return Slices();
    }
    if (x.K != w.K) throw std::runtime_error("matmul: activation width does not match the weight");
    // the tile kernels know two layouts; anything else handed over as tiles would be read as one of them, out of bounds
    if (!can_pack(w.type, w.K, w.N)) throw std::runtime_error("matmul: this matrix type or shape has no tile layout");
    if (T <= GEMV_MAX_T) {     // a very small step whose producer left the Q8_K blocks themselves
        const Act xg = x.operand(w.type);
        if ((mode == MM_STORE || mode == MM_ADD) && gemv_can(w, xg, T)) {
            gemv(s, w, xg, T, y, ldy, col0, mode, bias);
            return Slices();
        }
    }
    if (ws) return matmul_lds(s, w, x, T, y, ldy, col0, mode, bias, ws, may_slice);
    if (w.type == WT_Q6_K || w.type == WT_Q5_K)
        throw std::runtime_error("matmul: Q5_K and Q6_K tiles are multiplied by the LDS kernels only (pass the workspace)");
    const Act xo = x.operand(w.type);
    if (!xo.x) throw std::runtime_error("matmul: the activations were not prepared for this weight type");
    if (w.type == WT_Q4_K && !xo.sums) throw std::runtime_error("matmul: Q4_K needs block sums");
    MMArgs a {};
    a.w = w.packed; a.x = xo.x; a.sums = xo.sums; a.y = y; a.bias = bias;
    a.K = w.K; a.N = w.N; a.T = T; a.ldy = ldy; a.col0 = col0; a.mode = mode;
    a.n_row_tiles = w.N / 16;
    // Enough waves to cover the chip: split K across the waves of a workgroup
    // when there are few row tiles.
    const int nsb = w.K / 256;
    int ksplit = 1;
    if (a.n_row_tiles < 1024 && nsb >= 8) ksplit = 4;
    else if (a.n_row_tiles < 2048 && nsb >= 4) ksplit = 2;
    a.ksplit = ksplit;
    const int rows_per_wg = 4 / ksplit;
    dim3 grid((a.n_row_tiles + rows_per_wg - 1) / rows_per_wg, (T + 63) / 64);
    const int nt = T >= 49 ? 4 : (T + 15) / 16;
    const size_t lds = ksplit > 1 ? (size_t)(ksplit - 1) * rows_per_wg * nt * 4 * 64 * sizeof(float) : 0;
    switch (nt) {
        case 1: launch_mm<1>(s, w.type, a, grid, lds); break;
        case 2: launch_mm<2>(s, w.type, a, grid, lds); break;
        case 3: launch_mm<3>(s, w.type, a, grid, lds); break;
        default: launch_mm<4>(s, w.type, a, grid, lds); break;
    }
    check_launch("matmul");
    return Slices();
}

// ---------------------------------------------------------------------------
// embedding, RMSNorm, SwiGLU

__global__ void k_embed(int type, const uint8_t * __restrict__ raw, size_t rb, const int32_t * __restrict__ tok,
                        int E, float * __restrict__ x) {
    const int t = blockIdx.y;
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= E) return;
    x[(size_t)t * E + k] = decode_elem(type, raw + (size_t)tok[t] * rb, k);
}

void embed(hipStream_t s, const Weight & emb, const int32_t * tok, int T, float * x) {
    if (!emb.raw) throw std::runtime_error("embed: the embedding has no raw layout");
    if (T <= 0) return;
    hipLaunchKernelGGL(k_embed, dim3((emb.K + 255) / 256, T), dim3(256), 0, s, emb.type, emb.raw,
                       row_bytes(emb.type, emb.K), tok, emb.K, x);
    check_launch("embed");
}

__global__ void k_decode_rows(int type, const uint8_t * __restrict__ raw, size_t rb, int K, float * __restrict__ out) {
    const int r = blockIdx.y;
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= K) return;
    out[(size_t)r * K + k] = decode_elem(type, raw + (size_t)r * rb, k);
}

void decode_rows(hipStream_t s, int type, const uint8_t * raw, int K, int n_rows, float * out) {
    if (n_rows <= 0 || K <= 0) return;
    hipLaunchKernelGGL(k_decode_rows, dim3((K + 255) / 256, n_rows), dim3(256), 0, s, type, raw, row_bytes(type, K), K, out);
    check_launch("decode_rows");
}

// ---------------------------------------------------------------------------
// per-row LoRA

// The operand of a dot product with a factor of this storage type.
__device__ __forceinline__ float lora_operand(float hi, float lo, int type) {
    if (type == WT_F16) return hi;                   // hi is the f16 rounding of the value
    float v = hi + lo;
    if (type == WT_BF16) {
        uint32_t u = __float_as_uint(v);
        u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
        v = __uint_as_float(u);
    }
    return v;
}

// mid[t][r] = sum_k A[r][k] * x[t][k]: one workgroup per (token, four rank rows); its 256 threads stride over k in
// groups of eight, so the activations are read once for the four rows, and the partial sums meet through LDS.
// (Both LoRA products in one workgroup per token were measured slower: too few workgroups for the chain of loads.)
// Up to three targets that read the same activations (q, k, v) share a launch: blockIdx.z picks the target.
struct LoraTargets {
    const LoraEntry * table[3];
    int N[3], col0[3];
    int group;      // 0: output n is column col0 + n; g > 0: column col0 + (n / g) * 2g + n % g (gate and up interleaved by g)
};

__global__ __launch_bounds__(256) void k_lora_down(LoraTargets tg, const RowDesc * __restrict__ rows,
                                                   const int32_t * __restrict__ tok_row, Act x, float * __restrict__ mid_all,
                                                   int T) {
    __shared__ float red[4][4];
    const int t = blockIdx.x;
    const int route = rows[tok_row[t]].route;
    if (route <= 0) return;
    const LoraEntry e = tg.table[blockIdx.z][route - 1];
    const int r0 = blockIdx.y * 4;
    if (!e.A || r0 >= e.rank) return;                     // the same for every thread of the workgroup
    float * mid = mid_all + (size_t)blockIdx.z * T * LORA_MAX_RANK;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nr = min(4, e.rank - r0);
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (x.K % 8 == 0) {
        for (int k = threadIdx.x * 8; k < x.K; k += 2048) {
            const h8 hi = load_h8(x.x + act_at(t, k, 0, x.K)), lo = load_h8(x.x + act_at(t, k, 1, x.K));
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = lora_operand((float)hi[i], (float)lo[i], e.a_type);
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                if (rr >= nr) break;
                const float * a = e.A + (size_t)(r0 + rr) * x.K + k;
                const f4 a0 = *(const f4 *)a, a1 = *(const f4 *)(a + 4);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc[rr] = fmaf(a0[i], v[i], acc[rr]);
                    acc[rr] = fmaf(a1[i], v[4 + i], acc[rr]);
                }
            }
        }
    } else {
        for (int k = threadIdx.x; k < x.K; k += 256) {
            const float v = lora_operand(__half2float(x.x[act_at(t, k, 0, x.K)]), __half2float(x.x[act_at(t, k, 1, x.K)]), e.a_type);
            for (int rr = 0; rr < nr; ++rr) acc[rr] = fmaf(e.A[(size_t)(r0 + rr) * x.K + k], v, acc[rr]);
        }
    }
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
        const float s = wave_sum(acc[rr]);
        if (lane == 0) red[wave][rr] = s;
    }
    __syncthreads();
    if ((int)threadIdx.x < nr) mid[(size_t)t * LORA_MAX_RANK + r0 + threadIdx.x] = (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
}

// y[t][col0 + n] += scale * sum_r B[n][r] * mid[t][r]
__global__ __launch_bounds__(256) void k_lora_up(LoraTargets tg, const RowDesc * __restrict__ rows,
                                                 const int32_t * __restrict__ tok_row, const float * __restrict__ mid_all,
                                                 float * __restrict__ y, int ldy, int T) {
    __shared__ float ops[LORA_MAX_RANK];        // mid[t][r] as the factor B multiplies, once per workgroup
    const int t = blockIdx.x;
    const int route = rows[tok_row[t]].route;
    if (route <= 0) return;
    const LoraEntry e = tg.table[blockIdx.z][route - 1];
    const int N = tg.N[blockIdx.z], col0 = tg.col0[blockIdx.z];
    if (!e.A) return;
    const float * m = mid_all + (size_t)blockIdx.z * T * LORA_MAX_RANK + (size_t)t * LORA_MAX_RANK;
    if ((int)threadIdx.x < e.rank) {
        const float v = m[threadIdx.x];
        const float hi = (float)(_Float16)fminf(fmaxf(v, -65504.0f), 65504.0f);
        ops[threadIdx.x] = lora_operand(hi, v - hi, e.b_type);
    }
    __syncthreads();
    const int n = blockIdx.y * 256 + threadIdx.x;
    if (n >= N) return;
    const float * b = e.B + (size_t)n * e.rank;
    float acc = 0.0f;
    if (e.rank % 4 == 0) {
        for (int r = 0; r < e.rank; r += 4) {
            const f4 b4 = *(const f4 *)(b + r);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc = fmaf(b4[i], ops[r + i], acc);
        }
    } else {
        for (int r = 0; r < e.rank; ++r) acc = fmaf(b[r], ops[r], acc);
    }
    const int col = tg.group > 0 ? (n / tg.group) * 2 * tg.group + n % tg.group : n;
    y[(size_t)t * ldy + col0 + col] += e.scale * acc;
}

void lora_apply_targets(hipStream_t s, int n_targets, const LoraEntry * const * tables, const int * widths, const int * cols,
                        const RowDesc * rows, const int32_t * tok_row, const Act & x, int T, float * y, int ldy, float * mid,
                        int group) {
    if (T <= 0 || n_targets <= 0) return;
    if (group < 0) throw std::runtime_error("lora: the interleave group must not be negative");
    if (n_targets > 3) throw std::runtime_error("lora: at most three targets share a launch");
    if (!x.x) throw std::runtime_error("lora: the unconverted activations are missing");
    LoraTargets tg {};
    tg.group = group;
    int max_n = 0;
    for (int i = 0; i < n_targets; ++i) {
        tg.table[i] = tables[i]; tg.N[i] = widths[i]; tg.col0[i] = cols[i];
        max_n = std::max(max_n, widths[i]);
    }
    if (max_n <= 0) return;
    hipLaunchKernelGGL(k_lora_down, dim3(T, LORA_MAX_RANK / 4, n_targets), dim3(256), 0, s, tg, rows, tok_row, x, mid, T);
    check_launch("lora_down");
    hipLaunchKernelGGL(k_lora_up, dim3(T, (max_n + 255) / 256, n_targets), dim3(256), 0, s, tg, rows, tok_row, mid, y, ldy, T);
    check_launch("lora_up");
}

void lora_apply(hipStream_t s, const LoraEntry * table, const RowDesc * rows, const int32_t * tok_row,
                const Act & x, int T, int N, float * y, int ldy, int col0, float * mid) {
    lora_apply_targets(s, 1, &table, &N, &col0, rows, tok_row, x, T, y, ldy, mid, 0);
}

__global__ __launch_bounds__(256) void k_rmsnorm_act(float * x, const float * __restrict__ w,
                                                     int E, float eps, const int32_t * __restrict__ rows, Act out,
                                                     Slices add) {
    __shared__ float red[4];
    const int o = blockIdx.x;
    const int row = rows ? rows[o] : o;
    float * xr = x + (size_t)row * E;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < E; i += 256) {
        float v = xr[i];
        if (add.n > 0) {
            if (add.weight) {
                float c = 0.0f;
                for (int k = 0; k < add.n; ++k) {
                    const size_t term = (size_t)row * add.n + k;
                    c = fmaf(add.weight[term], add.data[(add.gather ? (size_t)add.gather[term] : term) * E + i], c);
                }
                v += c;
            } else {
                for (int k = 0; k < add.n; ++k) v += add.data[(size_t)k * add.stride + (size_t)row * E + i];
            }
            xr[i] = v;          // re-read below by the same thread
        }
        ss += v * v;
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float total = (red[0] + red[1]) + (red[2] + red[3]);
    const float scale = 1.0f / sqrtf(total / (float)E + eps);
    const int nblk = (E + 31) / 32;
    for (int b = threadIdx.x; b < nblk; b += 256) {
        const int k0 = b * 32;
        const int count = min(32, E - k0);
        float v[32];
        for (int i = 0; i < count; ++i) v[i] = (xr[k0 + i] * scale) * w[k0 + i];
        store_act_block(v, count, out, o, k0);
    }
}

// E % 32 == 0: 8 elements per lane, 16-byte loads and stores. NW waves per row:
// a row is read by one workgroup, and a workgroup's bandwidth grows with the
// loads it has in flight, so wide rows get more waves.
template <int NW>
__global__ __launch_bounds__(NW * 64) void k_rmsnorm_act8(float * x, const float * __restrict__ w,
                                                          int E, float eps, const int32_t * __restrict__ rows, Act out,
                                                          Slices add) {
    constexpr int STEP = NW * 64 * 8;
    __shared__ float red[NW];
    const int o = blockIdx.x;
    const int row = rows ? rows[o] : o;
    float * xr = x + (size_t)row * E;
    float ss = 0.0f;
    // the first 2 x STEP elements of the row stay in registers between the two passes
    constexpr int KEEP = 2;
    f4 ka[KEEP], kb[KEEP], wa[KEEP], wb[KEEP];
#pragma unroll
    for (int c = 0; c < KEEP; ++c) {
        const int k = threadIdx.x * 8 + c * STEP;
        if (k < E) { wa[c] = *(const f4 *)(w + k); wb[c] = *(const f4 *)(w + k + 4); }   // independent of everything: issued first
    }
    // eight elements of the row: the residual value plus what `add` holds for it; c counts the thread's groups
    auto group = [&](int k, int c) __attribute__((always_inline)) {
        f4 a = *(const f4 *)(xr + k), b = *(const f4 *)(xr + k + 4);
        if (add.n > 0 && add.weight) {
            // the weighted sum of the row's terms, eight terms' loads in flight together
            f4 ca = {0.f, 0.f, 0.f, 0.f}, cb = {0.f, 0.f, 0.f, 0.f};
            const size_t term0 = (size_t)row * add.n;
            const float * gw = add.weight + term0;
            for (int j = 0; j < add.n; j += 8) {
                f4 sa[8], sb[8];
                float wj[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int jj = min(j + u, add.n - 1);
                    const float * src = add.data + (add.gather ? (size_t)add.gather[term0 + jj] : term0 + jj) * E + k;
                    wj[u] = gw[jj];
                    sa[u] = *(const f4 *)src;
                    sb[u] = *(const f4 *)(src + 4);
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    if (j + u >= add.n) break;
#pragma unroll
                    for (int i = 0; i < 4; ++i) { ca[i] = fmaf(wj[u], sa[u][i], ca[i]); cb[i] = fmaf(wj[u], sb[u][i], cb[i]); }
                }
            }
            a += ca;
            b += cb;
            *(f4 *)(xr + k) = a;
            *(f4 *)(xr + k + 4) = b;
        } else if (add.n > 0) {
            const float * sl = add.data + (size_t)row * E + k;
            // eight slices' loads in flight together, added in slice order
            auto add_eight = [&](int j) __attribute__((always_inline)) {
                f4 sa[8], sb[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    sa[u] = *(const f4 *)(sl + (size_t)(j + u) * add.stride);
                    sb[u] = *(const f4 *)(sl + (size_t)(j + u) * add.stride + 4);
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) { a += sa[u]; b += sb[u]; }
            };
            int j = 0;
            // The first eight outside the loop: ahead of a loop that adds to values still on their way the compiler
            // waits for them, and the row itself would have to arrive before its slices are even requested.
            if (add.n >= 8) { add_eight(0); j = 8; }
            for (; j + 8 <= add.n; j += 8) add_eight(j);
            for (; j + 4 <= add.n; j += 4) {          // four
                f4 sa[4], sb[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    sa[u] = *(const f4 *)(sl + (size_t)(j + u) * add.stride);
                    sb[u] = *(const f4 *)(sl + (size_t)(j + u) * add.stride + 4);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) { a += sa[u]; b += sb[u]; }
            }
            for (; j < add.n; ++j) {
                a += *(const f4 *)(sl + (size_t)j * add.stride);
                b += *(const f4 *)(sl + (size_t)j * add.stride + 4);
            }
            *(f4 *)(xr + k) = a;          // read again below (past the kept part) by the same thread
            *(f4 *)(xr + k + 4) = b;
        }
#pragma unroll
        for (int i = 0; i < KEEP; ++i)
            if (i == c) { ka[i] = a; kb[i] = b; }
        ss += a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w + b.x * b.x + b.y * b.y + b.z * b.z + b.w * b.w;
    };
    // A row of one group per thread (the common widths) is not a loop: inside a loop the compiler waits for
    // everything requested so far before the slices' loads go out (a load of the pass before could still be on its
    // way into their registers, for all it knows), and the row would arrive before its slices are even requested.
    if (E <= STEP) {
        if ((int)threadIdx.x * 8 < E) group(threadIdx.x * 8, 0);
    } else {
        int c = 0;
        for (int k = threadIdx.x * 8; k < E; k += STEP, ++c) group(k, c);
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < NW; ++i) total += red[i];
    const float scale = 1.0f / sqrtf(total / (float)E + eps);
#pragma unroll
    for (int i = 0; i < KEEP; ++i) {
        const int k = threadIdx.x * 8 + i * STEP;
        if (k >= E) break;
        const f4 a = ka[i], b = kb[i];
        const float v[8] = {(a.x * scale) * wa[i].x, (a.y * scale) * wa[i].y, (a.z * scale) * wa[i].z, (a.w * scale) * wa[i].w,
                            (b.x * scale) * wb[i].x, (b.y * scale) * wb[i].y, (b.z * scale) * wb[i].z, (b.w * scale) * wb[i].w};
        store_act8(v, out, o, k, threadIdx.x & 3);
    }
    for (int k = threadIdx.x * 8 + KEEP * STEP; k < E; k += STEP) {
        const f4 a = *(const f4 *)(xr + k), b = *(const f4 *)(xr + k + 4);
        const f4 xa = *(const f4 *)(w + k), xb = *(const f4 *)(w + k + 4);
        const float v[8] = {(a.x * scale) * xa.x, (a.y * scale) * xa.y, (a.z * scale) * xa.z, (a.w * scale) * xa.w,
                            (b.x * scale) * xb.x, (b.y * scale) * xb.y, (b.z * scale) * xb.z, (b.w * scale) * xb.w};
        store_act8(v, out, o, k, threadIdx.x & 3);
    }
}

void rmsnorm_act(hipStream_t s, float * x, const float * w, int E, float eps,
                 const int32_t * rows, int n_rows, const Act & out, const Slices & add) {
    if (n_rows <= 0) return;
    if (add.n > 0 && add.N != E) throw std::runtime_error("rmsnorm: the slices do not match the row width");
    check_act_out(out, E, "rmsnorm", n_rows);
    if (E % 32 == 0) {
        // eight waves where four would need two groups of eight elements per thread (a loop: see the kernel)
        if (E > 2048) hipLaunchKernelGGL(k_rmsnorm_act8<8>, dim3(n_rows), dim3(512), 0, s, x, w, E, eps, rows, out, add);
        else hipLaunchKernelGGL(k_rmsnorm_act8<4>, dim3(n_rows), dim3(256), 0, s, x, w, E, eps, rows, out, add);
        check_launch("rmsnorm");
        return;
    }
    Act o = out;
    o.sums = nullptr;
    hipLaunchKernelGGL(k_rmsnorm_act, dim3(n_rows), dim3(256), 0, s, x, w, E, eps, rows, o, add);
    check_launch("rmsnorm");
}

// gate c of a token sits at column (c / group) * 2 group + c % group and up c `group` columns further: group = F
// for the two matrices side by side, 64 for the interleaved matrix of the fused kernel.
__global__ __launch_bounds__(256) void k_swiglu_act(const float * __restrict__ gu, int T, int F, int group, Act out) {
    const int nblk = (F + 31) / 32;
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (size_t)T * nblk) return;
    const int t = (int)(gid / nblk), b = (int)(gid % nblk);
    const int k0 = b * 32;
    const int count = min(32, F - k0);
    const float * g = gu + (size_t)t * 2 * F + (k0 / group) * 2 * group + k0 % group;
    const float * u = g + group;
    float v[32];
    for (int i = 0; i < count; ++i) {
        const float gi = g[i];
        v[i] = (gi / (1.0f + __expf(-gi))) * u[i];
    }
    store_act_block(v, count, out, t, k0);
}

__global__ __launch_bounds__(256) void k_to_act(const float * __restrict__ x, int T, int K, Act out) {
    const int nblk = (K + 31) / 32;
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (size_t)T * nblk) return;
    const int t = (int)(gid / nblk), b = (int)(gid % nblk);
    const int k0 = b * 32;
    const int count = min(32, K - k0);
    float v[32];
    for (int i = 0; i < count; ++i) v[i] = x[(size_t)t * K + k0 + i];
    store_act_block(v, count, out, t, k0);
}

// K % 32 == 0: 8 elements per lane.
__global__ __launch_bounds__(256) void k_to_act8(const float * __restrict__ x, int T, int K, Act out) {
    const int per = K / 8;
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (size_t)T * per) return;      // whole groups of lanes that share a block leave together
    const int t = (int)(gid / per), k = (int)(gid % per) * 8;
    const f4 a = *(const f4 *)(x + (size_t)t * K + k), b = *(const f4 *)(x + (size_t)t * K + k + 4);
    const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    store_act8(v, out, t, k, threadIdx.x & 3);
}

void to_act(hipStream_t s, const float * x, int T, int K, const Act & out) {
    if (T <= 0) return;
    check_act_out(out, K, "to_act", T);
    if (K % 32 == 0) {
        const size_t n = (size_t)T * (K / 8);
        hipLaunchKernelGGL(k_to_act8, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, x, T, K, out);
        check_launch("to_act");
        return;
    }
    Act o = out;
    o.sums = nullptr;
    const size_t n = (size_t)T * ((K + 31) / 32);
    hipLaunchKernelGGL(k_to_act, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, x, T, K, o);
    check_launch("to_act");
}

// The rows in `src` (hi/lo planes) converted into out.qx; the two may be the same buffer.
__global__ __launch_bounds__(256) void k_requant_act8(const __half * src, int T, int K, Act out) {
    const int per = K / 8;
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (size_t)T * per) return;      // whole groups of lanes that share a block leave together
    const int t = (int)(gid / per), k = (int)(gid % per) * 8;
    const h8 hi = load_h8(src + act_at(t, k, 0, K)), lo = load_h8(src + act_at(t, k, 1, K));
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (float)hi[i] + (float)lo[i];
    store_act8(v, out, t, k, threadIdx.x & 3);
}

void requant_act(hipStream_t s, const __half * src, int T, const Act & out) {
    if (T <= 0) return;
    check_act_out(out, out.K, "requant_act", T);
    if (out.x || !out.qx) throw std::runtime_error("requant_act: writes the converted rows only");
    const size_t n = (size_t)T * (out.K / 8);
    hipLaunchKernelGGL(k_requant_act8, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, src, T, out.K, out);
    check_launch("requant_act");
}

// F % 32 == 0: 8 elements per lane.
__global__ __launch_bounds__(256) void k_swiglu_act8(const float * __restrict__ gu, int T, int F, int group, Act out) {
    const int per = F / 8;
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (size_t)T * per) return;      // whole groups of four lanes leave together (per % 4 == 0)
    const int t = (int)(gid / per), k = (int)(gid % per) * 8;
    const float * g = gu + (size_t)t * 2 * F + (k / group) * 2 * group + k % group;
    const float * u = g + group;
    const f4 ga = *(const f4 *)g, gb = *(const f4 *)(g + 4), ua = *(const f4 *)u, ub = *(const f4 *)(u + 4);
    const float gv[8] = {ga.x, ga.y, ga.z, ga.w, gb.x, gb.y, gb.z, gb.w};
    const float uv[8] = {ua.x, ua.y, ua.z, ua.w, ub.x, ub.y, ub.z, ub.w};
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (gv[i] / (1.0f + __expf(-gv[i]))) * uv[i];
    store_act8(v, out, t, k, threadIdx.x & 3);
}

// The same from a gate/up product left as K-slices (rows of sl.N columns in groups of 128: 64 gate, then the 64 up
// columns of the same hidden columns): the slices are added in slice order, and hidden column c of the product is
// column col0 + c of `out`. Eight columns per lane, the four lanes of a 32-wide block together.
__global__ __launch_bounds__(256) void k_swiglu_slices(Slices sl, int T, int col0, Act out) {
    const int per = sl.N / 16;
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (size_t)T * per) return;      // whole groups of four lanes leave together (per % 4 == 0)
    const int t = (int)(gid / per), c = (int)(gid % per) * 8;
    const float * g = sl.data + (size_t)t * sl.N + (c / 64) * 128 + c % 64;
    f4 ga = {0.f, 0.f, 0.f, 0.f}, gb = ga, ua = ga, ub = ga;
    for (int i = 0; i < sl.n; ++i, g += sl.stride) {
        ga += *(const f4 *)g; gb += *(const f4 *)(g + 4);
        ua += *(const f4 *)(g + 64); ub += *(const f4 *)(g + 68);
    }
    const float gv[8] = {ga.x, ga.y, ga.z, ga.w, gb.x, gb.y, gb.z, gb.w};
    const float uv[8] = {ua.x, ua.y, ua.z, ua.w, ub.x, ub.y, ub.z, ub.w};
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (gv[i] / (1.0f + __expf(-gv[i]))) * uv[i];
    store_act8(v, out, t, col0 + c, threadIdx.x & 3);
}

void swiglu_slices(hipStream_t s, const Slices & sl, int T, const Act & out, int col0) {
    if (T <= 0) return;
    if (!sl.data || sl.n < 1 || sl.weight || sl.N % 128 != 0 || col0 % 32 != 0 || col0 + sl.N / 2 > out.K || (!out.x && !out.qx)
        || (out.qx && out.quant == AQ_Q8_K))
        throw std::runtime_error("swiglu_slices: needs plain K-slices of whole groups of 128 columns inside the output row (and no 256-wide conversion)");
    const size_t n = (size_t)T * (sl.N / 16);
    hipLaunchKernelGGL(k_swiglu_slices, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, sl, T, col0, out);
    check_launch("swiglu_slices");
}

void swiglu_act(hipStream_t s, const float * gu, int T, int F, const Act & out, int group) {
    if (T <= 0) return;
    check_act_out(out, F, "swiglu", T);
    if (group <= 0) group = F;
    // a block of 32 (8) gate columns must not straddle two groups
    if (group != F && (F % group != 0 || group % 32 != 0)) throw std::runtime_error("swiglu: the interleave group must divide F and be a multiple of 32");
    if (F % 32 == 0) {
        const size_t n = (size_t)T * (F / 8);
        hipLaunchKernelGGL(k_swiglu_act8, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, gu, T, F, group, out);
        check_launch("swiglu");
        return;
    }
    Act o = out;
    o.sums = nullptr;
    const size_t n = (size_t)T * ((F + 31) / 32);
    hipLaunchKernelGGL(k_swiglu_act, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, gu, T, F, group, o);
    check_launch("swiglu");
}

// ---------------------------------------------------------------------------
// step packing

__device__ __forceinline__ int tile_splits(int kv_begin, int kv_hi, int split_pages) {
    const int p_first = kv_begin / PAGE;
    const int p_last = (kv_hi - 1) / PAGE;
    return (p_last - p_first + 1 + split_pages - 1) / split_pages;
}

// Inclusive scan of one int per thread over a 1024-thread block.
__device__ int block_scan_incl(int v, int * scratch) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int o = 1; o < 64; o <<= 1) {
        const int n = __shfl_up(v, o, 64);
        if (lane >= o) v += n;
    }
    if (lane == 63) scratch[wave] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int i = 0; i < 16; ++i) { const int c = scratch[i]; scratch[i] = run; run += c; }
    }
    __syncthreads();
    v += scratch[wave];
    __syncthreads();
    return v;
}

__global__ __launch_bounds__(1024) void k_pack(const RowDesc * __restrict__ rows, int n_rows,
                                               const int32_t * __restrict__ toks,
                                               const TableUpdate * __restrict__ upd, int n_upd,
                                               int32_t * __restrict__ table, int max_pages,
                                               int qt, int n_kv, const double * __restrict__ inv_freq, int pairs,
                                               PackBuffers o) {
    __shared__ int scratch[16];
    __shared__ int carry[3];
    __shared__ int len_count[MAX_SPLIT_PAGES + 1], len_base[MAX_SPLIT_PAGES + 1];
    __shared__ int row_len[1024];
    for (int i = threadIdx.x; i < n_upd; i += 1024) table[(size_t)upd[i].slot * max_pages + upd[i].index] = upd[i].page;
    if (threadIdx.x == 0) { carry[0] = 0; carry[1] = 0; carry[2] = 0; }
    __syncthreads();

    // rows in chunks of 1024: per-row tile / item / output counts -> bases
    for (int base = 0; base < n_rows; base += 1024) {
        const int r = base + threadIdx.x;
        int tiles = 0, items = 0, outs = 0;
        RowDesc d;
        if (r < n_rows) {
            d = rows[r];
            tiles = (d.n + qt - 1) / qt;
            for (int j = 0; j < tiles; ++j) {
                const int hi = d.pos0 + min(d.n, (j + 1) * qt);
                items += n_kv * tile_splits(d.kv_begin, hi, o.split_pages);
            }
            outs = d.sample ? 1 : 0;
        }
        const int tile_end = block_scan_incl(tiles, scratch);
        const int item_end = block_scan_incl(items, scratch);
        const int out_end = block_scan_incl(outs, scratch);
        if (r < n_rows) {
            int tile_at = carry[0] + tile_end - tiles;
            int item_at = carry[1] + item_end - items;
            const int out_at = carry[2] + out_end - outs;
            o.row_offset[r] = d.tok_off;
            o.last_index[r] = d.tok_off + d.n - 1;
            if (d.sample) o.out_tok[out_at] = d.tok_off + d.n - 1;
            for (int j = 0; j < tiles; ++j) {
                const int q0 = j * qt;
                const int nq = min(qt, d.n - q0);
                const int hi = d.pos0 + q0 + nq;
                const int ns = tile_splits(d.kv_begin, hi, o.split_pages);
                o.tile_t0[tile_at] = d.tok_off + q0;
                o.tile_nq[tile_at] = nq;
                o.tile_item0[tile_at] = item_at;
                o.tile_nsplit[tile_at] = ns;
                o.tile_page0[tile_at] = d.kv_begin / PAGE;
                o.tile_kv_begin[tile_at] = d.kv_begin;
                for (int i = 0; i < nq; ++i) {
                    o.tok_tile[d.tok_off + q0 + i] = tile_at;
                    o.tok_merge[d.tok_off + q0 + i] = make_int4(item_at, ns, i, 0);
                }
                item_at += n_kv * ns;
                ++tile_at;
            }
            for (int i = 0; i < d.n; ++i) {
                const int t = d.tok_off + i;
                const int p = d.pos0 + i;
                o.tok[t] = toks[t];
                o.pos[t] = p;
                o.seq[t] = d.slot;
                o.row[t] = r;
                o.cell[t] = table[(size_t)d.slot * max_pages + p / PAGE] * PAGE + p % PAGE;
                o.out_index[t] = (d.sample && i + 1 == d.n) ? out_at : -1;
            }
        }
        __syncthreads();
        // rows past n_rows contribute zero, so the last thread's inclusive
        // sums are the chunk totals
        if (threadIdx.x == 1023) {
            carry[0] += tile_end;
            carry[1] += item_end;
            carry[2] += out_end;
        }
        __syncthreads();
    }
    // the work items of every (tile, kv head), from the tile and token arrays written above
    __threadfence_block();
    __syncthreads();
    // The descriptors are stored longest first (by pages): workgroups start in index order, so the items that start
    // last - the tail of the launch, when few waves are left to hide each other's latency - are the short ones. An
    // item keeps its number (a tile's items of a kv head are consecutive numbers, which the merge relies on) inside
    // its descriptor; only the place of the descriptor changes. Two passes: count the items of every length, then
    // place them (the order among items of one length is whatever the atomics give: it changes no result).
    for (int i = threadIdx.x; i <= MAX_SPLIT_PAGES; i += 1024) len_count[i] = 0;
    __syncthreads();
    for (int pass = 0; pass < 2; ++pass) {
        for (int pair = threadIdx.x; pair < carry[0] * n_kv; pair += 1024) {
            const int tile = pair / n_kv, h = pair % n_kv;
            const int t0 = o.tile_t0[tile], nq = o.tile_nq[tile], ns = o.tile_nsplit[tile];
            const int kv_begin = o.tile_kv_begin[tile], pos0 = o.pos[t0], slot = o.seq[t0];
            const int item0 = o.tile_item0[tile] + h * ns;
            const int hi = pos0 + nq;
            for (int sp = 0; sp < ns; ++sp) {
                const int page_first = kv_begin / PAGE + sp * o.split_pages;
                const int page_end = min((hi - 1) / PAGE + 1, page_first + o.split_pages);
                const int len = min(max(page_end - page_first, 0), MAX_SPLIT_PAGES);
                if (pass == 0) {
                    atomicAdd(&len_count[len], 1);
                } else {
                    const int at = atomicAdd(&len_base[len], 1);
                    o.item_a[at] = make_int4(t0, nq | (h << 8), item0 + sp, slot);
                    o.item_b[at] = make_int4(pos0, kv_begin, page_first, page_end - page_first);
                }
            }
        }
        __syncthreads();
        if (pass == 0 && threadIdx.x == 0) {
            int at = 0;
            for (int len = MAX_SPLIT_PAGES; len >= 0; --len) { len_base[len] = at; at += len_count[len]; }
        }
        __syncthreads();
    }
    // the rows by resident length, longest first (ties in row order): the decode-step attention starts one
    // workgroup per row and kv head in this order, so that the launch's tail is made of short sequences
    // Beside the order, per row in that order: what a workgroup of that launch needs to start (token index, position,
    // first resident position, slot) and, with the row's pages dealt evenly to eight waves, the id of each wave's
    // first page - so that the workgroup's first loads depend on one lookup, not on a chain of three.
    auto describe = [&](int rank, const RowDesc & d) {
        o.dec_order[rank] = d.tok_off;
        const int pos = d.pos0 + d.n - 1;
        o.dec_desc[rank] = make_int4(d.tok_off + d.n - 1, pos, d.kv_begin, d.slot);
        const int page_first = d.kv_begin / PAGE, n_pages = pos / PAGE - page_first + 1;
        const int per_wave = (n_pages + 7) / 8;
        for (int w = 0; w < 8; ++w)
            o.dec_pid[rank * 8 + w] = w * per_wave < n_pages ? table[(size_t)d.slot * max_pages + page_first + w * per_wave] : 0;
    };
    if (n_rows <= 1024) {
        if ((int)threadIdx.x < n_rows) { const RowDesc d = rows[threadIdx.x]; row_len[threadIdx.x] = d.pos0 + d.n - d.kv_begin; }
        __syncthreads();
        if ((int)threadIdx.x < n_rows) {
            const int mine = row_len[threadIdx.x];
            int rank = 0;
            for (int j = 0; j < n_rows; ++j) rank += (row_len[j] > mine || (row_len[j] == mine && j < (int)threadIdx.x)) ? 1 : 0;
            describe(rank, rows[threadIdx.x]);
        }
    } else {
        for (int r = threadIdx.x; r < n_rows; r += 1024) describe(r, rows[r]);
    }
    if (threadIdx.x == 0) {
        const RowDesc last = rows[n_rows - 1];
        o.row_offset[n_rows] = last.tok_off + last.n;
        o.counts[0] = last.tok_off + last.n;
        o.counts[1] = carry[2];
        o.counts[2] = carry[0];
        o.counts[3] = carry[1];
    }
    // rotary table of the step: angle = pos * inv_freq[j] in double; inv_freq[pairs] is the magnitude factor of the
    // rotation (1 unless the model's frequency scaling rule asks for another)
    const double magnitude = inv_freq[pairs];
    const RowDesc lastd = rows[n_rows - 1];
    const int T = lastd.tok_off + lastd.n;
    for (int i = threadIdx.x; i < T * pairs; i += 1024) {
        const int t = i / pairs, j = i % pairs;
        // position of token t: recompute from its row (binary search over tok_off)
        int lo = 0, hi = n_rows - 1;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (rows[mid].tok_off <= t) lo = mid; else hi = mid - 1;
        }
        const double ang = (double)(rows[lo].pos0 + (t - rows[lo].tok_off)) * inv_freq[j];
        double sv, cv;
        sincos(ang, &sv, &cv);
        o.rope_cos[i] = (float)(cv * magnitude);
        o.rope_sin[i] = (float)(sv * magnitude);
    }
}

void pack_step(hipStream_t s, const RowDesc * rows, int n_rows, const int32_t * tokens_concat,
               const TableUpdate * updates, int n_updates, int32_t * table, int max_pages,
               int qt, int n_kv_heads, const double * inv_freq, int rope_pairs, const PackBuffers & out) {
    if (n_rows <= 0) return;
    hipLaunchKernelGGL(k_pack, dim3(1), dim3(1024), 0, s, rows, n_rows, tokens_concat, updates, n_updates,
                       table, max_pages, qt, n_kv_heads, inv_freq, rope_pairs, out);
    check_launch("pack_step");
}

// Counts the step's query tiles and, for the split it chooses, its attention
// work items. A work item is one wave; the attention kernel's time hardly
// depends on the split as long as the waves fill the chip, while every split
// costs the merge kernel a partial result to read, so the largest split that
// still leaves about a wave per SIMD slot wins, and small steps get the
// smallest one.
void count_attention_work(const RowDesc * rows, int n_rows, int qt, int n_kv_heads, int * n_tiles, int * n_items,
                          int * split_pages) {
    constexpr int kEnoughItems = 1536;
    int tiles = 0, items = 0, split = MAX_SPLIT_PAGES;
    for (;; split /= 2) {
        tiles = 0; items = 0;
        for (int r = 0; r < n_rows; ++r) {
            const RowDesc & d = rows[r];
            const int nt = (d.n + qt - 1) / qt;
            for (int j = 0; j < nt; ++j) {
                const int hi = d.pos0 + std::min(d.n, (j + 1) * qt);
                const int p_first = d.kv_begin / PAGE, p_last = (hi - 1) / PAGE;
                items += n_kv_heads * ((p_last - p_first + 1 + split - 1) / split);
            }
            tiles += nt;
        }
        if (items >= kEnoughItems || split <= 4) break;
    }
    *n_tiles = tiles;
    *n_items = items;
    *split_pages = split;
}

// ---------------------------------------------------------------------------
// RoPE + KV store

__device__ __forceinline__ size_t k_page_offset(int head_dim, int t32, int e) {
    // [dims/32][token half][g][token][8]
    const int j = e >> 5, g = (e >> 3) & 3, i = e & 7;
    const int tg = t32 >> 4, t = t32 & 15;
    (void)head_dim;
    return (size_t)((((j * 2 + tg) * 4 + g) * 16 + t) * 8 + i);
}

__device__ __forceinline__ size_t v_page_offset(int head_dim, int t32, int e) {
    // [dims/16][g][dim][8]; slot (g, i) = token 4g+i (i<4) or 16+4g+(i-4)
    const int dt = e >> 4, d = e & 15;
    const int tt = t32 & 15;
    const int g = tt >> 2;
    const int i = (tt & 3) + ((t32 >> 4) << 2);
    (void)head_dim;
    return (size_t)(((dt * 4 + g) * 16 + d) * 8 + i);
}

struct RopeArgs {
    const float * qkv;
    const float * q_norm;
    const float * k_norm;
    __half * q_out;
    __half * q_out_lo;
    __half * k_pool;
    __half * v_pool;
    const int32_t * cell;
    const float * rope_cos;
    const float * rope_sin;
    int n_head, n_kv, hd, rope_dim, neox;
    float eps, qscale;
    Slices from;
    size_t page_stride, head_stride;
    int kv_quant;    // KV_F16, KV_Q8 or KV_Q4
    int q_q8;        // the ggml arithmetic over a quantised cache: the query row is converted to Q8_0 as well
};

// One wave per head: lanes own element pairs.
__global__ __launch_bounds__(256) void k_rope_store(RopeArgs a) {
    __shared__ float stash[4][128];          // Q8_0 cache: a head's row in element order, per wave
    const int t = blockIdx.x;
    const int head = blockIdx.y * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int heads_total = a.n_head + 2 * a.n_kv;
    if (head >= heads_total) return;
    const int QD = a.n_head * a.hd, KD = a.n_kv * a.hd;
    const int pairs = a.hd / 2;
    const int rp = a.rope_dim / 2;
    const size_t src_at = (size_t)t * (QD + 2 * KD) + (size_t)head * a.hd;
    const bool is_q = head < a.n_head;
    const bool is_k = !is_q && head < a.n_head + a.n_kv;
    const bool active = lane < pairs;
    // element pair of this lane
    int i0, i1;
    if (is_q || is_k) {
        if (lane < rp) {
            i0 = a.neox ? lane : 2 * lane;
            i1 = a.neox ? lane + rp : 2 * lane + 1;
        } else {          // dims past the rotary width pass through
            i0 = a.rope_dim + 2 * (lane - rp);
            i1 = i0 + 1;
        }
    } else {
        i0 = 2 * lane;
        i1 = i0 + 1;
    }
    float x0 = 0.0f, x1 = 0.0f;
    if (active) {
        if (a.from.n > 0) {
            for (int k = 0; k < a.from.n; ++k) {
                const float * sl = a.from.data + (size_t)k * a.from.stride + src_at;
                x0 += sl[i0];
                x1 += sl[i1];
            }
        } else {
            x0 = a.qkv[src_at + i0];
            x1 = a.qkv[src_at + i1];
        }
    }
    const float * nw = is_q ? a.q_norm : (is_k ? a.k_norm : nullptr);
    if (nw) {
        const float ss = wave_sum(x0 * x0 + x1 * x1);
        const float scale = 1.0f / sqrtf(ss / (float)a.hd + a.eps);
        if (active) {
            x0 = (x0 * scale) * nw[i0];
            x1 = (x1 * scale) * nw[i1];
        }
    }
    if (!active) return;
    if ((is_q || is_k) && lane < rp) {
        const float c = a.rope_cos[(size_t)t * rp + lane];
        const float s = a.rope_sin[(size_t)t * rp + lane];
        const float r0 = x0 * c - x1 * s;
        const float r1 = x0 * s + x1 * c;
        x0 = r0;
        x1 = r1;
    }
    // Q8_0 blocks want neighbours where lanes hold rotation pairs: through LDS, then lane L owns elements 2 L and
    // 2 L + 1 and sixteen lanes a block of 32. d = amax / 127, code = roundf(x / d) with the unrounded d (ggml's
    // quantize_row_q8_0_ref); returns the codes, d through `d`.
    auto q8_pair = [&](float & v0, float & v1, float & d) {
        float * mine = stash[threadIdx.x >> 6];
        mine[i0] = x0;
        mine[i1] = x1;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        v0 = mine[2 * lane];
        v1 = mine[2 * lane + 1];
        float amax = fmaxf(fabsf(v0), fabsf(v1));
#pragma unroll
        for (int o = 1; o < 16; o <<= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
        d = __fdiv_rn(amax, 127.0f);
        const float id = d != 0.0f ? __fdiv_rn(1.0f, d) : 0.0f;
        v0 = roundf(__fmul_rn(v0, id));
        v1 = roundf(__fmul_rn(v1, id));
    };
    if (is_q) {
        const size_t at = (size_t)t * QD + (size_t)head * a.hd;
        if (a.q_q8) {
            // the query row as Q8_0, the companion format of a Q8_0 K row in ggml's CPU attention: scale times code
            float c0, c1, d;
            q8_pair(c0, c1, d);
            const float dh = __half2float(__float2half_rn(d));
            x0 = __fmul_rn(dh, c0);
            x1 = __fmul_rn(dh, c1);
            i0 = 2 * lane;
            i1 = i0 + 1;
        }
        const float s0 = fminf(fmaxf(x0 * a.qscale, -65504.0f), 65504.0f);
        const float s1 = fminf(fmaxf(x1 * a.qscale, -65504.0f), 65504.0f);
        const __half h0 = __float2half_rn(s0), h1 = __float2half_rn(s1);
        a.q_out[at + i0] = h0;
        a.q_out[at + i1] = h1;
        a.q_out_lo[at + i0] = __float2half_rn(s0 - __half2float(h0));
        a.q_out_lo[at + i1] = __float2half_rn(s1 - __half2float(h1));
        return;
    }
    const int cell = a.cell[t];
    const int page = cell / PAGE, t32 = cell % PAGE;
    const int kvh = is_k ? head - a.n_head : head - a.n_head - a.n_kv;
    if (a.kv_quant == KV_Q8) {
        float c0, c1, d;
        q8_pair(c0, c1, d);
        const int e = 2 * lane;
        const uint32_t b0 = (uint32_t)((int)c0 + 128), b1 = (uint32_t)((int)c1 + 128);
        uint8_t * blk = (uint8_t *)((is_k ? a.k_pool : a.v_pool) + (size_t)page * a.page_stride + (size_t)kvh * a.head_stride);
        const int tg = (t32 & 15) >> 2, ti = (t32 & 3) + 4 * (t32 >> 4);      // the token's place among a lane's eight
        const int blk_idx = e >> 5;
        if (is_k) {
            const int g = (e >> 3) & 3, i = e & 7;
            *(uint16_t *)(blk + blk_idx * 1024 + (g * 16 + (t32 & 15)) * 16 + (t32 >> 4) * 8 + i) = (uint16_t)(b0 | (b1 << 8));
        } else {
            const int hi = (e >> 4) & 1, dd = e & 15;
            blk[blk_idx * 1024 + (tg * 16 + dd) * 16 + hi * 8 + ti] = (uint8_t)b0;
            blk[blk_idx * 1024 + (tg * 16 + dd + 1) * 16 + hi * 8 + ti] = (uint8_t)b1;
        }
        if ((lane & 15) == 0) ((__half *)(blk + (a.hd / 32) * 1024))[blk_idx * 32 + tg * 8 + ti] = __float2half_rn(d);
        return;
    }
    if (a.kv_quant == KV_Q4) {
        // ggml's quantize_row_q4_0_ref: d = m / -8 for the element m of largest magnitude (the first of equals),
        // code = min(15, (int)(x / d + 8.5)) with the unrounded d. Lane L owns elements 2 L and 2 L + 1 after the
        // exchange through LDS, sixteen lanes a block.
        float * mine = stash[threadIdx.x >> 6];
        mine[i0] = x0;
        mine[i1] = x1;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        const float v0 = mine[2 * lane], v1 = mine[2 * lane + 1];
        float amax = fabsf(v0), mval = v0;
        int midx = 2 * lane;
        if (fabsf(v1) > amax) { amax = fabsf(v1); mval = v1; midx = 2 * lane + 1; }
#pragma unroll
        for (int o = 1; o < 16; o <<= 1) {
            const float oa = __shfl_xor(amax, o, 64), ov = __shfl_xor(mval, o, 64);
            const int oi = __shfl_xor(midx, o, 64);
            if (oa > amax || (oa == amax && oi < midx)) { amax = oa; mval = ov; midx = oi; }
        }
        const float d = __fdiv_rn(mval, -8.0f);
        const float id = d != 0.0f ? __fdiv_rn(1.0f, d) : 0.0f;
        const uint32_t q0 = (uint32_t)min(15, (int)(int8_t)__fadd_rn(__fmul_rn(v0, id), 8.5f));
        const uint32_t q1 = (uint32_t)min(15, (int)(int8_t)__fadd_rn(__fmul_rn(v1, id), 8.5f));
        const int e = 2 * lane;
        uint8_t * blk = (uint8_t *)((is_k ? a.k_pool : a.v_pool) + (size_t)page * a.page_stride + (size_t)kvh * a.head_stride);
        const int tg = (t32 & 15) >> 2, ti = (t32 & 3) + 4 * (t32 >> 4);      // the token's place among a lane's eight
        const int blk_idx = e >> 5;
        if (is_k) {
            // four lanes hold the eight codes of one 32-bit word (this token's dims 8 g .. 8 g + 7): joined, then one store
            const int g = (e >> 3) & 3, i = e & 7;
            uint32_t word = (q0 << (4 * kv_nibble(i))) | (q1 << (4 * kv_nibble(i + 1)));
            word |= __shfl_xor(word, 1, 64);
            word |= __shfl_xor(word, 2, 64);
            if ((lane & 3) == 0)
                *(uint32_t *)(blk + blk_idx * 512 + (g * 16 + (t32 & 15)) * 8 + (t32 >> 4) * 4) = word;
        } else {
            // a word of V holds one dimension of eight tokens: this token's nibble is replaced atomically, other
            // tokens of the step may be writing theirs into the same word
            const int hi = (e >> 4) & 1, dd = e & 15;
            const int sh = 4 * kv_nibble(ti);
            uint32_t * w0 = (uint32_t *)(blk + blk_idx * 512 + (tg * 16 + dd) * 8 + hi * 4);
            uint32_t * w1 = (uint32_t *)(blk + blk_idx * 512 + (tg * 16 + dd + 1) * 8 + hi * 4);
            atomicAnd(w0, ~(0xfu << sh));
            atomicOr(w0, q0 << sh);
            atomicAnd(w1, ~(0xfu << sh));
            atomicOr(w1, q1 << sh);
        }
        if ((lane & 15) == 0) ((__half *)(blk + (a.hd / 32) * 512))[blk_idx * 32 + tg * 8 + ti] = __float2half_rn(d);
        return;
    }
    if (is_k) {
        __half * dst = a.k_pool + (size_t)page * a.page_stride + (size_t)kvh * a.head_stride;
        dst[k_page_offset(a.hd, t32, i0)] = sat_half(x0);
        dst[k_page_offset(a.hd, t32, i1)] = sat_half(x1);
    } else {
        __half * dst = a.v_pool + (size_t)page * a.page_stride + (size_t)kvh * a.head_stride;
        dst[v_page_offset(a.hd, t32, i0)] = sat_half(x0);
        dst[v_page_offset(a.hd, t32, i1)] = sat_half(x1);
    }
}

void rope_store(hipStream_t s, const float * qkv, int T, const AttnShape & sh, const PackBuffers & pk,
                const float * q_norm, const float * k_norm, __half * q_out, __half * q_out_lo,
                __half * k_pool, __half * v_pool, const Slices & from) {
    if (T <= 0) return;
    if (sh.head_dim > 128 || sh.head_dim % 32 != 0) throw std::runtime_error("rope_store: head_dim must be 32, 64, 96 or 128");
    RopeArgs a;
    a.qkv = qkv; a.q_norm = q_norm; a.k_norm = k_norm; a.q_out = q_out; a.q_out_lo = q_out_lo;
    a.k_pool = k_pool; a.v_pool = v_pool;
    a.cell = pk.cell; a.rope_cos = pk.rope_cos; a.rope_sin = pk.rope_sin;
    a.n_head = sh.n_head; a.n_kv = sh.n_head_kv; a.hd = sh.head_dim; a.rope_dim = sh.rope_dim; a.neox = sh.rope_neox ? 1 : 0;
    a.eps = sh.eps;
    a.qscale = 1.4426950408889634f / sqrtf((float)sh.head_dim);
    a.from = from;
    a.page_stride = sh.page_stride; a.head_stride = sh.head_stride;
    a.kv_quant = sh.kv_quant;
    a.q_q8 = sh.kv_quant != KV_F16 && sh.q_q8 ? 1 : 0;
    if (sh.kv_quant != KV_F16 && sh.kv_quant != KV_Q8 && sh.kv_quant != KV_Q4) throw std::runtime_error("rope_store: unknown cache type");
    if (sh.page_stride == 0 || sh.head_stride == 0) throw std::runtime_error("rope_store: the pool's strides are missing");
    if (from.n > 0 && from.N != (sh.n_head + 2 * sh.n_head_kv) * sh.head_dim)
        throw std::runtime_error("rope_store: the slices are not a fused q, k, v product");
    const int heads = sh.n_head + 2 * sh.n_head_kv;
    hipLaunchKernelGGL(k_rope_store, dim3(T, (heads + 3) / 4), dim3(256), 0, s, a);
    check_launch("rope_store");
}

// ---------------------------------------------------------------------------
// paged attention

// The K (V) blocks a wave holds for one page: f16 operands, or - a Q8_0 / Q4_0 cache - codes and block scales.
typedef uint32_t kv_u2 __attribute__((ext_vector_type(2)));
template <int N, int KVQ> struct KvRegs { h8 r[N]; };
template <int N> struct KvRegs<N, KV_Q8> { u4 raw[N / 2]; u4 sc[N / 2]; };
template <int N> struct KvRegs<N, KV_Q4> { kv_u2 raw[N / 2]; u4 sc[N / 2]; };
// Eight bytes (code + 128) as eight f16 codes: 0x6400 | byte is 1024 + byte, exactly.
__device__ __forceinline__ h8 codes8(uint32_t w0, uint32_t w1) {
    const h2 bias = {(_Float16)(-1152.0f), (_Float16)(-1152.0f)};
    const h2 a0 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w0, 0x04010400u)) + bias;
    const h2 a1 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w0, 0x04030402u)) + bias;
    const h2 a2 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w1, 0x04010400u)) + bias;
    const h2 a3 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w1, 0x04030402u)) + bias;
    return (h8){a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
}

// Eight four-bit codes q of a word as eight f16 values q - 8, in the order kv_nibble stores them: a mask leaves
// nibbles 0 and 4 of the (shifted) word in the low bits of two halves whose other bits are those of 1024.
__device__ __forceinline__ h8 codes4(uint32_t w) {
    const h2 bias = {(_Float16)(-1032.0f), (_Float16)(-1032.0f)};
    const h2 a0 = __builtin_bit_cast(h2, (w & 0x000f000fu) | 0x64006400u) + bias;
    const h2 a1 = __builtin_bit_cast(h2, ((w >> 4) & 0x000f000fu) | 0x64006400u) + bias;
    const h2 a2 = __builtin_bit_cast(h2, ((w >> 8) & 0x000f000fu) | 0x64006400u) + bias;
    const h2 a3 = __builtin_bit_cast(h2, ((w >> 12) & 0x000f000fu) | 0x64006400u) + bias;
    return (h8){a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
}

struct AttnArgs {
    const __half * q;
    const __half * q_lo;
    const __half * k_pool;
    const __half * v_pool;
    const int32_t * table;
    const int4 * item_a;
    const int4 * item_b;
    float * partial;
    int n_tiles, n_items, max_pages;
    int n_head, n_kv, G;
    int split_pages;
    size_t page_stride, head_stride;
};

// ONE: every tile holds a single query token (a pure decode step).
// SPLIT (at most 8 query heads per kv head): a tile holds at most 8 / G tokens. Column c < 8 carries the hi
// half of the query of (token c / G, head c % G) and column 8 + c its lo half, so that one matrix instruction
// multiplies both; the two score halves are added across the two lanes before the softmax, column 8 + c
// multiplies the lo halves of the same probabilities, and the two output halves are added at the end. The
// arithmetic of a column does not depend on ONE or on what else is in its tile, so a token's result is the
// same bits in a decode step and in a mixed step. Without SPLIT a tile holds 16 / G tokens and the lo halves
// take a second instruction each.
// KVQ = KV_Q8 / KV_Q4: the pools hold Q8_0 / Q4_0 blocks (kernels.hpp). K enters the score products as its codes,
// one 32-wide k-step being one block, and the block's scale multiplies that step's products; V enters as its codes
// and its scales join the probabilities, one version of the probability operand per 32-wide block of dimensions.
template <int HD, bool ONE, bool SPLIT, int KVQ = KV_F16>
__global__ __launch_bounds__(64, 2) void k_attention(AttnArgs a) {
    constexpr bool Q8 = KVQ != KV_F16;       // a quantised cache of either width
    constexpr int KS = HD / 32;     // k-steps of QK^T
    constexpr int DT = HD / 16;     // dim tiles of PV
    const int lane = threadIdx.x;
    const int c = lane & 15, g = lane >> 4;
    // what the packing kernel left for the workgroup's place (the longest items come first): one round trip instead
    // of a search over the tiles; the item's own number, which places its partial results, is part of it
    const int4 ia = a.item_a[blockIdx.x], ib = a.item_b[blockIdx.x];
    const int item = ia.z;
    const int t0 = ia.x, nq = ONE ? 1 : (ia.y & 0xff), h = ia.y >> 8, slot = ia.w;
    const int kv_begin = ib.y;
    const int cc = SPLIT ? (c & 7) : c;            // the column's (token, head) index
    const int qi = cc / a.G, gi = cc % a.G;
    const bool col_ok = qi < nq;
    const bool lo_col = SPLIT && c >= 8;
    const int tq = t0 + (col_ok ? qi : 0);
    const int limit = ib.x + (col_ok ? qi : 0);         // this column attends positions <= its own (tokens of a row are consecutive)
    const int page_first = ib.z;
    const int page_end = page_first + ib.w;

    const int QD = a.n_head * HD;
    h8 qreg[KS], qreg_lo[KS];
#pragma unroll
    for (int j = 0; j < KS; ++j) {
        if (col_ok) {
            const size_t at = (size_t)tq * QD + (size_t)(h * a.G + gi) * HD + 32 * j + 8 * g;
            qreg[j] = load_h8((lo_col ? a.q_lo : a.q) + at);
            qreg_lo[j] = SPLIT ? qreg[j] : load_h8(a.q_lo + at);
        } else {
            qreg[j] = (h8){0, 0, 0, 0, 0, 0, 0, 0};
            qreg_lo[j] = (h8){0, 0, 0, 0, 0, 0, 0, 0};
        }
    }
    f4 o[DT];
#pragma unroll
    for (int d = 0; d < DT; ++d) o[d] = (f4){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.0f;

    // page ids of this split, one per lane
    const int n_pages = page_end - page_first;
    const int my_pid = lane < n_pages ? a.table[(size_t)slot * a.max_pages + page_first + lane] : 0;
    typedef KvRegs<2 * KS, KVQ> KSet;          // f16: [k-step][token half]
    typedef KvRegs<DT, KVQ> VSet;
    auto load_k = [&](int idx, KSet & ks) {
        const int pid = __builtin_amdgcn_readlane(my_pid, idx);
        const __half * kp = a.k_pool + (size_t)pid * a.page_stride + (size_t)h * a.head_stride;
        if constexpr (KVQ == KV_Q8) {
            const uint8_t * kb = (const uint8_t *)kp;
#pragma unroll
            for (int j = 0; j < KS; ++j) {
                ks.raw[j] = *(const u4 *)(kb + j * 1024 + lane * 16);
                ks.sc[j] = *(const u4 *)(kb + KS * 1024 + (j * 4 + g) * 16);
            }
        } else if constexpr (KVQ == KV_Q4) {
            const uint8_t * kb = (const uint8_t *)kp;
#pragma unroll
            for (int j = 0; j < KS; ++j) {
                ks.raw[j] = *(const kv_u2 *)(kb + j * 512 + lane * 8);
                ks.sc[j] = *(const u4 *)(kb + KS * 512 + (j * 4 + g) * 16);
            }
        } else {
#pragma unroll
            for (int j = 0; j < KS; ++j) {
                ks.r[2 * j] = load_h8(kp + ((j * 2 + 0) * 64 + lane) * 8);
                ks.r[2 * j + 1] = load_h8(kp + ((j * 2 + 1) * 64 + lane) * 8);
            }
        }
    };
    auto load_v = [&](int idx, VSet & vs) {
        const int pid = __builtin_amdgcn_readlane(my_pid, idx);
        const __half * vp = a.v_pool + (size_t)pid * a.page_stride + (size_t)h * a.head_stride;
        if constexpr (KVQ == KV_Q8) {
            const uint8_t * vb = (const uint8_t *)vp;
#pragma unroll
            for (int b = 0; b < KS; ++b) {
                vs.raw[b] = *(const u4 *)(vb + b * 1024 + lane * 16);
                vs.sc[b] = *(const u4 *)(vb + KS * 1024 + (b * 4 + g) * 16);
            }
        } else if constexpr (KVQ == KV_Q4) {
            const uint8_t * vb = (const uint8_t *)vp;
#pragma unroll
            for (int b = 0; b < KS; ++b) {
                vs.raw[b] = *(const kv_u2 *)(vb + b * 512 + lane * 8);
                vs.sc[b] = *(const u4 *)(vb + KS * 512 + (b * 4 + g) * 16);
            }
        } else {
#pragma unroll
            for (int d = 0; d < DT; ++d) vs.r[d] = load_h8(vp + (d * 64 + lane) * 8);
        }
    };
    auto attend = [&](int pi, const KSet & ks, const VSet & vs) {
        h8 kreg[KS][2], vreg[DT];
        // Q8: the scales of this lane's eight tokens per block stay packed (ks.sc, vs.sc) and are widened where used,
        // and the codes are widened one k-step (dim-tile pair) at a time: fewer registers, a third wave per SIMD
        if constexpr (!Q8) {
#pragma unroll
            for (int j = 0; j < KS; ++j) { kreg[j][0] = ks.r[2 * j]; kreg[j][1] = ks.r[2 * j + 1]; }
#pragma unroll
            for (int d = 0; d < DT; ++d) vreg[d] = vs.r[d];
        }
        f4 s0 = (f4){0.f, 0.f, 0.f, 0.f}, s1 = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < KS; ++j) {
            if constexpr (Q8) {
                const f4 zero = (f4){0.f, 0.f, 0.f, 0.f};
                h8 k0, k1;
                if constexpr (KVQ == KV_Q8) { k0 = codes8(ks.raw[j].x, ks.raw[j].y); k1 = codes8(ks.raw[j].z, ks.raw[j].w); }
                else { k0 = codes4(ks.raw[j].x); k1 = codes4(ks.raw[j].y); }
                f4 u0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(k0, qreg[j], zero, 0, 0, 0);
                f4 u1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(k1, qreg[j], zero, 0, 0, 0);
                if (!SPLIT) {
                    u0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(k0, qreg_lo[j], u0, 0, 0, 0);
                    u1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(k1, qreg_lo[j], u1, 0, 0, 0);
                }
                const h8 dk = __builtin_bit_cast(h8, ks.sc[j]);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    s0[i] = fmaf((float)dk[i], u0[i], s0[i]);
                    s1[i] = fmaf((float)dk[4 + i], u1[i], s1[i]);
                }
            } else {
                s0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kreg[j][0], qreg[j], s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kreg[j][1], qreg[j], s1, 0, 0, 0);
                if (!SPLIT) {
                    s0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kreg[j][0], qreg_lo[j], s0, 0, 0, 0);
                    s1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kreg[j][1], qreg_lo[j], s1, 0, 0, 0);
                }
            }
        }
        if (SPLIT) {
            // the hi and lo products of a query sit 8 columns apart: both lanes take the sum
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                s0[i] += __shfl_xor(s0[i], 8, 64);
                s1[i] += __shfl_xor(s1[i], 8, 64);
            }
        }
        // rows of s0 are tokens 4g+i, of s1 tokens 16+4g+i of this page
        const int pbase = pi * PAGE + 4 * g;
        float mx = -INFINITY;
        // only the first and the last page of a sequence hold positions a column must not see
        const bool edge = !ONE || pi * PAGE < kv_begin || pi * PAGE + PAGE - 1 > limit;     // (a tile of several tokens: causal mask everywhere)
        if (edge) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int p0 = pbase + i, p1 = pbase + 16 + i;
                if (!(col_ok && p0 >= kv_begin && p0 <= limit)) s0[i] = -INFINITY;
                if (!(col_ok && p1 >= kv_begin && p1 <= limit)) s1[i] = -INFINITY;
            }
        } else if (!col_ok) {
#pragma unroll
            for (int i = 0; i < 4; ++i) { s0[i] = -INFINITY; s1[i] = -INFINITY; }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) mx = fmaxf(mx, fmaxf(s0[i], s1[i]));
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        const float m_use = m_new == -INFINITY ? 0.0f : m_new;
        const float alpha = !col_ok ? 1.0f : exp2f(m_run - m_use);       // m_run = -inf -> 0
        float psum = 0.0f;
        float e[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            e[i] = exp2f(s0[i] - m_use);
            e[4 + i] = exp2f(s1[i] - m_use);
            psum += e[i] + e[4 + i];
        }
        // the probabilities (Q8: times the V scale of the token in block `b`) as f16 hi/lo pairs
        auto operand = [&](int b, h8 & pt, h8 & pt_lo) {
            h8 dv;
            if constexpr (Q8) dv = __builtin_bit_cast(h8, vs.sc[b]);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float p = Q8 ? e[i] * (float)dv[i] : e[i];
                const _Float16 hi = (_Float16)p;
                const _Float16 lo = (_Float16)(p - (float)hi);
                // SPLIT: the column of the lo query half multiplies the lo half of the same probabilities
                pt[i] = lo_col ? lo : hi;
                pt_lo[i] = lo;
            }
        };
        h8 pt, pt_lo;
        if constexpr (!Q8) operand(0, pt, pt_lo);
        m_run = m_new;
        // the running maximum rarely moves after the first pages: then every column's factor is exactly one,
        // and multiplying by it would change nothing
        if (__any(alpha != 1.0f)) {
            l_run *= alpha;
#pragma unroll
            for (int d = 0; d < DT; ++d)
#pragma unroll
                for (int i = 0; i < 4; ++i) o[d][i] *= alpha;
        }
        l_run += psum;
#pragma unroll
        for (int d = 0; d < DT; ++d) {
            h8 vd;
            if constexpr (Q8) {
                if ((d & 1) == 0) operand(d >> 1, pt, pt_lo);
                if constexpr (KVQ == KV_Q8) vd = (d & 1) ? codes8(vs.raw[d >> 1].z, vs.raw[d >> 1].w) : codes8(vs.raw[d >> 1].x, vs.raw[d >> 1].y);
                else vd = (d & 1) ? codes4(vs.raw[d >> 1].y) : codes4(vs.raw[d >> 1].x);
            } else {
                vd = vreg[d];
            }
            o[d] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vd, pt, o[d], 0, 0, 0);
            if (!SPLIT) o[d] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vd, pt_lo, o[d], 0, 0, 0);
        }
    };
    // V of a page loads while its scores are computed, K of the next page while
    // the page is multiplied: two K register sets, one V set
    // The request for the next K page is never skipped (past the end it repeats the last page): a load under a
    // condition makes the number of loads in flight differ between the paths into the arithmetic, the compiler
    // then waits as if the fewer had been issued, and since loads return in order that wait covered the V page
    // before the scores needed it and the next K page before the products did - nothing was in flight while a
    // page was computed.
    if (n_pages > 0) {
        KSet kA, kB;
        VSet v;
        load_k(0, kA);
        for (int i = 0; i < n_pages; i += 2) {
            load_v(i, v);
            load_k(min(i + 1, n_pages - 1), kB);
            attend(page_first + i, kA, v);
            if (i + 1 >= n_pages) break;
            load_v(i + 1, v);
            load_k(min(i + 2, n_pages - 1), kA);
            attend(page_first + i + 1, kB, v);
        }
    }
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    if (SPLIT) {
        // the outputs against the lo halves of the probabilities join those against the hi halves
#pragma unroll
        for (int d = 0; d < DT; ++d)
#pragma unroll
            for (int i = 0; i < 4; ++i) o[d][i] += __shfl_xor(o[d][i], 8, 64);
    }
    if (col_ok && !lo_col) {
        float * dst = a.partial + ((size_t)item * 16 + c) * (HD + 2);
        if (g == 0) { dst[0] = m_run; dst[1] = l_run; }
#pragma unroll
        for (int d = 0; d < DT; ++d)
#pragma unroll
            for (int i = 0; i < 4; ++i) dst[2 + d * 16 + 4 * g + i] = o[d][i];
    }
}

size_t attention_partial_floats(int n_items, int head_dim) {
    return (size_t)n_items * 16 * (head_dim + 2);
}

void attention(hipStream_t s, const __half * q, const __half * q_lo, const AttnShape & sh, const PackBuffers & pk,
               const int32_t * table, int max_pages, const __half * k_pool, const __half * v_pool,
               int n_items, int n_tiles, float * partial, bool one_token_rows) {
    if (n_items <= 0) return;
    AttnArgs a;
    a.q = q; a.q_lo = q_lo; a.k_pool = k_pool; a.v_pool = v_pool; a.table = table;
    a.item_a = pk.item_a; a.item_b = pk.item_b;
    if (!pk.item_a || !pk.item_b) throw std::runtime_error("attention: the step's work items were not packed");
    a.partial = partial; a.n_tiles = n_tiles; a.n_items = n_items; a.max_pages = max_pages;
    a.n_head = sh.n_head; a.n_kv = sh.n_head_kv; a.G = sh.n_head / sh.n_head_kv;
    a.split_pages = pk.split_pages;
    a.page_stride = sh.page_stride; a.head_stride = sh.head_stride;
    if (sh.page_stride == 0 || sh.head_stride == 0) throw std::runtime_error("attention: the pool's strides are missing");
    if (a.G > 16 || sh.n_head % sh.n_head_kv != 0) throw std::runtime_error("attention: unsupported head grouping");
#define ATTN_LAUNCH_Q(HD_, Q8_) \
    do { \
        if (a.G <= 8 && one_token_rows) hipLaunchKernelGGL((k_attention<HD_, true, true, Q8_>), dim3(n_items), dim3(64), 0, s, a); \
        else if (a.G <= 8) hipLaunchKernelGGL((k_attention<HD_, false, true, Q8_>), dim3(n_items), dim3(64), 0, s, a); \
        else hipLaunchKernelGGL((k_attention<HD_, false, false, Q8_>), dim3(n_items), dim3(64), 0, s, a); \
    } while (0)
#define ATTN_LAUNCH(HD_) \
    do { \
        if (sh.kv_quant == KV_Q8) ATTN_LAUNCH_Q(HD_, KV_Q8); \
        else if (sh.kv_quant == KV_Q4) ATTN_LAUNCH_Q(HD_, KV_Q4); \
        else if (sh.kv_quant == KV_F16) ATTN_LAUNCH_Q(HD_, KV_F16); \
        else throw std::runtime_error("attention: unknown cache type"); \
    } while (0)
    switch (sh.head_dim) {
        case 32:  ATTN_LAUNCH(32); break;
        case 64:  ATTN_LAUNCH(64); break;
        case 128: ATTN_LAUNCH(128); break;
        default: throw std::runtime_error("attention: head_dim must be 32, 64 or 128");
    }
#undef ATTN_LAUNCH
#undef ATTN_LAUNCH_Q
    check_launch("attention");
}

struct CombineArgs {
    const float * partial;
    const int4 * tok_merge;
    Act out;
    int n_head, G, hd;
};

// One wave per (token, query head): merges the KV splits and writes the
// attention output as the O-projection's activations. The (max, sum) pairs of
// the splits are read one per lane, the outputs two dimensions per lane.
__global__ __launch_bounds__(256) void k_attention_combine(CombineArgs a) {
    __shared__ float blk_amax[4], blk_first[4];
    const int t = blockIdx.x;
    const int wave = threadIdx.x >> 6;
    const int head = blockIdx.y * 4 + wave;
    const int lane = threadIdx.x & 63;
    const bool live = head < a.n_head;           // a wave without a head still meets the others at the barrier
    const int e0 = 2 * lane;
    float M = -INFINITY, L = 0.0f, v0 = 0.0f, v1 = 0.0f;
    if (live) {
        const int4 meta = a.tok_merge[t];                  // first item of the token's tile, splits, index in the tile
        const int ns = meta.y;
        const int kvh = head / a.G, gi = head % a.G;
        const int col = meta.z * a.G + gi;
        const int item0 = meta.x + kvh * ns;
        const int stride = a.hd + 2;
        for (int s0 = 0; s0 < ns; s0 += 64) {
            const int n = min(64, ns - s0);
            float m_s = -INFINITY, l_s = 0.0f;
            if (lane < n) {
                const float * p = a.partial + ((size_t)(item0 + s0 + lane) * 16 + col) * stride;
                m_s = p[0];
                l_s = p[1];
            }
            float cm = m_s;
            for (int o = 32; o > 0; o >>= 1) cm = fmaxf(cm, __shfl_xor(cm, o, 64));
            const float m_new = fmaxf(M, cm);
            const float keep = M == -INFINITY ? 0.0f : exp2f(M - m_new);
            L *= keep; v0 *= keep; v1 *= keep;
            M = m_new;
            const float w_s = m_s == -INFINITY ? 0.0f : exp2f(m_s - M);
            L += wave_sum(w_s * l_s);
            // the splits' outputs eight at a time: their loads are in flight together, the sums keep the split order
            for (int s1 = 0; s1 < n; s1 += 8) {
                float2 pv[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    pv[u] = make_float2(0.0f, 0.0f);
                    if (s1 + u < n && e0 < a.hd)
                        pv[u] = *(const float2 *)(a.partial + ((size_t)(item0 + s0 + s1 + u) * 16 + col) * stride + 2 + e0);
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    if (s1 + u < n) {
                        const float w = __shfl(w_s, s1 + u, 64);
                        v0 = fmaf(w, pv[u].x, v0);
                        v1 = fmaf(w, pv[u].y, v1);
                    }
                }
            }
        }
    }
    const float inv = L > 0.0f ? 1.0f / L : 0.0f;
    const int QD = a.n_head * a.hd;
    const bool mine = live && e0 < a.hd;
    const float f0 = mine ? v0 * inv : 0.0f, f1 = mine ? v1 * inv : 0.0f;
    const int k = head * a.hd + e0;            // even: k and k + 1 share a group of eight
    // 32 outputs = 16 lanes: the block sum of the stored values
    auto store = [&](__half * x, __half * sums, float g0, float g1) {
        float r0 = 0.0f, r1 = 0.0f;
        if (mine) {
            const float c0 = fminf(fmaxf(g0, -65504.0f), 65504.0f), c1 = fminf(fmaxf(g1, -65504.0f), 65504.0f);
            const __half h0 = __float2half_rn(c0), h1 = __float2half_rn(c1);
            const __half l0 = __float2half_rn(c0 - __half2float(h0)), l1 = __float2half_rn(c1 - __half2float(h1));
            const size_t at = act_at(t, k, 0, QD), at_lo = act_at(t, k, 1, QD);
            x[at] = h0;
            x[at + 1] = h1;
            x[at_lo] = l0;
            x[at_lo + 1] = l1;
            r0 = __half2float(h0) + __half2float(l0);
            r1 = __half2float(h1) + __half2float(l1);
        }
        if (sums) {
            float sum = r0 + r1;
#pragma unroll
            for (int o = 1; o < 16; o <<= 1) sum += __shfl_xor(sum, o, 64);
            if ((lane & 15) == 0 && mine) {
                const int b = k / 32;
                const __half hi = sat_half(sum);
                sums[act_sum_at(t, b, 0, QD)] = hi;
                sums[act_sum_at(t, b, 1, QD)] = __float2half_rn(sum - __half2float(hi));
            }
        }
    };
    if (a.out.x) store(a.out.x, a.out.sums, f0, f1);
    if (!a.out.qx) return;
    // the conversion ggml's CPU matmul applies to the row before the output projection (see requantise8)
    float q0, q1;
    if (a.out.quant == AQ_Q8_0) {
        float amax = fmaxf(fabsf(f0), fabsf(f1));
#pragma unroll
        for (int o = 1; o < 16; o <<= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
        const float d = __fdiv_rn(amax, 127.0f);
        const float id = d != 0.0f ? __fdiv_rn(1.0f, d) : 0.0f;
        const float dh = (float)(_Float16)d;
        const float c0 = roundf(__fmul_rn(f0, id)), c1 = roundf(__fmul_rn(f1, id));
        q0 = __fmul_rn(dh, c0);
        q1 = __fmul_rn(dh, c1);
        if (a.out.qc && mine) {      // the blocks themselves, for the integer matrix-vector kernel (see store_codes8)
            int8_t * at = a.out.qc + (size_t)t * QD + k;
            at[0] = (int8_t)(int)c0;
            at[1] = (int8_t)(int)c1;
            if ((lane & 15) == 0) a.out.qd[(size_t)t * (QD >> 5) + (k >> 5)] = dh;
        }
    } else {
        // a block of 256 = 256 / hd heads = that many waves of this workgroup, in head order
        float amax = fabsf(f0), first = f0;
        if (fabsf(f1) > amax) { amax = fabsf(f1); first = f1; }
        float wmax = amax;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) wmax = fmaxf(wmax, __shfl_xor(wmax, o, 64));
        const uint64_t holders = __ballot(amax == wmax);
        first = __shfl(first, __ffsll((long long)holders) - 1, 64);
        if (lane == 0) { blk_amax[wave] = wmax; blk_first[wave] = first; }
        __syncthreads();
        const int per = 256 / a.hd;                 // waves per block: 2 (hd 128) or 4 (hd 64)
        const int w0 = wave / per * per;
        float gmax = 0.0f, max = 0.0f;
        for (int w = w0; w < w0 + per; ++w)
            if (blk_amax[w] > gmax) { gmax = blk_amax[w]; max = blk_first[w]; }
        float c0 = 0.0f, c1 = 0.0f, d = 0.0f;
        if (gmax == 0.0f) {
            q0 = q1 = 0.0f;
        } else {
            const float iscale = __fdiv_rn(-127.0f, max);
            d = __fdiv_rn(1.0f, iscale);
            c0 = fminf(127.0f, rintf(__fmul_rn(iscale, f0)));
            c1 = fminf(127.0f, rintf(__fmul_rn(iscale, f1)));
            q0 = __fmul_rn(d, c0);
            q1 = __fmul_rn(d, c1);
        }
        if (a.out.qc) {      // the blocks themselves, for the integer matrix-vector kernel (see store_codes8)
            const int i0 = (int)c0, i1 = (int)c1;
            int sum = i0 + i1;          // of 16 codes: eight lanes
#pragma unroll
            for (int o = 1; o < 8; o <<= 1) sum += __shfl_xor(sum, o, 64);
            if (mine) {
                int8_t * grp = a.out.qc + (size_t)t * QD + (k & ~7);
                grp[act_code_pos(k & 7)] = (int8_t)i0;
                grp[act_code_pos((k & 7) + 1)] = (int8_t)i1;
                if ((lane & 7) == 0) a.out.qbs[(size_t)t * (QD >> 4) + (k >> 4)] = (int16_t)sum;
                if (wave == w0 && lane == 0) a.out.qd[(size_t)t * (QD >> 8) + (k >> 8)] = d;
            }
        }
    }
    store(a.out.qx, a.out.qsums, q0, q1);
}

void attention_combine(hipStream_t s, const float * partial, int T, const AttnShape & sh,
                       const PackBuffers & pk, const Act & out) {
    if (T <= 0) return;
    check_act_out(out, sh.n_head * sh.head_dim, "attention_combine", T);
    if (out.qx && out.quant == AQ_Q8_K && ((sh.head_dim != 64 && sh.head_dim != 128) || (sh.n_head * sh.head_dim) % 256 != 0))
        throw std::runtime_error("attention_combine: the Q8_K conversion needs heads of 64 or 128 dimensions");
    CombineArgs a;
    a.partial = partial; a.tok_merge = pk.tok_merge; a.out = out;
    a.n_head = sh.n_head; a.G = sh.n_head / sh.n_head_kv; a.hd = sh.head_dim;
    hipLaunchKernelGGL(k_attention_combine, dim3(T, (sh.n_head + 3) / 4), dim3(256), 0, s, a);
    check_launch("attention_combine");
}

// ---------------------------------------------------------------------------
// the attention of a pure decode step in one launch

struct DecodeAttnArgs {
    const float * qkv;                      // [T][QD + 2 KD] f32 (with the biases), when there are no slices
    Slices from;                            // or the K-slices of the fused q, k, v product, added in slice order
    const float * rope_cos, * rope_sin;     // [T][head_dim / 2]
    const int4 * desc;                      // per row, longest sequence first: {token index, position, first resident position, slot}
    const int32_t * first_pid;              // [row in that order][8]: the id of each wave's first page
    const int32_t * table;
    int max_pages;
    __half * k_pool, * v_pool;
    size_t page_stride, head_stride;
    Act out;                                // the output projection's activations (hi/lo planes and block sums)
    int n_head, n_kv, G, neox;
    float qscale;
    const float * q_norm, * k_norm;         // per-head RMSNorm weights of the q and k rows ([head_dim]), or null
    float eps;
    unsigned long long * stamps;            // null, or [workgroup][6]: the constant 100 MHz clock at the workgroup's start,
                                            // after the prologue's barrier, when its first wave has attended its pages, after
                                            // the barrier behind all waves, at the end; the row's pages
};

// One workgroup of eight waves per (row, kv head) of a step in which every row decodes one token, f16 cache, at
// most eight query heads per kv head; it does what k_rope_store, k_attention<HD, true, true> and
// k_attention_combine do for such a step in three launches:
//   * every lane builds its part of the query operand itself: the K-slices of the q columns added in slice order,
//     rotated (a rotation pair lies inside a lane's dims in both pairings), scaled, split into f16 hi and lo;
//   * the sequence's pages are divided evenly among the eight waves (a division that depends on the sequence alone,
//     so a row's result does not depend on what else the step holds); each wave runs the same online softmax over
//     its pages as k_attention does over a work item;
//   * the wave that owns the page of the new position also makes the new K and V row (slices, rotation, f16),
//     stores them into the page for later steps and puts them into the operand registers it loaded for that page -
//     no other wave of the launch reads that cell;
//   * the eight partial results meet in LDS and waves 0 .. G - 1 merge them, one query head each, with
//     k_attention_combine's arithmetic, and store the output projection's activations.
template <int HD, int NW>
__global__ __launch_bounds__(NW * 64, 8 / NW) void k_attention_decode(DecodeAttnArgs a) {
    unsigned long long * stamp = a.stamps && threadIdx.x == 0 ? a.stamps + (size_t)blockIdx.x * 6 : nullptr;
    if (stamp) stamp[0] = wall_clock64();
    constexpr int KS = HD / 32;     // k-steps of QK^T
    constexpr int DT = HD / 16;     // dim tiles of PV
    constexpr int PS = HD + 2;      // floats of one partial result: max, sum, output
    constexpr int NT = NW * 64;
    __shared__ float part[NW][8][PS];
    __shared__ __attribute__((aligned(16))) _Float16 q_hi[8][HD], q_lo[8][HD], k_row[HD], v_row[HD];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    static_assert(NW == 8, "k_pack deals a row's pages to eight waves");
    const int4 dd = a.desc[blockIdx.x / a.n_kv];
    const int t = dd.x, h = blockIdx.x % a.n_kv;
    const int pos = dd.y, kv_begin = dd.z, slot = dd.w;
    const int pid0 = a.first_pid[(blockIdx.x / a.n_kv) * 8 + wave];
    const int cc = c & 7;
    const bool col_ok = cc < a.G;
    const bool lo_col = c >= 8;
    const int QD = a.n_head * HD, KD = a.n_kv * HD, ROW = QD + 2 * KD;
    const int page_first = kv_begin / PAGE, n_pages = pos / PAGE - page_first + 1;
    const int per_wave = (n_pages + NW - 1) / NW;
    const int my_first = page_first + wave * per_wave;
    const int my_n = min(per_wave, max(0, n_pages - wave * per_wave));
    const int last_owner = (n_pages - 1) / per_wave;
    const int t32 = pos % PAGE;

    // page ids of this wave's share, one per lane
    const int my_pid = lane < my_n ? a.table[(size_t)slot * a.max_pages + my_first + lane] : 0;

    // The workgroup's part of the step's q, k, v row, one column per thread and turn: the G query heads of this
    // kv head, its k row and its v row ((G + 2) HD columns). A column is the sum of its K-slices in slice order; q
    // and k columns are rotated with their partner column (which the thread adds up as well), q is scaled and
    // split into f16 hi and lo. Everything lands in LDS, in element order.
    // The order of the memory requests matters, because a wave's loads return in the order they were issued: first
    // the columns (every slice of a column and of its partner at once - one after the other they cost eight trips to
    // the L2), then the wave's first K page, and only then the arithmetic on the columns, so that the page's trip to
    // HBM runs under the rotation, the LDS exchange and the barrier.
    constexpr int TURNS = (10 * HD + NT - 1) / NT;          // G <= 8
    const int n_cols = (a.G + 2) * HD;
    const bool fast = a.from.n >= 1 && a.from.n <= 4;
    float xs[TURNS][4], ys[TURNS][4], cvs[TURNS], svs[TURNS], nxs[TURNS], nys[TURNS];
    const float * cs = a.rope_cos + (size_t)t * (HD / 2), * sn = a.rope_sin + (size_t)t * (HD / 2);
    auto place = [&](int idx, int & col, int & partner, int & hh, int & d) {
        hh = idx / HD; d = idx % HD;          // hh < G: query head, G: k, G + 1: v
        const int col0 = hh < a.G ? (h * a.G + hh) * HD : (hh == a.G ? QD + h * HD : QD + KD + h * HD);
        // partner of the rotation pair (v columns have none: the column itself)
        const int pd = hh > a.G ? d : (a.neox ? (d < HD / 2 ? d + HD / 2 : d - HD / 2) : (d ^ 1));
        col = col0 + d; partner = col0 + pd;
    };
#pragma unroll
    for (int u = 0; u < TURNS; ++u) {
        const int idx = min((int)threadIdx.x + u * NT, n_cols - 1);
        int col, partner, hh, d;
        place(idx, col, partner, hh, d);
        const int i = a.neox ? (d < HD / 2 ? d : d - HD / 2) : (d >> 1);
        cvs[u] = cs[i];
        svs[u] = sn[i];
        // the norm weights of the column and of its partner, where the architecture normalises q and k per head
        // (else any valid word: the request is made on every path, and before the first pages are requested - a
        // load behind them would have to wait for them)
        const float * nw = hh < a.G ? a.q_norm : (hh == a.G ? a.k_norm : nullptr);
        nxs[u] = nw ? nw[d] : cs[0];
        nys[u] = nw ? nw[partner - (col - d)] : cs[0];
        if (fast) {
            const float * base = a.from.data + (size_t)t * ROW;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const size_t at = (size_t)min(k, a.from.n - 1) * a.from.stride;
                xs[u][k] = base[at + col];
                ys[u][k] = base[at + partner];
            }
        }
    }
    asm volatile("" : : : "memory");
    struct KSet { h8 r[2 * KS]; };
    struct VSet { h8 r[DT]; };
    auto load_k_page = [&](int pid, KSet & ks) {
        const __half * kp = a.k_pool + (size_t)pid * a.page_stride + (size_t)h * a.head_stride;
#pragma unroll
        for (int j = 0; j < KS; ++j) {
            ks.r[2 * j] = load_h8(kp + ((j * 2 + 0) * 64 + lane) * 8);
            ks.r[2 * j + 1] = load_h8(kp + ((j * 2 + 1) * 64 + lane) * 8);
        }
    };
    auto load_k = [&](int idx, KSet & ks) { load_k_page(__builtin_amdgcn_readlane(my_pid, idx), ks); };
    KSet kA;
    // The wave's first page by the id k_pack left, so that the request does not wait for the table lookup above.
    // (The new position's own cell in its page is not stored yet: the owner wave replaces it in registers below.)
    // A wave without pages requests page 0 and never looks at it: with a branch around the request the waits
    // below could not tell the two paths apart and would wait for everything.
    load_k_page(pid0, kA);
    // ... and its V page behind it (the pages of a wave are attended with the next page's K and V in flight)
    auto load_v_page = [&](int pid, VSet & vs) {
        const __half * vp = a.v_pool + (size_t)pid * a.page_stride + (size_t)h * a.head_stride;
#pragma unroll
        for (int d = 0; d < DT; ++d) vs.r[d] = load_h8(vp + (d * 64 + lane) * 8);
    };
    VSet vA;
    load_v_page(pid0, vA);
    asm volatile("" : : : "memory");
    // The column values are first looked at here: left alone, the compiler adds a turn's first slices right behind
    // their loads (to reuse the registers) and so waits a trip to memory per turn before it requests the next.
    if (fast) {
#pragma unroll
        for (int u = 0; u < TURNS; ++u)
#pragma unroll
            for (int k = 0; k < 4; ++k) asm volatile("" : "+v"(xs[u][k]), "+v"(ys[u][k]));
    }
    auto column_pair = [&](int col, int partner, float & x, float & y) {
        x = 0.0f; y = 0.0f;
        if (a.from.n > 0) {
            const float * base = a.from.data + (size_t)t * ROW;
            for (int k = 0; k < a.from.n; ++k) {
                x += base[(size_t)k * a.from.stride + col];
                y += base[(size_t)k * a.from.stride + partner];
            }
        } else {
            x = a.qkv[(size_t)t * ROW + col];
            y = a.qkv[(size_t)t * ROW + partner];
        }
    };
    // The columns' sums in slice order. One branch around all turns, not one per turn: where the two paths meet the
    // compiler treats the other path's loads as possibly in flight, and a meeting point per turn made every turn
    // wait for everything requested so far - the wave's first K and V page included.
    float xv[TURNS], yv[TURNS];
    if (fast) {
#pragma unroll
        for (int u = 0; u < TURNS; ++u) {
            float x = 0.0f, y = 0.0f;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                x += k < a.from.n ? xs[u][k] : 0.0f;
                y += k < a.from.n ? ys[u][k] : 0.0f;
            }
            xv[u] = x; yv[u] = y;
        }
    } else {
#pragma unroll
        for (int u = 0; u < TURNS; ++u) {
            const int idx = threadIdx.x + u * NT;
            float x = 0.0f, y = 0.0f;
            if (idx < n_cols) {
                int col, partner, hh, d;
                place(idx, col, partner, hh, d);
                column_pair(col, partner, x, y);
            }
            xv[u] = x; yv[u] = y;
        }
        // (this path's loads land before the paths meet: a load that could still be in flight into a register the
        // other path writes would make that path wait for every request before it)
#pragma unroll
        for (int u = 0; u < TURNS; ++u) asm volatile("" : "+v"(xv[u]), "+v"(yv[u]));
    }
    // Architectures that normalise the q and k rows per head (RMSNorm over the head's dims, before the rotation): a
    // head's columns sit in consecutive threads of one turn - one wave for 64 dims, an even and an odd wave for 128 -
    // so the sum of squares is a wave sum, and for 128 dims the two halves meet in LDS.
    if (a.q_norm || a.k_norm) {
        float * half_ss = &part[0][0][0];          // free until the waves leave their partial results there
#pragma unroll
        for (int u = 0; u < TURNS; ++u) {
            const int idx = threadIdx.x + u * NT;
            const float mine = idx < n_cols ? xv[u] * xv[u] : 0.0f;
            const float ws = wave_sum(mine);
            if (lane == 0) half_ss[u * NW + wave] = ws;
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < TURNS; ++u) {
            const int idx = min((int)threadIdx.x + u * NT, n_cols - 1);
            int col, partner, hh, d;
            place(idx, col, partner, hh, d);
            const float * nw = hh < a.G ? a.q_norm : (hh == a.G ? a.k_norm : nullptr);
            if (nw) {
                const float ss = HD == 128 ? half_ss[u * NW + (wave & ~1)] + half_ss[u * NW + (wave | 1)] : half_ss[u * NW + wave];
                const float scale = 1.0f / sqrtf(ss / (float)HD + a.eps);
                xv[u] = (xv[u] * scale) * nxs[u];
                yv[u] = (yv[u] * scale) * nys[u];
            }
        }
        __syncthreads();          // half_ss is read before the partial results may overwrite it
    }
#pragma unroll
    for (int u = 0; u < TURNS; ++u) {
        const int idx = threadIdx.x + u * NT;
        if (idx >= n_cols) break;
        int col, partner, hh, d;
        place(idx, col, partner, hh, d);
        const bool first = a.neox ? d < HD / 2 : (d & 1) == 0;
        const float cv = cvs[u], sv = svs[u];
        float x = xv[u];
        const float y = yv[u];
        if (hh <= a.G) x = first ? x * cv - y * sv : y * sv + x * cv;
        if (hh < a.G) {
            const float sc = fminf(fmaxf(x * a.qscale, -65504.0f), 65504.0f);
            const _Float16 hi = (_Float16)sc;
            q_hi[hh][d] = hi;
            q_lo[hh][d] = (_Float16)(sc - (float)hi);
        } else {
            const _Float16 v = (_Float16)fminf(fmaxf(x, -65504.0f), 65504.0f);
            if (hh == a.G) k_row[d] = v; else v_row[d] = v;
        }
    }
    __syncthreads();
    if (stamp) stamp[1] = wall_clock64();

    h8 qreg[KS];
#pragma unroll
    for (int j = 0; j < KS; ++j) {
        if (col_ok) qreg[j] = *(const h8 *)&(lo_col ? q_lo : q_hi)[cc][32 * j + 8 * g];
        else qreg[j] = (h8){0, 0, 0, 0, 0, 0, 0, 0};
    }

    // The new position's K and V row, by the wave that owns its page. K: lane (g, t32 % 16) holds dims 32 j + 8 g ..
    // of the token in operand register 2 j + t32 / 16; V: lane (g = (t32 % 16) / 4, d) holds the token in slot
    // (t32 % 4) + 4 (t32 / 16) of dim 16 dt + d. Those lanes keep the values for the operand registers of the page
    // and store them into it for later steps.
    const bool owner = wave == last_owner;
    const bool k_lane = owner && (lane & 15) == (t32 & 15);
    const bool v_lane = owner && g == ((t32 & 15) >> 2);
    const int v_slot = (t32 & 3) + 4 * (t32 >> 4);
    h8 k_new[KS];
    _Float16 v_new[DT];
#pragma unroll
    for (int j = 0; j < KS; ++j) k_new[j] = (h8){0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int d = 0; d < DT; ++d) v_new[d] = (_Float16)0.0f;
    if (owner) {
        const int pid = __builtin_amdgcn_readlane(my_pid, my_n - 1);
        if (k_lane) {
            __half * dst = a.k_pool + (size_t)pid * a.page_stride + (size_t)h * a.head_stride;
#pragma unroll
            for (int j = 0; j < KS; ++j) {
                k_new[j] = *(const h8 *)&k_row[32 * j + 8 * g];
                *(h8 *)(dst + ((((j * 2 + (t32 >> 4)) * 4 + g) * 16 + (t32 & 15)) * 8)) = k_new[j];
            }
        }
        if (v_lane) {
            __half * dst = a.v_pool + (size_t)pid * a.page_stride + (size_t)h * a.head_stride;
#pragma unroll
            for (int d = 0; d < DT; ++d) {
                v_new[d] = v_row[16 * d + (lane & 15)];
                dst[((d * 4 + g) * 16 + (lane & 15)) * 8 + v_slot] = __builtin_bit_cast(__half, v_new[d]);
            }
        }
    }

    f4 o[DT];
#pragma unroll
    for (int d = 0; d < DT; ++d) o[d] = (f4){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.0f;
    auto load_v = [&](int idx, VSet & vs) { load_v_page(__builtin_amdgcn_readlane(my_pid, idx), vs); };
    auto attend = [&](int pi, const KSet & ks, const VSet & vs, bool newest) {
        h8 kreg[KS][2], vreg[DT];
#pragma unroll
        for (int j = 0; j < KS; ++j) { kreg[j][0] = ks.r[2 * j]; kreg[j][1] = ks.r[2 * j + 1]; }
#pragma unroll
        for (int d = 0; d < DT; ++d) vreg[d] = vs.r[d];
        if (newest) {
            // the page of the new position: what was loaded from its cell is replaced by the row made above
            if (k_lane) {
#pragma unroll
                for (int j = 0; j < KS; ++j) {
                    if (t32 >> 4) kreg[j][1] = k_new[j]; else kreg[j][0] = k_new[j];
                }
            }
            if (v_lane) {
#pragma unroll
                for (int d = 0; d < DT; ++d)
#pragma unroll
                    for (int i = 0; i < 8; ++i) if (i == v_slot) vreg[d][i] = v_new[d];
            }
        }
        f4 s0 = (f4){0.f, 0.f, 0.f, 0.f}, s1 = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < KS; ++j) {
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kreg[j][0], qreg[j], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kreg[j][1], qreg[j], s1, 0, 0, 0);
        }
        // the hi and lo products of a query sit 8 columns apart: both lanes take the sum
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            s0[i] += __shfl_xor(s0[i], 8, 64);
            s1[i] += __shfl_xor(s1[i], 8, 64);
        }
        const int pbase = pi * PAGE + 4 * g;
        float mx = -INFINITY;
        // only the first and the last page of a sequence hold positions a column must not see
        const bool edge = pi * PAGE < kv_begin || pi * PAGE + PAGE - 1 > pos;
        if (edge) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int p0 = pbase + i, p1 = pbase + 16 + i;
                if (!(col_ok && p0 >= kv_begin && p0 <= pos)) s0[i] = -INFINITY;
                if (!(col_ok && p1 >= kv_begin && p1 <= pos)) s1[i] = -INFINITY;
            }
        } else if (!col_ok) {
#pragma unroll
            for (int i = 0; i < 4; ++i) { s0[i] = -INFINITY; s1[i] = -INFINITY; }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) mx = fmaxf(mx, fmaxf(s0[i], s1[i]));
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        const float m_use = m_new == -INFINITY ? 0.0f : m_new;
        const float alpha = !col_ok ? 1.0f : exp2f(m_run - m_use);       // m_run = -inf -> 0
        float psum = 0.0f;
        h8 pt;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float e0 = exp2f(s0[i] - m_use), e1 = exp2f(s1[i] - m_use);
            psum += e0 + e1;
            const _Float16 h0 = (_Float16)e0, h1 = (_Float16)e1;
            // the column of the lo query half multiplies the lo half of the same probabilities
            pt[i] = lo_col ? (_Float16)(e0 - (float)h0) : h0;
            pt[4 + i] = lo_col ? (_Float16)(e1 - (float)h1) : h1;
        }
        m_run = m_new;
        // the running maximum rarely moves after the first pages: then every column's factor is exactly one
        if (__any(alpha != 1.0f)) {
            l_run *= alpha;
#pragma unroll
            for (int d = 0; d < DT; ++d)
#pragma unroll
                for (int i = 0; i < 4; ++i) o[d][i] *= alpha;
        }
        l_run += psum;
#pragma unroll
        for (int d = 0; d < DT; ++d) o[d] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vreg[d], pt, o[d], 0, 0, 0);
    };
    // K and V of the next page load while a page is attended (never skipped: past the end the last page again, so
    // that the number of loads in flight is the same on every path)
    if (my_n > 0) {
        KSet kB;
        VSet vB;
        for (int i = 0; i < my_n; i += 2) {
            load_k(min(i + 1, my_n - 1), kB);
            load_v(min(i + 1, my_n - 1), vB);
            attend(my_first + i, kA, vA, owner && i == my_n - 1);
            if (i + 1 >= my_n) break;
            load_k(min(i + 2, my_n - 1), kA);
            load_v(min(i + 2, my_n - 1), vA);
            attend(my_first + i + 1, kB, vB, owner && i + 1 == my_n - 1);
        }
    }
    if (stamp) stamp[2] = wall_clock64();
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
#pragma unroll
    for (int d = 0; d < DT; ++d)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[d][i] += __shfl_xor(o[d][i], 8, 64);
    if (col_ok && !lo_col) {
        float * dst = part[wave][cc];
        if (g == 0) { dst[0] = m_run; dst[1] = l_run; }
#pragma unroll
        for (int d = 0; d < DT; ++d)
#pragma unroll
            for (int i = 0; i < 4; ++i) dst[2 + d * 16 + 4 * g + i] = o[d][i];
    }
    __syncthreads();
    if (stamp) { stamp[3] = wall_clock64(); stamp[5] = (unsigned long long)n_pages; }
    // wave gi merges the eight partial results of query head h G + gi (a wave without pages left max = -inf, sum = 0)
    for (int gi = wave; gi < a.G; gi += NW) {
    const int e0 = 2 * lane;
    float m_s = -INFINITY, l_s = 0.0f;
    if (lane < NW) { m_s = part[lane][gi][0]; l_s = part[lane][gi][1]; }
    float M = m_s;
    for (int ofs = 32; ofs > 0; ofs >>= 1) M = fmaxf(M, __shfl_xor(M, ofs, 64));
    const float w_s = m_s == -INFINITY ? 0.0f : exp2f(m_s - M);
    const float L = wave_sum(w_s * l_s);
    float v0 = 0.0f, v1 = 0.0f;
    if (e0 < HD) {
#pragma unroll
        for (int sp = 0; sp < NW; ++sp) {
            const float w = __shfl(w_s, sp, 64);
            v0 = fmaf(w, part[sp][gi][2 + e0], v0);
            v1 = fmaf(w, part[sp][gi][2 + e0 + 1], v1);
        }
    } else {
#pragma unroll
        for (int sp = 0; sp < NW; ++sp) (void)__shfl(w_s, sp, 64);
    }
    const float inv = L > 0.0f ? 1.0f / L : 0.0f;
    const bool mine = e0 < HD;
    const float f0 = mine ? v0 * inv : 0.0f, f1 = mine ? v1 * inv : 0.0f;
    const int k = (h * a.G + gi) * HD + e0;
    float r0 = 0.0f, r1 = 0.0f;
    if (mine) {
        const float c0 = fminf(fmaxf(f0, -65504.0f), 65504.0f), c1 = fminf(fmaxf(f1, -65504.0f), 65504.0f);
        const __half h0 = __float2half_rn(c0), h1 = __float2half_rn(c1);
        const __half l0 = __float2half_rn(c0 - __half2float(h0)), l1 = __float2half_rn(c1 - __half2float(h1));
        const size_t at = act_at(t, k, 0, QD), at_lo = act_at(t, k, 1, QD);
        a.out.x[at] = h0;
        a.out.x[at + 1] = h1;
        a.out.x[at_lo] = l0;
        a.out.x[at_lo + 1] = l1;
        r0 = __half2float(h0) + __half2float(l0);
        r1 = __half2float(h1) + __half2float(l1);
    }
    if (a.out.sums) {
        float sum = r0 + r1;
#pragma unroll
        for (int ofs = 1; ofs < 16; ofs <<= 1) sum += __shfl_xor(sum, ofs, 64);
        if ((lane & 15) == 0 && mine) {
            const int b = k / 32;
            const __half hi = sat_half(sum);
            a.out.sums[act_sum_at(t, b, 0, QD)] = hi;
            a.out.sums[act_sum_at(t, b, 1, QD)] = __float2half_rn(sum - __half2float(hi));
        }
    }
    }
    if (stamp) stamp[4] = wall_clock64();
}

bool attention_decode_can(const AttnShape & sh, int max_positions) {
    const int G = sh.n_head_kv > 0 ? sh.n_head / sh.n_head_kv : 0;
    return sh.kv_quant == KV_F16 && (sh.head_dim == 128 || sh.head_dim == 64) && sh.rope_dim == sh.head_dim
        && G >= 1 && G <= 8 && sh.n_head % sh.n_head_kv == 0 && max_positions <= 8 * 64 * PAGE;       // a wave holds one page id per lane, a workgroup has eight waves
}

void attention_decode(hipStream_t s, const float * qkv, const Slices & from, int n_rows, const AttnShape & sh,
                      const PackBuffers & pk, const int32_t * table, int max_pages, __half * k_pool, __half * v_pool,
                      const float * q_norm, const float * k_norm, const Act & out, unsigned long long * stamps) {
    if (n_rows <= 0) return;
    if (!attention_decode_can(sh, 0)) throw std::runtime_error("attention_decode: unsupported shape or cache type");
    check_act_out(out, sh.n_head * sh.head_dim, "attention_decode", n_rows);
    if (!out.x) throw std::runtime_error("attention_decode: needs the plain activation planes");
    if (sh.page_stride == 0 || sh.head_stride == 0) throw std::runtime_error("attention_decode: the pool's strides are missing");
    const int ROW = (sh.n_head + 2 * sh.n_head_kv) * sh.head_dim;
    if (from.n > 0 && from.N != ROW) throw std::runtime_error("attention_decode: the slices are not a fused q, k, v product");
    if (!pk.dec_desc || !pk.dec_pid) throw std::runtime_error("attention_decode: the step's rows were not described");
    DecodeAttnArgs a;
    a.qkv = qkv; a.from = from; a.rope_cos = pk.rope_cos; a.rope_sin = pk.rope_sin;
    a.desc = pk.dec_desc; a.first_pid = pk.dec_pid;
    a.table = table; a.max_pages = max_pages; a.k_pool = k_pool; a.v_pool = v_pool;
    a.page_stride = sh.page_stride; a.head_stride = sh.head_stride;
    a.out = out;
    a.n_head = sh.n_head; a.n_kv = sh.n_head_kv; a.G = sh.n_head / sh.n_head_kv; a.neox = sh.rope_neox ? 1 : 0;
    a.qscale = 1.4426950408889634f / sqrtf((float)sh.head_dim);
    a.q_norm = q_norm; a.k_norm = k_norm; a.eps = sh.eps;
    a.stamps = stamps;
    const dim3 grid(n_rows * sh.n_head_kv);
    // eight waves per workgroup, one workgroup per CU (four waves and two workgroups per CU measured slower)
    if (sh.head_dim == 128) hipLaunchKernelGGL((k_attention_decode<128, 8>), grid, dim3(512), 0, s, a);
    else hipLaunchKernelGGL((k_attention_decode<64, 8>), grid, dim3(512), 0, s, a);
    check_launch("attention_decode");
}

// ---------------------------------------------------------------------------
// KV page utilities

__global__ void k_kv_gather(const __half * pool, KvStrides st, int n_kv, int hd, int is_v, const int32_t * cells, int n,
                            __half * out, int scatter) {
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int kd = n_kv * hd;
    if (gid >= (size_t)n * kd) return;
    const int idx = (int)(gid / kd), e_all = (int)(gid % kd);
    const int kvh = e_all / hd, e = e_all % hd;
    const int cell = cells[idx];
    const int page = cell / PAGE, t32 = cell % PAGE;
    const size_t off = (size_t)page * st.page + (size_t)kvh * st.head
        + (is_v ? v_page_offset(hd, t32, e) : k_page_offset(hd, t32, e));
    __half * cache = const_cast<__half *>(pool) + off;
    if (scatter) *cache = out[gid];
    else out[gid] = *cache;
}

// The Q8_0 pool: one 16-bit unit per thread - a pair of code bytes (elements 2u, 2u + 1 of the head's row) or,
// past the codes, one block scale. Rows of kv_row_halves units.
__global__ void k_kv_gather_q8(const __half * pool, KvStrides st, int n_kv, int hd, int is_v, const int32_t * cells, int n,
                               uint16_t * out, int scatter) {
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int per_head = hd / 2 + hd / 32;
    if (gid >= (size_t)n * n_kv * per_head) return;
    const int idx = (int)(gid / ((size_t)n_kv * per_head)), rest = (int)(gid % ((size_t)n_kv * per_head));
    const int kvh = rest / per_head, u = rest % per_head;
    const int cell = cells[idx];
    const int page = cell / PAGE, t32 = cell % PAGE;
    uint8_t * blk = (uint8_t *)(const_cast<__half *>(pool) + (size_t)page * st.page + (size_t)kvh * st.head);
    const int tg = (t32 & 15) >> 2, ti = (t32 & 3) + 4 * (t32 >> 4);
    if (u >= hd / 2) {
        uint16_t * sc = (uint16_t *)(blk + (hd / 32) * 1024) + (u - hd / 2) * 32 + tg * 8 + ti;
        if (scatter) *sc = out[gid]; else out[gid] = *sc;
        return;
    }
    const int e = 2 * u, b = e >> 5;
    if (!is_v) {
        uint16_t * c = (uint16_t *)(blk + b * 1024 + (((e >> 3) & 3) * 16 + (t32 & 15)) * 16 + (t32 >> 4) * 8 + (e & 7));
        if (scatter) *c = out[gid]; else out[gid] = *c;
    } else {
        uint8_t * c0 = blk + b * 1024 + (tg * 16 + (e & 15)) * 16 + ((e >> 4) & 1) * 8 + ti;
        if (scatter) { c0[0] = (uint8_t)(out[gid] & 0xff); c0[16] = (uint8_t)(out[gid] >> 8); }
        else out[gid] = (uint16_t)(c0[0] | (c0[16] << 8));
    }
}

// The Q4_0 pool: one 16-bit unit per thread - four codes (elements 4u .. 4u + 3 of the head's row, element 2 k in
// the low nibble of byte k) or, past the codes, one block scale. Rows of kv_row_halves units. Scattered codes
// replace their nibbles atomically: the words they sit in hold other elements (K) or other tokens (V) as well.
__global__ void k_kv_gather_q4(const __half * pool, KvStrides st, int n_kv, int hd, int is_v, const int32_t * cells, int n,
                               uint16_t * out, int scatter) {
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int per_head = hd / 4 + hd / 32;
    if (gid >= (size_t)n * n_kv * per_head) return;
    const int idx = (int)(gid / ((size_t)n_kv * per_head)), rest = (int)(gid % ((size_t)n_kv * per_head));
    const int kvh = rest / per_head, u = rest % per_head;
    const int cell = cells[idx];
    const int page = cell / PAGE, t32 = cell % PAGE;
    uint8_t * blk = (uint8_t *)(const_cast<__half *>(pool) + (size_t)page * st.page + (size_t)kvh * st.head);
    const int tg = (t32 & 15) >> 2, ti = (t32 & 3) + 4 * (t32 >> 4);
    if (u >= hd / 4) {
        uint16_t * sc = (uint16_t *)(blk + (hd / 32) * 512) + (u - hd / 4) * 32 + tg * 8 + ti;
        if (scatter) *sc = out[gid]; else out[gid] = *sc;
        return;
    }
    const int e0 = 4 * u, b = e0 >> 5;
    uint32_t unit = scatter ? out[gid] : 0;
    for (int k = 0; k < 4; ++k) {
        const int e = e0 + k;
        uint32_t * word;
        int sh;
        if (!is_v) {
            word = (uint32_t *)(blk + b * 512 + (((e >> 3) & 3) * 16 + (t32 & 15)) * 8 + (t32 >> 4) * 4);
            sh = 4 * kv_nibble(e & 7);
        } else {
            word = (uint32_t *)(blk + b * 512 + (tg * 16 + (e & 15)) * 8 + ((e >> 4) & 1) * 4);
            sh = 4 * kv_nibble(ti);
        }
        if (scatter) {
            atomicAnd(word, ~(0xfu << sh));
            atomicOr(word, ((unit >> (4 * k)) & 0xfu) << sh);
        } else {
            unit |= ((*word >> sh) & 0xfu) << (4 * k);
        }
    }
    if (!scatter) out[gid] = (uint16_t)unit;
}

void kv_gather(hipStream_t s, const __half * pool, KvStrides st, int n_kv_heads, int head_dim, bool is_v,
               const int32_t * cells, int n, __half * out, int kvq) {
    if (n <= 0) return;
    if (kvq == KV_Q8 || kvq == KV_Q4) {
        const size_t total = (size_t)n * kv_row_halves(n_kv_heads, head_dim, kvq);
        hipLaunchKernelGGL(kvq == KV_Q8 ? k_kv_gather_q8 : k_kv_gather_q4, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s,
                           pool, st, n_kv_heads, head_dim, is_v ? 1 : 0, cells, n, (uint16_t *)out, 0);
        check_launch("kv_gather");
        return;
    }
    if (kvq != KV_F16) throw std::runtime_error("kv_gather: unknown cache type");
    const size_t total = (size_t)n * n_kv_heads * head_dim;
    hipLaunchKernelGGL(k_kv_gather, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, pool, st, n_kv_heads,
                       head_dim, is_v ? 1 : 0, cells, n, out, 0);
    check_launch("kv_gather");
}

void kv_scatter(hipStream_t s, __half * pool, KvStrides st, int n_kv_heads, int head_dim, bool is_v,
                const int32_t * cells, int n, const __half * in, int kvq) {
    if (n <= 0) return;
    if (kvq == KV_Q8 || kvq == KV_Q4) {
        const size_t total = (size_t)n * kv_row_halves(n_kv_heads, head_dim, kvq);
        hipLaunchKernelGGL(kvq == KV_Q8 ? k_kv_gather_q8 : k_kv_gather_q4, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s,
                           pool, st, n_kv_heads, head_dim, is_v ? 1 : 0, cells, n, (uint16_t *)const_cast<__half *>(in), 1);
        check_launch("kv_scatter");
        return;
    }
    if (kvq != KV_F16) throw std::runtime_error("kv_scatter: unknown cache type");
    const size_t total = (size_t)n * n_kv_heads * head_dim;
    hipLaunchKernelGGL(k_kv_gather, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, pool, st, n_kv_heads,
                       head_dim, is_v ? 1 : 0, cells, n, const_cast<__half *>(in), 1);
    check_launch("kv_scatter");
}

__global__ void k_kv_copy_page(__half * k_pool, __half * v_pool, size_t head_halves, KvStrides st, int src, int dst) {
    const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (i >= head_halves) return;
    const size_t from = (size_t)src * st.page + (size_t)blockIdx.y * st.head + i;
    const size_t to = (size_t)dst * st.page + (size_t)blockIdx.y * st.head + i;
    *(u4 *)(k_pool + to) = *(const u4 *)(k_pool + from);
    *(u4 *)(v_pool + to) = *(const u4 *)(v_pool + from);
}

void kv_copy_page(hipStream_t s, __half * k_pool, __half * v_pool, KvStrides st, int n_kv_heads, int head_dim,
                  int src_page, int dst_page, int kvq) {
    const size_t head_halves = kv_block_halves(head_dim, kvq);       // one head's share of a page (a multiple of 8)
    hipLaunchKernelGGL(k_kv_copy_page, dim3((unsigned)((head_halves / 8 + 255) / 256), n_kv_heads), dim3(256), 0, s,
                       k_pool, v_pool, head_halves, st, src_page, dst_page);
    check_launch("kv_copy_page");
}

// ---------------------------------------------------------------------------
// sampling preparation

// (value desc, id asc) order on (float, int) pairs
__device__ __forceinline__ bool better(float va, int ia, float vb, int ib) {
    return va > vb || (va == vb && ia < ib);
}

__global__ __launch_bounds__(1024) void k_sample_prepare(const float * __restrict__ logits, int V,
                                                         const int32_t * __restrict__ kreq, SampleOut * out) {
    __shared__ float s_val[16];
    __shared__ int s_idx[16];
    __shared__ double s_sum[16];
    __shared__ float b_val;
    __shared__ int b_idx;
    const int row = blockIdx.x;
    const float * l = logits + (size_t)row * V;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int k = min(kreq ? kreq[row] : 0, MAX_TOPK);
    float prev_v = INFINITY;
    int prev_i = -1;
    float row_max = 0.0f;
    // selection 0 is the argmax; each later selection is the best entry
    // strictly after the previous one in (value desc, id asc) order
    // one selection more than asked for when k > 1: an entry right behind the k-th with the k-th's value means
    // the cut falls inside a run of equal logits, where which of them survive is the host algorithm's business
    const int n_sel = k > 1 ? k + 1 : 1;
    for (int sel = 0; sel < n_sel; ++sel) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
        for (int i = threadIdx.x; i < V; i += 1024) {
            const float v = l[i];
            const bool after_prev = sel == 0 || better(prev_v, prev_i, v, i);
            if (after_prev && better(v, i, bv, bi)) { bv = v; bi = i; }
        }
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o, 64);
            const int oi = __shfl_xor(bi, o, 64);
            if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
        }
        if (lane == 0) { s_val[wave] = bv; s_idx[wave] = bi; }
        __syncthreads();
        if (threadIdx.x == 0) {
            float fv = s_val[0];
            int fi = s_idx[0];
            for (int w = 1; w < 16; ++w) if (better(s_val[w], s_idx[w], fv, fi)) { fv = s_val[w]; fi = s_idx[w]; }
            b_val = fv;
            b_idx = fi;
            if (sel == 0) { out[row].argmax = fi; out[row].max = fv; out[row].edge_tie = 0; }
            if (sel < k) { out[row].top_id[sel] = fi; out[row].top_logit[sel] = fv; }
            else if (sel > 0) out[row].edge_tie = (fi != 0x7fffffff && fv == prev_v) ? 1 : 0;
        }
        __syncthreads();
        prev_v = b_val;
        prev_i = b_idx;
        if (sel == 0) row_max = b_val;
        __syncthreads();
    }
    double acc = 0.0;
    for (int i = threadIdx.x; i < V; i += 1024) acc += exp((double)l[i] - (double)row_max);
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
    if (lane == 0) s_sum[wave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double total = 0.0;
        for (int w = 0; w < 16; ++w) total += s_sum[w];
        out[row].sum_exp = total;
    }
}

// Rows that ask for at most one candidate: the vocabulary is cut into slices, one workgroup each, so that a
// 64-row step fills the chip instead of 64 compute units. A slice leaves its best entry and the sum of
// exp(double(logit) - its own maximum); the merge rescales the sums to the row maximum.
struct SamplePartial { float max; int32_t idx; double sum; };

__global__ __launch_bounds__(256) void k_sample_slices(const float * __restrict__ logits, int V, int len,
                                                       SamplePartial * __restrict__ part) {
    __shared__ float s_val[4];
    __shared__ int s_idx[4];
    __shared__ double s_sum[4];
    __shared__ float b_val;
    const int row = blockIdx.x, slice = blockIdx.y, n_slices = gridDim.y;
    const int lo = slice * len, hi = min(V, lo + len);
    const float * l = logits + (size_t)row * V;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = lo + threadIdx.x; i < hi; i += 256) {
        const float v = l[i];
        if (better(v, i, bv, bi)) { bv = v; bi = i; }
    }
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, 64);
        const int oi = __shfl_xor(bi, o, 64);
        if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
    if (lane == 0) { s_val[wave] = bv; s_idx[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        float fv = s_val[0];
        int fi = s_idx[0];
        for (int w = 1; w < 4; ++w) if (better(s_val[w], s_idx[w], fv, fi)) { fv = s_val[w]; fi = s_idx[w]; }
        b_val = fv;
        part[(size_t)row * n_slices + slice].max = fv;
        part[(size_t)row * n_slices + slice].idx = fi;
    }
    __syncthreads();
    const float slice_max = b_val;
    double acc = 0.0;
    // a slice whose logits are all -inf adds nothing (exp(-inf - -inf) would be a NaN that the merge multiplies by 0)
    if (slice_max != -INFINITY)
        for (int i = lo + threadIdx.x; i < hi; i += 256) acc += exp((double)l[i] - (double)slice_max);
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
    if (lane == 0) s_sum[wave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) part[(size_t)row * n_slices + slice].sum = (s_sum[0] + s_sum[1]) + (s_sum[2] + s_sum[3]);
}

__global__ __launch_bounds__(64) void k_sample_merge(const SamplePartial * __restrict__ part, int n_slices,
                                                     const int32_t * __restrict__ kreq, SampleOut * out) {
    const int row = blockIdx.x;
    if (threadIdx.x != 0) return;
    const SamplePartial * p = part + (size_t)row * n_slices;
    float fv = -INFINITY;
    int fi = 0x7fffffff;
    for (int s = 0; s < n_slices; ++s)
        if (p[s].idx != 0x7fffffff && better(p[s].max, p[s].idx, fv, fi)) { fv = p[s].max; fi = p[s].idx; }
    double total = 0.0;
    for (int s = 0; s < n_slices; ++s)
        if (p[s].idx != 0x7fffffff && p[s].max != -INFINITY) total += p[s].sum * exp((double)p[s].max - (double)fv);
    out[row].argmax = fi;
    out[row].max = fv;
    out[row].sum_exp = total;
    out[row].edge_tie = 0;
    if (kreq && kreq[row] >= 1) { out[row].top_id[0] = fi; out[row].top_logit[0] = fv; }
}

size_t sample_scratch_bytes(int n_rows) { return (size_t)std::max(n_rows, 1) * 32 * sizeof(SamplePartial); }

// Slices per row of the sliced scan: as many as keep about a thousand workgroups in flight, at most 32.
static int sample_slices_for(int n_rows) {
    int n_slices = 1;
    while (n_slices < 32 && n_rows * n_slices * 2 <= 1024) n_slices *= 2;
    return n_slices;
}

// ---- the greedy scan for callers that cannot allocate ---------------------------------------------
// The slice partials of k_sample_slices / the merge live in this file-scope device array instead of a
// buffer the library allocates. Every GPU the library runs on holds its own copy at its own address until
// the process ends; host code never uses the array's name as an address, only what hipGetSymbolAddress
// returned for the device that is current.
constexpr int SAMPLE_STATIC_MAX_ROWS = 4096;
constexpr size_t SAMPLE_STATIC_PARTIALS = SAMPLE_STATIC_MAX_ROWS;      // rows * slices never exceeds max(rows, 1024): see sample_slices_for
static __device__ __align__(256) unsigned char scratch[SAMPLE_STATIC_PARTIALS * sizeof(SamplePartial)];

int sample_static_max_rows() { return SAMPLE_STATIC_MAX_ROWS; }

// The address of `scratch` on the current device, looked up once per device: at engine creation
// (sample_static_prepare) or, in a process that creates no engine, by the first call - which must then be made
// outside stream capture, since the lookup may load the code object.
static void * sample_static_scratch() {
    constexpr int MAX_DEVICES = 64;
    static std::mutex lock;
    static void * ptr_of[MAX_DEVICES] = {};
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) throw std::runtime_error(std::string("hipGetDevice: ") + hipGetErrorString(e));
    if (dev < 0 || dev >= MAX_DEVICES) throw std::runtime_error("sample_greedy_static: device index out of range");
    std::lock_guard<std::mutex> hold(lock);
    if (!ptr_of[dev]) {
        void * ptr = nullptr;
        e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            throw std::runtime_error(std::string("hipGetSymbolAddress(scratch): ") + hipGetErrorString(e));
        ptr_of[dev] = ptr;
    }
    return ptr_of[dev];
}

void sample_static_prepare() { (void)sample_static_scratch(); }

__global__ __launch_bounds__(64) void k_sample_merge_arrays(const SamplePartial * __restrict__ part, int n_slices,
                                                            int32_t * __restrict__ out_argmax, float * __restrict__ out_max,
                                                            double * __restrict__ out_sum) {
    const int row = blockIdx.x;
    if (threadIdx.x != 0) return;
    const SamplePartial * p = part + (size_t)row * n_slices;
    float fv = -INFINITY;
    int fi = 0x7fffffff;
    for (int s = 0; s < n_slices; ++s)
        if (p[s].idx != 0x7fffffff && better(p[s].max, p[s].idx, fv, fi)) { fv = p[s].max; fi = p[s].idx; }
    double total = 0.0;
    for (int s = 0; s < n_slices; ++s)
        if (p[s].idx != 0x7fffffff && p[s].max != -INFINITY) total += p[s].sum * exp((double)p[s].max - (double)fv);
    out_argmax[row] = fi;
    out_max[row] = fv;
    out_sum[row] = total;
}

// argmax (lowest id on ties), max and sum exp(double(logit) - max) per row, all pointers device memory of the
// caller, the launches on the caller's stream; no allocation, no synchronisation. Every (row, slice) partial is
// written by its own workgroup before the merge reads it, so the array needs no clearing between calls; two
// calls that overlap on one GPU (different streams, or threads) race on it.
void sample_greedy_static(hipStream_t s, const float * logits, int n_rows, int n_vocab, int32_t * out_argmax,
                          float * out_max, double * out_sum) {
    if (n_rows <= 0 || n_rows > SAMPLE_STATIC_MAX_ROWS)
        throw std::runtime_error("sample_greedy_static: between 1 and " + std::to_string(SAMPLE_STATIC_MAX_ROWS)
                                 + " rows per call (the static scratch array holds no more), got " + std::to_string(n_rows));
    if (n_vocab <= 0) throw std::runtime_error("sample_greedy_static: the vocabulary must not be empty");
    if (!logits || !out_argmax || !out_max || !out_sum) throw std::runtime_error("sample_greedy_static: null pointer");
    const int n_slices = sample_slices_for(n_rows);
    if ((size_t)n_rows * n_slices > SAMPLE_STATIC_PARTIALS)
        throw std::runtime_error("sample_greedy_static: internal error, partials exceed the static scratch array");
    SamplePartial * part = (SamplePartial *)sample_static_scratch();
    const int len = ((n_vocab + n_slices - 1) / n_slices + 3) & ~3;
    hipLaunchKernelGGL(k_sample_slices, dim3(n_rows, n_slices), dim3(256), 0, s, logits, n_vocab, len, part);
    check_launch("sample_slices");
    hipLaunchKernelGGL(k_sample_merge_arrays, dim3(n_rows), dim3(64), 0, s, (const SamplePartial *)part, n_slices,
                       out_argmax, out_max, out_sum);
    check_launch("sample_merge_arrays");
}

void sample_prepare(hipStream_t s, const float * logits, int n_rows, int n_vocab, const int32_t * k,
                    SampleOut * out, int max_k, void * scratch) {
    if (n_rows <= 0) return;
    if (max_k <= 1 && scratch && n_vocab >= 8192) {
        const int n_slices = sample_slices_for(n_rows);
        const int len = ((n_vocab + n_slices - 1) / n_slices + 3) & ~3;
        hipLaunchKernelGGL(k_sample_slices, dim3(n_rows, n_slices), dim3(256), 0, s, logits, n_vocab, len, (SamplePartial *)scratch);
        check_launch("sample_slices");
        hipLaunchKernelGGL(k_sample_merge, dim3(n_rows), dim3(64), 0, s, (const SamplePartial *)scratch, n_slices, k, out);
        check_launch("sample_merge");
        return;
    }
    hipLaunchKernelGGL(k_sample_prepare, dim3(n_rows), dim3(1024), 0, s, logits, n_vocab, k, out);
    check_launch("sample_prepare");
}

}  // namespace rk
