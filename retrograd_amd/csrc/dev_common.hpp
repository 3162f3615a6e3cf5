// Device-side helpers shared by the kernel translation units.
#pragma once

#include "kernels.hpp"

#include <stdexcept>
#include <string>

namespace rk {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));

#define HIP_OK(expr)                                                                        \
    do {                                                                                    \
        hipError_t err__ = (expr);                                                          \
        if (err__ != hipSuccess)                                                            \
            throw std::runtime_error(std::string("HIP error: ") + hipGetErrorString(err__)  \
                                     + " at " #expr);                                       \
    } while (0)

static inline void check_launch(const char * what) {
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        throw std::runtime_error(std::string("kernel launch failed (") + what + "): " + hipGetErrorString(err));
}

__device__ __forceinline__ float h2f(uint16_t bits) {
    return __half2float(__ushort_as_half(bits));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// f32 -> f16 with saturation, so nothing non-finite is ever stored.
__device__ __forceinline__ __half sat_half(float v) {
    v = fminf(fmaxf(v, -65504.0f), 65504.0f);
    return __float2half_rn(v);
}

__device__ __forceinline__ h8 load_h8(const __half * p) {
    return *(const h8 *)p;
}

// Arguments of the tile matmuls.
// Index, in halves, of element (token, k, hi/lo) of an operand-order activation buffer.
__device__ __forceinline__ size_t act_chunk_halves(int K) { return (size_t)((K + 31) & ~31) * 128; }
__device__ __forceinline__ size_t act_at(int tok, int k, int hl, int K) {
    return (size_t)(tok >> 6) * act_chunk_halves(K) + (size_t)(((k >> 5) * 2 + hl) * 4 + ((tok >> 4) & 3)) * 512
         + ((((k >> 3) & 3) * 16 + (tok & 15)) * 8) + (k & 7);
}
// ... and of the hi/lo sum of 32-wide block `blk` of a token.
__device__ __forceinline__ size_t act_sum_chunk_halves(int K) { return (size_t)((K + 255) >> 8) * 2048; }
__device__ __forceinline__ size_t act_sum_at(int tok, int blk, int hl, int K) {
    return (size_t)(tok >> 6) * act_sum_chunk_halves(K) + (size_t)((blk >> 3) * 4 + ((tok >> 4) & 3)) * 512
         + ((hl * 16 + (tok & 15)) * 8) + (blk & 7);
}

// Scales and mins of the eight sub-blocks of a Q4_K super-block, one value per
// byte (sc[0] = sub-blocks 0-3, sc[1] = 4-7, likewise mn), from a row's tile
// header: word 0 is d | dmin << 16; the bytes of words 1, 2, 3 hold sc0-3, sc4-7
// and mn0-3 in their low six bits, and the top two bits of byte j of the three
// words are bits 0-1, 2-3 and 4-5 of mn(4+j).
struct Q4KScales { uint32_t sc[2]; uint32_t mn[2]; };
__device__ __forceinline__ Q4KScales q4k_scales(const u4 & hdr) {
    Q4KScales s;
    s.sc[0] = hdr.y & 0x3f3f3f3fu;
    s.sc[1] = hdr.z & 0x3f3f3f3fu;
    s.mn[0] = hdr.w & 0x3f3f3f3fu;
    s.mn[1] = ((hdr.y >> 6) & 0x03030303u) | ((hdr.z >> 4) & 0x0c0c0c0cu) | ((hdr.w >> 2) & 0x30303030u);
    return s;
}

// The conversion ggml's CPU matmul applies to an activation row before the dot
// product, on eight consecutive values per lane. The lanes that share a block
// (4 for the 32-wide Q8_0 blocks, 32 for the 256-wide Q8_K blocks) must be
// consecutive, aligned to the group size, hold consecutive pieces of one row
// and all be here. Returns the values the codes stand for, scale times code.
//   Q8_0: d = amax / 127, code = roundf(v / d) with the unrounded d (half away
//         from zero), value = f16(d) * code.
//   Q8_K: `max` = the first value of largest magnitude, iscale = -127 / max,
//         code = min(127, rint(iscale * v)) (half to even), value = code / iscale.
// With `codes` the integer codes are returned as well; the function's value is the block scale (Q8_K: 1 / iscale,
// 0 for a block of zeros; Q8_0: d rounded to f16).
__device__ __forceinline__ float requantise8(float (&v)[8], int quant, float * codes = nullptr) {
    float amax = 0.0f, first = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float ax = fabsf(v[i]);
        if (ax > amax) { amax = ax; first = v[i]; }
    }
    if (quant == AQ_Q8_0) {
        amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
        amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
        const float d = __fdiv_rn(amax, 127.0f);
        const float id = d != 0.0f ? __fdiv_rn(1.0f, d) : 0.0f;
        const float dh = (float)(_Float16)d;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float c = roundf(__fmul_rn(v[i], id));
            if (codes) codes[i] = c;
            v[i] = __fmul_rn(dh, c);
        }
        return dh;
    }
    float gmax = amax;
#pragma unroll
    for (int o = 1; o < 32; o <<= 1) gmax = fmaxf(gmax, __shfl_xor(gmax, o, 64));
    // the lowest lane of the group that holds the extreme has the first occurrence
    const int lane = __lane_id();
    const uint64_t holders = __ballot(amax == gmax);
    const uint32_t in_group = (uint32_t)(holders >> (lane & 32));
    const float max = __shfl(first, (lane & 32) + __ffs((int)in_group) - 1, 64);
    if (gmax == 0.0f) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = 0.0f;
        if (codes) {
#pragma unroll
            for (int i = 0; i < 8; ++i) codes[i] = 0.0f;
        }
        return 0.0f;
    }
    const float iscale = __fdiv_rn(-127.0f, max);
    const float d = __fdiv_rn(1.0f, iscale);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float c = fminf(127.0f, rintf(__fmul_rn(iscale, v[i])));
        if (codes) codes[i] = c;
        v[i] = __fmul_rn(d, c);
    }
    return d;
}

// The codes of eight consecutive values (k a multiple of 8) into the buffers of the integer matrix-vector kernel
// (Act::qc, qd, qbs). Q8_K: 8 bytes in the order of act_code_pos, the sum of every 16 codes from their two lanes (ggml's
// Q8_K bsums), the block scale from the lane that holds the block's first values. Q8_0: 8 bytes in element order, the scale of the
// 32-wide block from its first lane.
__device__ __forceinline__ void store_codes8(const float (&c)[8], float d, const Act & out, int tok, int k, int lane_in_block) {
    uint32_t w0 = 0, w1 = 0;
    int sum = 0;
    const bool natural = out.quant == AQ_Q8_0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int q = (int)c[i];
        sum += q;
        const uint32_t byte = (uint32_t)q & 0xffu;
        const int pos = natural ? i : act_code_pos(i);
        if (pos < 4) w0 |= byte << (8 * pos); else w1 |= byte << (8 * (pos - 4));
    }
    *(uint2 *)(out.qc + (size_t)tok * out.K + k) = make_uint2(w0, w1);
    if (natural) {
        if (lane_in_block == 0) out.qd[(size_t)tok * (out.K >> 5) + (k >> 5)] = d;
        return;
    }
    sum += __shfl_xor(sum, 1, 64);
    if ((lane_in_block & 1) == 0) out.qbs[(size_t)tok * (out.K >> 4) + (k >> 4)] = (int16_t)sum;
    if ((k & 255) == 0) out.qd[(size_t)tok * (out.K >> 8) + (k >> 8)] = d;
}

// Eight consecutive values per lane (k a multiple of 8) into one pair of planes:
// hi/lo as two 16-byte stores; the four lanes that own one 32-wide block add
// their sums with two xor-shuffles.
__device__ __forceinline__ void store_act8_planes(const float (&v)[8], __half * x, __half * sums, int K,
                                                  int tok, int k, int lane_in_block) {
    h8 a, b;
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float c = fminf(fmaxf(v[i], -65504.0f), 65504.0f);
        const _Float16 h = (_Float16)c;
        const _Float16 l = (_Float16)(c - (float)h);
        a[i] = h;
        b[i] = l;
        sum += (float)h + (float)l;
    }
    *(h8 *)(x + act_at(tok, k, 0, K)) = a;
    *(h8 *)(x + act_at(tok, k, 1, K)) = b;
    if (sums) {
        sum += __shfl_xor(sum, 1, 64);
        sum += __shfl_xor(sum, 2, 64);
        if (lane_in_block == 0) {
            const __half s = sat_half(sum);
            sums[act_sum_at(tok, k >> 5, 0, K)] = s;
            sums[act_sum_at(tok, k >> 5, 1, K)] = __float2half_rn(sum - __half2float(s));
        }
    }
}

// Writes the versions of the row that `out` asks for: the values themselves
// and / or their conversion (see requantise8 for what the lanes must satisfy).
__device__ __forceinline__ void store_act8(const float (&v)[8], const Act & out, int tok, int k, int lane_in_block) {
    if (out.x) store_act8_planes(v, out.x, out.sums, out.K, tok, k, lane_in_block);
    if (out.qx) {
        float q[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = v[i];
        if (out.qc) {
            float c[8];
            const float d = requantise8(q, out.quant, c);
            store_codes8(c, d, out, tok, k, lane_in_block);
        } else {
            requantise8(q, out.quant);
        }
        store_act8_planes(q, out.qx, out.qsums, out.K, tok, k, lane_in_block);
    }
}

// A direct-to-LDS request issued from inline assembly. The compiler's own wait
// insertion cannot tell which staging buffer an LDS read touches, so with the
// builtin it waits for every request (and, loads retiring in order, for every
// weight load before it) ahead of each barrier: s_waitcnt vmcnt(0) per
// super-block, the whole latency of the weight prefetch exposed. Requests it
// does not see leave only the waits written in the kernels. M0 carries the LDS
// address. base is wave-uniform; every lane adds its own byte offset.
__device__ __forceinline__ void lds_dma16(const void * base, uint32_t lane_off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(lane_off), "s"(base), "s"(lds_addr) : "memory");
}
__device__ __forceinline__ uint32_t lds_offset(const void * p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) uint8_t *)p;
}

struct MMArgs {
    const uint8_t * w;
    const __half * x;         // operand-order activations and block sums (see Act)
    const __half * sums;
    float * y;
    const float * bias;
    int K, N, T, ldy, col0, mode;
    int n_row_tiles;
    int ksplit;       // v1: waves of a workgroup sharing a row tile along K; v2: workgroups sharing a row group
    // v2 only
    int n_row_groups;
    float * partial;          // [ksplit][slice_rows][pld] K-slices of a split matmul; this matrix fills columns pcol .. pcol + N
    int pld, pcol;            // (pld = N, pcol = 0 unless several matrices share the slices)
    int slice_rows;           // token rows of a slice: 64 per chunk of the step
    // mode MM_SWIGLU: rows come in groups of 128, 64 gate rows then the 64 up rows of the same
    // columns; the epilogue writes silu(gate) * up as the activations of the next matmul
    Act act_out;
    float * act_f32;          // instead of act_out: the products as f32 rows of act_out.K (when the next matmul's
                              // conversion needs blocks wider than the 64 columns a workgroup holds)
};

}  // namespace rk
