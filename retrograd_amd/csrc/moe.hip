// Mixture-of-experts feed-forward (qwen3moe): softmax router, top-k experts with
// renormalised weights, SwiGLU experts with MXFP4 or Q8_0 weights.
//
// The expert weights dominate the bytes of a step (all experts are touched once
// a batch has a few dozen tokens), so the work is organised by expert: the
// (token, choice) pairs of a step are grouped by expert, every expert's range
// padded to whole 16-token MFMA tiles, and one wave owns one 16-row weight tile
// of one expert and streams it exactly once per 32 tokens of that expert; the
// four waves of a workgroup own four tiles of the same expert and share its
// activations through LDS (read from global memory per wave they cost several
// times the bytes of the weights):
//
//   k_moe_route     per token: top-k of the router logits, weights in double
//   k_moe_group     stable counting sort of the pairs by expert (one workgroup)
//   k_moe_gate_up   h[q][f] = silu(gate_e x) * (up_e x)       q = slot of a pair
//   k_moe_down      out[q][:] = down_e h[q]
//   k_moe_combine   x[t] += sum_j w[t][j] * out[q(t, j)]       in choice order (in the engine's steps the next
//                   RMSNorm launch adds this sum instead: k_moe_down leaves its rows in pair order for it)
//
// Expert tensors [K][N][n_expert] are tiled as one matrix of n_expert * N rows.
// MXFP4 tile (16 rows x 256 columns, 2176 B = the GGUF byte count): 16 x 8 E8M0
// scale bytes, then two 1 KiB loads; lane (r = l % 16, g = l / 16) of load h
// holds one dword per k-step 4h + j: byte b of it carries element 8g + 2b in its
// low nibble and element 8g + 2b + 1 in its high nibble, the order in which
// v_cvt_scalef32_pk_f16_fp4 turns a byte into two f16 numbers (exactly; with the
// factor 2 they are the doubled E2M1 magnitudes 0 1 2 3 4 6 8 12 that ggml's
// half scale multiplies): four instructions decode a lane's eight weights.
#include "dev_common.hpp"

namespace rk {

bool moe_can_pack(int type, int64_t K, int64_t N) {
    return (type == WT_MXFP4 || type == WT_Q8_0 || type == WT_Q4_K || type == WT_Q5_K || type == WT_Q6_K) && K % 256 == 0 && N % 16 == 0 && K > 0 && N > 0;
}

__global__ void k_repack_mxfp4(const uint8_t * __restrict__ raw, uint8_t * __restrict__ dst, int nsb, size_t n_tiles) {
    // one thread per output dword: 544 per (tile, super-block): 32 header + 512 payload
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t total = n_tiles * (size_t)nsb * 544;
    if (gid >= total) return;
    const int w = (int)(gid % 544);
    const size_t ts = gid / 544;
    const int sb = (int)(ts % nsb);
    const size_t rt = ts / nsb;
    const size_t row_bytes = (size_t)nsb * 8 * 17;
    uint32_t out = 0;
    if (w < 32) {                       // row r, scales of blocks 4*half .. +3
        const int r = w >> 1, half = w & 1;
        const uint8_t * row = raw + (rt * 16 + r) * row_bytes + (size_t)sb * 8 * 17;
        for (int i = 0; i < 4; ++i) out |= (uint32_t)row[(size_t)(4 * half + i) * 17] << (8 * i);
    } else {
        const int v = w - 32;
        const int h = v >> 8, lane = (v >> 2) & 63, j = v & 3;
        const int r = lane & 15, g = lane >> 4;
        const uint8_t * blk = raw + (rt * 16 + r) * row_bytes + (size_t)(sb * 8 + 4 * h + j) * 17;
        auto elem = [&](int e) -> uint32_t {
            const uint8_t byte = blk[1 + (e & 15)];
            return e < 16 ? (byte & 0x0f) : (byte >> 4);
        };
        for (int b = 0; b < 4; ++b) out |= (elem(8 * g + 2 * b) | (elem(8 * g + 2 * b + 1) << 4)) << (8 * b);
    }
    *(uint32_t *)(dst + ts * 2176 + (size_t)w * 4) = out;
}

void moe_repack(hipStream_t s, int type, const uint8_t * raw, uint8_t * packed, int K, int64_t n_rows) {
    if (!moe_can_pack(type, K, n_rows)) throw std::runtime_error("moe_repack: shape or type has no tile layout");
    if (type != WT_MXFP4) {
        // the dense tile layouts (Q8_0, Q4_K, Q6_K), in slabs the dense repack's 32-bit sizes can hold
        const int64_t slab = 1 << 20;
        for (int64_t r0 = 0; r0 < n_rows; r0 += slab) {
            const int64_t n = std::min(slab, n_rows - r0);
            const size_t off = (size_t)r0 * row_bytes(type, K);
            repack(s, type, raw + off, packed + off, K, (int)n);
        }
        return;
    }
    const int nsb = K / 256;
    const size_t n_tiles = (size_t)n_rows / 16;
    const size_t total = n_tiles * (size_t)nsb * 544;
    hipLaunchKernelGGL(k_repack_mxfp4, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, raw, packed, nsb, n_tiles);
    check_launch("moe_repack");
}

namespace {

template <int TYPE> struct Tile;

// What a tile contributes per 32-wide step: the weight operand(s) and the factors applied after the products.
// prep(s) decodes once per step, mac() multiplies one token tile (hi and lo halves) and adds into acc.
struct ScaledOperand { h8 b; float d; };

__device__ __forceinline__ f4 mfma2(const h8 & a_hi, const h8 & a_lo, const h8 & b);

__device__ __forceinline__ void mac(const ScaledOperand & o, const h8 & hi, const h8 & lo, f4 & acc) {
    const f4 p = mfma2(hi, lo, o.b);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = fmaf(o.d, p[i], acc[i]);
}

template <> struct Tile<WT_MXFP4> {
    static constexpr int BYTES = 2176;
    uint2 hdr;
    u4 q0, q1;
    __device__ __forceinline__ void load(const uint8_t * tile, int lane) {
        hdr = *(const uint2 *)(tile + (lane & 15) * 8);
        q0 = *(const u4 *)(tile + 128 + lane * 16);
        q1 = *(const u4 *)(tile + 128 + 1024 + lane * 16);
    }
    // half of 2^(x - 127): the E8M0 scale of doubled magnitudes
    __device__ __forceinline__ float scale(int s) const {
        const uint32_t x = ((s < 4 ? hdr.x : hdr.y) >> (8 * (s & 3))) & 0xff;
        return __builtin_ldexpf(0.5f, (int)x - 127);      // one instruction; exponents 0 and 1 give the subnormals 2^-128, 2^-127
    }
    __device__ __forceinline__ h8 frag(int s) const {
        const uint32_t w = s < 4 ? q0[s & 3] : q1[s & 3];
        // byte b: (low nibble, high nibble) -> the doubled magnitudes of elements 2b, 2b + 1
        const h2 p0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 2.0f, 0);
        const h2 p1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 2.0f, 1);
        const h2 p2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 2.0f, 2);
        const h2 p3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 2.0f, 3);
        return (h8){p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
    }
    __device__ __forceinline__ ScaledOperand prep(int s) const { return {frag(s), scale(s)}; }
};

template <> struct Tile<WT_Q8_0> {
    static constexpr int BYTES = 4352;
    u4 hdr;
    u4 q[4];
    __device__ __forceinline__ void load(const uint8_t * tile, int lane) {
        hdr = *(const u4 *)(tile + (lane & 15) * 16);
#pragma unroll
        for (int j = 0; j < 4; ++j) q[j] = *(const u4 *)(tile + 256 + j * 1024 + lane * 16);
    }
    __device__ __forceinline__ float scale(int s) const {
        const uint32_t sw = hdr[s >> 1];
        return h2f((uint16_t)((s & 1) ? (sw >> 16) : (sw & 0xffff)));
    }
    __device__ __forceinline__ h8 frag(int s) const {
        const u4 d4 = q[s >> 1];
        const int half = s & 1;
        const uint32_t w0 = d4[2 * half] ^ 0x80808080u, w1 = d4[2 * half + 1] ^ 0x80808080u;
        const h2 bias = {(_Float16)(-1152.0f), (_Float16)(-1152.0f)};
        const h2 a0 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w0, 0x04010400u)) + bias;
        const h2 a1 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w0, 0x04030402u)) + bias;
        const h2 a2 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w1, 0x04010400u)) + bias;
        const h2 a3 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w1, 0x04030402u)) + bias;
        return (h8){a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
    }
    __device__ __forceinline__ ScaledOperand prep(int s) const { return {frag(s), scale(s)}; }
};

__device__ __forceinline__ f4 mfma2(const h8 & a_hi, const h8 & a_lo, const h8 & b) {
    f4 p = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_hi, b, (f4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a_lo, b, p, 0, 0, 0);
}

__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t bits) { return (x & mask) | bits; }

// Q4_K, the dense tile (2304 bytes): value = d * sc * e - dmin * m per 32-wide sub-block. sc * e goes into the
// operand as an exact f16 (at most 945); the min term needs the sum of the activations of the sub-block, which a
// product with an operand of ones supplies for every token of the tile.
struct Q4KOperand { h8 b; float d, dm; };
__device__ __forceinline__ void mac(const Q4KOperand & o, const h8 & hi, const h8 & lo, f4 & acc) {
    const _Float16 one = (_Float16)1.0f;
    const h8 ones = {one, one, one, one, one, one, one, one};
    const f4 p = mfma2(hi, lo, o.b), sum = mfma2(hi, lo, ones);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = fmaf(-o.dm, sum[i], fmaf(o.d, p[i], acc[i]));
}
// FIVE: Q5_K, the same tile followed by a plane of fifth bits (one dword per k-half and lane).
template <bool FIVE> struct TileQ45 {
    static constexpr int BYTES = FIVE ? 2816 : 2304;
    u4 hdr;
    u4 q0, q1;
    uint32_t top0, top1;
    __device__ __forceinline__ void load(const uint8_t * tile, int lane) {
        hdr = *(const u4 *)(tile + (lane & 15) * 16);
        q0 = *(const u4 *)(tile + 256 + lane * 16);
        q1 = *(const u4 *)(tile + 256 + 1024 + lane * 16);
        top0 = FIVE ? *(const uint32_t *)(tile + 2304 + lane * 4) : 0u;
        top1 = FIVE ? *(const uint32_t *)(tile + 2304 + 256 + lane * 4) : 0u;
    }
    __device__ __forceinline__ Q4KOperand prep(int s) const {
        const Q4KScales s4 = q4k_scales(hdr);
        const int j = s & 3;
        const uint32_t scw = s < 4 ? s4.sc[0] : s4.sc[1], mnw = s < 4 ? s4.mn[0] : s4.mn[1];
        const h2 m1024 = {(_Float16)(-1024.0f), (_Float16)(-1024.0f)};
        // (1024 + sc, 1024 + sc) from byte j, then (sc, sc)
        const h2 k1 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, scw, 0x04000400u + 0x00010001u * j)) + m1024;
        const h2 c1 = k1 * (_Float16)(-1024.0f), c2 = k1 * (_Float16)(-64.0f);
        const uint32_t wq = s < 4 ? q0[j] : q1[j];
        const uint32_t w8 = wq >> 8;
        uint32_t v0 = and_or(wq, 0x000F000Fu, 0x64006400u), v1 = and_or(wq, 0x00F000F0u, 0x54005400u);   // 1024 + e; 64 + e (nibble one place up)
        uint32_t v2 = and_or(w8, 0x000F000Fu, 0x64006400u), v3 = and_or(w8, 0x00F000F0u, 0x54005400u);
        if (FIVE) {
            // fifth bits of this k-step: elements 0, 4 (1, 5) at bits 2j, 2j + 1 (16 + 2j ..) of the plane dword,
            // wanted at bit 4 (20); elements 2, 6 (3, 7) at 8 + 2j .. (24 + 2j ..), wanted at bit 8 (24)
            const uint32_t top = s < 4 ? top0 : top1;
            const uint32_t ta = j < 2 ? top << ((4 - 2 * j) & 31) : top >> ((2 * j - 4) & 31);
            const uint32_t tb = top >> (2 * j);
            v0 = and_or(ta, 0x00100010u, v0);
            v2 = and_or(ta >> 1, 0x00100010u, v2);
            v1 = and_or(tb, 0x01000100u, v1);
            v3 = and_or(tb >> 1, 0x01000100u, v3);
        }
        const h2 u0 = __builtin_bit_cast(h2, v0), u1 = __builtin_bit_cast(h2, v1);
        const h2 u2 = __builtin_bit_cast(h2, v2), u3 = __builtin_bit_cast(h2, v3);
        const h2 a0 = __builtin_elementwise_fma(u0, k1, c1), a1 = __builtin_elementwise_fma(u1, k1, c2);
        const h2 a2 = __builtin_elementwise_fma(u2, k1, c1), a3 = __builtin_elementwise_fma(u3, k1, c2);
        Q4KOperand o;
        o.b = (h8){a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
        o.d = h2f((uint16_t)(hdr.x & 0xffff));
        o.dm = h2f((uint16_t)(hdr.x >> 16)) * (float)((mnw >> (8 * j)) & 0xffu);
        return o;
    }
};

template <> struct Tile<WT_Q4_K> : TileQ45<false> {};
template <> struct Tile<WT_Q5_K> : TileQ45<true> {};

// Q6_K, the dense tile (3360 bytes): value = d * scale * (code - 32) per 16-wide block; the i8 scale goes into the
// operand in two parts whose products with a code are exact f16 numbers (its low four bits, and the rest).
struct Q6KOperand { h8 b_rest, b_low; float d; };
__device__ __forceinline__ void mac(const Q6KOperand & o, const h8 & hi, const h8 & lo, f4 & acc) {
    f4 p = mfma2(hi, lo, o.b_rest);
    p = __builtin_amdgcn_mfma_f32_16x16x32_f16(hi, o.b_low, p, 0, 0, 0);
    p = __builtin_amdgcn_mfma_f32_16x16x32_f16(lo, o.b_low, p, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = fmaf(o.d, p[i], acc[i]);
}
template <> struct Tile<WT_Q6_K> {
    static constexpr int BYTES = 3360;
    u4 sc;
    uint32_t dpair;
    u4 ql0, ql1;
    uint2 qh0, qh1;
    int lane_;
    __device__ __forceinline__ void load(const uint8_t * tile, int lane) {
        lane_ = lane;
        sc = *(const u4 *)(tile + (lane & 15) * 16);
        dpair = *(const uint32_t *)(tile + 256 + ((lane & 15) >> 1) * 4);
        ql0 = *(const u4 *)(tile + 288 + lane * 16);
        ql1 = *(const u4 *)(tile + 288 + 1024 + lane * 16);
        qh0 = *(const uint2 *)(tile + 2336 + lane * 8);
        qh1 = *(const uint2 *)(tile + 2336 + 512 + lane * 8);
    }
    __device__ __forceinline__ Q6KOperand prep(int s) const {
        const int j = s & 3;
        // scale of block 2 s + lane / 32: byte 2 (j & 1) + lane / 32 of scale dword s / 2
        const int scale = __builtin_amdgcn_sbfe((int)sc[s >> 1], 16 * (j & 1) + 8 * (lane_ >> 5), 8);
        const _Float16 s_low = (_Float16)(short)(scale & 15), s_rest = (_Float16)(short)(scale & ~15);
        const h2 k_low = {s_low, s_low}, k_rest = {s_rest, s_rest};
        const uint32_t lo = s < 4 ? ql0[j] : ql1[j];
        const uint32_t pair = s < 4 ? (j < 2 ? qh0.x : qh0.y) : (j < 2 ? qh1.x : qh1.y);
        const uint32_t top = (j & 1) ? __builtin_amdgcn_alignbit(pair, pair, 8) : pair;
        const h2 bias1056 = {(_Float16)(-1056.0f), (_Float16)(-1056.0f)};
        h2 q[4];
#pragma unroll
        for (int p = 0; p < 4; ++p)
            q[p] = __builtin_bit_cast(h2, and_or(top >> (2 * p), 0x00300030u, and_or(lo >> (4 * p), 0x000F000Fu, 0x64006400u))) + bias1056;
        const h2 b0 = q[0] * k_rest, b1 = q[1] * k_rest, b2 = q[2] * k_rest, b3 = q[3] * k_rest;
        const h2 c0 = q[0] * k_low, c1 = q[1] * k_low, c2 = q[2] * k_low, c3 = q[3] * k_low;
        Q6KOperand o;
        o.b_rest = (h8){b0.x, b0.y, b1.x, b1.y, b2.x, b2.y, b3.x, b3.y};
        o.b_low = (h8){c0.x, c0.y, c1.x, c1.y, c2.x, c2.y, c3.x, c3.y};
        o.d = h2f((uint16_t)((lane_ & 1) ? (dpair >> 16) : (dpair & 0xffff)));
        return o;
    }
};

}  // namespace

struct MoeArgs {
    const uint8_t * w0;        // gate (gate_up) or down
    const uint8_t * w1;        // up
    Act x;                     // gate_up: the normalised activations by token; down: h by pair slot
    Act h;                     // gate_up output
    float * out_pair;          // down output [slot][E]
    const int32_t * expert_n;  // pairs per expert
    const int32_t * off_pad;   // first slot of each expert (multiples of 16)
    const int32_t * tok_of_q;  // token of a slot, -1 for padding
    const int32_t * pair_of_q; // down: the output row of a slot (its pair), or null: the slot itself
    int n_expert, K, N;        // N output features per expert, K inputs
};

// The activations of one super-block (256 k) for up to two 16-token tiles, staged once per workgroup: its four
// waves own four row tiles of the same expert and multiply them with the same rows. A tile's share is 8 k-steps
// x (hi, lo) x 64 lanes of 16 bytes, in the order the MFMA operand wants them, so a wave reads its fragments
// back with one conflict-free 16-byte read per lane.
constexpr int kStageTile = 8 * 2 * 64 * 16;        // bytes per token tile and super-block

template <int NTMAX> struct StageRegs { u4 v[4 * NTMAX]; };
// where a thread's 16-byte pieces of super-block 0 lie in the activation buffer (in halves); super-block sb lies
// kStageStep halves further per step
template <int NTMAX> struct StageAt { uint32_t off[4 * NTMAX]; };
constexpr uint32_t kStageStep = 8 * 2 * 4 * 512;

// NTMAX = 1 halves the LDS of a workgroup (more of them per compute unit, more weight bytes in flight) and
// makes an expert with more than 16 pairs stream its weights once per 16 of them: the host picks it for
// decode-sized steps. rows[32]: for every row of the (up to) two tiles, the row of the activation buffer it reads.
template <int NTMAX>
__device__ __forceinline__ void stage_prepare(int K, const int * rows, int nt, StageAt<NTMAX> & at) {
#pragma unroll
    for (int c = 0; c < 4 * NTMAX; ++c) {
        if (c >= 4 * nt) break;
        const int chunk = c * 256 + threadIdx.x;
        const int t = chunk >> 10, rem = chunk & 1023;
        const int s = rem >> 7, hl = (rem >> 6) & 1, ln = rem & 63;
        at.off[c] = (uint32_t)act_at(rows[t * 16 + (ln & 15)], s * 32 + 8 * (ln >> 4), hl, K);
    }
}

template <int NTMAX>
__device__ __forceinline__ void stage_load(const __half * x, const StageAt<NTMAX> & at, int sb, int nt, StageRegs<NTMAX> & regs) {
    const __half * xs = x + (size_t)sb * kStageStep;
#pragma unroll
    for (int c = 0; c < 4 * NTMAX; ++c) {
        if (c >= 4 * nt) break;
        regs.v[c] = *(const u4 *)(xs + at.off[c]);
    }
}

template <int NTMAX>
__device__ __forceinline__ void stage_store(uint8_t * buf, int nt, const StageRegs<NTMAX> & regs) {
#pragma unroll
    for (int c = 0; c < 4 * NTMAX; ++c) {
        if (c >= 4 * nt) break;
        *(u4 *)(buf + (size_t)(c * 256 + threadIdx.x) * 16) = regs.v[c];
    }
}

__device__ __forceinline__ h8 staged(const uint8_t * buf, int t, int s, int hl, int lane) {
    return *(const h8 *)(buf + t * kStageTile + ((s * 2 + hl) * 64 + lane) * 16);
}

// The rotating weight sets of the MXFP4 pipeline (members only where the pipeline is built: as plain locals of every
// instantiation they cost the other weight types registers).
template <int TYPE, bool ON> struct GateUpSets { Tile<TYPE> g0, u0, g1, u1, g2, u2; };
template <int TYPE> struct GateUpSets<TYPE, false> {};
template <int TYPE, bool ON> struct DownSets { Tile<TYPE> w0, w1, w2; };
template <int TYPE> struct DownSets<TYPE, false> {};

// One workgroup per (expert, four consecutive tiles of 16 output features), one wave per tile: gate and up
// tiles together, SwiGLU in the epilogue. The weights of the next super-block and the activations of the next
// super-block are requested before the current one is multiplied.
// (Two workgroups fit a CU's LDS, two waves a SIMD: told so, the compiler keeps the products in vector registers
// instead of parking them in accumulation registers and copying them back.)
template <int TYPE, int NTMAX>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void k_moe_gate_up(MoeArgs a) {
    __shared__ __attribute__((aligned(16))) uint8_t stage[2][NTMAX * kStageTile];
    __shared__ int rows[32];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r16 = lane & 15, g = lane >> 4;
    const int n_tiles = a.N / 16;
    const int item0 = blockIdx.x * 4;
    const int e = item0 / n_tiles, ft = item0 % n_tiles + wave;     // n_tiles % 4 == 0: one expert per workgroup
    if (e >= a.n_expert) return;
    const int nsb = a.K >> 8;
    const uint8_t * wg = a.w0 + ((size_t)e * n_tiles + ft) * nsb * Tile<TYPE>::BYTES;
    const uint8_t * wu = a.w1 + ((size_t)e * n_tiles + ft) * nsb * Tile<TYPE>::BYTES;
    // MXFP4: three weight sets in rotation (below); the first two are requested before the expert's pair count and
    // slots are looked up - two trips to memory that the weights' own trip then runs under
    GateUpSets<TYPE, TYPE == WT_MXFP4> ws;
    auto request_w = [&](int sb, Tile<TYPE> & tg, Tile<TYPE> & tu) __attribute__((always_inline)) {
        const size_t o = (size_t)min(sb, nsb - 1) * Tile<TYPE>::BYTES;
        tg.load(wg + o, lane);
        tu.load(wu + o, lane);
    };
    if constexpr (TYPE == WT_MXFP4) {
        request_w(0, ws.g0, ws.u0);
        request_w(1, ws.g1, ws.u1);
    }
    const int n_e = a.expert_n[e];
    if (n_e == 0) return;
    const int qb = a.off_pad[e];
    for (int t0 = 0; t0 < n_e; t0 += 16 * NTMAX) {
        const int nt = (NTMAX == 2 && n_e - t0 > 16) ? 2 : 1;
        __syncthreads();                       // the last pass is done with rows and the staging buffers
        if constexpr (TYPE == WT_MXFP4) {
            if (t0 > 0) { request_w(0, ws.g0, ws.u0); request_w(1, ws.g1, ws.u1); }
        }
        if (threadIdx.x < 32) {
            const int at = t0 + threadIdx.x;
            const int tk = at < n_e ? a.tok_of_q[qb + at] : -1;
            rows[threadIdx.x] = tk < 0 ? 0 : tk;        // padding rows read token 0 and are never stored
        }
        __syncthreads();
        StageAt<NTMAX> at;
        stage_prepare(a.K, rows, nt, at);
        f4 ag[2], au[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) { ag[t] = (f4){0.f, 0.f, 0.f, 0.f}; au[t] = (f4){0.f, 0.f, 0.f, 0.f}; }
        auto multiply = [&](int sb, const Tile<TYPE> & cg, const Tile<TYPE> & cu) __attribute__((always_inline)) {
            const uint8_t * cur = stage[sb & 1];
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const auto og = cg.prep(s), ou = cu.prep(s);
#pragma unroll
                for (int t = 0; t < NTMAX; ++t) {
                    if (t >= nt) break;
                    const h8 hi = staged(cur, t, s, 0, lane), lo = staged(cur, t, s, 1, lane);
                    mac(og, hi, lo, ag[t]);
                    mac(ou, hi, lo, au[t]);
                }
            }
        };
        if constexpr (TYPE == WT_MXFP4) {
            // The small tiles are multiplied faster than a request returns: the activations go global -> LDS directly
            // (no registers, no store phase), the weights are requested two super-blocks ahead into three sets in
            // rotation, and the waits are written here - the compiler does not see the direct requests, and its own
            // waits for the weight loads it does see come after these and find them done. A wave's requests return in
            // order: at the top of super-block sb > 0 everything but the six loads of set sb + 1 must have landed.
            const uint32_t lds0 = lds_offset(&stage[0][0]);
            auto request_x = [&](int sb) __attribute__((always_inline)) {
                const __half * xs = a.x.x + (size_t)sb * kStageStep;
#pragma unroll
                for (int c = 0; c < 4 * NTMAX; ++c) {
                    if (c >= 4 * nt) break;
                    lds_dma16(xs, at.off[c] * 2u, lds0 + (uint32_t)(sb & 1) * (NTMAX * kStageTile) + (uint32_t)(c * 256 + wave * 64) * 16u);
                }
            };
            request_x(0);
            __builtin_amdgcn_sched_barrier(0);
            auto body = [&](int sb, Tile<TYPE> & cg, Tile<TYPE> & cu, Tile<TYPE> & fg, Tile<TYPE> & fu) __attribute__((always_inline)) {
                // super-block 0: its activations were requested last, after both weight sets - everything lands
                if (sb == 0) __builtin_amdgcn_s_waitcnt(0x0F70); else __builtin_amdgcn_s_waitcnt(0x0F70 | 6);
                asm volatile("" : "+v"(cg.hdr.x), "+v"(cg.hdr.y), "+v"(cg.q0), "+v"(cg.q1), "+v"(cu.hdr.x), "+v"(cu.hdr.y), "+v"(cu.q0), "+v"(cu.q1));
                __syncthreads();           // every wave's part of super-block sb is in LDS, and none still reads the other buffer
                if (sb + 1 < nsb) request_x(sb + 1);
                request_w(sb + 2, fg, fu);
                __builtin_amdgcn_sched_barrier(0);
                if (sb >= nsb) return;     // past the end: the round of three is only kept whole
                multiply(sb, cg, cu);
            };
            for (int sb = 0; sb < nsb; sb += 3) {
                body(sb, ws.g0, ws.u0, ws.g2, ws.u2);
                body(sb + 1, ws.g1, ws.u1, ws.g0, ws.u0);
                body(sb + 2, ws.g2, ws.u2, ws.g1, ws.u1);
            }
        } else {
            StageRegs<NTMAX> regs;
            stage_load(a.x.x, at, 0, nt, regs);
            Tile<TYPE> tg, tu;
            tg.load(wg, lane);
            tu.load(wu, lane);
            stage_store(stage[0], nt, regs);
            __syncthreads();
            for (int sb = 0; sb < nsb; ++sb) {
                const bool more = sb + 1 < nsb;
                Tile<TYPE> ng = tg, nu = tu;
                if (more) {
                    stage_load(a.x.x, at, sb + 1, nt, regs);
                    ng.load(wg + (size_t)(sb + 1) * Tile<TYPE>::BYTES, lane);
                    nu.load(wu + (size_t)(sb + 1) * Tile<TYPE>::BYTES, lane);
                }
                const uint8_t * cur = stage[sb & 1];
#pragma unroll
                for (int s = 0; s < 8; ++s) {
                    const auto og = tg.prep(s), ou = tu.prep(s);
#pragma unroll
                    for (int t = 0; t < NTMAX; ++t) {
                        if (t >= nt) break;
                        const h8 hi = staged(cur, t, s, 0, lane), lo = staged(cur, t, s, 1, lane);
                        mac(og, hi, lo, ag[t]);
                        mac(ou, hi, lo, au[t]);
                    }
                }
                if (more) stage_store(stage[(sb + 1) & 1], nt, regs);
                __syncthreads();
                tg = ng;
                tu = nu;
            }
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int at = t0 + t * 16 + 4 * g + i;
                if (t >= nt || at >= n_e) continue;
                const float gv = ag[t][i];
                const float v = fminf(fmaxf((gv / (1.0f + __expf(-gv))) * au[t][i], -65504.0f), 65504.0f);
                const __half hh = __float2half_rn(v);
                const int f = ft * 16 + r16;
                a.h.x[act_at(qb + at, f, 0, a.N)] = hh;
                a.h.x[act_at(qb + at, f, 1, a.N)] = __float2half_rn(v - __half2float(hh));
            }
    }
}

// One workgroup per (expert, four consecutive tiles of 16 output features of the model width), one wave per
// tile; the hidden rows of the expert's pairs are staged like the activations above.
constexpr int down_waves(int type, int ntmax) {
    return ntmax != 1 ? 2 : (type == WT_MXFP4 || type == WT_Q8_0 ? 4 : (type == WT_Q6_K ? 3 : 2));
}
// (One token tile of MXFP4 or Q8_0 weights fits 128 registers without spilling: four waves a SIMD instead of the
// three the compiler settles for; measured 40.6 -> 37.6 us per layer at the 128-expert shape. Q6_K fits three; everything else
// runs two waves a SIMD and may use their 256 registers, which keeps the products out of the accumulation registers.)
template <int TYPE, int NTMAX>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(down_waves(TYPE, NTMAX), down_waves(TYPE, NTMAX))))
void k_moe_down(MoeArgs a) {
    __shared__ __attribute__((aligned(16))) uint8_t stage[2][NTMAX * kStageTile];
    __shared__ int rows[32], out_rows[32];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r16 = lane & 15, g = lane >> 4;
    const int n_tiles = a.N / 16;
    const int item0 = blockIdx.x * 4;
    const int e = item0 / n_tiles, et = item0 % n_tiles + wave;
    if (e >= a.n_expert) return;
    const int nsb = a.K >> 8;
    const uint8_t * wd = a.w0 + ((size_t)e * n_tiles + et) * nsb * Tile<TYPE>::BYTES;
    DownSets<TYPE, TYPE == WT_MXFP4> ws;          // (MXFP4, as in k_moe_gate_up: the first two sets requested before the lookups)
    auto request_w = [&](int sb, Tile<TYPE> & tw) __attribute__((always_inline)) {
        tw.load(wd + (size_t)min(sb, nsb - 1) * Tile<TYPE>::BYTES, lane);
    };
    if constexpr (TYPE == WT_MXFP4) {
        request_w(0, ws.w0);
        request_w(1, ws.w1);
    }
    const int n_e = a.expert_n[e];
    if (n_e == 0) return;
    const int qb = a.off_pad[e];
    for (int t0 = 0; t0 < n_e; t0 += 16 * NTMAX) {
        const int nt = (NTMAX == 2 && n_e - t0 > 16) ? 2 : 1;
        __syncthreads();
        if constexpr (TYPE == WT_MXFP4) {
            if (t0 > 0) { request_w(0, ws.w0); request_w(1, ws.w1); }
        }
        // every row of a tile lies in the expert's padded slot range
        if (threadIdx.x < 32) {
            const int slot = qb + t0 + ((int)threadIdx.x < 16 * nt ? threadIdx.x : 0);
            rows[threadIdx.x] = slot;
            out_rows[threadIdx.x] = a.pair_of_q && t0 + (int)threadIdx.x < n_e ? a.pair_of_q[slot] : slot;
        }
        __syncthreads();
        StageAt<NTMAX> at;
        stage_prepare(a.K, rows, nt, at);
        f4 acc[2] = {(f4){0.f, 0.f, 0.f, 0.f}, (f4){0.f, 0.f, 0.f, 0.f}};
        auto multiply = [&](int sb, const Tile<TYPE> & cw) __attribute__((always_inline)) {
            const uint8_t * cur = stage[sb & 1];
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const auto ow = cw.prep(s);
#pragma unroll
                for (int t = 0; t < NTMAX; ++t) {
                    if (t >= nt) break;
                    mac(ow, staged(cur, t, s, 0, lane), staged(cur, t, s, 1, lane), acc[t]);
                }
            }
        };
        if constexpr (TYPE == WT_MXFP4) {
            // (as in k_moe_gate_up: direct requests into LDS, three weight sets, the waits written here; a set is three loads)
            const uint32_t lds0 = lds_offset(&stage[0][0]);
            auto request_x = [&](int sb) __attribute__((always_inline)) {
                const __half * xs = a.x.x + (size_t)sb * kStageStep;
#pragma unroll
                for (int c = 0; c < 4 * NTMAX; ++c) {
                    if (c >= 4 * nt) break;
                    lds_dma16(xs, at.off[c] * 2u, lds0 + (uint32_t)(sb & 1) * (NTMAX * kStageTile) + (uint32_t)(c * 256 + wave * 64) * 16u);
                }
            };
            request_x(0);
            __builtin_amdgcn_sched_barrier(0);
            auto body = [&](int sb, Tile<TYPE> & cw, Tile<TYPE> & fw) __attribute__((always_inline)) {
                if (sb == 0) __builtin_amdgcn_s_waitcnt(0x0F70); else __builtin_amdgcn_s_waitcnt(0x0F70 | 3);
                asm volatile("" : "+v"(cw.hdr.x), "+v"(cw.hdr.y), "+v"(cw.q0), "+v"(cw.q1));
                __syncthreads();
                if (sb + 1 < nsb) request_x(sb + 1);
                request_w(sb + 2, fw);
                __builtin_amdgcn_sched_barrier(0);
                if (sb >= nsb) return;
                multiply(sb, cw);
            };
            for (int sb = 0; sb < nsb; sb += 3) {
                body(sb, ws.w0, ws.w2);
                body(sb + 1, ws.w1, ws.w0);
                body(sb + 2, ws.w2, ws.w1);
            }
        } else {
            StageRegs<NTMAX> regs;
            stage_load(a.x.x, at, 0, nt, regs);
            Tile<TYPE> tw;
            tw.load(wd, lane);
            stage_store(stage[0], nt, regs);
            __syncthreads();
            for (int sb = 0; sb < nsb; ++sb) {
                const bool more = sb + 1 < nsb;
                Tile<TYPE> nw = tw;
                if (more) {
                    stage_load(a.x.x, at, sb + 1, nt, regs);
                    nw.load(wd + (size_t)(sb + 1) * Tile<TYPE>::BYTES, lane);
                }
                const uint8_t * cur = stage[sb & 1];
#pragma unroll
                for (int s = 0; s < 8; ++s) {
                    const auto ow = tw.prep(s);
#pragma unroll
                    for (int t = 0; t < NTMAX; ++t) {
                        if (t >= nt) break;
                        mac(ow, staged(cur, t, s, 0, lane), staged(cur, t, s, 1, lane), acc[t]);
                    }
                }
                if (more) stage_store(stage[(sb + 1) & 1], nt, regs);
                __syncthreads();
                tw = nw;
            }
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int at = t0 + t * 16 + 4 * g + i;
                if (t < nt && at < n_e) a.out_pair[(size_t)out_rows[t * 16 + 4 * g + i] * a.N + et * 16 + r16] = acc[t][i];
            }
    }
}

// Router logits on the f32 matrix instruction (32x32x2: exact f32 products, f32 sums): one wave per (32 experts,
// 32 tokens, 128 columns of K) leaves its sums as a K-slice [slice][token][expert]; k_moe_route adds the slices
// in slice order. The rows are the f32 router weights, the tokens' values hi + lo of the activation planes.
typedef float f16v __attribute__((ext_vector_type(16)));
constexpr int ROUTER_KSLICE = 128;
__global__ __launch_bounds__(64) void k_moe_router(const float * __restrict__ wm, const __half * __restrict__ x, int K, int N, int T,
                                                   float * __restrict__ slices) {
    const int lane = threadIdx.x, j = lane & 31, g = lane >> 5;
    const int t = min((int)blockIdx.y * 32 + j, T - 1);
    const float * wr = wm + (size_t)(blockIdx.x * 32 + j) * K;
    const int k0 = blockIdx.z * ROUTER_KSLICE + 8 * g;
    f4 wa[8], wb[8];
    h8 hi[8], lo[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {          // lanes 0-31 take columns 16u .. 16u+7 of the slice, lanes 32-63 the next eight
        const int k = k0 + 16 * u;
        wa[u] = *(const f4 *)(wr + k);
        wb[u] = *(const f4 *)(wr + k + 4);
        hi[u] = load_h8(x + act_at(t, k, 0, K));
        lo[u] = load_h8(x + act_at(t, k, 1, K));
    }
    f16v acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const float w[8] = {wa[u].x, wa[u].y, wa[u].z, wa[u].w, wb[u].x, wb[u].y, wb[u].z, wb[u].w};
#pragma unroll
        for (int i = 0; i < 8; ++i)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(w[i], (float)hi[u][i] + (float)lo[u][i], acc, 0, 0, 0);
    }
    // acc[4 b + i] = expert 8 b + 4 g + i of the tile, token j
    const int tok = blockIdx.y * 32 + j;
    if (tok >= T) return;
    float * dst = slices + ((size_t)blockIdx.z * T + tok) * N + blockIdx.x * 32 + 4 * g;
#pragma unroll
    for (int b = 0; b < 4; ++b) *(f4 *)(dst + 8 * b) = (f4){acc[4 * b], acc[4 * b + 1], acc[4 * b + 2], acc[4 * b + 3]};
}

// Per token: the top-k experts by router logit (ties to the lower index - the
// order of the softmax probabilities) and their weights renormalised over the
// selection, exp and the sums in double. The logits are the sum of n_slices
// K-slices `stride` floats apart, added in slice order.
__global__ __launch_bounds__(64) void k_moe_route(const float * __restrict__ logits, int n_slices, size_t stride, int n_expert,
                                                  int k_used, int32_t * __restrict__ sel, float * __restrict__ wgt) {
    const int t = blockIdx.x, lane = threadIdx.x;
    float v[4];
    bool taken[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int e = lane + 64 * i;
        v[i] = e < n_expert ? 0.0f : -INFINITY;
        taken[i] = e >= n_expert;
    }
    for (int s0 = 0; s0 < n_slices; s0 += 8) {       // eight slices' loads in flight together, added in slice order
        float part[8][4];
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int e = min(lane + 64 * i, n_expert - 1);
                part[u][i] = logits[(size_t)min(s0 + u, n_slices - 1) * stride + (size_t)t * n_expert + e];
            }
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (s0 + u < n_slices && lane + 64 * i < n_expert) v[i] = s0 + u == 0 ? part[u][i] : v[i] + part[u][i];
    }
    float mine = -INFINITY;       // lane j keeps the j-th largest logit
    float mx = -INFINITY;
    for (int j = 0; j < k_used; ++j) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (!taken[i] && (bi == 0x7fffffff || v[i] > bv)) { bv = v[i]; bi = lane + 64 * i; }
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o, 64);
            const int oi = __shfl_xor(bi, o, 64);
            if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (bi == lane + 64 * i) taken[i] = true;
        if (j == 0) mx = bv;
        if (lane == j) mine = bv;
        if (lane == 0) sel[(size_t)t * k_used + j] = bi;
    }
    // every lane below k_used its own exp; the sum in selection order, the same in every lane
    const double p = lane < k_used ? exp((double)mine - (double)mx) : 0.0;
    double sum = 0.0;
    for (int j = 0; j < k_used; ++j) sum += __shfl(p, j, 64);
    if (lane < k_used) wgt[(size_t)t * k_used + lane] = (float)(p / sum);
}

// Stable counting sort of the pairs by expert, every expert's range padded to a
// multiple of 16 slots. One workgroup of 1024 threads.
__global__ __launch_bounds__(1024) void k_moe_group(const int32_t * __restrict__ sel, int n_pairs, int n_expert, int k_used,
                                                    int32_t * __restrict__ expert_n, int32_t * __restrict__ off_pad,
                                                    int32_t * __restrict__ tok_of_q, int32_t * __restrict__ q_of_pair,
                                                    int32_t * __restrict__ pair_of_q) {
    __shared__ int cnt[256];
    __shared__ int base[256];
    __shared__ int wcnt[16][256];
    __shared__ int total_pad;
    __shared__ int wsum[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid < 256) cnt[tid] = 0;
    for (int i = tid; i < 16 * 256; i += 1024) (&wcnt[0][0])[i] = 0;
    __syncthreads();
    for (int p = tid; p < n_pairs; p += 1024) atomicAdd(&cnt[sel[p]], 1);
    __syncthreads();
    // exclusive prefix sums of the padded counts: a scan inside each of the first four waves, then the waves' totals
    int padded = 0, incl = 0;
    if (tid < 256) {
        padded = tid < n_expert ? (cnt[tid] + 15) & ~15 : 0;
        incl = padded;
        for (int o = 1; o < 64; o <<= 1) {
            const int up = __shfl_up(incl, o, 64);
            if (lane >= o) incl += up;
        }
        if (lane == 63) wsum[wave] = incl;
    }
    __syncthreads();
    if (tid < 256) {
        int before = 0;
        for (int w = 0; w < wave; ++w) before += wsum[w];
        const int at = before + incl - padded;
        if (tid < n_expert) {
            off_pad[tid] = at;
            base[tid] = at;
            expert_n[tid] = cnt[tid];
        }
        if (tid == n_expert - 1) {
            off_pad[n_expert] = at + padded;
            total_pad = at + padded;
        }
    }
    __syncthreads();
    for (int q = tid; q < total_pad; q += 1024) tok_of_q[q] = -1;
    __syncthreads();
    for (int c0 = 0; c0 < n_pairs; c0 += 1024) {
        const int p = c0 + tid;
        const int e = p < n_pairs ? sel[p] : -1;
        int rank = 0;
        for (int i = 0; i < 64; ++i) {
            const int other = __shfl(e, i, 64);
            if (other == e && i < lane) ++rank;
        }
        if (e >= 0) atomicMax(&wcnt[wave][e], rank + 1);
        __syncthreads();
        if (e >= 0) {
            int pos = base[e] + rank;
            for (int w = 0; w < wave; ++w) pos += wcnt[w][e];
            q_of_pair[p] = pos;
            tok_of_q[pos] = p / k_used;
            if (pair_of_q) pair_of_q[pos] = p;
        }
        __syncthreads();
        if (tid < n_expert) {
            int add = 0;
            for (int w = 0; w < 16; ++w) { add += wcnt[w][tid]; wcnt[w][tid] = 0; }
            base[tid] += add;
        }
        __syncthreads();
    }
}

__global__ __launch_bounds__(256) void k_moe_combine(const float * __restrict__ out_pair, const int32_t * __restrict__ q_of_pair,
                                                     const float * __restrict__ wgt, int k_used, int E, float * __restrict__ x) {
    const int t = blockIdx.x;
    const int c = (blockIdx.y * 256 + threadIdx.x) * 4;
    if (c >= E) return;
    f4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < k_used; ++j) {
        const float w = wgt[(size_t)t * k_used + j];
        const f4 v = *(const f4 *)(out_pair + (size_t)q_of_pair[(size_t)t * k_used + j] * E + c);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = fmaf(w, v[i], acc[i]);
    }
    f4 * dst = (f4 *)(x + (size_t)t * E + c);
    *dst += acc;
}

size_t moe_slots(int n_tokens, int k_used, int n_expert) {
    return ((size_t)n_tokens * k_used + (size_t)16 * n_expert + 63) / 64 * 64;
}

Slices moe_ffn(hipStream_t s, const MoeLayer & L, const MoeShape & sh, const Act & xn, int T, float * x, const MoeBuffers & b,
               bool defer_combine) {
    if (T <= 0) return Slices();
    // the weighted sum over a token's experts: added to x here, or left to the next RMSNorm launch as gathered slices
    auto combine = [&](bool pair_order) -> Slices {
        if (defer_combine) {
            Slices sl;
            sl.data = b.out_pair; sl.n = sh.k_used; sl.N = sh.E; sl.weight = b.wgt;
            sl.gather = pair_order ? nullptr : b.q_of_pair;
            return sl;
        }
        if (pair_order) throw std::runtime_error("moe: rows in pair order are combined by the next RMSNorm");
        hipLaunchKernelGGL(k_moe_combine, dim3(T, (sh.E / 4 + 255) / 256), dim3(256), 0, s, b.out_pair, b.q_of_pair, b.wgt,
                           sh.k_used, sh.E, x);
        check_launch("moe_combine");
        return Slices();
    };
    if (sh.n_expert > 256 || sh.k_used > 16 || sh.k_used > sh.n_expert) throw std::runtime_error("moe: unsupported expert count");
    // multiples of 256: whole super-blocks along K, and the four waves of a workgroup share an expert (N / 16 % 4 == 0)
    if (sh.E % 256 != 0 || sh.F % 256 != 0) throw std::runtime_error("moe: widths must be multiples of 256");
    auto tiled = [](int t) { return t == WT_MXFP4 || t == WT_Q8_0 || t == WT_Q4_K || t == WT_Q5_K || t == WT_Q6_K; };
    if (L.gate.type != L.up.type || !tiled(L.gate.type) || !tiled(L.down.type))
        throw std::runtime_error("moe: expert weights must be MXFP4, Q8_0, Q4_K, Q5_K or Q6_K, gate and up of one type");
    // The router: f32 rows on the f32 matrix instruction, K split into slices of 128 columns that the selection
    // adds (the slices borrow the pairs' output rows, which nothing holds yet); any other router by the generic kernel.
    const Act xr = xn.operand(L.router.type);
    const int r_slices = sh.E / ROUTER_KSLICE;
    if (L.router.type == WT_F32 && L.router.raw && ((uintptr_t)L.router.raw & 15) == 0 && xr.x && sh.n_expert % 32 == 0
        && L.router.K == sh.E && L.router.N == sh.n_expert
        && (size_t)r_slices * T * sh.n_expert <= moe_slots(T, sh.k_used, sh.n_expert) * (size_t)sh.E) {
        hipLaunchKernelGGL(k_moe_router, dim3(sh.n_expert / 32, (T + 31) / 32, r_slices), dim3(64), 0, s,
                           (const float *)L.router.raw, xr.x, sh.E, sh.n_expert, T, b.out_pair);
        check_launch("moe_router");
        hipLaunchKernelGGL(k_moe_route, dim3(T), dim3(64), 0, s, b.out_pair, r_slices, (size_t)T * sh.n_expert, sh.n_expert,
                           sh.k_used, b.sel, b.wgt);
    } else {
        matmul_generic(s, L.router, xn, T, b.logits, sh.n_expert, 0, MM_STORE, nullptr);
        hipLaunchKernelGGL(k_moe_route, dim3(T), dim3(64), 0, s, b.logits, 1, (size_t)0, sh.n_expert, sh.k_used, b.sel, b.wgt);
    }
    check_launch("moe_route");
    hipLaunchKernelGGL(k_moe_group, dim3(1), dim3(1024), 0, s, b.sel, T * sh.k_used, sh.n_expert, sh.k_used, b.expert_n,
                       b.off_pad, b.tok_of_q, b.q_of_pair, b.pair_of_q);
    check_launch("moe_group");
    MoeArgs a {};
    a.expert_n = b.expert_n; a.off_pad = b.off_pad; a.tok_of_q = b.tok_of_q; a.n_expert = sh.n_expert;
    // the experts multiply the rows after ggml's Q8_0 conversion, the router the rows themselves
    a.w0 = L.gate.packed; a.w1 = L.up.packed; a.x = xn.operand(L.gate.type); a.h = b.h; a.K = sh.E; a.N = sh.F;
    if (!a.x.x || !b.h.x) throw std::runtime_error("moe: the activations were not prepared for the expert weights");
    const unsigned gu_blocks = (unsigned)(((size_t)sh.n_expert * (sh.F / 16) + 3) / 4);
    // few pairs per expert (a decode step): one token tile per pass
    const bool one_tile = (size_t)T * sh.k_used <= (size_t)12 * sh.n_expert;
    // MXFP4 experts in such a step, exact arithmetic: the block-scaled FP4 x FP8 matrix instruction takes the stored
    // codes and exponents as they are (no decode), the activations as hexadecimal digits
    const size_t slots = moe_slots(T, sh.k_used, sh.n_expert);
    if (one_tile && !xn.faithful && L.gate.type == WT_MXFP4 && L.down.type == WT_MXFP4 && L.gate.records && L.up.records
        && L.down.records && b.mx_ops && slots <= b.mx_slots && mxe_moe_can(sh.E, sh.F)) {
        mxe_moe_gate_up(s, L.gate.records, L.up.records, xn, sh.E, sh.F, sh.n_expert, b.off_pad, b.tok_of_q, slots, b.mx_ops,
                        b.mx_scales, b.mx_h);
        mxe_moe_down(s, L.down.records, b.mx_h, sh.E, sh.F, sh.n_expert, b.off_pad, b.tok_of_q, slots, b.mx_ops, b.mx_scales,
                     b.out_pair);
        return combine(false);
    }
    // (measured on the 128-expert shape at 128 rows: the down projection gains a fifth from the smaller
    // workgroups, gate/up - two weight tiles per wave - loses a tenth, so it keeps two tiles)
    switch (L.gate.type) {
        case WT_MXFP4: hipLaunchKernelGGL((k_moe_gate_up<WT_MXFP4, 2>), dim3(gu_blocks), dim3(256), 0, s, a); break;
        case WT_Q4_K:  hipLaunchKernelGGL((k_moe_gate_up<WT_Q4_K, 2>), dim3(gu_blocks), dim3(256), 0, s, a); break;
        case WT_Q5_K:  hipLaunchKernelGGL((k_moe_gate_up<WT_Q5_K, 2>), dim3(gu_blocks), dim3(256), 0, s, a); break;
        case WT_Q6_K:  hipLaunchKernelGGL((k_moe_gate_up<WT_Q6_K, 2>), dim3(gu_blocks), dim3(256), 0, s, a); break;
        default:       hipLaunchKernelGGL((k_moe_gate_up<WT_Q8_0, 2>), dim3(gu_blocks), dim3(256), 0, s, a); break;
    }
    check_launch("moe_gate_up");
    if (xn.faithful) {
        // ggml's arithmetic: the hidden rows are converted, in place, for the down projection
        Act hq;
        hq.K = sh.F; hq.qx = b.h.x; hq.qsums = nullptr; hq.quant = act_quant_of(L.down.type);
        requant_act(s, b.h.x, (int)moe_slots(T, sh.k_used, sh.n_expert), hq);
    }
    a.w0 = L.down.packed; a.w1 = nullptr; a.x = b.h; a.out_pair = b.out_pair; a.K = sh.F; a.N = sh.E;
    // deferred: the rows leave in pair order, so that the norm reads a token's rows without looking up their slots
    a.pair_of_q = defer_combine ? b.pair_of_q : nullptr;
    const unsigned d_blocks = (unsigned)(((size_t)sh.n_expert * (sh.E / 16) + 3) / 4);
#define RK_MOE_DOWN(TYPE)                                                                                        \
    do {                                                                                                         \
        if (one_tile) hipLaunchKernelGGL((k_moe_down<TYPE, 1>), dim3(d_blocks), dim3(256), 0, s, a);              \
        else hipLaunchKernelGGL((k_moe_down<TYPE, 2>), dim3(d_blocks), dim3(256), 0, s, a);                       \
    } while (0)
    switch (L.down.type) {
        case WT_MXFP4: RK_MOE_DOWN(WT_MXFP4); break;
        case WT_Q4_K:  RK_MOE_DOWN(WT_Q4_K); break;
        case WT_Q5_K:  RK_MOE_DOWN(WT_Q5_K); break;
        case WT_Q6_K:  RK_MOE_DOWN(WT_Q6_K); break;
        default:       RK_MOE_DOWN(WT_Q8_0); break;
    }
#undef RK_MOE_DOWN
    check_launch("moe_down");
    return combine(a.pair_of_q != nullptr);
}

}  // namespace rk
