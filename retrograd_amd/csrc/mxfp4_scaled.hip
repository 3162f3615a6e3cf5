// MXFP4 weights times Q8_0 activation blocks on the block-scaled matrix instruction
// (v_mfma_scale_f32_16x16x128_f8f6f4), for decode-sized steps of at most 16 tokens under ggml's
// activation arithmetic (ggml's vec_dot for MXFP4 multiplies the E2M1 codes with Q8_0 codes and
// scales the integer sum by both block scales; the Q8_0 conversion is quantize_row_q8_0_ref's).
//
// One instruction takes one weight block of 32 values for 16 rows, in one half of its k range:
//   A (FP4, 16 rows x 128 k): lane groups 0 and 1 (k 0..31 and 32..63) both hold the 16 nibble bytes of
//     block b as GGUF stores them, lane groups 2 and 3 (k 64..95 and 96..127) those of block b + 1.
//     Nibble 2i of an operand is the low nibble of byte i, so k = 2j is a block's value j and
//     k = 2j + 1 its value j + 16. The E2M1 codes are the hardware's FP4 format; a block's E8M0 byte
//     is the hardware's block scale (2^(e-127) on 0.5-steps equals GGUF's 2^(e-128) on doubled values).
//   B (FP8 E4M3, 128 k x 16 tokens): an int8 code c = 16 hi + lo with hi in [-8, 7] and lo in
//     [0, 15], both exact in E4M3. For block b, k 0..31 holds hi (block scale 2^4), k 32..63 holds lo
//     (block scale 2^0) and k 64..127 is zero; for block b + 1 the same bytes sit in k 64..127 (the
//     operand's upper four registers) and k 0..63 is zero. All products and the sum are exact in f32.
//   The 16 x 16 result is then multiplied by the tokens' f16 block scales and added to the
//   accumulators by one fma per value.
// So one 16-byte load per lane feeds two instructions, and every byte of the weights is fetched by two
// lanes instead of four. The weights are stored for this kernel in records of 2176 B per (16-row tile,
// eight blocks): four pairs of blocks' nibbles (2 x 16 rows x 16 B each) and 16 x 8 exponent bytes
// (a row's even blocks, then its odd blocks), so that a lane loads the four exponents of its half as one
// dword and names the pair's byte in the instruction.
#include "kernels.hpp"
#include "dev_common.hpp"

namespace rk {

namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float f4v __attribute__((ext_vector_type(4)));

constexpr int MXS_RECORD = 2176;

// the integer v in [-8, 15] as an OCP E4M3 byte (bias 7, three mantissa bits)
__device__ inline uint8_t e4m3_of_small_int(int v) {
    if (v == 0) return 0;
    const int sign = v < 0 ? 0x80 : 0, m = v < 0 ? -v : v;
    const int p = 31 - __builtin_clz(m);
    return (uint8_t)(sign | ((p + 7) << 3) | (((m << 3) >> p) & 7));
}

__global__ void k_mxs_repack(const uint8_t * __restrict__ raw, uint8_t * __restrict__ dst, int nb, size_t total) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const size_t row = i / nb;
    const int b = (int)(i % nb), r = (int)(row % 16);
    const uint8_t * src = raw + i * 17;
    uint8_t * rec = dst + ((row / 16) * (nb / 8) + b / 8) * MXS_RECORD;
    rec[2048 + 8 * r + 4 * (b & 1) + ((b & 7) >> 1)] = src[0];
    uint8_t * q = rec + 256 * (b & 7) + 16 * r;
    for (int j = 0; j < 16; ++j) q[j] = src[1 + j];
}

// One thread per (block, token slot): the Q8_0 conversion of 32 values and the operand bytes of the slot's
// four lanes. Slots past the step's tokens hold zeros.
__global__ void k_mxs_quantise(const float * __restrict__ x, int T, int K, uint8_t * __restrict__ bop, float * __restrict__ dx) {
    const int nb = K / 32, i = blockIdx.x * 256 + threadIdx.x;
    if (i >= nb * 16) return;
    const int b = i / 16, n = i % 16;
    int code[32];
    float dh = 0.0f;
    if (n < T) {
        const float * src = x + (size_t)n * K + 32 * b;
        float amax = 0.0f;
        for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(src[j]));
        const float d = __fdiv_rn(amax, 127.0f);
        const float id = d != 0.0f ? __fdiv_rn(1.0f, d) : 0.0f;
        dh = __half2float(__float2half_rn(d));
        for (int j = 0; j < 32; ++j) code[j] = (int)roundf(src[j] * id);
    } else {
        for (int j = 0; j < 32; ++j) code[j] = 0;
    }
    dx[i] = dh;
    for (int q = 0; q < 4; ++q) {
        uint8_t * o = bop + ((size_t)(b * 64 + 16 * q + n)) * 16;
        for (int j = 0; j < 16; ++j) {
            const int k = 16 * (q & 1) + j;
            const int c = code[(k & 1) ? 16 + k / 2 : k / 2];
            o[j] = e4m3_of_small_int(q < 2 ? (c >> 4) : (c & 15));
        }
    }
}

struct MxsArgs {
    const uint8_t * w;      // records
    const uint8_t * bop;    // [block][lane][16 B]
    const float * dx;       // [block][16]
    float * y;              // [T][N]
    int nb, n_tiles, T, N;
};

template <int OPSEL, bool UPPER>
__device__ inline void mxs_block(const uint4 & a, int e, const uint4 & b, float d, int scale_b, f4v & acc) {
    const v8i A = {(int)a.x, (int)a.y, (int)a.z, (int)a.w, 0, 0, 0, 0};
    const v8i B = UPPER ? v8i{0, 0, 0, 0, (int)b.x, (int)b.y, (int)b.z, (int)b.w} : v8i{(int)b.x, (int)b.y, (int)b.z, (int)b.w, 0, 0, 0, 0};
    const f4v zero = {0.0f, 0.0f, 0.0f, 0.0f};
    const f4v o = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A, B, zero, 4, 0, OPSEL, e, 0, scale_b);
    for (int i = 0; i < 4; ++i) acc[i] = fmaf(d, o[i], acc[i]);
}

struct MxsGroup {
    uint4 a[4];
    int e;
};

// lane_at = 256 (lane / 32) + 16 (lane % 16): the lane's nibble bytes within a pair of blocks, and
// 2048 + 8 (lane % 16) + 4 (lane / 32): its four exponent bytes
__device__ inline void mxs_load(MxsGroup & g, const uint8_t * rec, int lane_at) {
    for (int u = 0; u < 4; ++u) g.a[u] = *(const uint4 *)(rec + 512 * u + lane_at);
    g.e = *(const int *)(rec + 2048 + ((lane_at & 0xf0) >> 1) + ((lane_at >> 8) << 2));
}

__device__ inline void mxs_group(const MxsGroup & c, const uint4 * lb, const float * ld, int scale_b, f4v & acc) {
    mxs_block<0, false>(c.a[0], c.e, lb[0], ld[0], scale_b, acc);
    mxs_block<0, true>(c.a[0], c.e, lb[64], ld[16], scale_b, acc);
    mxs_block<1, false>(c.a[1], c.e, lb[128], ld[32], scale_b, acc);
    mxs_block<1, true>(c.a[1], c.e, lb[192], ld[48], scale_b, acc);
    mxs_block<2, false>(c.a[2], c.e, lb[256], ld[64], scale_b, acc);
    mxs_block<2, true>(c.a[2], c.e, lb[320], ld[80], scale_b, acc);
    mxs_block<3, false>(c.a[3], c.e, lb[384], ld[96], scale_b, acc);
    mxs_block<3, true>(c.a[3], c.e, lb[448], ld[112], scale_b, acc);
}

// One workgroup of 16 waves keeps the step's activation operands in LDS. A wave takes whole 16-row tiles (tile
// blockIdx * 16 + wave, then every gridDim * 16 th) and reads their records as one stream, MXS_DEPTH groups of eight
// blocks in flight across tile boundaries; the first groups are requested before the workgroup meets at the barrier
// behind the staging. Past the stream's end the loads repeat its last record (no branch around a load, so the waits stay exact).
constexpr int MXS_DEPTH = 4;

__global__ __launch_bounds__(1024, 1) void k_mxs(MxsArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, nb = a.nb;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), r = lane & 15, q = lane >> 4;
    const int ng = nb / 8, lane_at = 256 * (lane >> 5) + 16 * r;
    const int tile0 = blockIdx.x * 16 + wave, stride = gridDim.x * 16;
    const int my_tiles = tile0 < a.n_tiles ? (a.n_tiles - tile0 + stride - 1) / stride : 0;
    const int total = my_tiles * ng;
    const size_t tile_bytes = (size_t)ng * MXS_RECORD;

    // the load stream's position: record `lg` of tile `lt`; it stops on the last record
    int lt = tile0, lg = 0, issued = 0;
    const uint8_t * lp = a.w + (size_t)(my_tiles ? tile0 : 0) * tile_bytes;
    auto advance = [&]() {
        if (issued + 1 < total) {
            ++issued;
            if (++lg == ng) { lg = 0; lt += stride; lp = a.w + (size_t)lt * tile_bytes; }
            else lp += MXS_RECORD;
        }
    };
    // The step's operands go to LDS first, four loads per thread in flight (LDS holds at least 4096 operand entries
    // and 1024 scales, so this pass stores without a bounds test); the first weight groups are requested before the
    // workgroup meets at the barrier.
    uint4 * l4 = (uint4 *)lds;
    float * ldx = (float *)(lds + (size_t)max(nb, 64) * 1024);
    const uint4 * src = (const uint4 *)a.bop;
    const int n4 = nb * 64, n_dx = nb * 16;
    {
        uint4 st[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) st[u] = src[min(tid + 1024 * u, n4 - 1)];
        const float sdx = a.dx[min(tid, n_dx - 1)];
#pragma unroll
        for (int u = 0; u < 4; ++u) l4[tid + 1024 * u] = st[u];
        ldx[tid] = sdx;
        if (n4 > 4096) {         // rows longer than 2048: the rest of the operands
            for (int i = tid + 4096; i < n4; i += 1024) l4[i] = src[i];
            for (int i = tid + 1024; i < n_dx; i += 1024) ldx[i] = a.dx[i];
        }
    }
    asm volatile("" : : : "memory");
    MxsGroup G[MXS_DEPTH];
#pragma unroll
    for (int j = 0; j < MXS_DEPTH; ++j) { mxs_load(G[j], lp, lane_at); advance(); }
    __syncthreads();

    const int scale_b = (q & 1) ? 127 : 131;
    f4v acc = {0.0f, 0.0f, 0.0f, 0.0f};
    int ct = tile0, cg = 0;
    // Whole rounds of MXS_DEPTH groups with no branch around a load or a product: a last round that runs past the
    // stream's end multiplies the repeated last record into an accumulator that is never stored.
    for (int s = 0; s < total; s += MXS_DEPTH) {
#pragma unroll
        for (int j = 0; j < MXS_DEPTH; ++j) {
            mxs_group(G[j], l4 + (size_t)(8 * cg) * 64 + lane, ldx + 8 * cg * 16 + r, scale_b, acc);
            // the group's registers are free only now: its reload must not be moved above the products
            asm volatile("" : "+v"(acc) : : "memory");
            __builtin_amdgcn_sched_barrier(0);
            mxs_load(G[j], lp, lane_at);
            __builtin_amdgcn_sched_barrier(0);
            advance();
            if (++cg == ng) {
                // lane l holds token l % 16, rows 4 (l / 16) .. + 3 of the tile
                if (r < a.T && ct < a.n_tiles) *(float4 *)(a.y + (size_t)r * a.N + ct * 16 + 4 * q) = make_float4(acc[0], acc[1], acc[2], acc[3]);
                acc = f4v{0.0f, 0.0f, 0.0f, 0.0f};
                cg = 0;
                ct += stride;
            }
        }
    }
}


// ---------------------------------------------------------------------------------------------------------------
// The same weights times f32 activations, to f32 accumulation accuracy ("exact" arithmetic): an activation is
// written, per token and block of 32, as 2^E times six signed hexadecimal digits c1 .. c6 in [-8, 8]
// (x = 2^E sum c_i 16^-i, |x| <= 2^(E-1) for the block's largest value: 24 bits below the block's top, an absolute
// error of at most 2^(E-25) per value); a digit is exact in E4M3 and 16^-i 2^E is a power of two, i.e. a block scale
// of the instruction. One instruction multiplies the weight blocks b (lane groups 0, 1) and b + 1 (lane groups 2, 3)
// with two digits each (k 0..31: digit 2j+1 of block b, k 32..63: digit 2j+2 of block b, k 64..95 and 96..127 the same
// of block b + 1) and adds to the running accumulator: three instructions per pair of blocks, nothing else - no
// decode and no arithmetic outside the matrix unit. A wave multiplies two 16-row tiles with the same activation
// operands, so that every operand read from LDS serves 32 rows.
// Activation operands of one pair of blocks: [j = 0..2][lane][32 B] (bytes 0..15: the lane's k-slots of the first
// block's digit, 16..31 of the second block's; lane groups 0, 1 hold digit 2j+1, groups 2, 3 digit 2j+2) and one dword
// per lane whose byte j is the E8M0 scale of the k-block its lane group supplies (group g: block b + g / 2, digit
// 2j + 1 + g % 2). 6400 B per pair: a workgroup holds at most 24 pairs (six records) in LDS at a time, so longer
// rows are multiplied in chunks of columns, the accumulators staying in registers.
constexpr int MXE_PAIR_BYTES = 3 * 64 * 32, MXE_PAIR_SCALES = 64 * 4;

// The operand bytes and scale bytes of one (block b, token slot n) of a row set: v are the block's 32 values.
__device__ inline void mxe_write_block(const float * v, int b, int n, uint8_t * ops, uint8_t * scales) {
    float amax = 0.0f;
    for (int k = 0; k < 32; ++k) amax = fmaxf(amax, fabsf(v[k]));
    int ex = 0;
    if (amax > 0.0f) (void)frexpf(amax, &ex);          // amax = m 2^ex with m in [0.5, 1)
    const int E = amax > 0.0f ? ex + 1 : 0;            // |v| <= 2^(E - 1)
    const float down = ldexpf(1.0f, -E);
    float r[32];
    for (int k = 0; k < 32; ++k) {
        const int el = (k & 1) ? 16 + k / 2 : k / 2;    // the weight operand's k-slot k is the block's value el
        r[k] = v[el] * down;                            // exact: a power of two (values so small that this underflows are lost)
    }
    const int pair = b / 2, hb = b & 1;
    uint8_t * pair_ops = ops + (size_t)pair * MXE_PAIR_BYTES;
    uint8_t * pair_scales = scales + (size_t)pair * MXE_PAIR_SCALES;
    for (int d = 1; d <= 6; ++d) {
        const int j = (d - 1) / 2, second = (d - 1) & 1;      // instruction and which of its two digits
        uint32_t words[8];
        for (int wd = 0; wd < 8; ++wd) {
            uint32_t packed = 0;
            for (int i = 0; i < 4; ++i) {
                const int k = 4 * wd + i;
                const float t = r[k] * 16.0f;
                const float c = rintf(t);
                r[k] = t - c;
                packed |= (uint32_t)e4m3_of_small_int((int)c) << (8 * i);
            }
            words[wd] = packed;
        }
        for (int half = 0; half < 2; ++half) {                // k-slots 0..15 and 16..31 sit in two lane groups
            const int lane = 16 * (2 * second + half) + n;
            *(uint4 *)(pair_ops + ((size_t)j * 64 + lane) * 32 + 16 * hb) =
                make_uint4(words[4 * half], words[4 * half + 1], words[4 * half + 2], words[4 * half + 3]);
        }
        // the scale of k-block 2 hb + second comes from lane group 2 hb + second
        const int e8 = 127 + E - 4 * d;
        pair_scales[(size_t)(16 * (2 * hb + second) + n) * 4 + j] = (uint8_t)min(max(e8, 0), 254);
    }
    if (hb == 0) {
        // byte 3 of the scale dwords is never selected
        for (int g = 0; g < 4; ++g) pair_scales[(size_t)(16 * g + n) * 4 + 3] = 127;
    }
}

__global__ void k_mxe_pieces(const float * __restrict__ x, int T, int K, uint8_t * __restrict__ ops, uint8_t * __restrict__ scales) {
    const int nb = K / 32, i = blockIdx.x * 256 + threadIdx.x;
    if (i >= nb * 16) return;
    const int b = i / 16, n = i % 16;
    float v[32];
    for (int k = 0; k < 32; ++k) v[k] = n < T ? x[(size_t)n * K + 32 * b + k] : 0.0f;
    mxe_write_block(v, b, n, ops, scales);
}

// The same for the rows of a mixture-of-experts step: group g holds the 16 pair slots 16 g .. of one expert
// (tok_of_q: the slot's token, -1 for padding; off_pad[n_expert]: the slots in use). FROM_ACT: the rows are the
// step's activations by token, as hi/lo planes (the value is hi + lo); else f32 rows by slot.
template <bool FROM_ACT>
__global__ void k_mxe_moe_pieces(const __half * __restrict__ xa, const float * __restrict__ xf, int K,
                                 const int32_t * __restrict__ off_pad, const int32_t * __restrict__ tok_of_q, int n_expert,
                                 uint8_t * __restrict__ ops, uint8_t * __restrict__ scales) {
    const int nb = K / 32;
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int g = (int)(i / ((size_t)nb * 16)), rem = (int)(i % ((size_t)nb * 16));
    if (16 * g >= off_pad[n_expert]) return;
    const int b = rem / 16, n = rem % 16;
    const int slot = 16 * g + n, t = tok_of_q[slot];
    float v[32];
    if (t < 0) {
        for (int k = 0; k < 32; ++k) v[k] = 0.0f;
    } else if (FROM_ACT) {
        for (int k8 = 0; k8 < 4; ++k8) {
            const h8 hi = load_h8(xa + act_at(t, 32 * b + 8 * k8, 0, K)), lo = load_h8(xa + act_at(t, 32 * b + 8 * k8, 1, K));
            for (int k = 0; k < 8; ++k) v[8 * k8 + k] = (float)hi[k] + (float)lo[k];
        }
    } else {
        const float4 * src = (const float4 *)(xf + (size_t)slot * K + 32 * b);
        for (int k4 = 0; k4 < 8; ++k4) { const float4 f = src[k4]; v[4 * k4] = f.x; v[4 * k4 + 1] = f.y; v[4 * k4 + 2] = f.z; v[4 * k4 + 3] = f.w; }
    }
    mxe_write_block(v, b, n, ops + (size_t)g * (nb / 2) * MXE_PAIR_BYTES, scales + (size_t)g * (nb / 2) * MXE_PAIR_SCALES);
}

struct MxeArgs {
    const uint8_t * w;          // records (see above)
    const uint8_t * ops;        // [pair][3][64][32 B]
    const uint8_t * scales;     // [pair][64][4 B]
    float * y;                  // [T][N]
    int nb, n_tiles, T, N;
    int chunk_records, n_chunks;
};

struct MxeHalf {          // half a record of one tile: two pairs of blocks and the record's exponent dword
    uint4 a[2];
    int e;
};

__device__ inline void mxe_load(MxeHalf & g, const uint8_t * rec, int half, int lane_at) {
    g.a[0] = *(const uint4 *)(rec + 1024 * half + lane_at);
    g.a[1] = *(const uint4 *)(rec + 1024 * half + 512 + lane_at);
    g.e = *(const int *)(rec + 2048 + ((lane_at & 0xf0) >> 1) + ((lane_at >> 8) << 2));
}

template <int OPSEL_A, int J>
__device__ inline void mxe_mfma(const uint4 & a, int e, const v8i & b, int sb, f4v & acc) {
    const v8i A = {(int)a.x, (int)a.y, (int)a.z, (int)a.w, 0, 0, 0, 0};
    acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A, b, acc, 4, 0, OPSEL_A, e, J, sb);
}

// one pair of blocks of both tiles: three instructions each, the activation operands read once
template <int OPSEL_A>
__device__ inline void mxe_pair(const uint4 & a0, int e0, const uint4 & a1, int e1, const uint8_t * pair_ops, const int * pair_scales,
                                int lane, f4v & acc0, f4v & acc1) {
    const int sb = pair_scales[lane];
    const uint4 * o = (const uint4 *)(pair_ops + (size_t)lane * 32);
    const uint4 b0l = o[0], b0h = o[1], b1l = o[128], b1h = o[129], b2l = o[256], b2h = o[257];
    const v8i B0 = {(int)b0l.x, (int)b0l.y, (int)b0l.z, (int)b0l.w, (int)b0h.x, (int)b0h.y, (int)b0h.z, (int)b0h.w};
    const v8i B1 = {(int)b1l.x, (int)b1l.y, (int)b1l.z, (int)b1l.w, (int)b1h.x, (int)b1h.y, (int)b1h.z, (int)b1h.w};
    const v8i B2 = {(int)b2l.x, (int)b2l.y, (int)b2l.z, (int)b2l.w, (int)b2h.x, (int)b2h.y, (int)b2h.z, (int)b2h.w};
    mxe_mfma<OPSEL_A, 0>(a0, e0, B0, sb, acc0);
    mxe_mfma<OPSEL_A, 0>(a1, e1, B0, sb, acc1);
    mxe_mfma<OPSEL_A, 1>(a0, e0, B1, sb, acc0);
    mxe_mfma<OPSEL_A, 1>(a1, e1, B1, sb, acc1);
    mxe_mfma<OPSEL_A, 2>(a0, e0, B2, sb, acc0);
    mxe_mfma<OPSEL_A, 2>(a1, e1, B2, sb, acc1);
}

// A workgroup of 16 waves; a wave takes up to two pairs of adjacent 16-row tiles per turn of the workgroup and keeps
// their four accumulators while the workgroup walks the row's chunks of columns (operands of a chunk staged in LDS).
__global__ __launch_bounds__(1024, 1) void k_mxe(MxeArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), r = lane & 15, q = lane >> 4;
    const int lane_at = 256 * (lane >> 5) + 16 * r;
    const int ng = a.nb / 8;                                 // records of a tile
    const size_t tile_bytes = (size_t)ng * MXS_RECORD;
    const int n_tp = a.n_tiles / 2;
    const int chunk_pairs = a.chunk_records * 4;
    uint8_t * l_ops = lds;
    const int * l_scales = (const int *)(lds + (size_t)chunk_pairs * MXE_PAIR_BYTES);
    for (int base = blockIdx.x * 32; base < n_tp; base += gridDim.x * 32) {
        const int tp0 = base + 2 * wave;
        const int n_mine = min(2, max(0, n_tp - tp0));      // this wave's tile pairs of the turn
        f4v acc[2][2];
#pragma unroll
        for (int i = 0; i < 2; ++i) { acc[i][0] = f4v{0.f, 0.f, 0.f, 0.f}; acc[i][1] = f4v{0.f, 0.f, 0.f, 0.f}; }
        for (int c = 0; c < a.n_chunks; ++c) {
            const int rec0 = c * a.chunk_records, n_rec = min(a.chunk_records, ng - rec0);
            // the wave's stream of this chunk: its tile pairs one after the other, the chunk's half records in order
            const int n_items = n_mine * n_rec * 2;
            int l_tp = 0, l_half = 0, issued = 0;
            const uint8_t * lp = a.w + (size_t)(2 * (n_mine ? tp0 : 0)) * tile_bytes + (size_t)rec0 * MXS_RECORD;
            auto advance = [&]() {
                if (issued + 1 < n_items) {
                    ++issued;
                    if (++l_half == 2 * n_rec) { l_half = 0; ++l_tp; lp = a.w + (size_t)(2 * (tp0 + l_tp)) * tile_bytes + (size_t)rec0 * MXS_RECORD; }
                    else if ((l_half & 1) == 0) lp += MXS_RECORD;
                }
            };
            MxeHalf G0[2], G1[2];          // two items in flight: [tile of the pair]
            mxe_load(G0[0], lp, l_half & 1, lane_at); mxe_load(G0[1], lp + tile_bytes, l_half & 1, lane_at); advance();
            mxe_load(G1[0], lp, l_half & 1, lane_at); mxe_load(G1[1], lp + tile_bytes, l_half & 1, lane_at); advance();
            // the chunk's operands: pairs rec0 * 4 .. of the row, contiguous in global memory
            {
                const uint4 * src = (const uint4 *)(a.ops + (size_t)rec0 * 4 * MXE_PAIR_BYTES);
                uint4 * dst = (uint4 *)l_ops;
                // whole passes of the workgroup, three loads per thread in flight, then what is left (no test around
                // the loads of a full pass: a tested load waits for its own data before the next is requested)
                const int n16 = n_rec * 4 * MXE_PAIR_BYTES / 16, n_full = n16 / 1024;
                int p = 0;
                for (; p + 3 <= n_full; p += 3) {
                    const uint4 s0 = src[(p + 0) * 1024 + tid], s1 = src[(p + 1) * 1024 + tid], s2 = src[(p + 2) * 1024 + tid];
                    dst[(p + 0) * 1024 + tid] = s0; dst[(p + 1) * 1024 + tid] = s1; dst[(p + 2) * 1024 + tid] = s2;
                }
                for (; p < n_full; ++p) dst[p * 1024 + tid] = src[p * 1024 + tid];
                if (p * 1024 + tid < n16) dst[p * 1024 + tid] = src[p * 1024 + tid];
                const int * ssrc = (const int *)(a.scales + (size_t)rec0 * 4 * MXE_PAIR_SCALES);
                int * sdst = (int *)(lds + (size_t)chunk_pairs * MXE_PAIR_BYTES);
                for (int i0 = tid; i0 < n_rec * 4 * 64; i0 += 1024) sdst[i0] = ssrc[i0];
            }
            __syncthreads();
            int cg = 0;          // half record of the chunk being multiplied
            int ct = 0;          // tile pair being multiplied
            for (int it = 0; it < n_items; it += 2) {
                // even items are first halves of a record (exponent bytes 0, 1), odd items second halves (2, 3)
                {
                    const uint8_t * po = l_ops + (size_t)(2 * cg) * MXE_PAIR_BYTES;
                    const int * ps = l_scales + (2 * cg) * 64;
                    f4v & x0 = acc[ct][0], & x1 = acc[ct][1];
                    mxe_pair<0>(G0[0].a[0], G0[0].e, G0[1].a[0], G0[1].e, po, ps, lane, x0, x1);
                    mxe_pair<1>(G0[0].a[1], G0[0].e, G0[1].a[1], G0[1].e, po + MXE_PAIR_BYTES, ps + 64, lane, x0, x1);
                    asm volatile("" : "+v"(x0), "+v"(x1) : : "memory");
                    __builtin_amdgcn_sched_barrier(0);
                    mxe_load(G0[0], lp, 0, lane_at); mxe_load(G0[1], lp + tile_bytes, 0, lane_at);
                    __builtin_amdgcn_sched_barrier(0);
                    advance();
                    ++cg;
                }
                {
                    const uint8_t * po = l_ops + (size_t)(2 * cg) * MXE_PAIR_BYTES;
                    const int * ps = l_scales + (2 * cg) * 64;
                    f4v & x0 = acc[ct][0], & x1 = acc[ct][1];
                    mxe_pair<2>(G1[0].a[0], G1[0].e, G1[1].a[0], G1[1].e, po, ps, lane, x0, x1);
                    mxe_pair<3>(G1[0].a[1], G1[0].e, G1[1].a[1], G1[1].e, po + MXE_PAIR_BYTES, ps + 64, lane, x0, x1);
                    asm volatile("" : "+v"(x0), "+v"(x1) : : "memory");
                    __builtin_amdgcn_sched_barrier(0);
                    mxe_load(G1[0], lp, 1, lane_at); mxe_load(G1[1], lp + tile_bytes, 1, lane_at);
                    __builtin_amdgcn_sched_barrier(0);
                    advance();
                    if (++cg == 2 * n_rec) { cg = 0; ++ct; }
                }
            }
            __syncthreads();          // every wave is done with the chunk's operands
        }
        // lane l holds token l % 16, rows 4 (l / 16) .. + 3 of a tile
        for (int i = 0; i < n_mine; ++i)
            for (int tl = 0; tl < 2; ++tl)
                if (r < a.T) *(float4 *)(a.y + (size_t)r * a.N + (size_t)(2 * (tp0 + i) + tl) * 16 + 4 * q) =
                    make_float4(acc[i][tl][0], acc[i][tl][1], acc[i][tl][2], acc[i][tl][3]);
    }
}


// The expert products of a mixture-of-experts step on the same instruction stream: a workgroup takes group g of 16
// pair slots (all of one expert) and a part of that expert's tile pairs - for gate and up the tiles of the same 16
// hidden columns in the two matrices (SwiGLU on the two accumulators, f32 rows by slot out), for down two adjacent tiles.
struct MxeMoeArgs {
    const uint8_t * w0, * w1;     // records of every expert's rows: gate and up, or down (w1 unused)
    const uint8_t * ops, * scales;
    const int32_t * off_pad;
    int n_expert;
    float * out;                  // [slot][N]
    int nb, tiles_per_expert, N, parts, chunk_records, n_chunks;
};

template <bool GATE_UP, int MAXP>
__global__ __launch_bounds__(1024, 1) void k_mxe_moe(MxeMoeArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    __shared__ int s_expert;
    const int tid = threadIdx.x;
    const int g = blockIdx.x / a.parts, part = blockIdx.x % a.parts, slot0 = 16 * g;
    if (slot0 >= a.off_pad[a.n_expert]) return;
    if (tid < a.n_expert && a.off_pad[tid] <= slot0 && slot0 < a.off_pad[tid + 1]) s_expert = tid;
    __syncthreads();
    const int expert = s_expert;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), r = lane & 15, q = lane >> 4;
    const int lane_at = 256 * (lane >> 5) + 16 * r;
    const int ng = a.nb / 8;
    const size_t tile_bytes = (size_t)ng * MXS_RECORD;
    const int n_pairs = GATE_UP ? a.tiles_per_expert : a.tiles_per_expert / 2;
    const int per_part = (n_pairs + a.parts - 1) / a.parts;
    // a wave's tile pairs of the part: MAXP consecutive ones
    const int ip0 = part * per_part + MAXP * wave;
    const int n_mine = min(MAXP, max(0, min(per_part - MAXP * wave, n_pairs - ip0)));
    // first tile of a pair and the distance to its second
    auto tile_of = [&](int ip) { return (size_t)expert * a.tiles_per_expert + (GATE_UP ? ip : 2 * ip); };
    const ptrdiff_t second = GATE_UP ? (a.w1 - a.w0) : (ptrdiff_t)tile_bytes;
    const int chunk_pairs = a.chunk_records * 4;
    uint8_t * l_ops = lds;
    const int * l_scales = (const int *)(lds + (size_t)chunk_pairs * MXE_PAIR_BYTES);
    const uint8_t * g_ops = a.ops + (size_t)g * (a.nb / 2) * MXE_PAIR_BYTES;
    const uint8_t * g_scales = a.scales + (size_t)g * (a.nb / 2) * MXE_PAIR_SCALES;
    f4v acc[MAXP][2];
#pragma unroll
    for (int i = 0; i < MAXP; ++i) { acc[i][0] = f4v{0.f, 0.f, 0.f, 0.f}; acc[i][1] = f4v{0.f, 0.f, 0.f, 0.f}; }
    for (int c = 0; c < a.n_chunks; ++c) {
        const int rec0 = c * a.chunk_records, n_rec = min(a.chunk_records, ng - rec0);
        const int n_items = n_mine * n_rec * 2;
        int l_tp = 0, l_half = 0, issued = 0;
        const uint8_t * lp = a.w0 + tile_of(n_mine ? ip0 : 0) * tile_bytes + (size_t)rec0 * MXS_RECORD;
        auto advance = [&]() {
            if (issued + 1 < n_items) {
                ++issued;
                if (++l_half == 2 * n_rec) { l_half = 0; ++l_tp; lp = a.w0 + tile_of(ip0 + l_tp) * tile_bytes + (size_t)rec0 * MXS_RECORD; }
                else if ((l_half & 1) == 0) lp += MXS_RECORD;
            }
        };
        MxeHalf G0[2], G1[2];
        mxe_load(G0[0], lp, l_half & 1, lane_at); mxe_load(G0[1], lp + second, l_half & 1, lane_at); advance();
        mxe_load(G1[0], lp, l_half & 1, lane_at); mxe_load(G1[1], lp + second, l_half & 1, lane_at); advance();
        {
            const uint4 * src = (const uint4 *)(g_ops + (size_t)rec0 * 4 * MXE_PAIR_BYTES);
            uint4 * dst = (uint4 *)l_ops;
            const int n16 = n_rec * 4 * MXE_PAIR_BYTES / 16, n_full = n16 / 1024;
            int p = 0;
            for (; p + 3 <= n_full; p += 3) {
                const uint4 s0 = src[(p + 0) * 1024 + tid], s1 = src[(p + 1) * 1024 + tid], s2 = src[(p + 2) * 1024 + tid];
                dst[(p + 0) * 1024 + tid] = s0; dst[(p + 1) * 1024 + tid] = s1; dst[(p + 2) * 1024 + tid] = s2;
            }
            for (; p < n_full; ++p) dst[p * 1024 + tid] = src[p * 1024 + tid];
            if (p * 1024 + tid < n16) dst[p * 1024 + tid] = src[p * 1024 + tid];
            const int * ssrc = (const int *)(g_scales + (size_t)rec0 * 4 * MXE_PAIR_SCALES);
            int * sdst = (int *)(lds + (size_t)chunk_pairs * MXE_PAIR_BYTES);
            for (int i0 = tid; i0 < n_rec * 4 * 64; i0 += 1024) sdst[i0] = ssrc[i0];
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < MAXP; ++i) {
            if (i >= n_mine) break;
            f4v & x0 = acc[i][0], & x1 = acc[i][1];
            for (int cg = 0; cg < 2 * n_rec; cg += 2) {
                {
                    const uint8_t * po = l_ops + (size_t)(2 * cg) * MXE_PAIR_BYTES;
                    const int * ps = l_scales + (2 * cg) * 64;
                    mxe_pair<0>(G0[0].a[0], G0[0].e, G0[1].a[0], G0[1].e, po, ps, lane, x0, x1);
                    mxe_pair<1>(G0[0].a[1], G0[0].e, G0[1].a[1], G0[1].e, po + MXE_PAIR_BYTES, ps + 64, lane, x0, x1);
                    asm volatile("" : "+v"(x0), "+v"(x1) : : "memory");
                    __builtin_amdgcn_sched_barrier(0);
                    mxe_load(G0[0], lp, 0, lane_at); mxe_load(G0[1], lp + second, 0, lane_at);
                    __builtin_amdgcn_sched_barrier(0);
                    advance();
                }
                {
                    const uint8_t * po = l_ops + (size_t)(2 * cg + 2) * MXE_PAIR_BYTES;
                    const int * ps = l_scales + (2 * cg + 2) * 64;
                    mxe_pair<2>(G1[0].a[0], G1[0].e, G1[1].a[0], G1[1].e, po, ps, lane, x0, x1);
                    mxe_pair<3>(G1[0].a[1], G1[0].e, G1[1].a[1], G1[1].e, po + MXE_PAIR_BYTES, ps + 64, lane, x0, x1);
                    asm volatile("" : "+v"(x0), "+v"(x1) : : "memory");
                    __builtin_amdgcn_sched_barrier(0);
                    mxe_load(G1[0], lp, 1, lane_at); mxe_load(G1[1], lp + second, 1, lane_at);
                    __builtin_amdgcn_sched_barrier(0);
                    advance();
                }
            }
        }
        __syncthreads();
    }
    // lane l holds pair slot slot0 + l % 16, rows 4 (l / 16) .. + 3 of a tile
    float * row = a.out + (size_t)(slot0 + r) * a.N;
#pragma unroll
    for (int i = 0; i < MAXP; ++i) {
        if (i >= n_mine) break;
        if (GATE_UP) {
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float gv = acc[i][0][e];
                v[e] = fminf(fmaxf((gv / (1.0f + __expf(-gv))) * acc[i][1][e], -65504.0f), 65504.0f);
            }
            *(float4 *)(row + (size_t)(ip0 + i) * 16 + 4 * q) = make_float4(v[0], v[1], v[2], v[3]);
        } else {
#pragma unroll
            for (int tl = 0; tl < 2; ++tl)
                *(float4 *)(row + (size_t)(2 * (ip0 + i) + tl) * 16 + 4 * q) = make_float4(acc[i][tl][0], acc[i][tl][1], acc[i][tl][2], acc[i][tl][3]);
        }
    }
}

}  // namespace

bool mxs_can(int64_t K, int64_t N, int n_tokens) {
    return K > 0 && N > 0 && K % 256 == 0 && N % 16 == 0 && n_tokens >= 1 && n_tokens <= MXS_MAX_TOKENS &&
           mxs_lds_bytes((int)K) <= 160 * 1024;
}

size_t mxs_packed_bytes(int64_t K, int64_t N) { return (size_t)(N / 16) * (size_t)(K / 256) * MXS_RECORD; }
size_t mxs_operand_bytes(int K) { return (size_t)(K / 32) * 1024; }
size_t mxs_scale_bytes(int K) { return (size_t)(K / 32) * 16 * sizeof(float); }
size_t mxs_lds_bytes(int K) { return std::max<size_t>(mxs_operand_bytes(K), 64 * 1024) + std::max<size_t>(mxs_scale_bytes(K), 4096); }

void mxs_repack(hipStream_t s, const uint8_t * raw, uint8_t * packed, int K, int64_t N) {
    const size_t total = (size_t)N * (K / 32);
    hipLaunchKernelGGL(k_mxs_repack, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, raw, packed, K / 32, total);
    check_launch("k_mxs_repack");
}

void mxs_quantise(hipStream_t s, const float * x, int n_tokens, int K, uint8_t * operands, float * scales) {
    const int total = K / 32 * 16;
    hipLaunchKernelGGL(k_mxs_quantise, dim3((total + 255) / 256), dim3(256), 0, s, x, n_tokens, K, operands, scales);
    check_launch("k_mxs_quantise");
}

void mxs_matmul(hipStream_t s, const uint8_t * packed, const uint8_t * operands, const float * scales, int K, int64_t N,
                int n_tokens, float * y) {
    if (!mxs_can(K, N, n_tokens)) throw std::runtime_error("mxfp4 scaled: rows in 16s, columns in 256s, 1..16 tokens, operands within LDS");
    static bool raised = false;
    if (!raised) {
        HIP_OK(hipFuncSetAttribute((const void *)k_mxs, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        raised = true;
    }
    MxsArgs a{packed, operands, scales, y, K / 32, (int)(N / 16), n_tokens, (int)N};
    const int groups = std::min(256, (a.n_tiles + 15) / 16);
    hipLaunchKernelGGL(k_mxs, dim3(groups), dim3(1024), mxs_lds_bytes(K), s, a);
    check_launch("k_mxs");
}


// ---- the exact arithmetic (k_mxe)
size_t mxe_operand_bytes(int K) { return (size_t)(K / 64) * MXE_PAIR_BYTES; }
size_t mxe_scale_bytes(int K) { return (size_t)(K / 64) * MXE_PAIR_SCALES; }
bool mxe_can(int64_t K, int64_t N, int n_tokens) {
    return K > 0 && N > 0 && K % 256 == 0 && N % 32 == 0 && n_tokens >= 1 && n_tokens <= MXS_MAX_TOKENS;
}

void mxe_pieces(hipStream_t s, const float * x, int n_tokens, int K, uint8_t * operands, uint8_t * scales) {
    const int total = K / 32 * 16;
    hipLaunchKernelGGL(k_mxe_pieces, dim3((total + 255) / 256), dim3(256), 0, s, x, n_tokens, K, operands, scales);
    check_launch("k_mxe_pieces");
}

void mxe_matmul(hipStream_t s, const uint8_t * packed, const uint8_t * operands, const uint8_t * scales, int K, int64_t N,
                int n_tokens, float * y) {
    if (!mxe_can(K, N, n_tokens)) throw std::runtime_error("mxfp4 scaled, exact: rows in 32s, columns in 256s, 1..16 tokens");
    static bool raised = false;
    if (!raised) {
        HIP_OK(hipFuncSetAttribute((const void *)k_mxe, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        raised = true;
    }
    const int ng = K / 256;
    const int n_chunks = (ng + 5) / 6, chunk_records = (ng + n_chunks - 1) / n_chunks;      // at most six records' operands in LDS
    MxeArgs a{packed, operands, scales, y, K / 32, (int)(N / 16), n_tokens, (int)N, chunk_records, n_chunks};
    const int groups = std::min(256, (a.n_tiles / 2 + 31) / 32);
    const size_t lds = (size_t)chunk_records * 4 * (MXE_PAIR_BYTES + MXE_PAIR_SCALES);
    hipLaunchKernelGGL(k_mxe, dim3(groups), dim3(1024), lds, s, a);
    check_launch("k_mxe");
}

// ---- the expert block of a mixture-of-experts step on k_mxe_moe
bool mxe_moe_can(int E, int F) { return E % 256 == 0 && F % 256 == 0 && E > 0 && F > 0; }
size_t mxe_moe_operand_bytes(int K, size_t slots) { return slots / 16 * (size_t)(K / 64) * MXE_PAIR_BYTES; }
size_t mxe_moe_scale_bytes(int K, size_t slots) { return slots / 16 * (size_t)(K / 64) * MXE_PAIR_SCALES; }

template <bool GATE_UP, int MAXP>
static void mxe_moe_launch_as(hipStream_t s, const MxeMoeArgs & a, unsigned grid, size_t lds) {
    static bool raised = false;
    if (!raised) {
        // (the kernel also holds a word of static LDS: six records' operands are 150 KiB)
        HIP_OK(hipFuncSetAttribute((const void *)k_mxe_moe<GATE_UP, MAXP>, hipFuncAttributeMaxDynamicSharedMemorySize, 152 * 1024));
        raised = true;
    }
    hipLaunchKernelGGL((k_mxe_moe<GATE_UP, MAXP>), dim3(grid), dim3(1024), lds, s, a);
}

static void mxe_moe_launch(hipStream_t s, bool gate_up, const uint8_t * w0, const uint8_t * w1, const uint8_t * ops,
                           const uint8_t * scales, const int32_t * off_pad, int n_expert, size_t slots, int K, int N, float * out) {
    MxeMoeArgs a {};
    a.w0 = w0; a.w1 = w1; a.ops = ops; a.scales = scales; a.off_pad = off_pad; a.n_expert = n_expert; a.out = out;
    a.nb = K / 32; a.tiles_per_expert = N / 16; a.N = N;
    // a workgroup of 16 waves takes a group of 16 pair slots and, when it can, all tile pairs of the expert (up to
    // four per wave): the fewer workgroups share a group, the less its operands are re-read, and about one
    // workgroup per expert fits the chip in one turn
    const int n_pairs = gate_up ? N / 16 : N / 32;
    const int maxp = std::min(4, (n_pairs + 15) / 16);
    a.parts = (n_pairs + 16 * maxp - 1) / (16 * maxp);
    const int ng = K / 256;
    a.n_chunks = (ng + 5) / 6;
    a.chunk_records = (ng + a.n_chunks - 1) / a.n_chunks;
    const size_t lds = (size_t)a.chunk_records * 4 * (MXE_PAIR_BYTES + MXE_PAIR_SCALES);
    const unsigned grid = (unsigned)(slots / 16 * a.parts);
#define RK_MXE_MOE(GU)                                                          \
    switch (maxp) {                                                             \
        case 1: mxe_moe_launch_as<GU, 1>(s, a, grid, lds); break;               \
        case 2: mxe_moe_launch_as<GU, 2>(s, a, grid, lds); break;               \
        case 3: mxe_moe_launch_as<GU, 3>(s, a, grid, lds); break;               \
        default: mxe_moe_launch_as<GU, 4>(s, a, grid, lds); break;              \
    }
    if (gate_up) { RK_MXE_MOE(true) } else { RK_MXE_MOE(false) }
#undef RK_MXE_MOE
    check_launch("k_mxe_moe");
}

void mxe_moe_gate_up(hipStream_t s, const uint8_t * gate, const uint8_t * up, const Act & x, int E, int F, int n_expert,
                     const int32_t * off_pad, const int32_t * tok_of_q, size_t slots, uint8_t * ops, uint8_t * scales, float * h) {
    if (!mxe_moe_can(E, F) || !x.x) throw std::runtime_error("mxe_moe_gate_up: widths in 256s and plain activation planes");
    const size_t threads = slots * (size_t)(E / 32);
    hipLaunchKernelGGL(k_mxe_moe_pieces<true>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, x.x, (const float *)nullptr, E,
                       off_pad, tok_of_q, n_expert, ops, scales);
    check_launch("k_mxe_moe_pieces");
    mxe_moe_launch(s, true, gate, up, ops, scales, off_pad, n_expert, slots, E, F, h);
}

void mxe_moe_down(hipStream_t s, const uint8_t * down, const float * h, int E, int F, int n_expert, const int32_t * off_pad,
                  const int32_t * tok_of_q, size_t slots, uint8_t * ops, uint8_t * scales, float * out_pair) {
    if (!mxe_moe_can(E, F) || E % 32 != 0) throw std::runtime_error("mxe_moe_down: widths in 256s");
    const size_t threads = slots * (size_t)(F / 32);
    hipLaunchKernelGGL(k_mxe_moe_pieces<false>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, (const __half *)nullptr, h, F,
                       off_pad, tok_of_q, n_expert, ops, scales);
    check_launch("k_mxe_moe_pieces");
    mxe_moe_launch(s, false, down, nullptr, ops, scales, off_pad, n_expert, slots, F, E, out_pair);
}

}  // namespace rk
