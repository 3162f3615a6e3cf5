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

}  // namespace rk
