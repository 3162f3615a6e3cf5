// Tile matmul with the activations staged through LDS.
//
// y[t][n] = sum_k W[n][k] * x[t][k] for one chunk of up to 64 tokens. At batch
// 64 the activations (64 tokens x K x hi/lo f16 = 256 B per k) outweigh the
// 16-row weight tile of a wave (9 B per k), so the activations are what must
// be reused:
//
//   * a workgroup of 4 waves covers 4*R row tiles of 16 weight rows and all
//     token tiles; the activations of one 256-wide super-block column are
//     copied global -> LDS once per workgroup with direct-to-LDS loads
//     (global_load_lds_dwordx4), already in MFMA operand order, double buffered;
//   * each wave reads an operand from LDS once per k-step and uses it for its R
//     row tiles;
//   * the weights of the next super-block are prefetched into registers while
//     the current one is multiplied.
//
// Few row tiles (N = 4096 at batch 64) do not give every CU a workgroup, so K
// can also be split across workgroups: each writes its partial sums to a
// workspace, and the workgroup that finishes last for a row group adds the
// partials in slice order - the result does not depend on which one is last.
#include "dev_common.hpp"

namespace rk {

namespace {

template <int NT> struct XStage {
    // 1 KiB blocks: [kstep 8][hi/lo 2][tile NT] activations, then [tile NT] block sums
    static constexpr int X_BLOCKS = 8 * 2 * NT;
    static constexpr int BLOCKS = X_BLOCKS + NT;
    static constexpr int BYTES = BLOCKS * 1024;
};

// Per-lane source pointers of the activation staging, computed once per kernel:
// wave w always stages token tile w % NT, and 4/NT waves share the sixteen
// (k-step, hi/lo) blocks of a tile.
template <int NT> struct StageSrc {
    const __half * x;        // row of this lane's token in a.x, at k = 8g
    ptrdiff_t lo_delta;      // a.x_lo - a.x (halves)
    const __half * sum;      // this lane's block-sum source (hi, lo or zeros)
    int sum_stride;          // halves to advance per super-block (0 for the zeros)
    int tile, slot;
};

template <int NT>
__device__ __forceinline__ StageSrc<NT> stage_prepare(const MMArgs & a, int tbase, int lane, int wave) {
    static_assert(NT == 1 || NT == 2 || NT == 4, "token tiles per chunk");
    StageSrc<NT> s;
    const int r16 = lane & 15, g = lane >> 4;
    s.tile = wave % NT;
    s.slot = wave / NT;
    const int tok = min(tbase + s.tile * 16 + r16, a.T - 1);
    s.x = a.x + (size_t)tok * a.K + 8 * g;
    s.lo_delta = a.x_lo - a.x;
    const int nblk = a.K >> 5;
    if (g == 0) { s.sum = a.xs_hi + (size_t)tok * nblk; s.sum_stride = 8; }
    else if (g == 1) { s.sum = a.xs_lo + (size_t)tok * nblk; s.sum_stride = 8; }
    else { s.sum = a.zeros; s.sum_stride = 0; }
    return s;
}

// Issues the direct-to-LDS loads of one super-block column of activations.
template <int NT>
__device__ __forceinline__ void stage_x(const StageSrc<NT> & s, int sb, uint8_t * buf, bool with_sums) {
    constexpr int WAVES_PER_TILE = 4 / NT;
    constexpr int PER_WAVE = 16 / WAVES_PER_TILE;
#pragma unroll
    for (int j = 0; j < PER_WAVE; ++j) {
        const int c = s.slot + WAVES_PER_TILE * j;      // (k-step, hi/lo) combination, wave-uniform
        const int ks = c >> 1, hl = c & 1;
        const __half * src = s.x + (size_t)sb * 256 + ks * 32 + (hl ? s.lo_delta : 0);
        __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)src,
                                         (void __attribute__((address_space(3))) *)(buf + ((ks * 2 + hl) * NT + s.tile) * 1024),
                                         16, 0, 0);
    }
    if (with_sums && s.slot == 0) {
        const __half * src = s.sum + (size_t)sb * s.sum_stride;
        __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)src,
                                         (void __attribute__((address_space(3))) *)(buf + (XStage<NT>::X_BLOCKS + s.tile) * 1024),
                                         16, 0, 0);
    }
}

__device__ __forceinline__ h8 lds_h8(const uint8_t * buf, int block, int lane) {
    return *(const h8 *)(buf + block * 1024 + lane * 16);
}

// Stores or reduces the accumulators. acc[r][t][i] is token tbase + 16t + 4g + i,
// weight row 16 * rt[r] + r16.
template <int NT, int R>
__device__ __forceinline__ void finish(const MMArgs & a, f4 (&acc)[R][NT], const int (&rt)[R], int tbase, int nt,
                                       int rg, int ks, int * flag) {
    const int lane = threadIdx.x & 63;
    const int r16 = lane & 15, g = lane >> 4;
    if (a.ksplit > 1) {
        const size_t tpad = (size_t)gridDim.y * 64;
        float * mine = a.partial + (size_t)ks * tpad * a.N;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (rt[r] >= a.n_row_tiles) continue;
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const size_t tok = (size_t)tbase + t * 16 + 4 * g + i;
                    mine[tok * a.N + rt[r] * 16 + r16] = acc[r][t][i];
                }
        }
        __threadfence();
        __syncthreads();
        if (threadIdx.x == 0) {
            int32_t * c = a.counters + rg * gridDim.y + blockIdx.y;
            const int prev = atomicAdd(c, 1);
            const int last = prev == a.ksplit - 1;
            if (last) *c = 0;              // ready for the next launch
            *flag = last;
        }
        __syncthreads();
        if (!*flag) return;
        __threadfence();
        // Every partial address was written exactly once, by one workgroup, before
        // its counter increment: plain loads see it. Slice order is the sum order.
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < NT; ++t) acc[r][t] = (f4){0.f, 0.f, 0.f, 0.f};
        for (int k = 0; k < a.ksplit; ++k) {
            const float * slice = a.partial + (size_t)k * tpad * a.N;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (rt[r] >= a.n_row_tiles) continue;
#pragma unroll
                for (int t = 0; t < NT; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const size_t tok = (size_t)tbase + t * 16 + 4 * g + i;
                        acc[r][t][i] += slice[tok * a.N + rt[r] * 16 + r16];
                    }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (rt[r] >= a.n_row_tiles) continue;
        const int n = rt[r] * 16 + r16;
        const float bias = a.bias ? a.bias[n] : 0.0f;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            if (t >= nt) break;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int tok = tbase + t * 16 + 4 * g + i;
                if (tok < a.T) {
                    float * p = a.y + (size_t)tok * a.ldy + a.col0 + n;
                    const float v = acc[r][t][i] + bias;
                    *p = a.mode == MM_ADD ? *p + v : v;
                }
            }
        }
    }
}

}  // namespace

template <int NT, int R>
__global__ __launch_bounds__(256, 1) void k_mm2_q4k(MMArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ int flag;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int rg = blockIdx.x % a.n_row_groups, ks = blockIdx.x / a.n_row_groups;
    const int tbase = blockIdx.y * 64;
    const int nt = min(NT, (a.T - tbase + 15) >> 4);
    const int nsb = a.K >> 8;
    const int per = (nsb + a.ksplit - 1) / a.ksplit;
    const int sb0 = ks * per, sb1 = min(nsb, sb0 + per);

    int rt[R];
#pragma unroll
    for (int r = 0; r < R; ++r) rt[r] = (rg * 4 + wave) * R + r;
    const StageSrc<NT> stage = stage_prepare<NT>(a, tbase, lane, wave);

    f4 acc[R][NT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[r][t] = (f4){0.f, 0.f, 0.f, 0.f};

    const uint8_t * wbase[R];
#pragma unroll
    for (int r = 0; r < R; ++r) wbase[r] = a.w + (size_t)min(rt[r], a.n_row_tiles - 1) * nsb * 2304;
    // weights of one super-block of every row tile: header, two payload loads
    u4 hdr[R], q0[R], q1[R], n_hdr[R], n_q0[R], n_q1[R];
    auto load_w = [&](int sb, u4 (&h)[R], u4 (&p0)[R], u4 (&p1)[R]) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            // rows past the matrix read the last tile; their results are never stored
            const uint8_t * tile = wbase[r] + (size_t)sb * 2304;
            h[r] = *(const u4 *)(tile + r16 * 16);
            p0[r] = *(const u4 *)(tile + 256 + lane * 16);
            p1[r] = *(const u4 *)(tile + 1280 + lane * 16);
        }
    };

    if (sb0 < sb1) {
        stage_x<NT>(stage, sb0, smem, true);
        load_w(sb0, hdr, q0, q1);
    }
    for (int sb = sb0; sb < sb1; ++sb) {
        uint8_t * cur = smem + ((sb - sb0) & 1) * XStage<NT>::BYTES;
        uint8_t * nxt = smem + ((sb - sb0 + 1) & 1) * XStage<NT>::BYTES;
        // everything issued for this super-block has landed, and every wave is
        // done reading the buffer the next loads overwrite
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (sb + 1 < sb1) {
            if (!(a.debug & 1)) stage_x<NT>(stage, sb + 1, nxt, true);
            load_w(sb + 1, n_hdr, n_q0, n_q1);
        }
        if (a.debug & 1) cur = smem;

        f4 accq[R][NT];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < NT; ++t) accq[r][t] = (f4){0.f, 0.f, 0.f, 0.f};
        // 6-bit scales and mins of the 8 sub-blocks, as bytes: sc in the low, min in the high half-word pairs
        uint32_t sc[R][8], mn[R][8];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t lo_b = (hdr[r].y >> (8 * j)) & 0xff;
                const uint32_t md_b = (hdr[r].z >> (8 * j)) & 0xff;
                const uint32_t hi_b = (hdr[r].w >> (8 * j)) & 0xff;
                sc[r][j] = lo_b & 63;
                mn[r][j] = md_b & 63;
                sc[r][j + 4] = (hi_b & 0x0f) | ((lo_b >> 6) << 4);
                mn[r][j + 4] = (hi_b >> 4) | ((md_b >> 6) << 4);
            }
        // min term: k-slots of lane group 0 carry the hi block sums, group 1 the lo sums
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const h8 sA = lds_h8(cur, XStage<NT>::X_BLOCKS + t, lane);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                h8 mB;
#pragma unroll
                for (int i = 0; i < 8; ++i) mB[i] = g < 2 ? (_Float16)(float)mn[r][i] : (_Float16)0.0f;
                const f4 m4 = __builtin_amdgcn_mfma_f32_16x16x32_f16(sA, mB, (f4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                const float ndmin = -h2f((uint16_t)(hdr[r].x >> 16));
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[r][t][i] = fmaf(ndmin, m4[i], acc[r][t][i]);
            }
        }
        if (!(a.debug & 2))
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            h8 A[NT], Al[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                A[t] = lds_h8(cur, (s * 2 + 0) * NT + t, lane);
                Al[t] = lds_h8(cur, (s * 2 + 1) * NT + t, lane);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t wq = s < 4 ? q0[r][s & 3] : q1[r][s & 3];
                const _Float16 sch = (_Float16)(float)sc[r][s];
                const h2 k1 = {sch, sch};
                const h2 c1 = k1 * (_Float16)(-1024.0f);
                const h2 k2 = k1 * (_Float16)(0.0625f);
                const h2 c2 = k1 * (_Float16)(-64.0f);
                const uint32_t w8 = wq >> 8;
                const h2 u0 = __builtin_bit_cast(h2, (wq & 0x000F000Fu) | 0x64006400u);
                const h2 u1 = __builtin_bit_cast(h2, (wq & 0x00F000F0u) | 0x64006400u);
                const h2 u2 = __builtin_bit_cast(h2, (w8 & 0x000F000Fu) | 0x64006400u);
                const h2 u3 = __builtin_bit_cast(h2, (w8 & 0x00F000F0u) | 0x64006400u);
                const h2 a0 = __builtin_elementwise_fma(u0, k1, c1);   // exactly sc * e (<= 945)
                const h2 a1 = __builtin_elementwise_fma(u1, k2, c2);
                const h2 a2 = __builtin_elementwise_fma(u2, k1, c1);
                const h2 a3 = __builtin_elementwise_fma(u3, k2, c2);
                const h8 B = {a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    accq[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[t], B, accq[r][t], 0, 0, 0);
                    accq[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Al[t], B, accq[r][t], 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float d = h2f((uint16_t)(hdr[r].x & 0xffff));
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[r][t][i] = fmaf(d, accq[r][t][i], acc[r][t][i]);
        }
#pragma unroll
        for (int r = 0; r < R; ++r) { hdr[r] = n_hdr[r]; q0[r] = n_q0[r]; q1[r] = n_q1[r]; }
    }
    finish<NT, R>(a, acc, rt, tbase, nt, rg, ks, &flag);
}

template <int NT, int R>
__global__ __launch_bounds__(256, 1) void k_mm2_q8_0(MMArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ int flag;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15;
    const int rg = blockIdx.x % a.n_row_groups, ks = blockIdx.x / a.n_row_groups;
    const int tbase = blockIdx.y * 64;
    const int nt = min(NT, (a.T - tbase + 15) >> 4);
    const int nsb = a.K >> 8;
    const int per = (nsb + a.ksplit - 1) / a.ksplit;
    const int sb0 = ks * per, sb1 = min(nsb, sb0 + per);

    int rt[R];
#pragma unroll
    for (int r = 0; r < R; ++r) rt[r] = (rg * 4 + wave) * R + r;
    const StageSrc<NT> stage = stage_prepare<NT>(a, tbase, lane, wave);
    f4 acc[R][NT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[r][t] = (f4){0.f, 0.f, 0.f, 0.f};

    const uint8_t * wbase[R];
#pragma unroll
    for (int r = 0; r < R; ++r) wbase[r] = a.w + (size_t)min(rt[r], a.n_row_tiles - 1) * nsb * 4352;
    u4 hdr[R], q[R][4], n_hdr[R], n_q[R][4];
    auto load_w = [&](int sb, u4 (&h)[R], u4 (&p)[R][4]) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint8_t * tile = wbase[r] + (size_t)sb * 4352;
            h[r] = *(const u4 *)(tile + r16 * 16);
#pragma unroll
            for (int j = 0; j < 4; ++j) p[r][j] = *(const u4 *)(tile + 256 + j * 1024 + lane * 16);
        }
    };
    const h2 bias1152 = {(_Float16)(-1152.0f), (_Float16)(-1152.0f)};

    if (sb0 < sb1) {
        stage_x<NT>(stage, sb0, smem, false);
        load_w(sb0, hdr, q);
    }
    for (int sb = sb0; sb < sb1; ++sb) {
        uint8_t * cur = smem + ((sb - sb0) & 1) * XStage<NT>::BYTES;
        uint8_t * nxt = smem + ((sb - sb0 + 1) & 1) * XStage<NT>::BYTES;
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (sb + 1 < sb1) {
            stage_x<NT>(stage, sb + 1, nxt, false);
            load_w(sb + 1, n_hdr, n_q);
        }
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            h8 A[NT], Al[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                A[t] = lds_h8(cur, (s * 2 + 0) * NT + t, lane);
                Al[t] = lds_h8(cur, (s * 2 + 1) * NT + t, lane);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t sw = hdr[r][s >> 1];
                const float d = h2f((uint16_t)((s & 1) ? (sw >> 16) : (sw & 0xffff)));
                const u4 d4 = q[r][s >> 1];
                const int half = s & 1;
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
                    f4 part = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[t], B, (f4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                    part = __builtin_amdgcn_mfma_f32_16x16x32_f16(Al[t], B, part, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[r][t][i] = fmaf(d, part[i], acc[r][t][i]);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            hdr[r] = n_hdr[r];
#pragma unroll
            for (int j = 0; j < 4; ++j) q[r][j] = n_q[r][j];
        }
    }
    finish<NT, R>(a, acc, rt, tbase, nt, rg, ks, &flag);
}

template <int NT, int R>
static void launch2(hipStream_t s, int type, const MMArgs & a, dim3 grid) {
    const size_t lds = 2 * (size_t)XStage<NT>::BYTES;
    if (type == WT_Q4_K) {
        static bool once = false;
        if (!once) {
            HIP_OK(hipFuncSetAttribute((const void *)k_mm2_q4k<NT, R>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            once = true;
        }
        hipLaunchKernelGGL((k_mm2_q4k<NT, R>), grid, dim3(256), lds, s, a);
    } else {
        static bool once = false;
        if (!once) {
            HIP_OK(hipFuncSetAttribute((const void *)k_mm2_q8_0<NT, R>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            once = true;
        }
        hipLaunchKernelGGL((k_mm2_q8_0<NT, R>), grid, dim3(256), lds, s, a);
    }
}

size_t matmul_workspace_bytes() {
    // partial sums of a split matmul (<= 64 tokens x 16 slices x 8192 columns), counters, zeros
    return (size_t)64 * 16 * 8192 * 4 + 65536 + 256;
}

// The LDS-staged path; ws must be zero-initialised once.
int g_mm_debug = 0;
int g_mm_force_ksplit = 0;
int g_mm_force_r = 0;

template <int R>
static void dispatch_nt(hipStream_t s, int type, int nt, const MMArgs & a, dim3 grid) {
    switch (nt) {
        case 1: launch2<1, R>(s, type, a, grid); break;
        case 2: launch2<2, R>(s, type, a, grid); break;
        default: launch2<4, R>(s, type, a, grid); break;
    }
}

void matmul_lds(hipStream_t s, const Weight & w, const Act & x, int T, float * y, int ldy, int col0,
                int mode, const float * bias, void * ws) {
    MMArgs a {};
    a.debug = g_mm_debug;
    a.w = w.packed; a.x = x.x; a.x_lo = x.x_lo; a.xs_hi = x.xs_hi; a.xs_lo = x.xs_lo; a.y = y; a.bias = bias;
    a.K = w.K; a.N = w.N; a.T = T; a.ldy = ldy; a.col0 = col0; a.mode = mode;
    a.n_row_tiles = w.N / 16;
    const size_t partial_bytes = (size_t)64 * 16 * 8192 * 4;
    a.partial = (float *)ws;
    a.counters = (int32_t *)((uint8_t *)ws + partial_bytes);
    a.zeros = (const __half *)((uint8_t *)ws + partial_bytes + 65536);
    const int nsb = w.K / 256;
    const int nt = T > 32 ? 4 : (T > 16 ? 2 : 1);
    const int chunks = (T + 63) / 64;
    const int R = g_mm_force_r == 4 ? 4 : 2;
    a.n_row_groups = (a.n_row_tiles + 4 * R - 1) / (4 * R);
    // Split K across workgroups when the row groups alone leave most CUs idle
    // (decode-sized batches only: the partial buffer holds one 64-token chunk).
    int ksplit = 1;
    if (chunks == 1) {
        while (a.n_row_groups * ksplit < 192 && ksplit * 2 <= 16 && nsb / (ksplit * 2) >= 2
               && (size_t)ksplit * 2 * 64 * w.N * 4 <= partial_bytes && a.n_row_groups * ksplit * 2 <= 16384) {
            ksplit *= 2;
        }
    }
    if (g_mm_force_ksplit > 0 && chunks == 1) ksplit = g_mm_force_ksplit;
    if ((size_t)ksplit * 64 * w.N * 4 > partial_bytes || (ksplit > 1 && a.n_row_groups > 16384)) {
        throw std::runtime_error("matmul_lds: the split does not fit the workspace");
    }
    a.ksplit = ksplit;
    dim3 grid(a.n_row_groups * ksplit, chunks);
    if (R == 4) dispatch_nt<4>(s, w.type, nt, a, grid);
    else dispatch_nt<2>(s, w.type, nt, a, grid);
    check_launch("matmul_lds");
}

}  // namespace rk
