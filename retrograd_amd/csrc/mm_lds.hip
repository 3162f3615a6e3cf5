// Tile matmul with the activations staged through LDS.
//
// y[t][n] = sum_k W[n][k] * x[t][k] for one chunk of up to 64 tokens. At batch
// 64 the activations (64 tokens x K x hi/lo f16 = 256 B per k) outweigh the
// 16-row weight tile of a wave (9 B per k), so the activations are what must
// be reused:
//
//   * a workgroup of 8 waves (4 row waves x 2 halves of every 256-wide
//     super-block) covers 4*R row tiles of 16 weight rows and all token tiles;
//     the activations of one super-block column are copied global -> LDS once
//     per workgroup with direct-to-LDS loads (global_load_lds_dwordx4),
//     already in MFMA operand order, double buffered;
//   * each wave reads an operand from LDS once per k-step and uses it for its R
//     row tiles;
//   * the weights of the next super-blocks are prefetched into registers while
//     the current one is multiplied;
//   * the two halves add their accumulators through LDS, and the sums leave
//     the workgroup as whole token rows.
//
// k_mm2_* are the general kernels (any number of token tiles, Q4_K and Q8_0);
// k_mm5_q4k is the kernel of the decode step (Q4_K, a full 64-token chunk).
//
// Few row tiles (N = 4096 at batch 64) do not give every CU a workgroup, so K
// can also be split across workgroups: each writes its sums over its slice of K
// to a workspace, and whoever consumes the result adds the slices in slice
// order (the next kernel of the step, or reduce_slices) - no workgroup waits
// for another and the sum order is fixed.
#include <type_traits>
#include "dev_common.hpp"

namespace rk {

namespace {

constexpr int kWaves = 8;      // 4 row waves x 2 halves of every super-block
constexpr int kThreads = kWaves * 64;

// In the general kernels the weight loads are loads the compiler knows: a load issued from
// inline assembly hands the compiler a register whose value arrives later, and
// any copy the register allocator makes of it before the wait (one was seen at
// a loop latch) reads stale data. The compiler counts only the loads it knows,
// so its own waits can only be stricter than needed, never too weak. (The
// decode kernel k_mm5_q4k keeps its prefetch in registers the compiler does not
// allocate at all.) They go through a buffer descriptor: `n_bytes` from `base` on
// (under 4 GiB), wave-uniform; a lane reads at lane_off + uniform_off, and a read
// past n_bytes returns zero instead of touching memory.
typedef __amdgpu_buffer_rsrc_t WeightRows;
__device__ __forceinline__ WeightRows weight_rows(const void * base, uint32_t n_bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)n_bytes, 0x00020000);
}
__device__ __forceinline__ u4 load16(WeightRows rows, uint32_t lane_off, uint32_t uniform_off) {
    return __builtin_bit_cast(u4, __builtin_amdgcn_raw_buffer_load_b128(rows, (int)lane_off, (int)uniform_off, 0));
}
typedef uint32_t u2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u2 load8(WeightRows rows, uint32_t lane_off, uint32_t uniform_off) {
    return __builtin_bit_cast(u2, __builtin_amdgcn_raw_buffer_load_b64(rows, (int)lane_off, (int)uniform_off, 0));
}
__device__ __forceinline__ uint32_t load4(WeightRows rows, uint32_t lane_off, uint32_t uniform_off) {
    return __builtin_amdgcn_raw_buffer_load_b32(rows, (int)lane_off, (int)uniform_off, 0);
}

template <int NT> struct XStage {
    // 1 KiB blocks: [kstep 8][hi/lo 2][tile NT] activations, then [tile NT] block sums
    static constexpr int X_BLOCKS = 8 * 2 * NT;
    static constexpr int BLOCKS = X_BLOCKS + NT;
    static constexpr int BYTES = BLOCKS * 1024;
};

// Activation staging of a workgroup: wave w of the eight always stages token
// tile w % NT, and 8/NT waves share the sixteen (k-step, hi/lo) blocks of a
// tile. The activations are stored in operand order, so every request copies
// one contiguous 1 KiB block; the bases are wave-uniform, the lanes add lane * 16.
template <int NT> struct StageSrc {
    const __half * x;        // block (k-step 0, hi) of this wave's tile
    const __half * sum;      // block sums of super-block 0 of this wave's tile
    int tile, slot;
    uint32_t lane16;
    uint32_t lds0;           // LDS address of the first staging buffer
};

template <int NT>
__device__ __forceinline__ StageSrc<NT> stage_prepare(const MMArgs & a, int chunk, int lane, int wave, const uint8_t * smem) {
    static_assert(NT == 1 || NT == 2 || NT == 4, "token tiles per chunk");
    StageSrc<NT> s;
    s.tile = wave % NT;
    s.slot = wave / NT;
    s.x = a.x + (size_t)chunk * act_chunk_halves(a.K) + s.tile * 512;
    s.sum = a.sums ? a.sums + (size_t)chunk * act_sum_chunk_halves(a.K) + s.tile * 512 : nullptr;
    s.lane16 = lane * 16;
    s.lds0 = lds_offset(smem);
    return s;
}

// Requests one super-block column of activations into staging buffer `which`.
template <int NT>
__device__ __forceinline__ void stage_x(const StageSrc<NT> & s, int sb, int which, bool with_sums) {
    constexpr int WAVES_PER_TILE = 8 / NT;
    constexpr int PER_WAVE = 16 / WAVES_PER_TILE;
    const uint32_t buf = s.lds0 + which * XStage<NT>::BYTES;
#pragma unroll
    for (int j = 0; j < PER_WAVE; ++j) {
        const int c = s.slot + WAVES_PER_TILE * j;      // (k-step, hi/lo) block of the super-block, wave-uniform
        lds_dma16(s.x + (size_t)(sb * 16 + c) * 2048, s.lane16, buf + (c * NT + s.tile) * 1024);
    }
    if (with_sums && s.slot == 0) lds_dma16(s.sum + (size_t)sb * 2048, s.lane16, buf + (XStage<NT>::X_BLOCKS + s.tile) * 1024);
}

__device__ __forceinline__ h8 lds_h8(const uint8_t * buf, int block, int lane) {
    return *(const h8 *)(buf + block * 1024 + lane * 16);
}

// Second half of the epilogue: both k-halves have left their accumulators in
// LDS as [half][token][row of the group]; every wave stores whole token rows.
template <int NT, int R>
__device__ __forceinline__ void store_token_rows(const MMArgs & a, uint8_t * smem, int rg, int tbase, int ks) {
    constexpr int S = 64 * R + 4;
    constexpr int LPR = 16 * R;            // lanes per token row
    constexpr int TPI = 64 / LPR;          // token rows per store instruction
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
    const float * h0 = (const float *)smem, * h1 = h0 + NT * 16 * S;
    if (a.mode == MM_SWIGLU) {
        // eight lanes per token, eight hidden columns each: gate in columns c, up in columns 64 + c of the group
        static_assert(R == 2, "a row group is 64 gate rows and 64 up rows");
        const int c = (threadIdx.x & 7) * 8;
        const Act & out = a.act_out;
        for (int tk = threadIdx.x >> 3; tk < NT * 16; tk += kThreads / 8) {
            const int tok = tbase + tk;
            if (tok >= a.T || rg * 64 + c >= out.K) continue;      // the four lanes of a 32-wide block leave together
            const float * g0 = h0 + tk * S + c, * g1 = h1 + tk * S + c;
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; i += 4) {
                const f4 g = *(const f4 *)(g0 + i) + *(const f4 *)(g1 + i);
                const f4 u = *(const f4 *)(g0 + 64 + i) + *(const f4 *)(g1 + 64 + i);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[i + e] = (g[e] / (1.0f + __expf(-g[e]))) * u[e];
            }
            if (a.act_f32) {
                float * dst = a.act_f32 + (size_t)tok * out.K + rg * 64 + c;
                *(f4 *)dst = (f4){v[0], v[1], v[2], v[3]};
                *(f4 *)(dst + 4) = (f4){v[4], v[5], v[6], v[7]};
            } else {
                store_act8(v, out, tok, rg * 64 + c, threadIdx.x & 3);
            }
        }
        return;
    }
    const int col = (lane % LPR) * 4;
    const int n = rg * 64 * R + col;
    if (n >= a.N) return;
    const bool sliced = a.ksplit > 1;
    float * slice = sliced ? a.partial + (size_t)ks * a.slice_rows * a.pld + a.pcol : nullptr;
    const f4 bias = (a.bias && ks == 0) ? *(const f4 *)(a.bias + n) : (f4){0.f, 0.f, 0.f, 0.f};
    const int nrows = min(NT * 16, a.T - tbase);
    for (int tk = wave * TPI + lane / LPR; tk < nrows; tk += kWaves * TPI) {
        f4 v = *(const f4 *)(h0 + tk * S + col);
        v += *(const f4 *)(h1 + tk * S + col);
        v += bias;
        const int tok = tbase + tk;
        if (sliced) {
            *(f4 *)(slice + (size_t)tok * a.pld + n) = v;
        } else {
            float * p = a.y + (size_t)tok * a.ldy + a.col0 + n;
            if (a.mode == MM_ADD) v = *(const f4 *)p + v;
            *(f4 *)p = v;
        }
    }
}

// Adds the accumulators of the two k-halves of every row wave and stores the
// sums: to y, or (split K) to this workgroup's slice of the workspace, the
// bias going into slice 0. Both halves leave their accumulators in LDS as
// [token][row of the group]; then every wave stores whole token rows, 16 R
// lanes per row with four columns each, so each store instruction writes full
// cache lines (an accumulator tile stored from its registers covers only a
// 64-byte piece of four different rows per instruction, which was measured to
// cost several microseconds per launch at 64 tokens).
// acc[r][t][i] is token 16t + 4g + i of the chunk, row 16 (rw R + r) + r16 of the group.
template <int NT, int R>
__device__ __forceinline__ void join_and_store(const MMArgs & a, f4 (&acc)[R][NT], uint8_t * smem, int rg, int rw, int kh,
                                               int tbase, int ks) {
    constexpr int S = 64 * R + 4;          // floats per token row in LDS; the pad spreads the four token rows a store touches over the banks
    static_assert(2 * NT * 16 * S * 4 <= 2 * XStage<NT>::BYTES, "both halves' accumulators fit the staging buffers");
    const int lane = threadIdx.x & 63;
    const int r16 = lane & 15, g = lane >> 4;
    __syncthreads();       // every wave is done with the staged activations
    float * mine = (float *)smem + kh * (NT * 16 * S);
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) mine[(t * 16 + 4 * g + i) * S + (rw * R + r) * 16 + r16] = acc[r][t][i];
    store_token_rows<NT, R>(a, smem, rg, tbase, ks);
}

// The super-blocks sb0 .. sb1-1 of a K-slice through `body(sb, current set, set to request into)` with three
// weight sets in rotation: w0 and w1 hold (or are loading) sb0 and sb0 + 1 on entry. Always whole rounds of
// three: a body past the end of the slice still waits, synchronises and repeats the request for the last
// super-block, and only skips its arithmetic. The loop therefore has no exit in the middle of a round; with
// one, the compiled loop has an edge from mid-round back to its head on which the set about to be read looks
// as if it were still loading, and the compiler then waits at the head of every round until the requests
// just issued (the staging requests among them) have landed.
template <class WSet, class Body>
__device__ __forceinline__ void rotate_sets(int sb0, int sb1, WSet & w0, WSet & w1, WSet & w2, Body body) {
    for (int sb = sb0; sb < sb1; sb += 3) {
        body(sb, w0, w2);
        body(sb + 1, w1, w0);
        body(sb + 2, w2, w1);
    }
}

// (x & mask) | bits in one instruction
__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t bits) {
    uint32_t d;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(d) : "v"(x), "s"(mask), "v"(bits));
    return d;
}

// f16 pair (1024 + byte a, 1024 + byte b) of a word, bytes chosen by the selector
__device__ __forceinline__ h2 magic_pair(uint32_t word, uint32_t sel) {
    return __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, word, sel));
}


}  // namespace

// Which (row group, K-slice) a workgroup takes. The hardware hands workgroups to the eight XCDs in turn (workgroup b
// to XCD b % 8) and every XCD has an L2 of its own, so the activations of a K-slice are fetched once by every XCD
// that multiplies the slice: with row groups in the fast index every XCD staged every slice (measured: the
// down projection fetched 31 MB of activations beside 33 MB of weights). Here the slices are dealt to the XCDs first -
// with 8 slices XCD x multiplies slice x only - and an XCD's workgroups walk the row groups. The slice and the row
// group decide where a result goes, not the workgroup's number, so results do not change.
__device__ __forceinline__ void wg_place(const MMArgs & a, int b, int & rg, int & ks) {
    const int total = a.n_row_groups * a.ksplit;
    if (a.ksplit == 1 || (total & 7)) { rg = b % a.n_row_groups; ks = b / a.n_row_groups; return; }
    const int g = (a.ksplit & 7) == 0 ? 8 : (a.ksplit & 3) == 0 ? 4 : (a.ksplit & 1) == 0 ? 2 : 1;   // gcd(ksplit, 8)
    const int xcd = b & 7, j = b >> 3;
    const int idx = j * (8 / g) + xcd / g;       // the workgroup's number among those of its slice class xcd % g
    rg = idx % a.n_row_groups;
    ks = xcd % g + g * (idx / a.n_row_groups);
}


// FIVE: Q5_K - the same tile followed by a plane of fifth bits (one dword per k-half and lane), which one shift
// per use puts above the nibbles; sc * e stays an exact f16 (at most 63 * 31).
template <int NT, int R, bool FIVE = false>
__global__ __launch_bounds__(kThreads, NT <= 2 ? 4 : 1) void k_mm2_q4k(MMArgs a) {
    constexpr uint32_t TILE = FIVE ? 2816u : 2304u;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rw = wave & 3, kh = wave >> 2;
    const int r16 = lane & 15;
    int rg, ks;
    wg_place(a, blockIdx.x, rg, ks);
    const int tbase = blockIdx.y * 64;
    const int nsb = a.K >> 8;
    const int per = (nsb + a.ksplit - 1) / a.ksplit;
    const int sb0 = ks * per, sb1 = min(nsb, sb0 + per);

    int rt[R];
#pragma unroll
    for (int r = 0; r < R; ++r) rt[r] = (rg * 4 + rw) * R + r;
    const StageSrc<NT> stage = stage_prepare<NT>(a, blockIdx.y, lane, wave, smem);

    f4 acc[R][NT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[r][t] = (f4){0.f, 0.f, 0.f, 0.f};

    // rows past the matrix read the last tile; their results are never stored
    // A row tile's super-blocks are one buffer: the loads take the lane's offset and the super-block's as
    // they are, so no load needs an address computed into a vector register first. (With plain pointers the
    // compiler built each 64-bit address in the register the load was about to fill, and waited there for
    // loads it believed were still writing it: the staging requests it had just issued, every third super-block.)
    WeightRows wbase[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
        wbase[r] = weight_rows(a.w + (size_t)min(rt[r], a.n_row_tiles - 1) * nsb * TILE, (uint32_t)nsb * TILE);
    // this wave's weights of one super-block: the row headers and its half of the payload
    struct WSet { u4 hdr[R]; u4 q[R]; uint32_t top[R]; };
    constexpr int LOADS = FIVE ? 3 : 2;        // per row tile and set
    const uint32_t off_hdr = r16 * 16, off_q = 256 + kh * 1024 + lane * 16, off_top = 2304 + kh * 256 + lane * 4;
    auto load_w = [&](int sb, WSet & w) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            w.hdr[r] = load16(wbase[r], off_hdr, (uint32_t)sb * TILE);
            w.q[r] = load16(wbase[r], off_q, (uint32_t)sb * TILE);
            if (FIVE) w.top[r] = load4(wbase[r], off_top, (uint32_t)sb * TILE);
            else w.top[r] = 0;
        }
    };
    const h2 m1024 = {(_Float16)(-1024.0f), (_Float16)(-1024.0f)};
    const uint32_t magic1024 = 0x64006400u, magic64 = 0x54005400u;

    // One super-block: wait for its activations, start the loads of what comes
    // next (activations one super-block ahead, weights two), multiply.
    auto body = [&](int sb, WSet & w, WSet & fut) __attribute__((always_inline)) {
        uint8_t * cur = smem + ((sb - sb0) & 1) * XStage<NT>::BYTES;
        // All but the newest LOADS x R loads (the weights one super-block ahead) have
        // landed: this super-block's activations and weights are in.
        __builtin_amdgcn_s_waitcnt(0x0F70 | (LOADS * R));
        // the set is usable from here on and not before (nothing of it is to be touched, and so waited
        // for, inside the super-block before)
#pragma unroll
        for (int r = 0; r < R; ++r) {
            asm volatile("" : "+v"(w.hdr[r]), "+v"(w.q[r]));
            if (FIVE) asm volatile("" : "+v"(w.top[r]));
        }
        __syncthreads();   // ... for every wave, and nobody still reads the other buffer
        if (sb + 1 < sb1) stage_x<NT>(stage, sb + 1, (sb - sb0 + 1) & 1, true);
        load_w(min(sb + 2, sb1 - 1), fut);
        __builtin_amdgcn_sched_barrier(0);   // requested now, not wherever the scheduler finds room among the arithmetic
        if (sb >= sb1) return;       // past the slice: the round is only kept whole

        Q4KScales s4[R];
#pragma unroll
        for (int r = 0; r < R; ++r) s4[r] = q4k_scales(w.hdr[r]);

        // min term: k-slots of lane group 0 carry the hi block sums, group 1 the
        // lo sums, groups 2-3 zeros; the token tiles are shared out between the halves
        {
            h8 mB[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const h2 p0 = magic_pair(s4[r].mn[0], 0x04010400u) + m1024;
                const h2 p1 = magic_pair(s4[r].mn[0], 0x04030402u) + m1024;
                const h2 p2 = magic_pair(s4[r].mn[1], 0x04010400u) + m1024;
                const h2 p3 = magic_pair(s4[r].mn[1], 0x04030402u) + m1024;
                mB[r] = (h8){p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
            }
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                if ((NT == 1 ? 0 : (t & 1)) != kh) continue;
                const h8 sA = lds_h8(cur, XStage<NT>::X_BLOCKS + t, lane);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const f4 m4 = __builtin_amdgcn_mfma_f32_16x16x32_f16(sA, mB[r], (f4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                    const float ndmin = -h2f((uint16_t)(w.hdr[r].x >> 16));
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[r][t][i] = fmaf(ndmin, m4[i], acc[r][t][i]);
                }
            }
        }

        f4 accq[R][NT];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < NT; ++t) accq[r][t] = (f4){0.f, 0.f, 0.f, 0.f};
        const uint8_t * xk = cur + kh * (8 * NT * 1024);      // this half's four k-steps
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            h8 A[NT], Al[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                A[t] = lds_h8(xk, (j * 2 + 0) * NT + t, lane);
                Al[t] = lds_h8(xk, (j * 2 + 1) * NT + t, lane);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t scw = kh ? s4[r].sc[1] : s4[r].sc[0];
                const h2 k1 = magic_pair(scw, 0x04000400u + 0x00010001u * j) + m1024;   // (sc, sc)
                const h2 c1 = k1 * (_Float16)(-1024.0f);
                const h2 c2 = k1 * (_Float16)(-64.0f);
                const uint32_t wq = w.q[r][j];
                const uint32_t w8 = wq >> 8;
                // 1024 + e in the low nibble positions, 64 + e in the high ones
                uint32_t v0 = and_or(wq, 0x000F000Fu, magic1024), v1 = and_or(wq, 0x00F000F0u, magic64);
                uint32_t v2 = and_or(w8, 0x000F000Fu, magic1024), v3 = and_or(w8, 0x00F000F0u, magic64);
                if (FIVE) {
                    // the fifth bits of this k-step: elements 0, 4 (1, 5) at bits 2j, 2j + 1 (16 + 2j ..), wanted at
                    // bit 4 (20); elements 2, 6 (3, 7) at 8 + 2j .. (24 + 2j ..), wanted at bit 8 (24)
                    const uint32_t ta = j < 2 ? w.top[r] << ((4 - 2 * j) & 31) : w.top[r] >> ((2 * j - 4) & 31);
                    const uint32_t tb = w.top[r] >> (2 * j);
                    v0 = and_or(ta, 0x00100010u, v0);
                    v2 = and_or(ta >> 1, 0x00100010u, v2);
                    v1 = and_or(tb, 0x01000100u, v1);
                    v3 = and_or(tb >> 1, 0x01000100u, v3);
                }
                const h2 u0 = __builtin_bit_cast(h2, v0), u1 = __builtin_bit_cast(h2, v1);
                const h2 u2 = __builtin_bit_cast(h2, v2), u3 = __builtin_bit_cast(h2, v3);
                const h2 a0 = __builtin_elementwise_fma(u0, k1, c1);   // exactly sc * e (<= 945)
                const h2 a1 = __builtin_elementwise_fma(u1, k1, c2);
                const h2 a2 = __builtin_elementwise_fma(u2, k1, c1);
                const h2 a3 = __builtin_elementwise_fma(u3, k1, c2);
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
            const float d = h2f((uint16_t)(w.hdr[r].x & 0xffff));
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[r][t][i] = fmaf(d, accq[r][t][i], acc[r][t][i]);
        }
    };

    if (sb0 < sb1) {
        WSet w0, w1, w2;
        stage_x<NT>(stage, sb0, 0, true);
        load_w(sb0, w0);
        // The waits in `body` count loads in program order. Left free, the scheduler interleaves the loads of
        // the two sets here, and the compiler then has to wait in the loop for the newest loads as well
        // (the staging requests just issued among them) before it may touch what it believes is still arriving.
        __builtin_amdgcn_sched_barrier(0);
        load_w(min(sb0 + 1, sb1 - 1), w1);
        __builtin_amdgcn_sched_barrier(0);
        rotate_sets(sb0, sb1, w0, w1, w2, body);
    }
    join_and_store<NT, R>(a, acc, smem, rg, rw, kh, tbase, ks);
}

typedef float f16v __attribute__((ext_vector_type(16)));

// a * b + c into a register of the allocator's choice: left to itself the
// compiler picks the two-operand form for some of the accumulator updates and
// pays a register copy in front of each
__device__ __forceinline__ float fma3(float a, float b, float c) {
    float d;
    asm("v_fma_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}

// Q4_K for a full chunk of 64 tokens on v_mfma_f32_32x32x16_f16: half as many
// matrix instructions as with 16x16x32 tiles for the same products, which
// matters because matrix and vector instructions of the two waves of a SIMD
// share one issue port; with 16x16x32 the decode's vector instructions and the
// matrix instructions together need more issue cycles than the matrix pipe
// needs to execute.
// A row wave owns 32 weight rows (two row tiles); lane l works for row
// n32 = l % 32 and, p = l / 32, for the k-groups g = p and g = 2 + p of every
// 32-wide k-step, so MFMA (j, h) multiplies k = 32 j + 16 h .. + 15. The staged
// activations and the weight tiles keep the 16x16x32 operand order; only the
// per-lane addresses differ.
// acc[tb][i] is token 32 tb + 8 (i / 4) + 4 p + i % 4, row n32.
__global__ __launch_bounds__(kThreads, 1) __attribute__((amdgpu_num_vgpr(232))) void k_mm5_q4k(MMArgs a) {
    constexpr int NT = 4;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rw = wave & 3, kh = wave >> 2;
    const int n32 = lane & 31, p = lane >> 5;
    const int r16 = n32 & 15;
    int rg, ks;
    wg_place(a, blockIdx.x, rg, ks);
    const int tbase = blockIdx.y * 64;
    const int nsb = a.K >> 8;
    const int per = (nsb + a.ksplit - 1) / a.ksplit;
    const int sb0 = ks * per, sb1 = min(nsb, sb0 + per);
    constexpr int WAVES_PER_TILE = 8 / NT;
    // wave w of the eight stages token tile w % NT; the two waves of a tile share its sixteen (k-step, hi/lo) blocks
    const int st_tile = wave % NT, st_slot = wave / NT;
    const __half * xu = a.x + (size_t)blockIdx.y * act_chunk_halves(a.K) + st_tile * 512;
    const __half * su = a.sums + (size_t)blockIdx.y * act_sum_chunk_halves(a.K) + st_tile * 512;
    const uint32_t lds0 = lds_offset(smem);

    f16v acc[2];
    float accm[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) { acc[0][i] = 0.0f; acc[1][i] = 0.0f; accm[i] = 0.0f; }

    // rows past the matrix read the last tile; their results are never stored
    const int tile0 = min((rg * 4 + rw) * 2, a.n_row_tiles - 1), tile1 = min((rg * 4 + rw) * 2 + 1, a.n_row_tiles - 1);
    const uint8_t * wu = a.w + (size_t)tile0 * nsb * 2304;
    const uint32_t off_tile = (n32 >> 4) * (uint32_t)(tile1 - tile0) * nsb * 2304;
    const uint32_t off_hdr = off_tile + r16 * 16, off_q = off_tile + 256 + kh * 1024 + (p * 16 + r16) * 16;
    // The two prefetched weight sets live in v[232:243] and v[244:255], above the
    // registers the compiler may allocate (amdgpu_num_vgpr above): their loads are
    // issued from inline assembly so that the compiler's wait insertion does not
    // see them, and a register it knows nothing about cannot be copied, spilled
    // or reused while its load is still in flight. `take` is the only way a
    // value gets out: it waits until at most the newest set is pending and hands
    // the other set over.
    struct WSet { u4 hdr; u4 q[2]; };
    auto load_w = [&](int sb, auto set) __attribute__((always_inline)) {
        const uint8_t * t = wu + (size_t)sb * 2304;
        const uint32_t oh = off_hdr, oq = off_q;      // named here: an asm operand does not capture in a generic lambda
        if (decltype(set)::value == 0) {
            asm volatile("global_load_dwordx4 v[232:235], %0, %2\n\tglobal_load_dwordx4 v[236:239], %1, %2\n\t"
                         "global_load_dwordx4 v[240:243], %1, %2 offset:512"
                         :: "v"(oh), "v"(oq), "s"(t)
                         : "memory", "v232", "v233", "v234", "v235", "v236", "v237", "v238", "v239", "v240", "v241", "v242", "v243");
        } else {
            asm volatile("global_load_dwordx4 v[244:247], %0, %2\n\tglobal_load_dwordx4 v[248:251], %1, %2\n\t"
                         "global_load_dwordx4 v[252:255], %1, %2 offset:512"
                         :: "v"(oh), "v"(oq), "s"(t)
                         : "memory", "v244", "v245", "v246", "v247", "v248", "v249", "v250", "v251", "v252", "v253", "v254", "v255");
        }
    };
    auto take = [&](auto set) __attribute__((always_inline)) {
        WSet w;
        if (decltype(set)::value == 0)
            asm volatile("s_waitcnt vmcnt(3)" : "={v[232:235]}"(w.hdr), "={v[236:239]}"(w.q[0]), "={v[240:243]}"(w.q[1]) :: "memory");
        else
            asm volatile("s_waitcnt vmcnt(3)" : "={v[244:247]}"(w.hdr), "={v[248:251]}"(w.q[0]), "={v[252:255]}"(w.q[1]) :: "memory");
        return w;
    };
    const h2 m1024 = {(_Float16)(-1024.0f), (_Float16)(-1024.0f)};
    const uint32_t magic1024 = 0x64006400u, magic64 = 0x54005400u;

    // One of this wave's activation requests for super-block sb (clamped to the
    // last one, whose repeated request lands in the buffer nobody reads any
    // more): block idx of its share, or (idx 8) the block sums.
    const uint32_t lane16 = lane * 16;
    auto request = [&](int sb, int idx) __attribute__((always_inline)) {
        const uint32_t buf = lds0 + ((sb - sb0) & 1) * XStage<NT>::BYTES;
        sb = min(sb, sb1 - 1);
        if (idx < 8) {
            const int c = st_slot + WAVES_PER_TILE * idx;
            lds_dma16(xu + (size_t)(sb * 16 + c) * 2048, lane16, buf + (c * NT + st_tile) * 1024);
        } else {
            // every wave requests sums (waves past slot 0 repeat slot 0's block): no branch in the stream
            lds_dma16(su + (size_t)sb * 2048, lane16, buf + (XStage<NT>::X_BLOCKS + st_tile) * 1024);
        }
    };
    // this lane's part of the staged activations: token n32 of a 32-token block is row n32 % 16 of tile n32 / 16
    const uint32_t lane_x = kh * (8 * NT * 1024) + (n32 >> 4) * 1024 + (p * 16 + r16) * 16;
    const uint32_t lane_s = (XStage<NT>::X_BLOCKS + 2 * kh + (n32 >> 4)) * 1024 + (p * 16 + r16) * 16;

    // q: this super-block's products (sc e x), scaled by the row's d while the
    // next super-block multiplies; pq, pd: the products and d left by the one before
    auto body = [&](int sb, auto set, f16v (&q)[2], float & d, const f16v (&pq)[2], float pd) __attribute__((always_inline)) {
        const uint8_t * cur = smem + ((sb - sb0) & 1) * XStage<NT>::BYTES;
        // All but the newest three loads (the other weight set) have landed:
        // this super-block's weights and this wave's activation requests.
        const WSet w = take(set);
        __syncthreads();   // ... for every wave, and nobody still reads the other buffer
        const uint8_t * xk = cur + lane_x;
        // fragments of step s = 2 j + h: [hi, lo][token block]
        h8 A[2][2][2];
        auto read_step = [&](int s) __attribute__((always_inline)) {
            const int j = s >> 1, h = s & 1;
#pragma unroll
            for (int hl = 0; hl < 2; ++hl)
#pragma unroll
                for (int tb = 0; tb < 2; ++tb)
                    A[s & 1][hl][tb] = *(const h8 *)(xk + ((j * 2 + hl) * NT + 2 * tb) * 1024 + h * 512);
        };
        const h8 sA = *(const h8 *)(cur + lane_s);      // block sums of token block kh: hi (p = 0) or lo (p = 1) of the 8 sub-blocks
        read_step(0);

        const Q4KScales s4 = q4k_scales(w.hdr);
        const h2 p0 = magic_pair(s4.mn[0], 0x04010400u) + m1024;
        const h2 p1 = magic_pair(s4.mn[0], 0x04030402u) + m1024;
        const h2 p2 = magic_pair(s4.mn[1], 0x04010400u) + m1024;
        const h2 p3 = magic_pair(s4.mn[1], 0x04030402u) + m1024;
        const h8 mB = {p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
        d = h2f((uint16_t)(w.hdr.x & 0xffff));
        float ndmin = -h2f((uint16_t)(w.hdr.x >> 16));
        // as f32 values of their own: folded into the mixed-precision FMAs they
        // would keep the header word alive into the next super-block, and the
        // weight registers could not take the next load without a copy behind a full wait
        asm volatile("" : "+v"(d), "+v"(ndmin));
        const uint32_t scw = kh ? s4.sc[1] : s4.sc[0];
        // scales of the four k-steps as f16 pairs (sc 2i, sc 2i + 1) and their products with the two magic
        // offsets; the packed FMAs below pick the half they need, so nothing is duplicated per k-step
        h2 kp[2], c1p[2], c2p[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            kp[i] = magic_pair(scw, i ? 0x04030402u : 0x04010400u) + m1024;
            c1p[i] = kp[i] * (_Float16)(-1024.0f);
            c2p[i] = kp[i] * (_Float16)(-64.0f);
        }
        auto decode = [&](int s) __attribute__((always_inline)) {
            const int j = s >> 1;
            const h2 kk = kp[j >> 1], cc1 = c1p[j >> 1], cc2 = c2p[j >> 1];
            const h2 k1 = (j & 1) ? __builtin_shufflevector(kk, kk, 1, 1) : __builtin_shufflevector(kk, kk, 0, 0);
            const h2 c1 = (j & 1) ? __builtin_shufflevector(cc1, cc1, 1, 1) : __builtin_shufflevector(cc1, cc1, 0, 0);
            const h2 c2 = (j & 1) ? __builtin_shufflevector(cc2, cc2, 1, 1) : __builtin_shufflevector(cc2, cc2, 0, 0);
            const uint32_t wq = w.q[s & 1][j];
            const uint32_t w8 = wq >> 8;
            // 1024 + e in the low nibble positions, 64 + e in the high ones
            const h2 u0 = __builtin_bit_cast(h2, and_or(wq, 0x000F000Fu, magic1024));
            const h2 u1 = __builtin_bit_cast(h2, and_or(wq, 0x00F000F0u, magic64));
            const h2 u2 = __builtin_bit_cast(h2, and_or(w8, 0x000F000Fu, magic1024));
            const h2 u3 = __builtin_bit_cast(h2, and_or(w8, 0x00F000F0u, magic64));
            const h2 a0 = __builtin_elementwise_fma(u0, k1, c1);   // exactly sc * e (<= 945)
            const h2 a1 = __builtin_elementwise_fma(u1, k1, c2);
            const h2 a2 = __builtin_elementwise_fma(u2, k1, c1);
            const h2 a3 = __builtin_elementwise_fma(u3, k1, c2);
            return (h8){a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
        };
        h8 B[2];
        B[0] = decode(0);
        // min term: the 16 k-slots are the 8 sub-blocks' hi sums and their lo sums, against the same 8 mins
        f16v zero;
#pragma unroll
        for (int i = 0; i < 16; ++i) zero[i] = 0.0f;
        const f16v m16 = __builtin_amdgcn_mfma_f32_32x32x16_f16(sA, mB, zero, 0, 0, 0);
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            // the LDS reads of the next step go first: they land while this step multiplies
            if (s + 1 < 8) read_step(s + 1);
            __builtin_amdgcn_sched_barrier(0);
            // the activation requests of the next super-block, early enough to have landed by its barrier
            if (s < 3) { request(sb + 1, 3 * s); request(sb + 1, 3 * s + 1); request(sb + 1, 3 * s + 2); }
            if (s + 1 < 8) {
                B[(s + 1) & 1] = decode(s + 1);
            }
            // a share of the scaling left by the last super-block, and of this one's min term
#pragma unroll
            for (int i = 2 * s; i < 2 * s + 2; ++i) {
                acc[0][i] = fma3(pd, pq[0][i], acc[0][i]);
                acc[1][i] = fma3(pd, pq[1][i], acc[1][i]);
            }
            if (s >= 2 && s < 6) {
#pragma unroll
                for (int i = 4 * (s - 2); i < 4 * (s - 2) + 4; ++i) accm[i] = fma3(ndmin, m16[i], accm[i]);
            }
#pragma unroll
            for (int tb = 0; tb < 2; ++tb)
                q[tb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[s & 1][0][tb], B[s & 1], s == 0 ? zero : q[tb], 0, 0, 0);
#pragma unroll
            for (int tb = 0; tb < 2; ++tb)
                q[tb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[s & 1][1][tb], B[s & 1], q[tb], 0, 0, 0);
            if (s == 7) load_w(min(sb + 2, sb1 - 1), set);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto scale_last = [&](const f16v (&q)[2], float d) __attribute__((always_inline)) {
#pragma unroll
        for (int tb = 0; tb < 2; ++tb)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[tb][i] = fmaf(d, q[tb][i], acc[tb][i]);
    };

    if (sb0 < sb1) {
        f16v qa[2], qb[2];
        float da = 0.0f, db = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) { qb[0][i] = 0.0f; qb[1][i] = 0.0f; }
        const std::integral_constant<int, 0> set0;
        const std::integral_constant<int, 1> set1;
        for (int i = 0; i <= 8; ++i) request(sb0, i);
        load_w(sb0, set0);
        load_w(min(sb0 + 1, sb1 - 1), set1);
        for (int sb = sb0; sb < sb1; sb += 2) {
            body(sb, set0, qa, da, qb, db);
            if (sb + 1 >= sb1) { scale_last(qa, da); break; }
            body(sb + 1, set1, qb, db, qa, da);
            if (sb + 2 >= sb1) scale_last(qb, db);
        }
        // the last, repeated requests have landed before the buffers are reused, and no load is in flight
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    // the min term of token block kh joins its accumulator
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        acc[0][i] += kh == 0 ? accm[i] : 0.0f;
        acc[1][i] += kh == 1 ? accm[i] : 0.0f;
    }
    constexpr int S = 64 * 2 + 4;
    __syncthreads();       // every wave is done with the staged activations
    float * mine = (float *)smem + kh * (NT * 16 * S);
#pragma unroll
    for (int tb = 0; tb < 2; ++tb)
#pragma unroll
        for (int i = 0; i < 16; ++i) mine[(32 * tb + 8 * (i >> 2) + 4 * p + (i & 3)) * S + rw * 32 + n32] = acc[tb][i];
    store_token_rows<NT, 2>(a, smem, rg, tbase, ks);
}

template <int NT, int R>
__global__ __launch_bounds__(kThreads, 1) void k_mm2_q8_0(MMArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rw = wave & 3, kh = wave >> 2;
    const int r16 = lane & 15;
    int rg, ks;
    wg_place(a, blockIdx.x, rg, ks);
    const int tbase = blockIdx.y * 64;
    const int nsb = a.K >> 8;
    const int per = (nsb + a.ksplit - 1) / a.ksplit;
    const int sb0 = ks * per, sb1 = min(nsb, sb0 + per);

    int rt[R];
#pragma unroll
    for (int r = 0; r < R; ++r) rt[r] = (rg * 4 + rw) * R + r;
    const StageSrc<NT> stage = stage_prepare<NT>(a, blockIdx.y, lane, wave, smem);
    f4 acc[R][NT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[r][t] = (f4){0.f, 0.f, 0.f, 0.f};

    WeightRows wbase[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
        wbase[r] = weight_rows(a.w + (size_t)min(rt[r], a.n_row_tiles - 1) * nsb * 4352, (uint32_t)nsb * 4352u);
    struct WSet { u4 hdr[R]; u4 q[R][2]; };
    const uint32_t off_hdr = r16 * 16, off_q = 256 + 2 * kh * 1024 + lane * 16;
    auto load_w = [&](int sb, WSet & w) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            w.hdr[r] = load16(wbase[r], off_hdr, (uint32_t)sb * 4352u);
            w.q[r][0] = load16(wbase[r], off_q, (uint32_t)sb * 4352u);
            w.q[r][1] = load16(wbase[r], off_q + 1024, (uint32_t)sb * 4352u);
        }
    };
    const h2 bias1152 = {(_Float16)(-1152.0f), (_Float16)(-1152.0f)};

    auto body = [&](int sb, WSet & w, WSet & fut) __attribute__((always_inline)) {
        uint8_t * cur = smem + ((sb - sb0) & 1) * XStage<NT>::BYTES;
        // all but the newest 3R loads (the weights one super-block ahead) have landed
        __builtin_amdgcn_s_waitcnt(0x0F70 | (3 * R));
        // The set is usable from here on and not before: without this the scheduler starts on the next
        // super-block's payload inside this one and waits for it there, the staging requests included.
#pragma unroll
        for (int r = 0; r < R; ++r) asm volatile("" : "+v"(w.hdr[r]), "+v"(w.q[r][0]), "+v"(w.q[r][1]));
        __syncthreads();
        if (sb + 1 < sb1) stage_x<NT>(stage, sb + 1, (sb - sb0 + 1) & 1, false);
        load_w(min(sb + 2, sb1 - 1), fut);
        __builtin_amdgcn_sched_barrier(0);   // requested now, not wherever the scheduler finds room among the arithmetic
        if (sb >= sb1) return;       // past the slice: the round is only kept whole
        const uint8_t * xk = cur + kh * (8 * NT * 1024);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            h8 A[NT], Al[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                A[t] = lds_h8(xk, (j * 2 + 0) * NT + t, lane);
                Al[t] = lds_h8(xk, (j * 2 + 1) * NT + t, lane);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                // scales of sub-blocks 4 kh + j: words 2 kh and 2 kh + 1 of the header
                const uint32_t sw = kh ? (j < 2 ? w.hdr[r].z : w.hdr[r].w) : (j < 2 ? w.hdr[r].x : w.hdr[r].y);
                const float d = h2f((uint16_t)((j & 1) ? (sw >> 16) : (sw & 0xffff)));
                const u4 d4 = w.q[r][j >> 1];
                const int half = j & 1;
                const uint32_t w0 = d4[2 * half] ^ 0x80808080u;
                const uint32_t w1 = d4[2 * half + 1] ^ 0x80808080u;
                const h2 a0 = magic_pair(w0, 0x04010400u) + bias1152, a1 = magic_pair(w0, 0x04030402u) + bias1152;
                const h2 a2 = magic_pair(w1, 0x04010400u) + bias1152, a3 = magic_pair(w1, 0x04030402u) + bias1152;
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
    };

    if (sb0 < sb1) {
        WSet w0, w1, w2;
        stage_x<NT>(stage, sb0, 0, false);
        load_w(sb0, w0);
        __builtin_amdgcn_sched_barrier(0);     // the waits in `body` count loads in program order
        load_w(min(sb0 + 1, sb1 - 1), w1);
        __builtin_amdgcn_sched_barrier(0);
        rotate_sets(sb0, sb1, w0, w1, w2, body);
    }
    join_and_store<NT, R>(a, acc, smem, rg, rw, kh, tbase, ks);
}

// Q6_K: value = (d * scale of the 16-wide block) * (code - 32), code of six bits, scale an i8. A lane's eight
// k-slots of a 32-wide step lie in one 16-wide block, so the block scale can be folded into the weight
// operand; the product scale * code reaches 4096 and is not always an f16, so the scale goes in as two
// parts whose products are: its low four bits (0..15, products up to 480) and the rest (a multiple of 16,
// products multiples of 16 up to 4096). Four matrix instructions per step and tile pair (two scale parts x
// hi/lo activations) accumulate sum(scale * code * x) exactly as far as f32 goes; d is applied per super-block.
template <int NT, int R>
__global__ __launch_bounds__(kThreads, 1) void k_mm2_q6k(MMArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rw = wave & 3, kh = wave >> 2;
    const int r16 = lane & 15;
    int rg, ks;
    wg_place(a, blockIdx.x, rg, ks);
    const int tbase = blockIdx.y * 64;
    const int nsb = a.K >> 8;
    const int per = (nsb + a.ksplit - 1) / a.ksplit;
    const int sb0 = ks * per, sb1 = min(nsb, sb0 + per);

    int rt[R];
#pragma unroll
    for (int r = 0; r < R; ++r) rt[r] = (rg * 4 + rw) * R + r;
    const StageSrc<NT> stage = stage_prepare<NT>(a, blockIdx.y, lane, wave, smem);
    f4 acc[R][NT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[r][t] = (f4){0.f, 0.f, 0.f, 0.f};

    WeightRows wbase[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
        wbase[r] = weight_rows(a.w + (size_t)min(rt[r], a.n_row_tiles - 1) * nsb * 3360, (uint32_t)nsb * 3360u);
    // this wave's weights of one super-block: the rows' scales, d (two rows to a dword), its half of the payload
    struct WSet { u4 sc[R]; uint32_t d[R]; u4 ql[R]; u2 qh[R]; };
    const uint32_t off_sc = r16 * 16, off_d = 256 + (r16 >> 1) * 4;
    const uint32_t off_ql = 288 + kh * 1024 + lane * 16, off_qh = 2336 + kh * 512 + lane * 8;
    auto load_w = [&](int sb, WSet & w) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            w.sc[r] = load16(wbase[r], off_sc, (uint32_t)sb * 3360u);
            w.d[r] = load4(wbase[r], off_d, (uint32_t)sb * 3360u);
            w.ql[r] = load16(wbase[r], off_ql, (uint32_t)sb * 3360u);
            w.qh[r] = load8(wbase[r], off_qh, (uint32_t)sb * 3360u);
        }
    };
    const h2 bias1056 = {(_Float16)(-1056.0f), (_Float16)(-1056.0f)};
    const uint32_t magic1024 = 0x64006400u;
    const int sc_shift = (lane >> 5) * 8;          // the lane's 16-wide block within a 32-wide step

    auto body = [&](int sb, WSet & w, WSet & fut) __attribute__((always_inline)) {
        uint8_t * cur = smem + ((sb - sb0) & 1) * XStage<NT>::BYTES;
        // all but the newest 4R loads (the weights one super-block ahead) have landed
        __builtin_amdgcn_s_waitcnt(0x0F70 | (4 * R));
        // the set is usable from here on and not before
#pragma unroll
        for (int r = 0; r < R; ++r) asm volatile("" : "+v"(w.sc[r]), "+v"(w.d[r]), "+v"(w.ql[r]), "+v"(w.qh[r]));
        __syncthreads();
        if (sb + 1 < sb1) stage_x<NT>(stage, sb + 1, (sb - sb0 + 1) & 1, false);
        load_w(min(sb + 2, sb1 - 1), fut);
        __builtin_amdgcn_sched_barrier(0);   // requested now, not wherever the scheduler finds room among the arithmetic
        if (sb >= sb1) return;       // past the slice: the round is only kept whole
        const uint8_t * xk = cur + kh * (8 * NT * 1024);
        f4 accq[R][NT];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < NT; ++t) accq[r][t] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            h8 A[NT], Al[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                A[t] = lds_h8(xk, (j * 2 + 0) * NT + t, lane);
                Al[t] = lds_h8(xk, (j * 2 + 1) * NT + t, lane);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                // scale of block 8 kh + 2 j + (lane / 32): byte 2 (j & 1) + lane / 32 of dword 2 kh + j / 2
                const uint32_t sw = kh ? (j < 2 ? w.sc[r].z : w.sc[r].w) : (j < 2 ? w.sc[r].x : w.sc[r].y);
                const int sc = __builtin_amdgcn_sbfe((int)sw, 16 * (j & 1) + sc_shift, 8);
                const _Float16 s_low = (_Float16)(short)(sc & 15), s_rest = (_Float16)(short)(sc & ~15);
                const h2 k_low = {s_low, s_low}, k_rest = {s_rest, s_rest};
                const uint32_t lo = w.ql[r][j];
                const uint32_t top = (j & 1) ? __builtin_amdgcn_alignbit(w.qh[r][j >> 1], w.qh[r][j >> 1], 8) : w.qh[r][j >> 1];
                h2 q[4];
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    // 1024 + code in both halves, then code - 32
                    const uint32_t u = and_or(top >> (2 * p), 0x00300030u, and_or(lo >> (4 * p), 0x000F000Fu, magic1024));
                    q[p] = __builtin_bit_cast(h2, u) + bias1056;
                }
                const h2 b0 = q[0] * k_rest, b1 = q[1] * k_rest, b2 = q[2] * k_rest, b3 = q[3] * k_rest;
                const h2 c0 = q[0] * k_low, c1 = q[1] * k_low, c2 = q[2] * k_low, c3 = q[3] * k_low;
                const h8 B = {b0.x, b0.y, b1.x, b1.y, b2.x, b2.y, b3.x, b3.y};
                const h8 Bl = {c0.x, c0.y, c1.x, c1.y, c2.x, c2.y, c3.x, c3.y};
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    accq[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[t], B, accq[r][t], 0, 0, 0);
                    accq[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Al[t], B, accq[r][t], 0, 0, 0);
                    accq[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[t], Bl, accq[r][t], 0, 0, 0);
                    accq[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Al[t], Bl, accq[r][t], 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float d = h2f((uint16_t)((r16 & 1) ? (w.d[r] >> 16) : (w.d[r] & 0xffff)));
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[r][t][i] = fmaf(d, accq[r][t][i], acc[r][t][i]);
        }
    };

    if (sb0 < sb1) {
        WSet w0, w1, w2;
        stage_x<NT>(stage, sb0, 0, false);
        load_w(sb0, w0);
        __builtin_amdgcn_sched_barrier(0);     // the waits in `body` count loads in program order
        load_w(min(sb0 + 1, sb1 - 1), w1);
        __builtin_amdgcn_sched_barrier(0);
        rotate_sets(sb0, sb1, w0, w1, w2, body);
    }
    join_and_store<NT, R>(a, acc, smem, rg, rw, kh, tbase, ks);
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
        if (NT == 4 && R == 2) {
            static bool once5 = false;
            if (!once5) {
                HIP_OK(hipFuncSetAttribute((const void *)k_mm5_q4k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
                once5 = true;
            }
            hipLaunchKernelGGL(k_mm5_q4k, grid, dim3(kThreads), lds, s, a);
            return;
        }
        hipLaunchKernelGGL((k_mm2_q4k<NT, R>), grid, dim3(kThreads), lds, s, a);
    } else if (type == WT_Q5_K) {
        static bool once = false;
        if (!once) {
            HIP_OK(hipFuncSetAttribute((const void *)k_mm2_q4k<NT, R, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            once = true;
        }
        hipLaunchKernelGGL((k_mm2_q4k<NT, R, true>), grid, dim3(kThreads), lds, s, a);
    } else if (type == WT_Q6_K) {
        static bool once = false;
        if (!once) {
            HIP_OK(hipFuncSetAttribute((const void *)k_mm2_q6k<NT, R>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            once = true;
        }
        hipLaunchKernelGGL((k_mm2_q6k<NT, R>), grid, dim3(kThreads), lds, s, a);
    } else {
        static bool once = false;
        if (!once) {
            HIP_OK(hipFuncSetAttribute((const void *)k_mm2_q8_0<NT, R>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            once = true;
        }
        hipLaunchKernelGGL((k_mm2_q8_0<NT, R>), grid, dim3(kThreads), lds, s, a);
    }
}

size_t matmul_workspace_bytes() {
    // K-slices of a split matmul: up to 16 slices x 64 tokens x 8192 columns
    return (size_t)64 * 16 * 8192 * 4;
}

thread_local int g_mm_force_ksplit = 0;

template <int R>
static void dispatch_nt(hipStream_t s, int type, int nt, const MMArgs & a, dim3 grid) {
    switch (nt) {
        case 1: launch2<1, R>(s, type, a, grid); break;
        case 2: launch2<2, R>(s, type, a, grid); break;
        default: launch2<4, R>(s, type, a, grid); break;
    }
}

// act_out: destination of mode MM_SWIGLU, else null
// One matrix of several that leave their K-slices side by side: the common slice count, the row width of the
// slices and this matrix's first column in them.
struct SharedSlices { int ksplit = 0, ld = 0, col = 0; };

static Slices lds_impl(hipStream_t s, const Weight & w, const Act & x_all, int T, float * y, int ldy, int col0,
                       int mode, const float * bias, void * ws, bool may_slice, const Act * act_out, float * act_f32,
                       const SharedSlices * shared = nullptr) {
    if (!w.packed || !can_pack(w.type, w.K, w.N))
        throw std::runtime_error("matmul_lds: needs a tile-packed Q4_K, Q5_K, Q6_K or Q8_0 matrix of whole super-blocks and 16-row tiles");
    const Act x = x_all.operand(w.type);
    if (!x.x) throw std::runtime_error("matmul: the activations were not prepared for this weight type");
    if ((w.type == WT_Q4_K || w.type == WT_Q5_K) && !x.sums) throw std::runtime_error("matmul: Q4_K and Q5_K need block sums");
    MMArgs a {};
    a.w = w.packed; a.x = x.x; a.sums = x.sums; a.y = y; a.bias = bias;
    a.K = w.K; a.N = w.N; a.T = T; a.ldy = ldy; a.col0 = col0; a.mode = mode;
    if (act_out) { a.act_out = *act_out; a.act_f32 = act_f32; }
    a.n_row_tiles = w.N / 16;
    // the epilogue stores four columns per lane
    if (mode != MM_SWIGLU && ((ldy & 3) || (col0 & 3) || ((uintptr_t)y & 15) || (bias && ((uintptr_t)bias & 15))))
        throw std::runtime_error("matmul_lds: y, ldy, col0 and bias must be aligned to four floats");
    a.partial = (float *)ws;
    if (mode == MM_SWIGLU) may_slice = false;
    const int nsb = w.K / 256;
    const int nt = T > 32 ? 4 : (T > 16 ? 2 : 1);
    const int chunks = (T + 63) / 64;
    constexpr int R = 2;
    a.n_row_groups = (a.n_row_tiles + 4 * R - 1) / (4 * R);
    // Few row groups and chunks of tokens: split K so that about every CU
    // gets a workgroup, each with at least two super-blocks.
    int ksplit = 1;
    a.slice_rows = chunks * 64;
    if (may_slice) {
        int want = std::min(16, 256 / (a.n_row_groups * chunks));
        if (g_mm_force_ksplit > 0) want = g_mm_force_ksplit;
        want = std::min(want, nsb / 2);
        if (want > 1) {
            const int per = (nsb + want - 1) / want;
            ksplit = (nsb + per - 1) / per;
        }
        if ((size_t)ksplit * a.slice_rows * w.N * 4 > matmul_workspace_bytes()) {
            if (g_mm_force_ksplit > 0) throw std::runtime_error("matmul_lds: the split does not fit the workspace");
            ksplit = 1;
        }
    }
    a.pld = w.N; a.pcol = 0;
    if (shared) {
        if (shared->ksplit < 2 || shared->ksplit > nsb || (shared->col & 3) || (shared->ld & 3) ||
            shared->col + w.N > shared->ld || (size_t)shared->ksplit * a.slice_rows * shared->ld * 4 > matmul_workspace_bytes())
            throw std::runtime_error("matmul_lds: the shared slices do not fit this matrix");
        const int per = (nsb + shared->ksplit - 1) / shared->ksplit;
        if ((nsb + per - 1) / per != shared->ksplit) throw std::runtime_error("matmul_lds: the shared slice count leaves an empty slice");
        ksplit = shared->ksplit;
        a.pld = shared->ld; a.pcol = shared->col;
    }
    a.ksplit = ksplit;
    dim3 grid(a.n_row_groups * ksplit, chunks);
    dispatch_nt<R>(s, w.type, nt, a, grid);
    check_launch("matmul_lds");
    Slices out;
    if (ksplit > 1) { out.data = a.partial; out.n = ksplit; out.stride = (size_t)a.slice_rows * a.pld; out.N = a.pld; }
    return out;
}

// Several tiled matrices over the same activations whose outputs sit side by side in y (q, k and v of different
// storage types): each is launched on its own, all with the same number of K-slices into one set of slices of
// the full row width, so that the consumer adds them as it would for one fused matrix. Returns no slices (and
// leaves the results in y) when the row groups and token chunks already fill the chip or K is too short to split.
Slices matmul_deferred_parts(hipStream_t s, const Weight * const * parts, int n_parts, const Act & x, int T, float * y,
                             int ldy, const float * bias, void * ws) {
    if (T <= 0 || n_parts <= 0) return Slices();
    int total = 0, K = parts[0]->K;
    for (int i = 0; i < n_parts; ++i) {
        if (!parts[i]->packed || parts[i]->K != K || !can_pack(parts[i]->type, K, parts[i]->N) || (parts[i]->N & 3))
            throw std::runtime_error("matmul_deferred_parts: needs tile-packed matrices of one width");
        total += parts[i]->N;
    }
    if (!ws || total > ldy) throw std::runtime_error("matmul_deferred_parts: needs the workspace and room for every part in y");
    if (T <= GEMV_MAX_T) {     // every part by the integer matrix-vector kernel, or none
        bool all = true;
        for (int i = 0; i < n_parts; ++i) all = all && gemv_can(*parts[i], x.operand(parts[i]->type), T);
        if (all) {
            int at = 0;
            for (int i = 0; i < n_parts; ++i) {
                gemv(s, *parts[i], x.operand(parts[i]->type), T, y, ldy, at, MM_STORE, bias ? bias + at : nullptr);
                at += parts[i]->N;
            }
            return Slices();
        }
    }
    const int nsb = K / 256, chunks = (T + 63) / 64;
    int ksplit = 1;
    {
        const int groups = (total / 16 + 7) / 8;
        int want = std::min(std::min(16, 256 / std::max(groups * chunks, 1)), nsb / 2);
        if (want > 1) {
            const int per = (nsb + want - 1) / want;
            ksplit = (nsb + per - 1) / per;
        }
        if ((size_t)ksplit * chunks * 64 * total * 4 > matmul_workspace_bytes()) ksplit = 1;
    }
    Slices out;
    int col = 0;
    for (int i = 0; i < n_parts; ++i) {
        const float * b = bias ? bias + col : nullptr;
        if (ksplit > 1) {
            SharedSlices sh;
            sh.ksplit = ksplit; sh.ld = total; sh.col = col;
            out = lds_impl(s, *parts[i], x, T, y, ldy, col, MM_STORE, b, ws, true, nullptr, nullptr, &sh);
        } else {
            lds_impl(s, *parts[i], x, T, y, ldy, col, MM_STORE, b, ws, false, nullptr, nullptr);
        }
        col += parts[i]->N;
    }
    if (ksplit > 1) { out.data = (const float *)ws; out.n = ksplit; out.stride = (size_t)chunks * 64 * total; out.N = total; }
    return out;
}

Slices matmul_lds(hipStream_t s, const Weight & w, const Act & x, int T, float * y, int ldy, int col0,
                  int mode, const float * bias, void * ws, bool may_slice) {
    if (mode == MM_SWIGLU) throw std::runtime_error("matmul_lds: use matmul_swiglu");
    return lds_impl(s, w, x, T, y, ldy, col0, mode, bias, ws, may_slice, nullptr, nullptr);
}

void matmul_swiglu(hipStream_t s, const Weight & w, const Act & x, int T, const Act & out, void * ws, float * h_f32) {
    if (T <= 0) return;
    if (!w.packed || !ws || w.N != 2 * out.K || out.K % 64 != 0 || (!out.x && !out.qx))
        throw std::runtime_error("matmul_swiglu: needs a tile-packed gate/up matrix interleaved by 64 columns");
    if (x.K != w.K) throw std::runtime_error("matmul_swiglu: activation width does not match the weight");
    // A workgroup holds 64 hidden columns of a token: enough for the 32-wide blocks of the Q8_0
    // conversion, not for the 256-wide ones of Q8_K. Those rows leave as f32 and are converted after.
    if (h_f32 && T <= GEMV_MAX_T && gemv_can(w, x.operand(w.type), T)) {
        // a very small step: gate and up as f32 rows (in their groups of 64) by the integer kernel, then the SiLU
        gemv(s, w, x.operand(w.type), T, h_f32, w.N, 0, MM_STORE, nullptr);
        swiglu_act(s, h_f32, T, out.K, out, 64);
        return;
    }
    const bool via_f32 = out.qx && out.quant == AQ_Q8_K;
    if (via_f32 && !h_f32) throw std::runtime_error("matmul_swiglu: the Q8_K conversion needs the f32 row buffer");
    // One workgroup per CU and more row groups than CUs: the last round of workgroups would run on a few CUs only
    // (18944 hidden columns: 296 groups, the second round 40 of 256 CUs for as long as the first). Whole rounds keep
    // the fused epilogue; the groups left over are multiplied with K split over as many workgroups as fill the chip,
    // and a small launch adds their slices and applies the SiLU.
    const int groups = w.N / 128, tail = groups % 256;
    if (!via_f32 && T > 32 && T <= 64 && w.N % 128 == 0 && groups > 256 && tail > 0 && tail <= 128 && w.K / 256 >= 4 && g_mm_force_ksplit == 0) {
        const size_t tile = w.type == WT_Q4_K ? 2304 : (w.type == WT_Q5_K ? 2816 : (w.type == WT_Q6_K ? 3360 : 4352));
        Weight head = w, rest = w;
        head.N = (groups - tail) * 128;
        rest.N = tail * 128;
        rest.packed = w.packed + (size_t)(groups - tail) * 8 * (size_t)(w.K / 256) * tile;
        head.bytes = rest.bytes = 0;       // views: the bytes belong to w
        lds_impl(s, head, x, T, nullptr, 0, 0, MM_SWIGLU, nullptr, ws, false, &out, nullptr);
        const Slices sl = lds_impl(s, rest, x, T, nullptr, rest.N, 0, MM_STORE, nullptr, ws, true, nullptr, nullptr);
        if (sl.n < 2) throw std::runtime_error("matmul_swiglu: the left-over row groups were not split");
        swiglu_slices(s, sl, T, out, (groups - tail) * 64);
        return;
    }
    lds_impl(s, w, x, T, nullptr, 0, 0, MM_SWIGLU, nullptr, ws, false, &out, via_f32 ? h_f32 : nullptr);
    if (via_f32) to_act(s, h_f32, T, out.K, out);
}

}  // namespace rk
