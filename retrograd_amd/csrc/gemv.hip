// The integer matrix-vector kernel of very small steps under ggml's arithmetic (gfx950, wave64).
//
// A step of one or two tokens reads every weight once and has nothing to amortise the conversion of the stored
// codes to f16 matrix operands over: the tile kernels then spend their time issuing vector instructions, not
// waiting for memory. When the activations are Q8_K / Q8_0 blocks anyway (what ggml's CPU dot products multiply:
// ggml-quants.c ggml_vec_dot_q4_K_q8_K, ggml_vec_dot_q8_0_q8_0), the products can stay integers and a four-way
// integer dot product (v_dot4c_i32_i8) multiplies four weight codes with four activation codes at a time.
//
// Q4_K (activations Q8_K):
//   sum_k w[n][k] x[k] = sum over super-blocks of
//       d_x * ( d_w * sum_s sc_s * (sum_{k in s} q_k c_k)  -  dmin_w * sum_s m_s * bsum_s )
// with q the 4-bit codes, c the activation codes, sc / m the 6-bit scales and mins of the eight sub-blocks s,
// bsum_s the sum of the activation codes of s: all integer up to the two float factors per super-block, exactly
// the quantities ggml's kernel forms (its order of the float additions is one of several, per instruction set).
// The matrix is the Q4_K tile layout of the tile kernels (16 rows x 256 columns, 16-byte row headers, then two
// 1 KiB loads in which lane (r = l % 16, g = l / 16) of load h holds, as dword j, the eight nibbles of columns
// 32 (4h + j) + 8g .. + 8 of row r, in the order e0 e2 e4 e6 e1 e3 e5 e7). Masking a dword with 0x0F0F0F0F gives
// the bytes e0 e4 e1 e5, the same after a shift by four e2 e6 e3 e7: the activation codes are stored in that
// byte order (act_code_pos), so no lane ever permutes anything: about a quarter of the tile kernels' vector
// instructions per weight.
//
// Q6_K (activations Q8_K; the finer type of a Q4_K_M file):
//   sum over super-blocks of  d_w d_x * sum_b sc_b * ( sum_{k in b} u_k c_k  -  32 bsum_b )
// over the sixteen blocks b of 16 with their i8 scales, u the unsigned 6-bit codes. The tile keeps the low nibbles
// in the Q4_K order and the top bit pairs in a plane of their own (see k_repack_q6k); two shifts and masks per dword
// move them above the nibbles of the two byte dwords, which costs about twice the Q4_K kernel's vector instructions
// per weight - still fewer than the tile kernel spends, and without its four matrix instructions per step.
//
// Q5_K (activations Q8_K; the main type of a Q5_K_M file): the Q4_K formula with 5-bit codes. The tile is the Q4_K
// tile of the low nibbles followed by one dword of fifth bits per k-half and lane (see k_repack_q4k); a shift by the
// k-step and two masked shifts per byte dword put them above the nibbles.
//
// Q8_0 (activations Q8_0):
//   sum_k w[n][k] x[k] = sum over blocks of 32 of  (d_w d_x) * sum_{k in block} q_k c_k
// The Q8_0 tile (16 x 8 f16 scales, then four 1 KiB loads in which lane (r, g) of load q holds columns 8g .. 8g + 8
// of blocks 2q and 2q + 1 of row r, bytes in element order) needs no unpacking at all; the activation codes stay in
// element order.
#include "dev_common.hpp"

namespace rk {

thread_local int g_gemv_max_t = GEMV_MAX_T;

struct GemvArgs {
    const uint8_t * w;         // tiles
    const int8_t * codes;      // [T][K]
    const float * d;           // [T][K / 256] (Q8_K) or [T][K / 32] (Q8_0)
    const int16_t * bsums;     // [T][K / 16] (Q8_K only)
    float * y;
    const float * bias;
    int K, N, T, ldy, col0, mode, n_tiles;
    // SRC_NORM / SRC_SWIGLU: the f32 rows the blocks are made from while they are staged
    const float * xin;         // NORM: rows of K floats; SWIGLU: rows of 2 K floats, gate and up in alternating groups
    const float * norm_w;      // NORM: the RMSNorm weights
    const int32_t * rows;      // NORM: row t is xin row rows[t] (null: t)
    float eps;
    int group;                 // SWIGLU: gate c at column (c / group) * 2 group + c % group, up c `group` columns further
    // SRC_COMBINE: the split partials of the step's single token (what attention_combine merges)
    const float * partial;     // per (item, column): m (log2 domain), l, head_dim unnormalised outputs
    int item0, n_split;        // the token's first work item; splits per kv head
    int att_G, att_hd;         // query heads per kv head, head_dim
    // k_gemv_f32, SRC_CODES: the hi / lo f16 planes a producer left (Act::x)
    const __half * planes;
};
enum : int { SRC_CODES = 0, SRC_NORM = 1, SRC_SWIGLU = 2, SRC_COMBINE = 3 };

template <int WT> struct GemvTile;
template <> struct GemvTile<WT_Q4_K> { static constexpr int BYTES = 2304, LOADS = 2, QUANT = AQ_Q8_K; };
template <> struct GemvTile<WT_Q8_0> { static constexpr int BYTES = 4352, LOADS = 4, QUANT = AQ_Q8_0; };
// Q6_K: register set = the row's sixteen scales | low nibbles of the two k-halves | top bits of the two k-halves
// (8 bytes a lane each, held as one 16-byte word) | d
template <> struct GemvTile<WT_Q6_K> { static constexpr int BYTES = 3360, LOADS = 3, QUANT = AQ_Q8_K; };
// Q5_K: the two loads of low nibbles; the two dwords of fifth bits travel apart (fifth[])
template <> struct GemvTile<WT_Q5_K> { static constexpr int BYTES = 2816, LOADS = 2, QUANT = AQ_Q8_K; };

// WT: the weight type. NT: tokens held (rows of the step beyond a.T read as zeros). PER: super-blocks of a tile per
// wave; a workgroup has nw waves (PER 2: half the row's super-blocks; wider rows: 16), wave w takes super-blocks
// w + u * nw. A matrix read once has nothing to hide the memory latency behind, so the loads are issued as early as
// they can be: a wave holds two super-blocks at a time and requests the next two as soon as those registers are
// free - the first pair before the step's rows are staged, the first pair of the next tile before the partial sums
// of this one meet in LDS (one barrier per tile: the sums alternate between two buffers). Holding all four of a wide
// row at once was slower.
// SRC: where the activation blocks come from. SRC_CODES: the buffers a producer left. SRC_NORM: every workgroup makes
// them itself from the residual rows - RMSNorm (the sum of squares in the order k_rmsnorm_act8 adds it, so a row of
// 4096 gives the same codes bit for bit) and the conversion, straight into LDS - which saves the step a launch of
// four to five microseconds for about one and a half of redundant work per workgroup. SRC_SWIGLU: likewise
// silu(gate) * up of the gate/up product's f32 rows. SRC_COMBINE (one token, few splits): the merge of the attention
// splits - what k_attention_combine computes - for the output projection. NT is exactly the token count then.
// Dynamic LDS: codes NT * K bytes | scales NT * nd floats (nd = K / 256 or K / 32) | Q8_K: block sums NT * K / 8
// bytes | 2 * nw * NT * 16 floats.
template <int WT, int NT, int PER, int SRC>
__global__ __launch_bounds__(1024) void k_gemv(GemvArgs a) {
    using Tile = GemvTile<WT>;
    constexpr bool Q5 = WT == WT_Q5_K, Q4 = WT == WT_Q4_K || Q5, Q6 = WT == WT_Q6_K, K8 = Tile::QUANT == AQ_Q8_K;
    extern __shared__ __align__(16) uint8_t lds[];
    const int K = a.K, nsb = K >> 8;
    const int nd = K8 ? nsb : (K >> 5);
    const int nthreads = blockDim.x, nw = nthreads >> 6;
    int8_t * l_codes = (int8_t *)lds;
    float * l_d = (float *)(lds + (size_t)NT * K);
    int16_t * l_bsums = (int16_t *)(l_d + NT * nd);
    float * l_red = K8 ? (float *)((uint8_t *)l_bsums + (size_t)NT * (K >> 3)) : (float *)l_bsums;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;

    // two super-blocks are held at a time: u0 and u0 + 1 of the wave's PER
    u4 hdr[2], q[2][Tile::LOADS];
    uint16_t dq6[2] = {0, 0};          // Q6_K: the row's d
    uint32_t fifth[2][2] = {{0, 0}, {0, 0}};      // Q5_K: the fifth bits of the two k-halves
    auto request = [&](int tile, int u0) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int sb = wave + (u0 + u) * nw;
            if (sb < nsb) {
                const uint8_t * tp = a.w + ((size_t)tile * nsb + sb) * Tile::BYTES;
                hdr[u] = *(const u4 *)(tp + r * 16);
                if constexpr (Q6) {
                    q[u][0] = *(const u4 *)(tp + 288 + lane * 16);
                    q[u][1] = *(const u4 *)(tp + 1312 + lane * 16);
                    const uint2 t0 = *(const uint2 *)(tp + 2336 + lane * 8), t1 = *(const uint2 *)(tp + 2848 + lane * 8);
                    q[u][2] = u4{t0.x, t0.y, t1.x, t1.y};
                    dq6[u] = *(const uint16_t *)(tp + 256 + 2 * r);
                } else {
#pragma unroll
                    for (int i = 0; i < Tile::LOADS; ++i) q[u][i] = *(const u4 *)(tp + 256 + i * 1024 + lane * 16);
                    if constexpr (Q5) {
                        fifth[u][0] = *(const uint32_t *)(tp + 2304 + lane * 4);
                        fifth[u][1] = *(const uint32_t *)(tp + 2560 + lane * 4);
                    }
                }
            }
        }
    };
    // The inputs of a thread's first eight values of row 0 are requested ahead of the weights: loads return in
    // order, so a wait for anything requested after the weights would be a wait for the weights as well.
    auto row_of = [&](int t) -> const float * {
        if (SRC == SRC_NORM) return a.xin + (size_t)(a.rows ? a.rows[t] : t) * K;
        return a.xin + (size_t)t * 2 * K;
    };
    // NORM: eight row values and their norm weights; SWIGLU: eight gate and eight up values
    auto load_in = [&](const float * xr, int k, f4 (&in)[4]) {
        if (SRC == SRC_NORM) {
            in[0] = *(const f4 *)(xr + k); in[1] = *(const f4 *)(xr + k + 4);
            in[2] = *(const f4 *)(a.norm_w + k); in[3] = *(const f4 *)(a.norm_w + k + 4);
        } else {
            const float * gp = xr + (size_t)(k / a.group) * 2 * a.group + k % a.group, * up = gp + a.group;
            in[0] = *(const f4 *)gp; in[1] = *(const f4 *)(gp + 4); in[2] = *(const f4 *)up; in[3] = *(const f4 *)(up + 4);
        }
    };
    f4 first[4];
    if (SRC != SRC_CODES && SRC != SRC_COMBINE && tid * 8 < K) load_in(row_of(0), tid * 8, first);
    int tile = blockIdx.x;
    if (tile < a.n_tiles) request(tile, 0);

    // The blocks a fused source makes: what store_codes8 writes for a producer, written to LDS (through LDS pointers,
    // so that the stores are LDS instructions and not flat ones, whose completion would be counted with the weight
    // requests in flight)
    auto store_lds = [&](const float (&c)[8], float d, int t, int k) {
        uint32_t w0 = 0, w1 = 0;
        int sum = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int q8 = (int)c[i];
            sum += q8;
            const uint32_t byte = (uint32_t)q8 & 0xffu;
            const int pos = K8 ? act_code_pos(i) : i;
            if (pos < 4) w0 |= byte << (8 * pos); else w1 |= byte << (8 * (pos - 4));
        }
        *(uint2 *)(l_codes + t * K + k) = make_uint2(w0, w1);
        if (K8) {
            sum += __shfl_xor(sum, 1, 64);
            if ((tid & 1) == 0) l_bsums[t * (K >> 4) + (k >> 4)] = (int16_t)sum;
            if ((k & 255) == 0) l_d[t * nsb + (k >> 8)] = d;
        } else if ((tid & 3) == 0) {
            l_d[t * nd + (k >> 5)] = d;
        }
    };
    if (SRC == SRC_CODES) {
        // stage the rows of the step: 16-byte words of codes, scales, dwords of block sums
        for (int i = tid; i < NT * (K >> 4); i += nthreads) {
            const int t = i / (K >> 4);
            u4 v = {0u, 0u, 0u, 0u};
            if (t < a.T) v = ((const u4 *)a.codes)[i];
            ((u4 *)l_codes)[i] = v;
        }
        for (int i = tid; i < NT * nd; i += nthreads) l_d[i] = i / nd < a.T ? a.d[i] : 0.0f;
        if (K8) {
            for (int i = tid; i < NT * (K >> 5); i += nthreads) {
                const int t = i / (K >> 5);
                ((uint32_t *)l_bsums)[i] = t < a.T ? ((const uint32_t *)a.bsums)[i] : 0u;
            }
        }
    } else if (SRC == SRC_COMBINE) {
        // eight consecutive dimensions of one query head per thread: the splits' (max, sum) pairs, the weights
        // 2^(m_s - M), the weighted outputs over the weighted sums, then the conversion as for any other row
        for (int k = tid * 8; k < K; k += nthreads * 8) {
            const int head = k / a.att_hd, e0 = k % a.att_hd;
            const int kvh = head / a.att_G, col = head % a.att_G;
            const int stride = a.att_hd + 2;
            const float * base = a.partial + ((size_t)(a.item0 + kvh * a.n_split) * 16 + col) * stride;
            float M = -INFINITY;
            for (int sp = 0; sp < a.n_split; ++sp) M = fmaxf(M, base[(size_t)sp * 16 * stride]);
            float L = 0.0f, v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (int sp = 0; sp < a.n_split; ++sp) {
                const float * p = base + (size_t)sp * 16 * stride;
                const float m_s = p[0];
                const float w_s = m_s == -INFINITY ? 0.0f : exp2f(m_s - M);
                L = fmaf(w_s, p[1], L);
                const float2 o0 = *(const float2 *)(p + 2 + e0), o1 = *(const float2 *)(p + 4 + e0);
                const float2 o2 = *(const float2 *)(p + 6 + e0), o3 = *(const float2 *)(p + 8 + e0);
                v[0] = fmaf(w_s, o0.x, v[0]); v[1] = fmaf(w_s, o0.y, v[1]); v[2] = fmaf(w_s, o1.x, v[2]); v[3] = fmaf(w_s, o1.y, v[3]);
                v[4] = fmaf(w_s, o2.x, v[4]); v[5] = fmaf(w_s, o2.y, v[5]); v[6] = fmaf(w_s, o3.x, v[6]); v[7] = fmaf(w_s, o3.y, v[7]);
            }
            const float inv = L > 0.0f ? 1.0f / L : 0.0f;
            float c[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] *= inv;
            const float d = requantise8(v, Tile::QUANT, c);
            store_lds(c, d, 0, k);
        }
    } else {
        // make the blocks here: eight consecutive values per thread, the threads of a block together (requantise8)
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const float * xr = row_of(t);
            float scale = 1.0f;
            if (SRC == SRC_NORM) {
                float ss = 0.0f;
                for (int k = tid * 8; k < K; k += nthreads * 8) {
                    f4 in[2];
                    if (t == 0 && k == tid * 8) { in[0] = first[0]; in[1] = first[1]; }
                    else { in[0] = *(const f4 *)(xr + k); in[1] = *(const f4 *)(xr + k + 4); }
                    const f4 p = in[0], q4 = in[1];
                    ss += p.x * p.x + p.y * p.y + p.z * p.z + p.w * p.w + q4.x * q4.x + q4.y * q4.y + q4.z * q4.z + q4.w * q4.w;
                }
                ss = wave_sum(ss);
                if (lane == 0) l_red[wave] = ss;
                __syncthreads();
                float total = 0.0f;
                for (int i = 0; i < nw; ++i) total += l_red[i];
                scale = 1.0f / sqrtf(total / (float)K + a.eps);
                if (t + 1 < NT) __syncthreads();   // l_red is written again for the next row (the tiles write it behind the barrier below)
            }
            for (int k = tid * 8; k < K; k += nthreads * 8) {
                f4 in[4];
                if (t == 0 && k == tid * 8) { in[0] = first[0]; in[1] = first[1]; in[2] = first[2]; in[3] = first[3]; }
                else load_in(xr, k, in);
                float v[8], c[8];
                if (SRC == SRC_NORM) {
                    v[0] = (in[0].x * scale) * in[2].x; v[1] = (in[0].y * scale) * in[2].y;
                    v[2] = (in[0].z * scale) * in[2].z; v[3] = (in[0].w * scale) * in[2].w;
                    v[4] = (in[1].x * scale) * in[3].x; v[5] = (in[1].y * scale) * in[3].y;
                    v[6] = (in[1].z * scale) * in[3].z; v[7] = (in[1].w * scale) * in[3].w;
                } else {
                    const float gv[8] = {in[0].x, in[0].y, in[0].z, in[0].w, in[1].x, in[1].y, in[1].z, in[1].w};
                    const float uv[8] = {in[2].x, in[2].y, in[2].z, in[2].w, in[3].x, in[3].y, in[3].z, in[3].w};
#pragma unroll
                    for (int i = 0; i < 8; ++i) v[i] = (gv[i] / (1.0f + __expf(-gv[i]))) * uv[i];
                }
                const float d = requantise8(v, Tile::QUANT, c);
                store_lds(c, d, t, k);
            }
        }
    }
    __syncthreads();

    float acc[NT];
    // super-block sb of the tile, held in register set u, times the rows of the step
    auto multiply = [&](int sb, int u) {
        if constexpr (Q4) {
            const Q4KScales S = q4k_scales(hdr[u]);
            int dot[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) dot[t] = 0;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t wq = j == 0 ? q[u][h].x : (j == 1 ? q[u][h].y : (j == 2 ? q[u][h].z : q[u][h].w));
                    int lo = (int)(wq & 0x0F0F0F0Fu), hi = (int)((wq >> 4) & 0x0F0F0F0Fu);
                    if constexpr (Q5) {
                        // after the shift by the k-step: the fifth bits of elements 0 4 | 2 6 | 1 5 | 3 7 at bits 0 1 | 8 9 | 16 17 | 24 25
                        const uint32_t f = fifth[u][h] >> (2 * j);
                        lo |= (int)(((f << 4) & 0x00100010u) | ((f << 11) & 0x10001000u));
                        hi |= (int)(((f >> 4) & 0x00100010u) | ((f << 3) & 0x10001000u));
                    }
                    const int sc = (int)((S.sc[h] >> (8 * j)) & 0xffu);
                    const int k0 = (sb << 8) + ((4 * h + j) << 5) + (g << 3);
#pragma unroll
                    for (int t = 0; t < NT; ++t) {
                        const uint2 c = *(const uint2 *)(l_codes + t * K + k0);
                        int is = __builtin_amdgcn_sdot4(lo, (int)c.x, 0, false);
                        is = __builtin_amdgcn_sdot4(hi, (int)c.y, is, false);
                        dot[t] += __mul24(sc, is);
                    }
                }
            }
            // the min term: lane group g takes sub-blocks 2g and 2g + 1
            const uint32_t mword = (g < 2 ? S.mn[0] : S.mn[1]) >> (16 * (g & 1));
            const int m0 = (int)(mword & 0xffu), m1 = (int)((mword >> 8) & 0xffu);
            const float dw = h2f((uint16_t)(hdr[u].x & 0xffffu)), dmin = h2f((uint16_t)(hdr[u].x >> 16));
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const int2 bs = *(const int2 *)(l_bsums + t * (K >> 4) + (sb << 4) + 4 * g);      // four sums of 16
                const int s0 = (int)(int16_t)(bs.x & 0xffff) + (bs.x >> 16), s1 = (int)(int16_t)(bs.y & 0xffff) + (bs.y >> 16);
                const int mins = __mul24(m0, s0) + __mul24(m1, s1);
                acc[t] += l_d[t * nsb + sb] * (dw * (float)dot[t] - dmin * (float)mins);
            }
        } else if constexpr (Q6) {
            int dot[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) dot[t] = 0;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t wq = j == 0 ? q[u][h].x : (j == 1 ? q[u][h].y : (j == 2 ? q[u][h].z : q[u][h].w));
                    // the top bit pairs of k-steps 2m and 2m + 1 share a dword, the odd step's rotated left by eight
                    const uint32_t tw = h == 0 ? (j < 2 ? q[u][2].x : q[u][2].y) : (j < 2 ? q[u][2].z : q[u][2].w);
                    const uint32_t top = (j & 1) ? __builtin_amdgcn_alignbit(tw, tw, 8) : tw;
                    // codes 0 4 1 5 and 2 6 3 7 as bytes: nibble | top pair << 4
                    const int lo = (int)((wq & 0x0F0F0F0Fu) | (top & 0x00300030u) | ((top << 4) & 0x30003000u));
                    const int hi = (int)(((wq >> 4) & 0x0F0F0F0Fu) | ((top >> 2) & 0x00300030u) | ((top << 2) & 0x30003000u));
                    // the block of 16 these eight columns belong to: 8h + 2j + g / 2; its i8 scale
                    const int b = 8 * h + 2 * j + (g >> 1);
                    const uint32_t sw = (b >> 2) == 0 ? hdr[u].x : ((b >> 2) == 1 ? hdr[u].y : ((b >> 2) == 2 ? hdr[u].z : hdr[u].w));
                    const int sc = (int)(int8_t)((sw >> (8 * (b & 3))) & 0xffu);
                    const int k0 = (sb << 8) + ((4 * h + j) << 5) + (g << 3);
#pragma unroll
                    for (int t = 0; t < NT; ++t) {
                        const uint2 c = *(const uint2 *)(l_codes + t * K + k0);
                        int is = __builtin_amdgcn_sdot4(lo, (int)c.x, 0, false);
                        is = __builtin_amdgcn_sdot4(hi, (int)c.y, is, false);
                        dot[t] += __mul24(sc, is);
                    }
                }
            }
            // the offset of 32: lane group g takes blocks 4g .. 4g + 3 (the bytes of header dword g)
            const uint32_t sw = g == 0 ? hdr[u].x : (g == 1 ? hdr[u].y : (g == 2 ? hdr[u].z : hdr[u].w));
            const float dw = h2f(dq6[u]);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const int2 bs = *(const int2 *)(l_bsums + t * (K >> 4) + (sb << 4) + 4 * g);
                int corr = __mul24((int)(int8_t)(sw & 0xffu), (int)(int16_t)(bs.x & 0xffff));
                corr += __mul24((int)(int8_t)((sw >> 8) & 0xffu), bs.x >> 16);
                corr += __mul24((int)(int8_t)((sw >> 16) & 0xffu), (int)(int16_t)(bs.y & 0xffff));
                corr += __mul24((int)(int8_t)(sw >> 24), bs.y >> 16);
                acc[t] += (dw * l_d[t * nsb + sb]) * (float)(dot[t] - 32 * corr);
            }
        } else {
            // the row's eight block scales: f16 pairs in the header's four dwords
#pragma unroll
            for (int qi = 0; qi < 4; ++qi) {
                const uint32_t pair = qi == 0 ? hdr[u].x : (qi == 1 ? hdr[u].y : (qi == 2 ? hdr[u].z : hdr[u].w));
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int blk = 2 * qi + half;
                    const float dw = h2f((uint16_t)(half ? pair >> 16 : pair & 0xffffu));
                    const int w0 = (int)(half ? q[u][qi].z : q[u][qi].x), w1 = (int)(half ? q[u][qi].w : q[u][qi].y);
                    const int k0 = (sb << 8) + (blk << 5) + (g << 3);
#pragma unroll
                    for (int t = 0; t < NT; ++t) {
                        const uint2 c = *(const uint2 *)(l_codes + t * K + k0);
                        int is = __builtin_amdgcn_sdot4(w0, (int)c.x, 0, false);
                        is = __builtin_amdgcn_sdot4(w1, (int)c.y, is, false);
                        acc[t] += (dw * l_d[t * nd + (sb << 3) + blk]) * (float)is;
                    }
                }
            }
        }
    };

    for (int turn = 0; tile < a.n_tiles; tile += gridDim.x, turn ^= 1) {
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = 0.0f;
#pragma unroll
        for (int u0 = 0; u0 < PER; u0 += 2) {
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int sb = wave + (u0 + u) * nw;
                if (sb < nsb) multiply(sb, u);
            }
            // the registers are free again: the wave's next pair of this tile, or its first of the next tile
            if (u0 + 2 < PER) request(tile, u0 + 2);
            else if (tile + (int)gridDim.x < a.n_tiles) request(tile + (int)gridDim.x, 0);
        }
        // the four lane groups of a row, then the waves of the workgroup
        float * red = l_red + turn * (nw * NT * 16);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            acc[t] += __shfl_xor(acc[t], 16, 64);
            acc[t] += __shfl_xor(acc[t], 32, 64);
            if (g == 0) red[(wave * NT + t) * 16 + r] = acc[t];
        }
        __syncthreads();
        if (tid < NT * 16) {
            const int t = tid >> 4, row = tid & 15;
            if (t < a.T) {
                float v = 0.0f;
                for (int w = 0; w < nw; ++w) v += red[(w * NT + t) * 16 + row];
                const int n = tile * 16 + row;
                if (a.bias) v += a.bias[n];
                float * dst = a.y + (size_t)t * a.ldy + a.col0 + n;
                *dst = a.mode == MM_ADD ? *dst + v : v;
            }
        }
    }
}

// The same kernel for the exact arithmetic: the rows of the step stay f32 in LDS and every weight code is converted
// (v_cvt_f32_ubyte) and multiplied by a fused multiply-add - about four times the integer kernel's vector
// instructions per weight, which one or two tokens still hide behind the memory. Per eight columns a lane forms
// p = sum q_k x_k in f32 and adds sc * p (Q4_K, Q5_K, Q6_K) to the super-block's sum; the offsets (Q4_K / Q5_K:
// dmin * m_s * sum of the sub-block's x; Q6_K: 32 * sc_b * sum of the block's x) come from the sums of every sixteen
// values made while the rows are staged. Q8_0: d_b * p per block. Sources: SRC_CODES - here the hi / lo planes a
// producer left (the value is hi + lo) -, SRC_NORM and SRC_SWIGLU as above, the values kept as they are computed.
// Dynamic LDS: NT * K floats | K-quants: NT * K / 16 floats | 2 * nw * NT * 16 floats.
template <int WT, int NT, int PER, int SRC>
__global__ __launch_bounds__(1024) void k_gemv_f32(GemvArgs a) {
    using Tile = GemvTile<WT>;
    constexpr bool Q5 = WT == WT_Q5_K, Q4 = WT == WT_Q4_K || Q5, Q6 = WT == WT_Q6_K, KQ = WT != WT_Q8_0;
    static_assert(SRC == SRC_CODES || SRC == SRC_NORM || SRC == SRC_SWIGLU, "planes, RMSNorm or SwiGLU");
    extern __shared__ __align__(16) uint8_t lds[];
    const int K = a.K, nsb = K >> 8;
    const int nthreads = blockDim.x, nw = nthreads >> 6;
    float * l_x = (float *)lds;
    float * l_s = l_x + NT * K;
    float * l_red = KQ ? l_s + NT * (K >> 4) : l_s;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;

    u4 hdr[2], q[2][Tile::LOADS];
    uint16_t dq6[2] = {0, 0};
    uint32_t fifth[2][2] = {{0, 0}, {0, 0}};
    auto request = [&](int tile, int u0) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int sb = wave + (u0 + u) * nw;
            if (sb < nsb) {
                const uint8_t * tp = a.w + ((size_t)tile * nsb + sb) * Tile::BYTES;
                hdr[u] = *(const u4 *)(tp + r * 16);
                if constexpr (Q6) {
                    q[u][0] = *(const u4 *)(tp + 288 + lane * 16);
                    q[u][1] = *(const u4 *)(tp + 1312 + lane * 16);
                    const uint2 t0 = *(const uint2 *)(tp + 2336 + lane * 8), t1 = *(const uint2 *)(tp + 2848 + lane * 8);
                    q[u][2] = u4{t0.x, t0.y, t1.x, t1.y};
                    dq6[u] = *(const uint16_t *)(tp + 256 + 2 * r);
                } else {
#pragma unroll
                    for (int i = 0; i < Tile::LOADS; ++i) q[u][i] = *(const u4 *)(tp + 256 + i * 1024 + lane * 16);
                    if constexpr (Q5) {
                        fifth[u][0] = *(const uint32_t *)(tp + 2304 + lane * 4);
                        fifth[u][1] = *(const uint32_t *)(tp + 2560 + lane * 4);
                    }
                }
            }
        }
    };
    // as in k_gemv: what a thread's first eight values of row 0 are made from is requested ahead of the weights
    auto row_of = [&](int t) -> const float * {
        if (SRC == SRC_NORM) return a.xin + (size_t)(a.rows ? a.rows[t] : t) * K;
        return a.xin + (size_t)t * 2 * K;
    };
    auto load_in = [&](int t, int k, f4 (&in)[4]) {
        if (SRC == SRC_NORM) {
            const float * xr = row_of(t);
            in[0] = *(const f4 *)(xr + k); in[1] = *(const f4 *)(xr + k + 4);
            in[2] = *(const f4 *)(a.norm_w + k); in[3] = *(const f4 *)(a.norm_w + k + 4);
        } else if (SRC == SRC_SWIGLU) {
            const float * gp = row_of(t) + (size_t)(k / a.group) * 2 * a.group + k % a.group, * up = gp + a.group;
            in[0] = *(const f4 *)gp; in[1] = *(const f4 *)(gp + 4); in[2] = *(const f4 *)up; in[3] = *(const f4 *)(up + 4);
        } else {
            // the hi and lo halves of eight values: sixteen bytes each
            in[0] = *(const f4 *)(a.planes + act_at(t, k, 0, K));
            in[1] = *(const f4 *)(a.planes + act_at(t, k, 1, K));
        }
    };
    f4 first[4];
    if (tid * 8 < K) load_in(0, tid * 8, first);
    int tile = blockIdx.x;
    if (tile < a.n_tiles) request(tile, 0);

    auto store8 = [&](const float (&v)[8], int t, int k) {
        *(f4 *)(l_x + t * K + k) = (f4){v[0], v[1], v[2], v[3]};
        *(f4 *)(l_x + t * K + k + 4) = (f4){v[4], v[5], v[6], v[7]};
        if (KQ) {
            float sum = ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
            sum += __shfl_xor(sum, 1, 64);
            if ((tid & 1) == 0) l_s[t * (K >> 4) + (k >> 4)] = sum;
        }
    };
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        float scale = 1.0f;
        if (SRC == SRC_NORM) {
            const float * xr = row_of(t);
            float ss = 0.0f;
            for (int k = tid * 8; k < K; k += nthreads * 8) {
                f4 in[2];
                if (t == 0 && k == tid * 8) { in[0] = first[0]; in[1] = first[1]; }
                else { in[0] = *(const f4 *)(xr + k); in[1] = *(const f4 *)(xr + k + 4); }
                const f4 p = in[0], q4 = in[1];
                ss += p.x * p.x + p.y * p.y + p.z * p.z + p.w * p.w + q4.x * q4.x + q4.y * q4.y + q4.z * q4.z + q4.w * q4.w;
            }
            ss = wave_sum(ss);
            if (lane == 0) l_red[wave] = ss;
            __syncthreads();
            float total = 0.0f;
            for (int i = 0; i < nw; ++i) total += l_red[i];
            scale = 1.0f / sqrtf(total / (float)K + a.eps);
            if (t + 1 < NT) __syncthreads();
        }
        for (int k = tid * 8; k < K; k += nthreads * 8) {
            f4 in[4];
            if (t == 0 && k == tid * 8) { in[0] = first[0]; in[1] = first[1]; in[2] = first[2]; in[3] = first[3]; }
            else load_in(t, k, in);
            float v[8];
            if (SRC == SRC_NORM) {
                v[0] = (in[0].x * scale) * in[2].x; v[1] = (in[0].y * scale) * in[2].y;
                v[2] = (in[0].z * scale) * in[2].z; v[3] = (in[0].w * scale) * in[2].w;
                v[4] = (in[1].x * scale) * in[3].x; v[5] = (in[1].y * scale) * in[3].y;
                v[6] = (in[1].z * scale) * in[3].z; v[7] = (in[1].w * scale) * in[3].w;
            } else if (SRC == SRC_SWIGLU) {
                const float gv[8] = {in[0].x, in[0].y, in[0].z, in[0].w, in[1].x, in[1].y, in[1].z, in[1].w};
                const float uv[8] = {in[2].x, in[2].y, in[2].z, in[2].w, in[3].x, in[3].y, in[3].z, in[3].w};
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = (gv[i] / (1.0f + __expf(-gv[i]))) * uv[i];
            } else {
                const h8 hi = __builtin_bit_cast(h8, in[0]), lo = __builtin_bit_cast(h8, in[1]);
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = t < a.T ? (float)hi[i] + (float)lo[i] : 0.0f;
            }
            store8(v, t, k);
        }
    }
    __syncthreads();

    float acc[NT];
    // eight codes as bytes in the order 0 4 1 5 (word a) and 2 6 3 7 (word b) times eight values
    auto dot8 = [&](uint32_t wa, uint32_t wb, const f4 & xa, const f4 & xb) {
        float p = (float)(wa & 0xffu) * xa.x;
        p = fmaf((float)((wa >> 16) & 0xffu), xa.y, p);
        p = fmaf((float)(wb & 0xffu), xa.z, p);
        p = fmaf((float)((wb >> 16) & 0xffu), xa.w, p);
        p = fmaf((float)((wa >> 8) & 0xffu), xb.x, p);
        p = fmaf((float)(wa >> 24), xb.y, p);
        p = fmaf((float)((wb >> 8) & 0xffu), xb.z, p);
        p = fmaf((float)(wb >> 24), xb.w, p);
        return p;
    };
    // The values of a lane's eight columns of sub-block d of super-block sb, every token's. A lane reads one group
    // ahead of the one it multiplies and no further, and converts a group's codes when the group before is done (the
    // fence in the loops below): left to itself the compiler requests the values and converts the codes of a whole
    // super-block at once, and with two tokens they do not fit the registers.
    struct X8 { f4 a[NT], b[NT]; };
    auto xload = [&](int sb, int d, X8 & x) {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const float * at = l_x + t * K + (sb << 8) + (d << 5) + (g << 3);
            x.a[t] = *(const f4 *)at; x.b[t] = *(const f4 *)(at + 4);
        }
    };
    auto multiply = [&](int sb, int u) {
        if constexpr (Q4) {
            const Q4KScales S = q4k_scales(hdr[u]);
            float dot[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) dot[t] = 0.0f;
            X8 x;
            xload(sb, 0, x);
#pragma unroll
            for (int d = 0; d < 8; ++d) {
                const int h = d >> 2, j = d & 3;
                X8 nx;
                if (d < 7) xload(sb, d + 1, nx);
                uint32_t wq = j == 0 ? q[u][h].x : (j == 1 ? q[u][h].y : (j == 2 ? q[u][h].z : q[u][h].w));
                asm volatile("" : "+v"(wq), "+v"(dot[0]) :: "memory");     // this group's codes behind the last group's products
                uint32_t lo = wq & 0x0F0F0F0Fu, hi = (wq >> 4) & 0x0F0F0F0Fu;
                if constexpr (Q5) {
                    const uint32_t f = fifth[u][h] >> (2 * j);
                    lo |= ((f << 4) & 0x00100010u) | ((f << 11) & 0x10001000u);
                    hi |= ((f >> 4) & 0x00100010u) | ((f << 3) & 0x10001000u);
                }
                const float sc = (float)((S.sc[h] >> (8 * j)) & 0xffu);
#pragma unroll
                for (int t = 0; t < NT; ++t) dot[t] = fmaf(sc, dot8(lo, hi, x.a[t], x.b[t]), dot[t]);
                if (d < 7) x = nx;
            }
            // the min term: lane group g takes sub-blocks 2g and 2g + 1 (sums of sixteen 4g .. 4g + 3)
            const uint32_t mword = (g < 2 ? S.mn[0] : S.mn[1]) >> (16 * (g & 1));
            const float m0 = (float)(mword & 0xffu), m1 = (float)((mword >> 8) & 0xffu);
            const float dw = h2f((uint16_t)(hdr[u].x & 0xffffu)), dmin = h2f((uint16_t)(hdr[u].x >> 16));
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const f4 bs = *(const f4 *)(l_s + t * (K >> 4) + (sb << 4) + 4 * g);
                const float mins = fmaf(m0, bs.x + bs.y, m1 * (bs.z + bs.w));
                acc[t] += dw * dot[t] - dmin * mins;
            }
        } else if constexpr (Q6) {
            float dot[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) dot[t] = 0.0f;
            X8 x;
            xload(sb, 0, x);
#pragma unroll
            for (int d = 0; d < 8; ++d) {
                const int h = d >> 2, j = d & 3;
                X8 nx;
                if (d < 7) xload(sb, d + 1, nx);
                uint32_t wq = j == 0 ? q[u][h].x : (j == 1 ? q[u][h].y : (j == 2 ? q[u][h].z : q[u][h].w));
                asm volatile("" : "+v"(wq), "+v"(dot[0]) :: "memory");     // this group's codes behind the last group's products
                const uint32_t tw = h == 0 ? (j < 2 ? q[u][2].x : q[u][2].y) : (j < 2 ? q[u][2].z : q[u][2].w);
                const uint32_t top = (j & 1) ? __builtin_amdgcn_alignbit(tw, tw, 8) : tw;
                const uint32_t lo = (wq & 0x0F0F0F0Fu) | (top & 0x00300030u) | ((top << 4) & 0x30003000u);
                const uint32_t hi = ((wq >> 4) & 0x0F0F0F0Fu) | ((top >> 2) & 0x00300030u) | ((top << 2) & 0x30003000u);
                const int b = 8 * h + 2 * j + (g >> 1);
                const uint32_t sw = (b >> 2) == 0 ? hdr[u].x : ((b >> 2) == 1 ? hdr[u].y : ((b >> 2) == 2 ? hdr[u].z : hdr[u].w));
                const float sc = (float)(int)(int8_t)((sw >> (8 * (b & 3))) & 0xffu);
#pragma unroll
                for (int t = 0; t < NT; ++t) dot[t] = fmaf(sc, dot8(lo, hi, x.a[t], x.b[t]), dot[t]);
                if (d < 7) x = nx;
            }
            // the offset of 32: lane group g takes blocks 4g .. 4g + 3 (the bytes of header dword g)
            const uint32_t sw = g == 0 ? hdr[u].x : (g == 1 ? hdr[u].y : (g == 2 ? hdr[u].z : hdr[u].w));
            const float dw = h2f(dq6[u]);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const f4 bs = *(const f4 *)(l_s + t * (K >> 4) + (sb << 4) + 4 * g);
                float corr = (float)(int)(int8_t)(sw & 0xffu) * bs.x;
                corr = fmaf((float)(int)(int8_t)((sw >> 8) & 0xffu), bs.y, corr);
                corr = fmaf((float)(int)(int8_t)((sw >> 16) & 0xffu), bs.z, corr);
                corr = fmaf((float)(int)(int8_t)(sw >> 24), bs.w, corr);
                acc[t] += dw * fmaf(-32.0f, corr, dot[t]);
            }
        } else {
#pragma unroll
            for (int qi = 0; qi < 4; ++qi) {
                const uint32_t pair = qi == 0 ? hdr[u].x : (qi == 1 ? hdr[u].y : (qi == 2 ? hdr[u].z : hdr[u].w));
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int blk = 2 * qi + half;
                    const float dw = h2f((uint16_t)(half ? pair >> 16 : pair & 0xffffu));
                    const uint32_t w0 = half ? q[u][qi].z : q[u][qi].x, w1 = half ? q[u][qi].w : q[u][qi].y;
                    const int k0 = (sb << 8) + (blk << 5) + (g << 3);
                    float c[8];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        c[i] = (float)(int)(int8_t)((w0 >> (8 * i)) & 0xffu);
                        c[4 + i] = (float)(int)(int8_t)((w1 >> (8 * i)) & 0xffu);
                    }
#pragma unroll
                    for (int t = 0; t < NT; ++t) {
                        const f4 xa = *(const f4 *)(l_x + t * K + k0), xb = *(const f4 *)(l_x + t * K + k0 + 4);
                        float p = c[0] * xa.x;
                        p = fmaf(c[1], xa.y, p); p = fmaf(c[2], xa.z, p); p = fmaf(c[3], xa.w, p);
                        p = fmaf(c[4], xb.x, p); p = fmaf(c[5], xb.y, p); p = fmaf(c[6], xb.z, p); p = fmaf(c[7], xb.w, p);
                        acc[t] = fmaf(dw, p, acc[t]);
                    }
                }
            }
        }
    };

    for (int turn = 0; tile < a.n_tiles; tile += gridDim.x, turn ^= 1) {
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = 0.0f;
#pragma unroll
        for (int u0 = 0; u0 < PER; u0 += 2) {
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int sb = wave + (u0 + u) * nw;
                if (sb < nsb) multiply(sb, u);
            }
            if (u0 + 2 < PER) request(tile, u0 + 2);
            else if (tile + (int)gridDim.x < a.n_tiles) request(tile + (int)gridDim.x, 0);
        }
        float * red = l_red + turn * (nw * NT * 16);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            acc[t] += __shfl_xor(acc[t], 16, 64);
            acc[t] += __shfl_xor(acc[t], 32, 64);
            if (g == 0) red[(wave * NT + t) * 16 + r] = acc[t];
        }
        __syncthreads();
        if (tid < NT * 16) {
            const int t = tid >> 4, row = tid & 15;
            if (t < a.T) {
                float v = 0.0f;
                for (int w = 0; w < nw; ++w) v += red[(w * NT + t) * 16 + row];
                const int n = tile * 16 + row;
                if (a.bias) v += a.bias[n];
                float * dst = a.y + (size_t)t * a.ldy + a.col0 + n;
                *dst = a.mode == MM_ADD ? *dst + v : v;
            }
        }
    }
}

constexpr size_t kGemvMaxLds = 96 * 1024;     // of the CU's 160 KiB; two tokens of 24,576 columns take 57 KiB
constexpr size_t kGemvMaxLdsF32 = 112 * 1024; // the f32 row: 24,576 columns take 104 KiB
constexpr int kGemvMaxSb = 16 * 6;            // sixteen waves, at most six super-blocks of a tile each
static size_t gemv_lds_bytes(int type, int NT, int NW, int K) {
    const size_t scales = type == WT_Q8_0 ? (size_t)NT * (K >> 5) * 4 : (size_t)NT * (K >> 8) * 4 + (size_t)NT * (K >> 3);
    return (size_t)NT * K + scales + (size_t)2 * NW * NT * 16 * 4;
}
static size_t gemv_f32_lds_bytes(int type, int NT, int NW, int K) {
    return (size_t)NT * K * 4 + (type == WT_Q8_0 ? 0 : (size_t)NT * (K >> 4) * 4) + (size_t)2 * NW * NT * 16 * 4;
}

bool gemv_can_weight(const Weight & w, int T) {
    return (w.type == WT_Q4_K || w.type == WT_Q5_K || w.type == WT_Q6_K || w.type == WT_Q8_0) && w.packed && T >= 1 && T <= g_gemv_max_t && T <= GEMV_MAX_T
        && w.K % 256 == 0 && w.N % 16 == 0 && w.K > 0 && w.N > 0
        && w.K <= 256 * kGemvMaxSb && gemv_lds_bytes(w.type, GEMV_MAX_T, 16, w.K) <= kGemvMaxLds;
}

bool gemv_f32_can_weight(const Weight & w, int T) {
    return (w.type == WT_Q4_K || w.type == WT_Q5_K || w.type == WT_Q6_K || w.type == WT_Q8_0) && w.packed && T == 1
        && w.K % 256 == 0 && w.N % 16 == 0 && w.K > 0 && w.N > 0
        && w.K <= 256 * kGemvMaxSb && gemv_f32_lds_bytes(w.type, T, 16, w.K) <= kGemvMaxLdsF32;
}

bool gemv_can(const Weight & w, const Act & x, int T) {
    if (!x.qc || !x.qd || x.K != w.K || !gemv_can_weight(w, T)) return false;
    return w.type == WT_Q8_0 ? x.quant == AQ_Q8_0 : (x.quant == AQ_Q8_K && x.qbs != nullptr);
}

template <int WT, int NT, int PER, int SRC>
static void launch_gemv(hipStream_t s, const GemvArgs & a) {
    const int nsb = a.K / 256;
    const int nw = PER == 2 ? (nsb + 1) / 2 : 16;
    const size_t lds = gemv_lds_bytes(WT, NT, nw, a.K);
    static bool once = false;
    if (!once) {
        HIP_OK(hipFuncSetAttribute((const void *)k_gemv<WT, NT, PER, SRC>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kGemvMaxLds));
        once = true;
    }
    // a workgroup stages the step's rows once and then walks tiles: as many workgroups as the chip holds at
    // once, fewer when that gives every workgroup the same number of tiles
    const int capacity = 256 * std::max(1, 2048 / (nw * 64));
    const int turns = (a.n_tiles + capacity - 1) / capacity;
    const unsigned grid = (unsigned)((a.n_tiles + turns - 1) / turns);
    hipLaunchKernelGGL((k_gemv<WT, NT, PER, SRC>), dim3(grid), dim3(nw * 64), lds, s, a);
}

template <int WT, int SRC>
static void launch_gemv_tokens(hipStream_t s, const GemvArgs & a) {
    static_assert(GEMV_MAX_T == 2, "one instantiation per token count");
    // two super-blocks of a tile per wave while sixteen waves cover the row, four or six beyond
    const int nsb = a.K / 256;
    if (a.T == 1) {
        if (nsb <= 32) launch_gemv<WT, 1, 2, SRC>(s, a);
        else if (nsb <= 64) launch_gemv<WT, 1, 4, SRC>(s, a);
        else launch_gemv<WT, 1, 6, SRC>(s, a);
    } else {
        if (nsb <= 32) launch_gemv<WT, 2, 2, SRC>(s, a);
        else if (nsb <= 64) launch_gemv<WT, 2, 4, SRC>(s, a);
        else launch_gemv<WT, 2, 6, SRC>(s, a);
    }
    check_launch("gemv");
}

template <int SRC>
static void launch_gemv_src(hipStream_t s, int type, const GemvArgs & a) {
    if (type == WT_Q4_K) launch_gemv_tokens<WT_Q4_K, SRC>(s, a);
    else if (type == WT_Q5_K) launch_gemv_tokens<WT_Q5_K, SRC>(s, a);
    else if (type == WT_Q6_K) launch_gemv_tokens<WT_Q6_K, SRC>(s, a);
    else launch_gemv_tokens<WT_Q8_0, SRC>(s, a);
}

template <int WT, int NT, int PER, int SRC>
static void launch_gemv_f32(hipStream_t s, const GemvArgs & a) {
    const int nsb = a.K / 256;
    const int nw = PER == 2 ? (nsb + 1) / 2 : 16;
    const size_t lds = gemv_f32_lds_bytes(WT, NT, nw, a.K);
    static bool once = false;
    if (!once) {
        HIP_OK(hipFuncSetAttribute((const void *)k_gemv_f32<WT, NT, PER, SRC>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kGemvMaxLdsF32));
        once = true;
    }
    // as many workgroups as the chip holds at once (by threads and by LDS), fewer when that gives every
    // workgroup the same number of tiles
    const int per_cu = std::max(1, std::min(2048 / (nw * 64), (int)((160 * 1024) / lds)));
    const int capacity = 256 * per_cu;
    const int turns = (a.n_tiles + capacity - 1) / capacity;
    const unsigned grid = (unsigned)((a.n_tiles + turns - 1) / turns);
    hipLaunchKernelGGL((k_gemv_f32<WT, NT, PER, SRC>), dim3(grid), dim3(nw * 64), lds, s, a);
}

template <int WT, int SRC>
static void launch_gemv_f32_tokens(hipStream_t s, const GemvArgs & a) {
    // single-token steps only: with two tokens' values and products the kernel does not fit the 128 registers a
    // workgroup of sixteen waves leaves a lane (the compiler spills the staged values), and the tile kernels take the step
    const int nsb = a.K / 256;
    if (a.T != 1) throw std::runtime_error("gemv_f32: one token");
    if (nsb <= 32) launch_gemv_f32<WT, 1, 2, SRC>(s, a);
    else if (nsb <= 64) launch_gemv_f32<WT, 1, 4, SRC>(s, a);
    else launch_gemv_f32<WT, 1, 6, SRC>(s, a);
    check_launch("gemv_f32");
}

template <int SRC>
static void launch_gemv_f32_src(hipStream_t s, int type, const GemvArgs & a) {
    if (type == WT_Q4_K) launch_gemv_f32_tokens<WT_Q4_K, SRC>(s, a);
    else if (type == WT_Q5_K) launch_gemv_f32_tokens<WT_Q5_K, SRC>(s, a);
    else if (type == WT_Q6_K) launch_gemv_f32_tokens<WT_Q6_K, SRC>(s, a);
    else launch_gemv_f32_tokens<WT_Q8_0, SRC>(s, a);
}

static GemvArgs gemv_args(const Weight & w, int T, float * y, int ldy, int col0, int mode, const float * bias) {
    if (mode != MM_STORE && mode != MM_ADD) throw std::runtime_error("gemv: stores or adds");
    if (col0 < 0 || col0 + w.N > ldy) throw std::runtime_error("gemv: the outputs do not fit the row");
    GemvArgs a {};
    a.w = w.packed; a.y = y; a.bias = bias;
    a.K = w.K; a.N = w.N; a.T = T; a.ldy = ldy; a.col0 = col0; a.mode = mode; a.n_tiles = w.N / 16;
    return a;
}

void gemv(hipStream_t s, const Weight & w, const Act & x, int T, float * y, int ldy, int col0, int mode, const float * bias) {
    if (!gemv_can(w, x, T))
        throw std::runtime_error("gemv: needs Q4_K, Q5_K, Q6_K or Q8_0 tiles, the code buffers of their conversion and at most " + std::to_string(GEMV_MAX_T) + " tokens");
    GemvArgs a = gemv_args(w, T, y, ldy, col0, mode, bias);
    a.codes = x.qc; a.d = x.qd; a.bsums = x.qbs;
    launch_gemv_src<SRC_CODES>(s, w.type, a);
}

void gemv_norm(hipStream_t s, const Weight & w, const float * x, const float * norm_w, float eps, const int32_t * rows, int T,
               float * y, int ldy, int col0, int mode, const float * bias) {
    if (!gemv_can_weight(w, T) || !x || !norm_w) throw std::runtime_error("gemv_norm: needs Q4_K, Q5_K, Q6_K or Q8_0 tiles, the rows and the norm weights");
    GemvArgs a = gemv_args(w, T, y, ldy, col0, mode, bias);
    a.xin = x; a.norm_w = norm_w; a.rows = rows; a.eps = eps;
    launch_gemv_src<SRC_NORM>(s, w.type, a);
}

void gemv_combine(hipStream_t s, const Weight & w, const float * partial, int item0, int n_split, int n_head, int G, int head_dim,
                  float * y, int ldy, int col0, int mode) {
    if (!gemv_can_weight(w, 1) || !partial || item0 < 0 || n_split < 1 || n_split > GEMV_COMBINE_MAX_SPLITS || G < 1 || n_head % G != 0
        || head_dim % 8 != 0 || w.K != n_head * head_dim)
        throw std::runtime_error("gemv_combine: needs Q4_K, Q5_K, Q6_K or Q8_0 tiles over the heads' outputs and at most "
                                 + std::to_string(GEMV_COMBINE_MAX_SPLITS) + " splits");
    GemvArgs a = gemv_args(w, 1, y, ldy, col0, mode, nullptr);
    a.partial = partial; a.item0 = item0; a.n_split = n_split; a.att_G = G; a.att_hd = head_dim;
    launch_gemv_src<SRC_COMBINE>(s, w.type, a);
}

void gemv_swiglu(hipStream_t s, const Weight & w, const float * gu, int group, int T, float * y, int ldy, int col0, int mode) {
    if (group <= 0) group = w.K;
    if (!gemv_can_weight(w, T) || !gu || w.K % group != 0 || group % 8 != 0)
        throw std::runtime_error("gemv_swiglu: needs Q4_K, Q5_K, Q6_K or Q8_0 tiles and gate / up rows in groups that divide the width");
    GemvArgs a = gemv_args(w, T, y, ldy, col0, mode, nullptr);
    a.xin = gu; a.group = group;
    launch_gemv_src<SRC_SWIGLU>(s, w.type, a);
}

void gemv_f32(hipStream_t s, const Weight & w, const Act & x, int T, float * y, int ldy, int col0, int mode, const float * bias) {
    if (!gemv_f32_can_weight(w, T) || !x.x || x.K != w.K)
        throw std::runtime_error("gemv_f32: needs Q4_K, Q5_K, Q6_K or Q8_0 tiles, the hi / lo planes of the row and a single token");
    GemvArgs a = gemv_args(w, T, y, ldy, col0, mode, bias);
    a.planes = x.x;
    launch_gemv_f32_src<SRC_CODES>(s, w.type, a);
}

void gemv_f32_norm(hipStream_t s, const Weight & w, const float * x, const float * norm_w, float eps, const int32_t * rows, int T,
                   float * y, int ldy, int col0, int mode, const float * bias) {
    if (!gemv_f32_can_weight(w, T) || !x || !norm_w) throw std::runtime_error("gemv_f32_norm: needs Q4_K, Q5_K, Q6_K or Q8_0 tiles, the rows and the norm weights");
    GemvArgs a = gemv_args(w, T, y, ldy, col0, mode, bias);
    a.xin = x; a.norm_w = norm_w; a.rows = rows; a.eps = eps;
    launch_gemv_f32_src<SRC_NORM>(s, w.type, a);
}

void gemv_f32_swiglu(hipStream_t s, const Weight & w, const float * gu, int group, int T, float * y, int ldy, int col0, int mode) {
    if (group <= 0) group = w.K;
    if (!gemv_f32_can_weight(w, T) || !gu || w.K % group != 0 || group % 8 != 0)
        throw std::runtime_error("gemv_f32_swiglu: needs Q4_K, Q5_K, Q6_K or Q8_0 tiles and gate / up rows in groups that divide the width");
    GemvArgs a = gemv_args(w, T, y, ldy, col0, mode, nullptr);
    a.xin = gu; a.group = group;
    launch_gemv_f32_src<SRC_SWIGLU>(s, w.type, a);
}

}  // namespace rk
