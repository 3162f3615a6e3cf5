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
struct MMArgs {
    const uint8_t * w;
    const __half * x;
    const __half * x_lo;
    const __half * xs_hi;
    const __half * xs_lo;
    float * y;
    const float * bias;
    int K, N, T, ldy, col0, mode;
    int n_row_tiles;
    int ksplit;       // v1: waves of a workgroup sharing a row tile along K; v2: workgroups sharing a row group
    // v2 only
    int n_row_groups;
    float * partial;          // [ksplit][gridDim.y * 64][N]
    int32_t * counters;       // [n_row_groups * gridDim.y], zero between launches
    const __half * zeros;     // 16 bytes of zeros
    int debug;                // timing experiments only: bit 0 stage activations once, bit 1 skip the multiplies
};

}  // namespace rk
