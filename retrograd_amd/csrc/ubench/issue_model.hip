// Micro-benchmarks of the gfx950 compute unit that the tile matmul kernels are designed around.
//
//   1. instruction issue: a loop of v_mfma_f32_32x32x16_f16 (or 16x16x32) with NV independent packed-f16 vector
//      instructions behind each, one and two waves per SIMD, with pseudo-random and with zero operands;
//   2. LDS read rate: ds_read_b128, every wave its own 16 KiB, eight reads in flight;
//   3. global -> LDS direct loads (global_load_lds_dwordx4) from a 1 MiB buffer that stays in L2.
//
// A block is one compute unit's worth (256 blocks; 128 KiB of LDS per block keep two blocks off one unit in parts 2
// and 3). Each wave stamps s_memtime (clock64: shader clocks) and s_memrealtime (wall_clock64: 100 MHz) around
// its loop; the program prints shader clocks per step, nanoseconds per step and the clock rate the two stamps
// imply. Timing only: results of the arithmetic are discarded.
//
// Build:  hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops \
//               -o retrograd_amd/lib/ubench_issue_model retrograd_amd/csrc/ubench/issue_model.hip
// (retrograd_amd/build.py does). Run on an MI355X:  ./retrograd_amd/lib/ubench_issue_model
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); std::exit(1); } } while (0)

// MF: 0 no matrix instruction, 1 32x32x16, 2 16x16x32. One step = one matrix instruction and NV vector instructions.
template <int NV, int MF>
__global__ void k_issue(int iters, const uint32_t * seed, uint64_t * out, float * sink) {
    const int lane = threadIdx.x & 63;
    const u4 s = ((const u4 *)seed)[threadIdx.x & 255];
    const h8 a = __builtin_bit_cast(h8, s), b = __builtin_bit_cast(h8, ((const u4 *)seed)[256 + (threadIdx.x & 255)]);
    f16v acc[4];
    f4v acc4[4];
    for (int m = 0; m < 4; ++m) { for (int i = 0; i < 16; ++i) acc[m][i] = 0.f; for (int i = 0; i < 4; ++i) acc4[m][i] = 0.f; }
    uint32_t x[8];
    for (int i = 0; i < 8; ++i) x[i] = s[i & 3] + i;
    const uint32_t y = s.y, z = s.z;
    const uint64_t t0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            if (MF == 1) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc[m]) : "v"(a), "v"(b));
            if (MF == 2) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc4[m]) : "v"(a), "v"(b));
#pragma unroll
            for (int v = 0; v < NV; ++v) asm volatile("v_pk_fma_f16 %0, %0, %1, %2" : "+v"(x[(m * NV + v) & 7]) : "v"(y), "v"(z));
        }
    }
    const uint64_t t1 = clock64(), w1 = wall_clock64();
    float f = 0.f;
    for (int m = 0; m < 4; ++m) { for (int i = 0; i < 16; ++i) f += acc[m][i]; for (int i = 0; i < 4; ++i) f += acc4[m][i]; }
    for (int i = 0; i < 8; ++i) f += (float)x[i];
    if (f == 12345.678f) sink[0] = f;
    if (lane == 0) {
        const int w = blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64;
        out[2 * w] = t1 - t0;
        out[2 * w + 1] = w1 - w0;
    }
}

__global__ void k_lds_read(int iters, uint64_t * out, uint32_t * sink) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    for (int i = threadIdx.x; i < 131072 / 16; i += blockDim.x) ((u4 *)lds)[i] = (u4){(uint32_t)i, 1u, 2u, 3u};
    __syncthreads();
    const uint32_t addr = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) uint8_t *)lds + (wave % 8) * 16384 + lane * 16;
    u4 r[8];
    for (int i = 0; i < 8; ++i) r[i] = (u4){0u, 0u, 0u, 0u};
    const uint64_t t0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
        asm volatile("ds_read_b128 %0, %8\n\tds_read_b128 %1, %8 offset:1024\n\tds_read_b128 %2, %8 offset:2048\n\tds_read_b128 %3, %8 offset:3072\n\t"
                     "ds_read_b128 %4, %8 offset:4096\n\tds_read_b128 %5, %8 offset:5120\n\tds_read_b128 %6, %8 offset:6144\n\tds_read_b128 %7, %8 offset:7168\n\t"
                     "s_waitcnt lgkmcnt(4)"
                     : "=v"(r[0]), "=v"(r[1]), "=v"(r[2]), "=v"(r[3]), "=v"(r[4]), "=v"(r[5]), "=v"(r[6]), "=v"(r[7]) : "v"(addr));
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const uint64_t t1 = clock64(), w1 = wall_clock64();
    uint32_t f = 0;
    for (int i = 0; i < 8; ++i) f += r[i].x;
    if (f == 0x12345) sink[0] = f;
    if (lane == 0) { const int w = blockIdx.x * (blockDim.x / 64) + wave; out[2 * w] = t1 - t0; out[2 * w + 1] = w1 - w0; }
}

// AHEAD requests of 1 KiB may be outstanding per wave
template <int AHEAD>
__global__ void k_lds_dma(int iters, const uint8_t * src, size_t span, uint64_t * out) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) uint8_t *)lds + (wave % 8) * 16384;
    const uint32_t lane16 = lane * 16;
    const uint64_t t0 = clock64(), w0 = wall_clock64();
    size_t off = (size_t)wave * 4096;
    for (int it = 0; it < iters; ++it) {
        const uint8_t * p = src + off;
        // the instruction's offset moves the global and the LDS address alike
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\t"
                     "global_load_lds_dwordx4 %0, %1\n\tglobal_load_lds_dwordx4 %0, %1 offset:1024\n\t"
                     "global_load_lds_dwordx4 %0, %1 offset:2048\n\tglobal_load_lds_dwordx4 %0, %1 offset:3072"
                     :: "v"(lane16), "s"(p), "s"(lds0 + (it & 3) * 4096) : "memory");
        if (AHEAD == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        off += 32768;
        if (off + 4096 > span) off = (size_t)wave * 4096;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const uint64_t t1 = clock64(), w1 = wall_clock64();
    if (lane == 0) { const int w = blockIdx.x * (blockDim.x / 64) + wave; out[2 * w] = t1 - t0; out[2 * w + 1] = w1 - w0; }
}

static void means(const uint64_t * out, int n_waves, double * clocks, double * wall_ns) {
    std::vector<uint64_t> h(2 * (size_t)n_waves);
    CK(hipMemcpy(h.data(), out, h.size() * 8, hipMemcpyDeviceToHost));
    double c = 0, w = 0;
    for (int i = 0; i < n_waves; ++i) { c += (double)h[2 * i]; w += (double)h[2 * i + 1]; }
    *clocks = c / n_waves;
    *wall_ns = w / n_waves * 10.0;
}

template <int NV, int MF>
static void issue(int threads, int iters, const uint32_t * seed, uint64_t * out, float * sink) {
    hipLaunchKernelGGL((k_issue<NV, MF>), dim3(256), dim3(threads), 0, 0, iters / 10, seed, out, sink);      // warm
    CK(hipDeviceSynchronize());
    hipLaunchKernelGGL((k_issue<NV, MF>), dim3(256), dim3(threads), 0, 0, iters, seed, out, sink);
    CK(hipDeviceSynchronize());
    double c, ns;
    means(out, 256 * threads / 64, &c, &ns);
    const double steps = iters * 4.0;
    std::printf("  %-10s + %d vector, %d wave(s) per SIMD: %6.1f clocks and %6.2f ns per step of a wave, clock %4.0f MHz\n",
                MF == 1 ? "32x32x16" : (MF == 2 ? "16x16x32" : "no matrix"), NV, threads / 256, c / steps, ns / steps, c / ns * 1e3);
    std::fflush(stdout);
}

int main() {
    uint32_t * seed; uint64_t * out; float * sink; uint8_t * src;
    const size_t span = (size_t)1 << 20;
    CK(hipMalloc(&seed, 512 * 16)); CK(hipMalloc(&out, 1 << 20)); CK(hipMalloc(&sink, 4)); CK(hipMalloc(&src, span));
    CK(hipMemset(src, 1, span));
    std::vector<uint32_t> hs(512 * 4);
    const int IT = 20000;
    for (int zero = 0; zero < 2; ++zero) {
        std::srand(1);
        for (auto & v : hs) {
            // f16 pairs of moderate magnitude: exponents 13..16, random mantissas and signs
            auto h = [&]() { return (uint32_t)(((std::rand() & 1) << 15) | ((13 + (std::rand() & 3)) << 10) | (std::rand() & 1023)); };
            v = zero ? 0u : (h() | (h() << 16));
        }
        CK(hipMemcpy(seed, hs.data(), hs.size() * 4, hipMemcpyHostToDevice));
        std::printf("instruction issue, %s operands (a step = one matrix instruction and its vector instructions):\n", zero ? "zero" : "pseudo-random");
        for (int threads : {256, 512}) {
            issue<0, 1>(threads, IT, seed, out, sink);
            issue<0, 2>(threads, IT, seed, out, sink);
            issue<8, 0>(threads, IT, seed, out, sink);
            issue<2, 1>(threads, IT, seed, out, sink);
            issue<4, 1>(threads, IT, seed, out, sink);
            issue<6, 1>(threads, IT, seed, out, sink);
            issue<8, 1>(threads, IT, seed, out, sink);
            issue<2, 2>(threads, IT, seed, out, sink);
            issue<4, 2>(threads, IT, seed, out, sink);
        }
    }
    CK(hipFuncSetAttribute((const void *)k_lds_read, hipFuncAttributeMaxDynamicSharedMemorySize, 131072));
    CK(hipFuncSetAttribute((const void *)k_lds_dma<8>, hipFuncAttributeMaxDynamicSharedMemorySize, 131072));
    CK(hipFuncSetAttribute((const void *)k_lds_dma<16>, hipFuncAttributeMaxDynamicSharedMemorySize, 131072));
    const int LT = 4000;
    std::printf("LDS reads (ds_read_b128, conflict-free, eight in flight per wave):\n");
    for (int threads : {256, 512, 1024}) {
        hipLaunchKernelGGL(k_lds_read, dim3(256), dim3(threads), 131072, 0, LT, out, (uint32_t *)sink);
        CK(hipDeviceSynchronize());
        double c, ns;
        means(out, 256 * threads / 64, &c, &ns);
        const double bytes = LT * 8.0 * 1024 * (threads / 64);
        std::printf("  %2d waves per compute unit: %6.1f B per clock per compute unit, %6.1f GB/s\n", threads / 64, bytes / c, bytes / ns);
    }
    std::printf("global -> LDS direct loads (global_load_lds_dwordx4, source resident in L2, every compute unit at once):\n");
    for (int threads : {256, 512}) {
        for (int ahead : {8, 16}) {
            if (ahead == 8) hipLaunchKernelGGL(k_lds_dma<8>, dim3(256), dim3(threads), 131072, 0, LT, src, span, out);
            else hipLaunchKernelGGL(k_lds_dma<16>, dim3(256), dim3(threads), 131072, 0, LT, src, span, out);
            CK(hipDeviceSynchronize());
            double c, ns;
            means(out, 256 * threads / 64, &c, &ns);
            const double bytes = LT * 4096.0 * (threads / 64);
            std::printf("  %2d waves per compute unit, %2d KiB in flight per wave: %5.1f B per clock per compute unit, %6.1f GB/s\n",
                        threads / 64, ahead, bytes / c, bytes / ns);
        }
    }
    return 0;
}
