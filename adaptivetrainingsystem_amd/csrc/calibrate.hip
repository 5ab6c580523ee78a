// Calibration loops for the benchmark: what the matrix cores sustain when nothing else is going on.
//
// The grouped expert GEMM at prefill sizes is limited by board power, not by instruction issue: with random
// bf16 operands the core clock settles well below its ceiling.  This kernel issues independent MFMAs on
// operands that live in registers (no memory traffic at all), so its rate is the ceiling that a GEMM with the
// same operand statistics can approach on the same machine, and the ratio between its two operand modes
// (all-zero bits vs random bits) shows how much of the nominal peak the power limit takes away.
#include "ats_common.hpp"

namespace ats {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 cal_bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float cal_f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float cal_f32x4_t;
typedef unsigned int cal_u32x4_t __attribute__((ext_vector_type(4)));

// externally visible, so that the stores below (which keep the products alive) are not removed
__device__ float ats_calibrate_sink[64];

// Two bf16 values per word, each a normal deviate of standard deviation 0.5 (Box-Muller on hashed uniforms):
// the operand statistics of activations and of scaled weights, which is what the power draw depends on.
__device__ __forceinline__ unsigned cal_hash(unsigned x) {
    x *= 2654435761u;
    x ^= x >> 15;
    x *= 2246822519u;
    x ^= x >> 13;
    x *= 3266489917u;
    x ^= x >> 16;
    return x;
}
__device__ __forceinline__ float cal_normal(unsigned seed) {
    const float u1 = ((cal_hash(seed) >> 8) + 1.0f) * (1.0f / 16777217.0f);
    const float u2 = (cal_hash(seed ^ 0x9e3779b9u) >> 8) * (1.0f / 16777216.0f);
    return 0.5f * sqrtf(-2.0f * logf(u1)) * cosf(6.28318530718f * u2);
}
__device__ __forceinline__ unsigned cal_word(unsigned seed) {
    return pack_bf16x2(cal_normal(2u * seed), cal_normal(2u * seed + 1u));
}

// SHAPE 0: v_mfma_f32_32x32x16_bf16, wave tile 128 x 64 (8 accumulator tiles);
// SHAPE 1: v_mfma_f32_16x16x32_bf16, wave tile 128 x 64 (32 accumulator tiles).  Both: 128 accumulator registers.
template <int SHAPE>
__global__ __launch_bounds__(512) void calibrate_mfma_kernel(int random_operands, int iters, unsigned long long* clocks) {
    constexpr int TA = SHAPE == 0 ? 4 : 8, TB = SHAPE == 0 ? 2 : 4;
    union {
        cal_u32x4_t u;
        cal_bf16x8_t v;
    } a[TA], b[TB];
    const unsigned t = blockIdx.x * 512u + threadIdx.x;
#pragma unroll
    for (int i = 0; i < TA; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c) a[i].u[c] = random_operands ? cal_word(t * 64u + i * 4 + c) : 0u;
#pragma unroll
    for (int i = 0; i < TB; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c) b[i].u[c] = random_operands ? cal_word(t * 64u + 32 + i * 4 + c) : 0u;
    float s = 0.f;
    const unsigned long long c0 = clock64(), w0 = wall_clock64();
    if constexpr (SHAPE == 0) {
        cal_f32x16_t acc[TB][TA];
#pragma unroll
        for (int j = 0; j < TB; ++j)
#pragma unroll
            for (int i = 0; i < TA; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[j][i][v] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int j = 0; j < TB; ++j)
#pragma unroll
                for (int i = 0; i < TA; ++i)
                    acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[j].v, a[i].v, acc[j][i], 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < TB; ++j)
#pragma unroll
            for (int i = 0; i < TA; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) s += acc[j][i][v];
    } else {
        cal_f32x4_t acc[TB][TA];
#pragma unroll
        for (int j = 0; j < TB; ++j)
#pragma unroll
            for (int i = 0; i < TA; ++i) acc[j][i] = cal_f32x4_t{0.f, 0.f, 0.f, 0.f};
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int j = 0; j < TB; ++j)
#pragma unroll
                for (int i = 0; i < TA; ++i)
                    acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[j].v, a[i].v, acc[j][i], 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < TB; ++j)
#pragma unroll
            for (int i = 0; i < TA; ++i)
#pragma unroll
                for (int v = 0; v < 4; ++v) s += acc[j][i][v];
    }
    asm volatile("" ::"v"(s));               // the clocks are read after the last product
    if (clocks && t == 0) {
        clocks[0] = clock64() - c0;          // core clock cycles
        clocks[1] = wall_clock64() - w0;     // ticks of the constant 100 MHz clock
    }
    if (s == 1.2345678e-30f) ats_calibrate_sink[threadIdx.x & 63] = s;   // keeps the products alive
}

// Plain streaming copy, 16 bytes per lane and four loads in flight per lane: the yardstick for the
// bandwidth-bound kernels (what a kernel that only moves its bytes reaches at the same size).
__global__ __launch_bounds__(256) void calibrate_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                             size_t n) {
    size_t i = (size_t)blockIdx.x * 1024 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 1024;
    for (; i < n; i += stride) {
        uint4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (i + u * 256 < n) v[u] = stream_load(src + i + u * 256);
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (i + u * 256 < n) stream_store(dst + i + u * 256, v[u]);
    }
}

// Plain streaming read, 16 bytes per lane and eight loads in flight per lane: the yardstick for the kernels
// that stream weights (what a kernel that only reads its bytes, front to back, reaches).  The values are folded
// into a word that is stored only if it takes one particular value, which keeps the loads alive.
__global__ __launch_bounds__(256) void calibrate_read_kernel(const uint4* __restrict__ src, size_t n,
                                                             unsigned* __restrict__ sink) {
    size_t i = (size_t)blockIdx.x * 2048 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 2048;
    unsigned acc = 0u;
    for (; i < n; i += stride) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            v[u] = make_uint4(0u, 0u, 0u, 0u);
            if (i + u * 256 < n) v[u] = stream_load(src + i + u * 256);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (acc == 0x9e3779b9u) sink[0] = acc;
}

}  // namespace ats

extern "C" int ats_calibrate_read(const void* src, size_t bytes, void* sink, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(src && sink && bytes % 16 == 0 && aligned16(src), ATS_ERR_INVALID_ARG,
                "ats_calibrate_read: a 16-byte aligned buffer of a multiple of 16 bytes and a 4-byte sink");
    if (bytes == 0) return ATS_OK;
    const size_t n = bytes / 16;
    size_t blocks = (n + 2047) / 2048;
    if (blocks > 2048) blocks = 2048;
    hipLaunchKernelGGL(calibrate_read_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                       static_cast<const uint4*>(src), n, static_cast<unsigned*>(sink));
    ATS_CHECK_LAUNCH("ats_calibrate_read");
    return ATS_OK;
}

extern "C" int ats_calibrate_copy(const void* src, void* dst, size_t bytes, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(src && dst && bytes % 16 == 0 && aligned16(src) && aligned16(dst), ATS_ERR_INVALID_ARG,
                "ats_calibrate_copy: 16-byte aligned buffers and a multiple of 16 bytes");
    if (bytes == 0) return ATS_OK;
    const size_t n = bytes / 16;
    size_t blocks = (n + 1023) / 1024;
    if (blocks > 2048) blocks = 2048;
    hipLaunchKernelGGL(calibrate_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                       static_cast<const uint4*>(src), static_cast<uint4*>(dst), n);
    ATS_CHECK_LAUNCH("ats_calibrate_copy");
    return ATS_OK;
}

extern "C" int ats_calibrate_mfma(int shape, int random_operands, int iters, uint64_t* clocks_dev, double* flop_out,
                                  ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE((shape == 0 || shape == 1) && iters > 0 && iters <= (1 << 24), ATS_ERR_INVALID_ARG,
                "ats_calibrate_mfma: shape=%d iters=%d", shape, iters);
    constexpr int kBlocks = 256;     // one 8-wave workgroup per compute unit, two waves per SIMD
    // per wave and iteration: 8 products of 2 x 32 x 32 x 16 flop, or 32 products of 2 x 16 x 16 x 32 flop
    if (flop_out) *flop_out = (double)kBlocks * 8.0 * (double)iters * (shape == 0 ? 8.0 * 32768.0 : 32.0 * 16384.0);
    hipStream_t s = as_stream(stream);
    auto* clk = reinterpret_cast<unsigned long long*>(clocks_dev);
    if (shape == 0) hipLaunchKernelGGL(calibrate_mfma_kernel<0>, dim3(kBlocks), dim3(512), 0, s, random_operands, iters, clk);
    else hipLaunchKernelGGL(calibrate_mfma_kernel<1>, dim3(kBlocks), dim3(512), 0, s, random_operands, iters, clk);
    ATS_CHECK_LAUNCH("ats_calibrate_mfma");
    return ATS_OK;
}
