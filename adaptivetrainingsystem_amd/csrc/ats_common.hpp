// Shared device/host helpers for the gfx950 sparse-layer kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <initializer_list>

#include "../../include/ats_gfx950.h"

namespace ats {

constexpr int kWave = 64;

void set_error(const char* fmt, ...);

#define ATS_REQUIRE(cond, code, ...)    \
    do {                                \
        if (!(cond)) {                  \
            ats::set_error(__VA_ARGS__); \
            return (code);              \
        }                               \
    } while (0)

// Checks the launch that was just issued; never synchronises.
#define ATS_CHECK_LAUNCH(name)                                                        \
    do {                                                                              \
        hipError_t e_ = hipGetLastError();                                            \
        if (e_ != hipSuccess) {                                                       \
            ats::set_error("%s: launch failed: %s", name, hipGetErrorString(e_));     \
            return ATS_ERR_LAUNCH;                                                    \
        }                                                                             \
    } while (0)

// A kernel that uses more than 64 KB of dynamic LDS needs the limit raised once per device (the attribute
// belongs to the function on the current device).  One LdsReservation per launch site remembers, as a
// bit per device id, where that has been done; racing first calls only repeat the idempotent request.
struct LdsReservation {
    std::atomic<uint64_t> done{0};
};
inline hipError_t reserve_lds(LdsReservation& r, std::initializer_list<const void*> kernels, int bytes) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const uint64_t bit = 1ull << (dev & 63);
    if (dev < 64 && (r.done.load(std::memory_order_relaxed) & bit)) return hipSuccess;
    for (const void* k : kernels) {
        e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (e != hipSuccess) return e;
    }
    if (dev < 64) r.done.fetch_or(bit, std::memory_order_relaxed);
    return hipSuccess;
}

inline hipStream_t as_stream(ats_stream_t s) { return reinterpret_cast<hipStream_t>(s); }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---------------------------------------------------------------- element types
struct bf16_t {
    uint16_t bits;
};

__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) { return __uint_as_float(b << 16); }

// float32 pair -> packed bf16 pair with the hardware converter (v_cvt_pk_bf16_f32: round to
// nearest even, NaN stays a quiet NaN).  lo goes to bits [15:0].
typedef __bf16 ats_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float ats_f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    union {
        ats_bf16x2_t b;
        uint32_t u;
    } cv;
    cv.b = __builtin_convertvector(ats_f32x2_t{lo, hi}, ats_bf16x2_t);
    return cv.u;
}
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) { return pack_bf16x2(f, 0.f) & 0xffffu; }

template <typename T>
struct Elem;
template <>
struct Elem<float> {
    static constexpr int kVec = 4;  // elements per 16-byte access
    __device__ static __forceinline__ float load(const float* p) { return *p; }
    __device__ static __forceinline__ void store(float* p, float v) { *p = v; }
    __device__ static __forceinline__ void unpack(const uint4& v, float* f) {
        f[0] = __uint_as_float(v.x);
        f[1] = __uint_as_float(v.y);
        f[2] = __uint_as_float(v.z);
        f[3] = __uint_as_float(v.w);
    }
    __device__ static __forceinline__ uint4 pack(const float* f) {
        return make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]),
                          __float_as_uint(f[3]));
    }
};
template <>
struct Elem<bf16_t> {
    static constexpr int kVec = 8;
    __device__ static __forceinline__ float load(const bf16_t* p) { return bf16_bits_to_float(p->bits); }
    __device__ static __forceinline__ void store(bf16_t* p, float v) {
        p->bits = static_cast<uint16_t>(float_to_bf16_bits(v));
    }
    __device__ static __forceinline__ void unpack(const uint4& v, float* f) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(w[i] << 16);
            f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    __device__ static __forceinline__ uint4 pack(const float* f) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = pack_bf16x2(f[2 * i], f[2 * i + 1]);
        return make_uint4(w[0], w[1], w[2], w[3]);
    }
};

// silu(g) = g / (1 + exp(-g)) with the hardware exp2 and reciprocal (each about 1 ulp): the
// result is within ~3e-7 relative of the correctly rounded value, far inside the float32 bar.
__device__ __forceinline__ float silu_f(float g) {
    const float e = __builtin_amdgcn_exp2f(g * -1.4426950408889634f);
    return g * __builtin_amdgcn_rcpf(1.0f + e);
}

// sigmoid with the hardware exp2 and reciprocal (each about 1 ulp): a few 1e-7 relative, well inside the
// float32 bar of the gradients.
__device__ __forceinline__ float sigmoid_f(float v) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(v * -1.4426950408889634f));
}

// 16-byte accesses of data that is touched once: the non-temporal hint keeps a stream from displacing what
// other kernels left in the caches (measured on a 67 MB copy: 1-3 % faster than plain accesses).
typedef unsigned int ats_u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 stream_load(const uint4* p) {
    const ats_u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const ats_u32x4_t*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void stream_store(uint4* p, const uint4& v) {
    const ats_u32x4_t t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<ats_u32x4_t*>(p));
}

// ---------------------------------------------------------------- wave helpers
// Whole-wave reductions without LDS traffic: four DPP steps leave the result of every row of 16 lanes in all of
// its lanes (the lane pairs, the quads, the mirrored half rows, the mirrored rows), the four row results are read
// back as scalars and folded in a fixed order.  All 64 lanes must be active.
template <int CTRL>
__device__ __forceinline__ unsigned dpp_u32(unsigned v) {
    return (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
constexpr int kDppSwapPairs = 0xB1, kDppSwapQuadHalves = 0x4E, kDppHalfMirror = 0x141, kDppRowMirror = 0x140;
__device__ __forceinline__ unsigned wave_max_u32(unsigned v) {
    v = max(v, dpp_u32<kDppSwapPairs>(v));
    v = max(v, dpp_u32<kDppSwapQuadHalves>(v));
    v = max(v, dpp_u32<kDppHalfMirror>(v));
    v = max(v, dpp_u32<kDppRowMirror>(v));
    const unsigned a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
    const unsigned c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
    return max(max(a, b), max(c, d));
}
__device__ __forceinline__ float wave_max_f32(float v) {
    v = fmaxf(v, dpp_f32<kDppSwapPairs>(v));
    v = fmaxf(v, dpp_f32<kDppSwapQuadHalves>(v));
    v = fmaxf(v, dpp_f32<kDppHalfMirror>(v));
    v = fmaxf(v, dpp_f32<kDppRowMirror>(v));
    const float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}
__device__ __forceinline__ float wave_sum_f32(float v) {
    v += dpp_f32<kDppSwapPairs>(v);
    v += dpp_f32<kDppSwapQuadHalves>(v);
    v += dpp_f32<kDppHalfMirror>(v);
    v += dpp_f32<kDppRowMirror>(v);
    const float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return ((a + b) + c) + d;
}
// Sum over the wave, the same value (bit for bit) in every lane.
__device__ __forceinline__ float wave_sum(float v) { return wave_sum_f32(v); }

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }

// Inclusive prefix sum over the 64 lanes of a wave, all of which must be active.  Four DPP row shifts scan every
// row of 16 lanes (a lane whose source lies outside its row adds 0), the three row totals are read back as
// scalars.  A shuffle scan costs six round trips through the LDS crossbar instead.
__device__ __forceinline__ int wave_inclusive_scan(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xF, 0xF, false);   // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xF, 0xF, false);   // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xF, 0xF, false);   // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xF, 0xF, false);   // row_shr:8
    const int r0 = __builtin_amdgcn_readlane(v, 15);
    const int r1 = r0 + __builtin_amdgcn_readlane(v, 31);
    const int r2 = r1 + __builtin_amdgcn_readlane(v, 47);
    const int row = (threadIdx.x & 63) >> 4;
    return v + (row == 0 ? 0 : row == 1 ? r0 : row == 2 ? r1 : r2);
}

}  // namespace ats
