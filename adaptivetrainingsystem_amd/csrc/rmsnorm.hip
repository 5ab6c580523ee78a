// RMSNorm forward for gfx950.  HBM-bound: every element is read once and
// written once.  One wave64 owns one row at a time, keeps the whole row in
// registers as 16-byte vectors (so x is fetched exactly once), reduces the sum
// of squares with cross-lane shuffles, and writes 16 bytes per lane.  The
// weight vector is loaded into registers once per wave and reused for every
// row that wave processes.
#include "ats_common.hpp"

namespace ats {

template <typename T, typename WT, int NV, bool HAS_W>
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const T* __restrict__ x,
                                                           const WT* __restrict__ w,
                                                           T* __restrict__ y, int64_t rows, int H,
                                                           float eps) {
    constexpr int V = Elem<T>::kVec;
    const int lane = lane_id();
    const int nvec = H / V;
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);

    float wreg[NV][V];
    if (HAS_W) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = lane + i * kWave;
            if (v < nvec) {
#pragma unroll
                for (int j = 0; j < V; ++j) wreg[i][j] = Elem<WT>::load(w + (int64_t)v * V + j);
            }
        }
    }

    for (int64_t row = wave; row < rows; row += nwaves) {
        const uint4* xr = reinterpret_cast<const uint4*>(x + row * H);
        uint4 raw[NV];
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = lane + i * kWave;
            if (v < nvec) raw[i] = xr[v];
        }
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = lane + i * kWave;
            if (v < nvec) {
                float f[V];
                Elem<T>::unpack(raw[i], f);
#pragma unroll
                for (int j = 0; j < V; ++j) ss += f[j] * f[j];
            }
        }
        ss = wave_sum(ss);
        const float r = 1.0f / sqrtf(ss / (float)H + eps);
        uint4* yr = reinterpret_cast<uint4*>(y + row * H);
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = lane + i * kWave;
            if (v < nvec) {
                float f[V];
                Elem<T>::unpack(raw[i], f);
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    float t = f[j] * r;
                    if (HAS_W) t = t * wreg[i][j];
                    f[j] = t;
                }
                yr[v] = Elem<T>::pack(f);
            }
        }
    }
}

// Any hidden size / alignment: one wave per row, scalar accesses, second pass
// re-reads the row (served by L2).
template <typename T, typename WT, bool HAS_W>
__global__ __launch_bounds__(256) void rmsnorm_generic_kernel(const T* __restrict__ x,
                                                              const WT* __restrict__ w,
                                                              T* __restrict__ y, int64_t rows, int H,
                                                              float eps) {
    const int lane = lane_id();
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
    for (int64_t row = wave; row < rows; row += nwaves) {
        const T* xr = x + row * H;
        float ss = 0.f;
        for (int h = lane; h < H; h += kWave) {
            const float f = Elem<T>::load(xr + h);
            ss += f * f;
        }
        ss = wave_sum(ss);
        const float r = 1.0f / sqrtf(ss / (float)H + eps);
        T* yr = y + row * H;
        for (int h = lane; h < H; h += kWave) {
            float t = Elem<T>::load(xr + h) * r;
            if (HAS_W) t = t * Elem<WT>::load(w + h);
            Elem<T>::store(yr + h, t);
        }
    }
}

template <typename T, typename WT, bool HAS_W>
static int launch_rmsnorm(const void* x, const void* w, void* y, int64_t rows, int H, float eps,
                          hipStream_t s) {
    constexpr int V = Elem<T>::kVec;
    const T* xp = static_cast<const T*>(x);
    const WT* wp = static_cast<const WT*>(w);
    T* yp = static_cast<T*>(y);
    const int64_t blocks64 = (rows + 3) / 4;
    const int blocks = (int)(blocks64 < 4096 ? blocks64 : 4096);
    const bool vec_ok = (H % V == 0) && aligned16(x) && aligned16(y) && (H / V) <= 16 * kWave;
    if (!vec_ok) {
        hipLaunchKernelGGL((rmsnorm_generic_kernel<T, WT, HAS_W>), dim3(blocks), dim3(256), 0, s, xp, wp,
                           yp, rows, H, eps);
        return ATS_OK;
    }
    const int per_lane = (H / V + kWave - 1) / kWave;
#define ATS_RMS_CASE(NV)                                                                            \
    hipLaunchKernelGGL((rmsnorm_rows_kernel<T, WT, NV, HAS_W>), dim3(blocks), dim3(256), 0, s, xp, wp, \
                       yp, rows, H, eps)
    if (per_lane <= 1) ATS_RMS_CASE(1);
    else if (per_lane <= 2) ATS_RMS_CASE(2);
    else if (per_lane <= 4) ATS_RMS_CASE(4);
    else if (per_lane <= 8) ATS_RMS_CASE(8);
    else ATS_RMS_CASE(16);
#undef ATS_RMS_CASE
    return ATS_OK;
}

}  // namespace ats

extern "C" int ats_rmsnorm_fwd(const void* x, const void* w, void* y, int64_t rows, int hidden,
                               float eps, int x_dtype, int w_dtype, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(rows >= 0 && hidden > 0, ATS_ERR_INVALID_ARG, "ats_rmsnorm_fwd: rows=%lld hidden=%d",
                (long long)rows, hidden);
    if (rows == 0) return ATS_OK;
    ATS_REQUIRE(x && y, ATS_ERR_INVALID_ARG, "ats_rmsnorm_fwd: null pointer");
    ATS_REQUIRE((x_dtype == ATS_F32 || x_dtype == ATS_BF16) && (w_dtype == ATS_F32 || w_dtype == ATS_BF16),
                ATS_ERR_UNSUPPORTED, "ats_rmsnorm_fwd: dtype tags %d/%d", x_dtype, w_dtype);
    hipStream_t s = as_stream(stream);
    int rc;
    if (x_dtype == ATS_F32) {
        if (!w) rc = launch_rmsnorm<float, float, false>(x, w, y, rows, hidden, eps, s);
        else if (w_dtype == ATS_F32) rc = launch_rmsnorm<float, float, true>(x, w, y, rows, hidden, eps, s);
        else rc = launch_rmsnorm<float, bf16_t, true>(x, w, y, rows, hidden, eps, s);
    } else {
        if (!w) rc = launch_rmsnorm<bf16_t, float, false>(x, w, y, rows, hidden, eps, s);
        else if (w_dtype == ATS_F32) rc = launch_rmsnorm<bf16_t, float, true>(x, w, y, rows, hidden, eps, s);
        else rc = launch_rmsnorm<bf16_t, bf16_t, true>(x, w, y, rows, hidden, eps, s);
    }
    if (rc != ATS_OK) return rc;
    ATS_CHECK_LAUNCH("ats_rmsnorm_fwd");
    return ATS_OK;
}
