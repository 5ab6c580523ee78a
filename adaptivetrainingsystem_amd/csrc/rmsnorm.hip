// RMSNorm forward for gfx950.  HBM-bound: every element is read once and
// written once.  One wave64 owns one row at a time, keeps the whole row in
// registers as 16-byte vectors (so x is fetched exactly once), reduces the sum
// of squares with cross-lane shuffles, and writes 16 bytes per lane.  The
// weight vector is fetched once per block into LDS as float32, behind the
// loads of every wave's first two rows, and kept in registers for every row
// a wave processes.
#include "ats_common.hpp"

namespace ats {

// V consecutive weights as float32, fetched with 16-byte loads where the alignment allows it.
template <typename WT, int V>
__device__ __forceinline__ void load_weight_vec(const WT* __restrict__ w, float (&out)[V]) {
    constexpr int kPer = 16 / (int)sizeof(WT);            // weights per 16-byte load
    if ((reinterpret_cast<uintptr_t>(w) & 15u) == 0 && V % kPer == 0) {
#pragma unroll
        for (int c = 0; c < V / kPer; ++c) {
            float f[kPer];
            Elem<WT>::unpack(reinterpret_cast<const uint4*>(w)[c], f);
#pragma unroll
            for (int j = 0; j < kPer; ++j) out[c * kPer + j] = f[j];
        }
    } else {
#pragma unroll
        for (int j = 0; j < V; ++j) out[j] = Elem<WT>::load(w + j);
    }
}

template <typename T, typename WT, int NV, bool HAS_W>
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const T* __restrict__ x,
                                                           const WT* __restrict__ w,
                                                           T* __restrict__ y, int64_t rows, int H,
                                                           float eps) {
    constexpr int V = Elem<T>::kVec;
    extern __shared__ float w_lds[];      // [H] float32 weights of the block
    const int lane = lane_id();
    const int nvec = H / V;
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);

    // Two rows of a wave (one when a row takes more than four vectors per lane: registers) are asked for before
    // anything else (loads return in order, so whatever is asked for first delays them), then the block's
    // weights: once per block, a 16-byte load or two per thread instead of up to eight per lane of every wave,
    // converted to float32 into LDS, from where every wave picks up its slices.  Later rows are fetched two
    // rows (one row) ahead.  [8192, 2048] bf16 with float32 weights: 13.3 -> 11.6 us.
    constexpr bool kPrefetch = NV <= 8;
    constexpr bool kTwoAhead = NV <= 4;
    constexpr int NP = kPrefetch ? NV : 1;
    constexpr int NP2 = kTwoAhead ? NV : 1;
    uint4 cur[NP], nxt[NP2];
    if (kPrefetch) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = lane + i * kWave;
            if (wave < rows && v < nvec) cur[kPrefetch ? i : 0] = stream_load(reinterpret_cast<const uint4*>(x + wave * H) + v);
        }
    }
    if (kTwoAhead) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = lane + i * kWave;
            if (wave + nwaves < rows && v < nvec)
                nxt[kTwoAhead ? i : 0] = stream_load(reinterpret_cast<const uint4*>(x + (wave + nwaves) * H) + v);
        }
    }
    float wreg[NV][V];
    if (HAS_W && !kTwoAhead) {
        // long rows: every wave loads its own slices (measured at [16384, 4096]: 46.5 us against 48.7 through LDS)
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = lane + i * kWave;
            if (v < nvec) load_weight_vec<WT, V>(w + (int64_t)v * V, wreg[i]);
        }
    }
    if (HAS_W && kTwoAhead) {
        constexpr int kPer = 16 / (int)sizeof(WT);
        if ((reinterpret_cast<uintptr_t>(w) & 15u) == 0 && H % kPer == 0) {
            for (int c = threadIdx.x; c < H / kPer; c += blockDim.x) {
                float f[kPer];
                Elem<WT>::unpack(reinterpret_cast<const uint4*>(w)[c], f);
#pragma unroll
                for (int j = 0; j < kPer; ++j) w_lds[c * kPer + j] = f[j];
            }
        } else {
            for (int h = threadIdx.x; h < H; h += blockDim.x) w_lds[h] = Elem<WT>::load(w + h);
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = lane + i * kWave;
            if (v < nvec) {
#pragma unroll
                for (int j = 0; j < V; j += 4) {
                    const float4 q = *reinterpret_cast<const float4*>(w_lds + v * V + j);
                    wreg[i][j] = q.x;
                    wreg[i][j + 1] = q.y;
                    wreg[i][j + 2] = q.z;
                    wreg[i][j + 3] = q.w;
                }
            }
        }
    }
    for (int64_t row = wave; row < rows; row += nwaves) {
        uint4 raw[NV];
        if (kTwoAhead) {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                raw[i] = cur[kPrefetch ? i : 0];
                cur[kPrefetch ? i : 0] = nxt[kTwoAhead ? i : 0];
            }
            if (row + 2 * nwaves < rows) {
                const uint4* xn = reinterpret_cast<const uint4*>(x + (row + 2 * nwaves) * H);
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    const int v = lane + i * kWave;
                    if (v < nvec) nxt[kTwoAhead ? i : 0] = stream_load(xn + v);
                }
            }
        } else if (kPrefetch) {
#pragma unroll
            for (int i = 0; i < NV; ++i) raw[i] = cur[kPrefetch ? i : 0];
            if (row + nwaves < rows) {
                const uint4* xn = reinterpret_cast<const uint4*>(x + (row + nwaves) * H);
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    const int v = lane + i * kWave;
                    if (v < nvec) cur[kPrefetch ? i : 0] = stream_load(xn + v);
                }
            }
        } else {
            const uint4* xr = reinterpret_cast<const uint4*>(x + row * H);
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int v = lane + i * kWave;
                if (v < nvec) raw[i] = stream_load(xr + v);
            }
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
                stream_store(yr + v, Elem<T>::pack(f));
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
    // resident waves that walk several rows each (with the next row in flight) instead of a wave per row
    // (measured on [8192, 2048] bf16 streamed from HBM: 14.4 us with 2048-4096 blocks, 13.9-14.0 us with 512-1024)
    constexpr int kRmsBlocks = 1024;
    const int blocks = (int)(blocks64 < kRmsBlocks ? blocks64 : kRmsBlocks);
    const bool vec_ok = (H % V == 0) && aligned16(x) && aligned16(y) && (H / V) <= 16 * kWave;
    if (!vec_ok) {
        hipLaunchKernelGGL((rmsnorm_generic_kernel<T, WT, HAS_W>), dim3(blocks), dim3(256), 0, s, xp, wp,
                           yp, rows, H, eps);
        return ATS_OK;
    }
    const int per_lane = (H / V + kWave - 1) / kWave;
    const size_t wl = HAS_W ? (size_t)H * sizeof(float) : 0;      // the block's weights as float32 (rows of up to 4 vectors per lane)
#define ATS_RMS_CASE(NV)                                                                            \
    hipLaunchKernelGGL((rmsnorm_rows_kernel<T, WT, NV, HAS_W>), dim3(blocks), dim3(256), wl, s, xp, wp, \
                       yp, rows, H, eps)
    if (per_lane <= 1) ATS_RMS_CASE(1);
    else if (per_lane <= 2) ATS_RMS_CASE(2);
    else if (per_lane <= 4) ATS_RMS_CASE(4);
    else if (per_lane <= 8) ATS_RMS_CASE(8);
    else ATS_RMS_CASE(16);
#undef ATS_RMS_CASE
    return ATS_OK;
}

// ---------------------------------------------------------------- backward
// y = x * r * w, r = rsqrt(mean(x^2) + eps).  With g = dy * w (dy alone when there is no weight):
//   dx = r * g - x * r^3 * mean(g * x)          dw = sum over rows of dy * x * r
// (RMSNormFunction.backward, cuda_opt_wrapper.py:119-142).  HBM-bound: x and dy are read once,
// dx written once.  A wave keeps its slice of dw in registers over all the rows it processes;
// the waves of a block add their slices in LDS in a fixed order and the block writes one
// partial row; a second kernel adds the partial rows in index order (no atomics, so the result
// does not depend on timing).
template <typename T, typename WT, int NV, bool HAS_W, bool WREG>
__global__ __launch_bounds__(256) void rmsnorm_bwd_rows_kernel(const T* __restrict__ x, const WT* __restrict__ w,
                                                               const T* __restrict__ dy, T* __restrict__ dx,
                                                               float* __restrict__ dw_partial, int64_t rows,
                                                               int H, float eps) {
    constexpr int V = Elem<T>::kVec;
    extern __shared__ float dw_lds[];  // [H] when dw_partial != nullptr
    const int lane = lane_id();
    const int nvec = H / V;
    const int wave_in_block = threadIdx.x >> 6;
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + wave_in_block;
    const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);

    // the weight slice lives in registers unless the row is so long that registers run out;
    // then it is re-read per row (it stays in the vector cache)
    // short rows: the next row is fetched while the current one is reduced and written; the first row's loads
    // go out before the weights' (loads return in order)
    constexpr bool kPrefetch = NV <= 4;
    uint4 xnext[kPrefetch ? NV : 1], gnext[kPrefetch ? NV : 1];
    if (kPrefetch && wave < rows) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = lane + i * kWave;
            if (v < nvec) {
                xnext[kPrefetch ? i : 0] = reinterpret_cast<const uint4*>(x + wave * H)[v];
                gnext[kPrefetch ? i : 0] = reinterpret_cast<const uint4*>(dy + wave * H)[v];
            }
        }
    }
    float wreg[WREG ? NV : 1][V];
    float dwacc[NV][V];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = lane + i * kWave;
#pragma unroll
        for (int j = 0; j < V; ++j) {
            dwacc[i][j] = 0.f;
            if (WREG) wreg[WREG ? i : 0][j] = 1.f;
        }
        if (WREG && HAS_W && v < nvec) load_weight_vec<WT, V>(w + (int64_t)v * V, wreg[WREG ? i : 0]);
    }
#define ATS_WVAL(i_, j_, v_) (!HAS_W ? 1.f : WREG ? wreg[WREG ? (i_) : 0][j_] : Elem<WT>::load(w + (int64_t)(v_) * V + (j_)))
    for (int64_t row = wave; row < rows; row += nwaves) {
        const uint4* xr = reinterpret_cast<const uint4*>(x + row * H);
        const uint4* gr = reinterpret_cast<const uint4*>(dy + row * H);
        uint4 xraw[NV], graw[NV];
        if (kPrefetch) {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                xraw[i] = xnext[kPrefetch ? i : 0];
                graw[i] = gnext[kPrefetch ? i : 0];
            }
            const int64_t nrow = row + nwaves;
            if (nrow < rows) {
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    const int v = lane + i * kWave;
                    if (v < nvec) {
                        xnext[kPrefetch ? i : 0] = reinterpret_cast<const uint4*>(x + nrow * H)[v];
                        gnext[kPrefetch ? i : 0] = reinterpret_cast<const uint4*>(dy + nrow * H)[v];
                    }
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int v = lane + i * kWave;
                if (v < nvec) {
                    xraw[i] = xr[v];
                    graw[i] = gr[v];
                }
            }
        }
        float ss = 0.f, dot = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = lane + i * kWave;
            if (v < nvec) {
                float xf[V], gf[V];
                Elem<T>::unpack(xraw[i], xf);
                Elem<T>::unpack(graw[i], gf);
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    ss += xf[j] * xf[j];
                    dot += gf[j] * ATS_WVAL(i, j, v) * xf[j];
                }
            }
        }
        ss = wave_sum(ss);
        dot = wave_sum(dot);
        const float r = 1.0f / sqrtf(ss / (float)H + eps);
        const float c = dot / (float)H * r * r * r;
        uint4* dxr = reinterpret_cast<uint4*>(dx + row * H);
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = lane + i * kWave;
            if (v < nvec) {
                float xf[V], gf[V], o[V];
                Elem<T>::unpack(xraw[i], xf);
                Elem<T>::unpack(graw[i], gf);
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    o[j] = gf[j] * ATS_WVAL(i, j, v) * r - xf[j] * c;
                    dwacc[i][j] += gf[j] * xf[j] * r;
                }
                dxr[v] = Elem<T>::pack(o);
            }
        }
    }

    if (dw_partial) {
        for (int wv = 0; wv < (int)(blockDim.x >> 6); ++wv) {
            if (wave_in_block == wv) {
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    const int v = lane + i * kWave;
                    if (v < nvec) {
#pragma unroll
                        for (int j = 0; j < V; ++j) {
                            const int h = v * V + j;
                            dw_lds[h] = (wv == 0 ? 0.f : dw_lds[h]) + dwacc[i][j];
                        }
                    }
                }
            }
            __syncthreads();
        }
        for (int h = threadIdx.x; h < H; h += blockDim.x) dw_partial[(int64_t)blockIdx.x * H + h] = dw_lds[h];
    }
}
#undef ATS_WVAL

// Long rows (256-1024 vectors): the 256 lanes of a team (4 waves) share a row, so a lane holds 1-4 vectors of x
// and of dy, few enough registers for 16 waves per CU; a block is two teams.  A team fetches its next row before
// the current row's two sums cross its waves through LDS (one block-wide barrier per row; the slots alternate
// with the row's parity, so a wave that runs ahead never overwrites sums still being read).  At the end team 1
// leaves its dw slice in LDS and team 0 adds its own: one partial row per block.
constexpr int kTeamLanes = 256;
template <typename T, typename WT, int NV, bool HAS_W>
__global__ __launch_bounds__(512, 2) void rmsnorm_bwd_team_kernel(const T* __restrict__ x, const WT* __restrict__ w,
                                                                  const T* __restrict__ dy, T* __restrict__ dx,
                                                                  float* __restrict__ dw_partial, int64_t rows,
                                                                  int H, float eps) {
    constexpr int V = Elem<T>::kVec;
    extern __shared__ float dw_lds[];  // [H] when dw_partial != nullptr
    __shared__ float red[2][2][8];     // [row parity][team][4 x sum of squares, 4 x dot]
    const int lane = lane_id();
    const int team = threadIdx.x >> 8, t = threadIdx.x & (kTeamLanes - 1), wv = t >> 6;
    const int nvec = H / V;
    const int64_t stride = (int64_t)gridDim.x * 2;
    const int64_t first = (int64_t)blockIdx.x * 2;
    // both teams make the same number of trips (the barrier is block-wide); team 1 may idle through the last one
    const int64_t trips = first < rows ? (rows - first + stride - 1) / stride : 0;

    // the first row's loads go out before the weights' (loads return in order, and a block lives for a few rows
    // only: with the weights first, as eight 2-byte loads per vector, [8192, 2048] took 22.4 instead of 20.6 us)
    uint4 xnext[NV], gnext[NV];
    int64_t row = first + team;
    if (row < rows) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = t + i * kTeamLanes;
            if (v < nvec) {
                xnext[i] = reinterpret_cast<const uint4*>(x + row * H)[v];
                gnext[i] = reinterpret_cast<const uint4*>(dy + row * H)[v];
            }
        }
    }
    float wreg[NV][V], dwacc[NV][V];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = t + i * kTeamLanes;
#pragma unroll
        for (int j = 0; j < V; ++j) {
            dwacc[i][j] = 0.f;
            wreg[i][j] = 1.f;
        }
        if (HAS_W && v < nvec) load_weight_vec<WT, V>(w + (int64_t)v * V, wreg[i]);
    }
    for (int64_t trip = 0; trip < trips; ++trip, row += stride) {
        const bool active = row < rows;
        uint4 xraw[NV], graw[NV];
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            xraw[i] = xnext[i];
            graw[i] = gnext[i];
        }
        const int64_t nrow = row + stride;
        if (nrow < rows) {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int v = t + i * kTeamLanes;
                if (v < nvec) {
                    xnext[i] = reinterpret_cast<const uint4*>(x + nrow * H)[v];
                    gnext[i] = reinterpret_cast<const uint4*>(dy + nrow * H)[v];
                }
            }
        }
        float ss = 0.f, dot = 0.f;
        if (active) {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                if (t + i * kTeamLanes < nvec) {
                    float xf[V], gf[V];
                    Elem<T>::unpack(xraw[i], xf);
                    Elem<T>::unpack(graw[i], gf);
#pragma unroll
                    for (int j = 0; j < V; ++j) {
                        ss += xf[j] * xf[j];
                        dot += gf[j] * wreg[i][j] * xf[j];
                    }
                }
            }
        }
        ss = wave_sum(ss);
        dot = wave_sum(dot);
        const int par = (int)(trip & 1);
        if (lane == 0) {
            red[par][team][wv] = ss;
            red[par][team][4 + wv] = dot;
        }
        __syncthreads();
        if (active) {
            const float* rd = red[par][team];
            ss = ((rd[0] + rd[1]) + rd[2]) + rd[3];
            dot = ((rd[4] + rd[5]) + rd[6]) + rd[7];
            const float r = 1.0f / sqrtf(ss / (float)H + eps);
            const float c = dot / (float)H * r * r * r;
            uint4* dxr = reinterpret_cast<uint4*>(dx + row * H);
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int v = t + i * kTeamLanes;
                if (v < nvec) {
                    float xf[V], gf[V], o[V];
                    Elem<T>::unpack(xraw[i], xf);
                    Elem<T>::unpack(graw[i], gf);
#pragma unroll
                    for (int j = 0; j < V; ++j) {
                        o[j] = gf[j] * wreg[i][j] * r - xf[j] * c;
                        dwacc[i][j] += gf[j] * xf[j] * r;
                    }
                    dxr[v] = Elem<T>::pack(o);
                }
            }
        }
    }

    if (dw_partial) {
        if (team == 1) {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int v = t + i * kTeamLanes;
                if (v < nvec) {
#pragma unroll
                    for (int j = 0; j < V; ++j) dw_lds[v * V + j] = dwacc[i][j];
                }
            }
        }
        __syncthreads();
        if (team == 0) {
            float* mine = dw_partial + (int64_t)blockIdx.x * H;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int v = t + i * kTeamLanes;
                if (v < nvec) {
                    // V is 4 or 8 and H a multiple of it, and the workspace is 16-byte aligned: whole float4s
#pragma unroll
                    for (int j = 0; j < V; j += 4) {
                        const float4 o = make_float4(dwacc[i][j] + dw_lds[v * V + j], dwacc[i][j + 1] + dw_lds[v * V + j + 1],
                                                     dwacc[i][j + 2] + dw_lds[v * V + j + 2],
                                                     dwacc[i][j + 3] + dw_lds[v * V + j + 3]);
                        *reinterpret_cast<float4*>(mine + v * V + j) = o;
                    }
                }
            }
        }
    }
}

// Any hidden size / alignment: one wave per row, two scalar passes over the row; every wave owns
// one partial row of dw in global memory and adds to it row after row.
template <typename T, typename WT, bool HAS_W>
__global__ __launch_bounds__(256) void rmsnorm_bwd_generic_kernel(const T* __restrict__ x, const WT* __restrict__ w,
                                                                  const T* __restrict__ dy, T* __restrict__ dx,
                                                                  float* __restrict__ dw_partial, int64_t rows,
                                                                  int H, float eps) {
    const int lane = lane_id();
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
    float* mine = dw_partial ? dw_partial + wave * H : nullptr;
    bool first = true;
    for (int64_t row = wave; row < rows; row += nwaves) {
        const T* xr = x + row * H;
        const T* gr = dy + row * H;
        float ss = 0.f, dot = 0.f;
        for (int h = lane; h < H; h += kWave) {
            const float xf = Elem<T>::load(xr + h);
            const float wf = HAS_W ? Elem<WT>::load(w + h) : 1.f;
            ss += xf * xf;
            dot += Elem<T>::load(gr + h) * wf * xf;
        }
        ss = wave_sum(ss);
        dot = wave_sum(dot);
        const float r = 1.0f / sqrtf(ss / (float)H + eps);
        const float c = dot / (float)H * r * r * r;
        T* dxr = dx + row * H;
        for (int h = lane; h < H; h += kWave) {
            const float xf = Elem<T>::load(xr + h);
            const float gf = Elem<T>::load(gr + h);
            const float wf = HAS_W ? Elem<WT>::load(w + h) : 1.f;
            Elem<T>::store(dxr + h, gf * wf * r - xf * c);
            if (mine) mine[h] = (first ? 0.f : mine[h]) + gf * xf * r;
        }
        first = false;
    }
    if (mine && first)
        for (int h = lane; h < H; h += kWave) mine[h] = 0.f;
}

// dw[h] = sum over the partial rows, in a fixed order: a block owns 32 columns; its 32 row groups each add
// every 32nd partial row (16 independent loads in flight), then the 32 sums are added in order.  (With 8 row
// groups of 256 threads a thread walked 64 partial rows in 8 dependent batches: 4.4 us for 512 rows of 2048.)
__global__ __launch_bounds__(1024) void rmsnorm_dw_reduce_kernel(const float* __restrict__ partial, int n_partial,
                                                                 float* __restrict__ dw, int H) {
    __shared__ float part[32][33];
    const int col = threadIdx.x & 31, grp = threadIdx.x >> 5;
    const int h = blockIdx.x * 32 + col;
    float s = 0.f;
    if (h < H) {
#pragma unroll 16
        for (int b = grp; b < n_partial; b += 32) s += partial[(int64_t)b * H + h];
    }
    part[grp][col] = s;
    __syncthreads();
    if (grp == 0 && h < H) {
        float t = part[0][col];
#pragma unroll
        for (int g = 1; g < 32; ++g) t += part[g][col];
        dw[h] = t;
    }
}

static void launch_dw_reduce(const float* partial, int n_partial, float* dw, int H, hipStream_t s) {
    hipLaunchKernelGGL(rmsnorm_dw_reduce_kernel, dim3((H + 31) / 32), dim3(1024), 0, s, partial, n_partial, dw, H);
}

constexpr int kBwdBlocksVec = 512;      // vector kernel: two blocks per CU, one partial row per block
constexpr int kBwdBlocksGeneric = 64;   // generic kernel: one partial row per wave (256 rows)

static bool rmsnorm_bwd_vec_ok(const void* x, const void* dy, const void* dx, int H, int V) {
    return (H % V == 0) && aligned16(x) && aligned16(dy) && aligned16(dx) && (H / V) <= 16 * kWave;
}

template <typename T, typename WT, bool HAS_W>
static int launch_rmsnorm_bwd(const void* x, const void* w, const void* dy, void* dx, float* dw, float* partial,
                              int64_t rows, int H, float eps, hipStream_t s) {
    constexpr int V = Elem<T>::kVec;
    const T* xp = static_cast<const T*>(x);
    const WT* wp = static_cast<const WT*>(w);
    const T* gp = static_cast<const T*>(dy);
    T* dxp = static_cast<T*>(dx);
    float* part = dw ? partial : nullptr;
    int n_partial;
    if (!rmsnorm_bwd_vec_ok(x, dy, dx, H, V)) {
        const int64_t want = (rows + 3) / 4;
        const int blocks = (int)(want < kBwdBlocksGeneric ? want : kBwdBlocksGeneric);
        hipLaunchKernelGGL((rmsnorm_bwd_generic_kernel<T, WT, HAS_W>), dim3(blocks), dim3(256), 0, s, xp, wp, gp, dxp,
                           part, rows, H, eps);
        n_partial = blocks * 4;
    } else {
        const size_t lds = part ? (size_t)H * sizeof(float) : 0;
        const int nvec = H / V;
        if (nvec >= kTeamLanes && nvec <= 4 * kTeamLanes) {
            const int64_t want = (rows + 1) / 2;
            const int blocks = (int)(want < kBwdBlocksVec ? want : kBwdBlocksVec);
            const int per_team_lane = (nvec + kTeamLanes - 1) / kTeamLanes;
#define ATS_RMSB_TEAM(NV)                                                                                        \
    hipLaunchKernelGGL((rmsnorm_bwd_team_kernel<T, WT, NV, HAS_W>), dim3(blocks), dim3(512), lds, s, xp, wp, gp, dxp, \
                       part, rows, H, eps)
            if (per_team_lane <= 1) ATS_RMSB_TEAM(1);
            else if (per_team_lane <= 2) ATS_RMSB_TEAM(2);
            else ATS_RMSB_TEAM(4);
#undef ATS_RMSB_TEAM
            if (dw)
                launch_dw_reduce(partial, blocks, dw, H, s);
            return ATS_OK;
        }
        const int64_t want = (rows + 3) / 4;
        const int blocks = (int)(want < kBwdBlocksVec ? want : kBwdBlocksVec);
        const int per_lane = (H / V + kWave - 1) / kWave;
#define ATS_RMSB_CASE(NV)                                                                                  \
    hipLaunchKernelGGL((rmsnorm_bwd_rows_kernel<T, WT, NV, HAS_W, (NV * V <= 32)>), dim3(blocks), dim3(256), lds, \
                       s, xp, wp, gp, dxp, part, rows, H, eps)
        if (per_lane <= 1) ATS_RMSB_CASE(1);
        else if (per_lane <= 2) ATS_RMSB_CASE(2);
        else if (per_lane <= 4) ATS_RMSB_CASE(4);
        else if (per_lane <= 8) ATS_RMSB_CASE(8);
        else ATS_RMSB_CASE(16);
#undef ATS_RMSB_CASE
        n_partial = blocks;
    }
    if (dw)
        launch_dw_reduce(partial, n_partial, dw, H, s);
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

extern "C" size_t ats_rmsnorm_bwd_workspace(int64_t rows, int hidden) {
    (void)rows;
    const size_t n = ats::kBwdBlocksVec > ats::kBwdBlocksGeneric * 4 ? ats::kBwdBlocksVec : ats::kBwdBlocksGeneric * 4;
    return n * (size_t)(hidden > 0 ? hidden : 0) * sizeof(float);
}

extern "C" int ats_rmsnorm_bwd(const void* x, const void* w, const void* dy, void* dx, float* dw, int64_t rows,
                               int hidden, float eps, int x_dtype, int w_dtype, void* workspace,
                               size_t workspace_bytes, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(rows >= 0 && hidden > 0, ATS_ERR_INVALID_ARG, "ats_rmsnorm_bwd: rows=%lld hidden=%d",
                (long long)rows, hidden);
    ATS_REQUIRE((x_dtype == ATS_F32 || x_dtype == ATS_BF16) && (w_dtype == ATS_F32 || w_dtype == ATS_BF16),
                ATS_ERR_UNSUPPORTED, "ats_rmsnorm_bwd: dtype tags %d/%d", x_dtype, w_dtype);
    hipStream_t s = as_stream(stream);
    if (rows == 0) {
        if (dw) launch_dw_reduce(nullptr, 0, dw, hidden, s);
        ATS_CHECK_LAUNCH("ats_rmsnorm_bwd");
        return ATS_OK;
    }
    ATS_REQUIRE(x && dy && dx, ATS_ERR_INVALID_ARG, "ats_rmsnorm_bwd: null pointer");
    ATS_REQUIRE(!dw || (workspace && workspace_bytes >= ats_rmsnorm_bwd_workspace(rows, hidden)), ATS_ERR_WORKSPACE,
                "ats_rmsnorm_bwd: workspace of %zu bytes, need %zu", workspace_bytes,
                ats_rmsnorm_bwd_workspace(rows, hidden));
    ATS_REQUIRE(hidden <= 32768 || !dw, ATS_ERR_UNSUPPORTED, "ats_rmsnorm_bwd: hidden=%d", hidden);
    ATS_REQUIRE(!dw || aligned16(workspace), ATS_ERR_INVALID_ARG, "ats_rmsnorm_bwd: the workspace must be 16-byte aligned");
    float* part = static_cast<float*>(workspace);
    int rc;
    if (x_dtype == ATS_F32) {
        if (!w) rc = launch_rmsnorm_bwd<float, float, false>(x, w, dy, dx, dw, part, rows, hidden, eps, s);
        else if (w_dtype == ATS_F32) rc = launch_rmsnorm_bwd<float, float, true>(x, w, dy, dx, dw, part, rows, hidden, eps, s);
        else rc = launch_rmsnorm_bwd<float, bf16_t, true>(x, w, dy, dx, dw, part, rows, hidden, eps, s);
    } else {
        if (!w) rc = launch_rmsnorm_bwd<bf16_t, float, false>(x, w, dy, dx, dw, part, rows, hidden, eps, s);
        else if (w_dtype == ATS_F32) rc = launch_rmsnorm_bwd<bf16_t, float, true>(x, w, dy, dx, dw, part, rows, hidden, eps, s);
        else rc = launch_rmsnorm_bwd<bf16_t, bf16_t, true>(x, w, dy, dx, dw, part, rows, hidden, eps, s);
    }
    if (rc != ATS_OK) return rc;
    ATS_CHECK_LAUNCH("ats_rmsnorm_bwd");
    return ATS_OK;
}
