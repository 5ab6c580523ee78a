// Backward-pass kernels of the sparse layer that are not GEMMs (gfx950, all HBM-bound):
//   silu(a) * b and its gradient on row-strided operands (expert activation, dense SwiGLU),
//   gradient of the weighted combine, gradient of the routing rule (+ load-balancing loss),
//   the router's input gradient and weight gradient.
// float32 math throughout; reductions run in a fixed order (no atomics), so results do not
// depend on timing.
#include "ats_common.hpp"

namespace ats {

// ---------------------------------------------------------------- silu(a) * b
// out[r, c] = silu(a[r, c]) * b[r, c]; operands addressed as base + r * ld + c.
template <typename T>
__global__ __launch_bounds__(256) void silu_mul_fwd_kernel(const T* __restrict__ a, int64_t lda,
                                                           const T* __restrict__ b, int64_t ldb, T* __restrict__ out,
                                                           int64_t ldo, int64_t rows, const int32_t* __restrict__ rows_dev, int cols,
                                                           bool vec) {
    constexpr int V = Elem<T>::kVec;
    if (rows_dev && rows_dev[0] < rows) rows = rows_dev[0] > 0 ? rows_dev[0] : 0;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (vec) {   // a block walks whole rows: no 64-bit divisions in the address math
        const int cv = cols / V;
        for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
            for (int cvi = threadIdx.x; cvi < cv; cvi += blockDim.x) {
                const int c = cvi * V;
                float av[V], bv[V];
                Elem<T>::unpack(*reinterpret_cast<const uint4*>(a + r * lda + c), av);
                Elem<T>::unpack(*reinterpret_cast<const uint4*>(b + r * ldb + c), bv);
#pragma unroll
                for (int j = 0; j < V; ++j) av[j] = av[j] * sigmoid_f(av[j]) * bv[j];
                *reinterpret_cast<uint4*>(out + r * ldo + c) = Elem<T>::pack(av);
            }
        }
    } else {
        const int64_t n = rows * cols;
        for (int64_t i = tid; i < n; i += stride) {
            const int64_t r = i / cols;
            const int c = (int)(i - r * cols);
            const float av = Elem<T>::load(a + r * lda + c);
            Elem<T>::store(out + r * ldo + c, av * sigmoid_f(av) * Elem<T>::load(b + r * ldb + c));
        }
    }
}

// da = dout * b * (s + a*s*(1-s)), db = dout * a * s, s = sigmoid(a)
// (SwiGLUFunction.backward, cuda_opt_wrapper.py:237-254, with a = the activated operand).
template <typename T>
__global__ __launch_bounds__(256) void silu_mul_bwd_kernel(const T* __restrict__ a, int64_t lda,
                                                           const T* __restrict__ b, int64_t ldb,
                                                           const T* __restrict__ dout, int64_t ldd,
                                                           T* __restrict__ da, int64_t ldda, T* __restrict__ db,
                                                           int64_t lddb, int64_t rows, const int32_t* __restrict__ rows_dev, int cols,
                                                           bool vec) {
    constexpr int V = Elem<T>::kVec;
    if (rows_dev && rows_dev[0] < rows) rows = rows_dev[0] > 0 ? rows_dev[0] : 0;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (vec) {
        const int cv = cols / V;
        for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
            for (int cvi = threadIdx.x; cvi < cv; cvi += blockDim.x) {
                const int c = cvi * V;
                float av[V], bv[V], gv[V], oa[V], ob[V];
                Elem<T>::unpack(*reinterpret_cast<const uint4*>(a + r * lda + c), av);
                Elem<T>::unpack(*reinterpret_cast<const uint4*>(b + r * ldb + c), bv);
                Elem<T>::unpack(*reinterpret_cast<const uint4*>(dout + r * ldd + c), gv);
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    const float s = sigmoid_f(av[j]);
                    oa[j] = gv[j] * bv[j] * (s + av[j] * s * (1.0f - s));
                    ob[j] = gv[j] * (av[j] * s);
                }
                *reinterpret_cast<uint4*>(da + r * ldda + c) = Elem<T>::pack(oa);
                *reinterpret_cast<uint4*>(db + r * lddb + c) = Elem<T>::pack(ob);
            }
        }
    } else {
        const int64_t n = rows * cols;
        for (int64_t i = tid; i < n; i += stride) {
            const int64_t r = i / cols;
            const int c = (int)(i - r * cols);
            const float av = Elem<T>::load(a + r * lda + c);
            const float bv = Elem<T>::load(b + r * ldb + c);
            const float gv = Elem<T>::load(dout + r * ldd + c);
            const float s = sigmoid_f(av);
            Elem<T>::store(da + r * ldda + c, gv * bv * (s + av * s * (1.0f - s)));
            Elem<T>::store(db + r * lddb + c, gv * (av * s));
        }
    }
}

// ---------------------------------------------------------------- combine backward
// Forward: out[t,:] = sum_j w[t,j] * y[row_of[t*k+j], :].  Row-major restatement of its gradient:
// for expert row r with assignment m = token_map[r] (t = m / k):
//   dy[r,:] = w[m] * dout[t,:],   dw[m] = dout[t,:] . y[r,:];   rows with m < 0 get zeros.
// One wave per row; dw entries of dropped assignments are cleared by a fill kernel beforehand.
template <typename TY, typename TO>
__global__ __launch_bounds__(256) void combine_bwd_kernel(const TO* __restrict__ dout, const TY* __restrict__ y,
                                                          const int32_t* __restrict__ token_map,
                                                          const float* __restrict__ w, TY* __restrict__ dy,
                                                          float* __restrict__ dw, int64_t n_rows, int k, int H,
                                                          bool vec) {
    const int lane = lane_id();
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
    for (int64_t r = wave; r < n_rows; r += nwaves) {
        const int m = token_map[r];
        TY* dyr = dy + r * H;
        if (m < 0) {
            for (int h = lane; h < H; h += kWave) Elem<TY>::store(dyr + h, 0.f);
            continue;
        }
        const int64_t t = m / k;
        const float wv = w[m];
        const TO* g = dout + t * H;
        const TY* yr = y + r * H;
        float dot = 0.f;
        if (vec) {
            constexpr int V = 8;
            for (int h0 = lane * V; h0 < H; h0 += kWave * V) {
                float gv[V], yv[V], o[V];
                if constexpr (sizeof(TO) == 2) {
                    Elem<TO>::unpack(*reinterpret_cast<const uint4*>(g + h0), gv);
                } else {
                    Elem<TO>::unpack(*reinterpret_cast<const uint4*>(g + h0), gv);
                    Elem<TO>::unpack(*reinterpret_cast<const uint4*>(g + h0 + 4), gv + 4);
                }
                if constexpr (sizeof(TY) == 2) {
                    Elem<TY>::unpack(*reinterpret_cast<const uint4*>(yr + h0), yv);
                } else {
                    Elem<TY>::unpack(*reinterpret_cast<const uint4*>(yr + h0), yv);
                    Elem<TY>::unpack(*reinterpret_cast<const uint4*>(yr + h0 + 4), yv + 4);
                }
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    dot += gv[j] * yv[j];
                    o[j] = wv * gv[j];
                }
                if constexpr (sizeof(TY) == 2) {
                    *reinterpret_cast<uint4*>(dyr + h0) = Elem<TY>::pack(o);
                } else {
                    *reinterpret_cast<uint4*>(dyr + h0) = Elem<TY>::pack(o);
                    *reinterpret_cast<uint4*>(dyr + h0 + 4) = Elem<TY>::pack(o + 4);
                }
            }
        } else {
            for (int h = lane; h < H; h += kWave) {
                const float gv = Elem<TO>::load(g + h);
                dot += gv * Elem<TY>::load(yr + h);
                Elem<TY>::store(dyr + h, wv * gv);
            }
        }
        dot = wave_sum(dot);
        if (lane == 0) dw[m] = dot;
    }
}

__global__ __launch_bounds__(256) void fill_f32_kernel(float* __restrict__ p, int64_t n, float v) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        p[i] = v;
}

// ---------------------------------------------------------------- routing backward
// mode 0 (softmax -> top-k -> renormalise, model.py:1200-1217):
//   p = softmax(z / tau), S = sum_j p[i_j], w_j = p[i_j] / (S + 1e-9)
//   dp[i_j] = (dw_j - sum_m dw_m w_m) / (S + 1e-9);  dz = p * (dp - sum_e dp_e p_e) / tau
// mode 1 (top-k -> softmax, moe_cuda_wrapper.py:229-233):
//   dz[i_j] = w_j * (dw_j - sum_m dw_m w_m) / tau
// Load-balancing loss (model.py:1244-1263) with q = softmax(z_aux), usage constant:
//   dz_aux[e] += aux_scale * q_e * (usage_e - sum_e' usage_e' q_e'),  aux_scale = dL/daux * E * weight / T
// (aux_scale = host factor times an optional device scalar, so dL/daux needs no host read-back)
// One thread per token (E is small).
__global__ __launch_bounds__(256) void route_bwd_kernel(const float* __restrict__ z_route,
                                                        const float* __restrict__ z_aux,
                                                        const int32_t* __restrict__ idx, const float* __restrict__ w,
                                                        const float* __restrict__ dw, const float* __restrict__ usage,
                                                        float aux_scale, const float* __restrict__ aux_scale_dev,
                                                        float inv_tau, int mode,
                                                        float* __restrict__ dz, int64_t T, int E, int k) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= T) return;
    const float* zr = z_route + t * E;
    const int32_t* it = idx + t * k;
    const float* wt = w + t * k;
    const float* dwt = dw + t * k;
    float* out = dz + t * E;
    float dot = 0.f;
    for (int j = 0; j < k; ++j) dot += dwt[j] * wt[j];
    if (mode == 0) {
        float mx = -INFINITY;
        for (int e = 0; e < E; ++e) mx = fmaxf(mx, zr[e] * inv_tau);
        float Z = 0.f;
        for (int e = 0; e < E; ++e) Z += expf(zr[e] * inv_tau - mx);
        const float invZ = 1.0f / Z;
        float S = 0.f;
        for (int j = 0; j < k; ++j) S += expf(zr[it[j]] * inv_tau - mx) * invZ;
        const float invS = 1.0f / (S + 1e-9f);
        float inner = 0.f;
        for (int j = 0; j < k; ++j) inner += (dwt[j] - dot) * invS * (expf(zr[it[j]] * inv_tau - mx) * invZ);
        for (int e = 0; e < E; ++e) out[e] = -(expf(zr[e] * inv_tau - mx) * invZ) * inner * inv_tau;
        for (int j = 0; j < k; ++j) {
            const int e = it[j];
            const float p = expf(zr[e] * inv_tau - mx) * invZ;
            out[e] += p * ((dwt[j] - dot) * invS) * inv_tau;
        }
    } else {
        for (int e = 0; e < E; ++e) out[e] = 0.f;
        for (int j = 0; j < k; ++j) out[it[j]] += wt[j] * (dwt[j] - dot) * inv_tau;
    }
    if (aux_scale_dev) aux_scale *= aux_scale_dev[0];
    if (usage && aux_scale != 0.f) {
        const float* za = z_aux + t * E;
        float mx = -INFINITY;
        for (int e = 0; e < E; ++e) mx = fmaxf(mx, za[e]);
        float Z = 0.f;
        for (int e = 0; e < E; ++e) Z += expf(za[e] - mx);
        const float invZ = 1.0f / Z;
        float uq = 0.f;
        for (int e = 0; e < E; ++e) uq += usage[e] * (expf(za[e] - mx) * invZ);
        for (int e = 0; e < E; ++e) {
            const float q = expf(za[e] - mx) * invZ;
            out[e] += aux_scale * q * (usage[e] - uq);
        }
    }
}

// ---------------------------------------------------------------- router input gradient
// out[t, h] = base[t, h] + sum_e dz[t, e] * Wg[e, h]   (base may be NULL or alias out).
// One wave per token; the E rows of Wg stay in L2.
template <typename T>
__global__ __launch_bounds__(256) void router_dx_kernel(const float* __restrict__ dz, const T* __restrict__ wg,
                                                        const T* base, T* out, int64_t Tn, int E, int H, bool vec) {
    constexpr int V = Elem<T>::kVec;
    const int lane = lane_id();
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
    for (int64_t t = wave; t < Tn; t += nwaves) {
        const float* dzt = dz + t * E;
        if (vec) {
            for (int h0 = lane * V; h0 < H; h0 += kWave * V) {
                float acc[V];
#pragma unroll
                for (int j = 0; j < V; ++j) acc[j] = 0.f;
                if (base) Elem<T>::unpack(*reinterpret_cast<const uint4*>(base + t * H + h0), acc);
                for (int e = 0; e < E; ++e) {
                    const float d = dzt[e];
                    float wv[V];
                    Elem<T>::unpack(*reinterpret_cast<const uint4*>(wg + (int64_t)e * H + h0), wv);
#pragma unroll
                    for (int j = 0; j < V; ++j) acc[j] += d * wv[j];
                }
                *reinterpret_cast<uint4*>(out + t * H + h0) = Elem<T>::pack(acc);
            }
        } else {
            for (int h = lane; h < H; h += kWave) {
                float acc = base ? Elem<T>::load(base + t * H + h) : 0.f;
                for (int e = 0; e < E; ++e) acc += dzt[e] * Elem<T>::load(wg + (int64_t)e * H + h);
                Elem<T>::store(out + t * H + h, acc);
            }
        }
    }
}

// Up to 8 experts: a thread owns V consecutive columns for a chunk of tokens and keeps its V x E gate weights in
// registers, so the gate rows are read once per chunk instead of once per token (they made up 8/9 of the loads);
// the next four tokens' base pieces travel while the current four are used.  A token's E gradients are wave
// uniform and come in as one scalar load: nothing in the loop over the experts is conditional (absent experts
// have zero weights and a zero gradient), since a test per expert made every value a load of its own with a
// wait behind it.  Per element the same sum in the same order as above.
constexpr int kDxExperts = 8;
constexpr int kDxChunk = 64;
template <typename T, bool FULL>   // FULL: exactly 8 experts (a token's gradients are one 32-byte scalar load)
__global__ __launch_bounds__(256) void router_dx_cols_kernel(const float* __restrict__ dz, const T* __restrict__ wg,
                                                             const T* base, T* out, int64_t Tn, int E, int H) {
    constexpr int V = Elem<T>::kVec;
    constexpr int U = 4;
    const int h = (blockIdx.x * blockDim.x + threadIdx.x) * V;
    if (h >= H) return;
    const int64_t t0 = (int64_t)blockIdx.y * kDxChunk;
    const int64_t t1 = t0 + kDxChunk < Tn ? t0 + kDxChunk : Tn;
    float wv[kDxExperts][V];
#pragma unroll
    for (int e = 0; e < kDxExperts; ++e) {
#pragma unroll
        for (int j = 0; j < V; ++j) wv[e][j] = 0.f;
        if (e < E) Elem<T>::unpack(*reinterpret_cast<const uint4*>(wg + (int64_t)e * H + h), wv[e]);
    }
    uint4 nxt[U];
#define ATS_DX_FETCH(tb_)                                                                              \
    if (base) {                                                                                        \
        _Pragma("unroll") for (int u = 0; u < U; ++u)                                                  \
            if ((tb_) + u < t1) nxt[u] = *reinterpret_cast<const uint4*>(base + ((tb_) + u) * H + h);  \
    }
#define ATS_DX_TOKEN(raw_, t_)                                                                         \
    {                                                                                                  \
        float acc[V];                                                                                  \
        _Pragma("unroll") for (int j = 0; j < V; ++j) acc[j] = 0.f;                                    \
        if (base) Elem<T>::unpack(raw_, acc);                                                          \
        const float* dzt = dz + (t_) * E;                                                              \
        float d[kDxExperts];                                                                           \
        _Pragma("unroll") for (int e = 0; e < kDxExperts; ++e) d[e] = dzt[FULL || e < E ? e : E - 1];  \
        _Pragma("unroll") for (int e = 0; e < kDxExperts; ++e) d[e] = FULL || e < E ? d[e] : 0.f;      \
        _Pragma("unroll") for (int e = 0; e < kDxExperts; ++e) {                                       \
            _Pragma("unroll") for (int j = 0; j < V; ++j) acc[j] += d[e] * wv[e][j];                   \
        }                                                                                              \
        *reinterpret_cast<uint4*>(out + (t_) * H + h) = Elem<T>::pack(acc);                            \
    }
    ATS_DX_FETCH(t0);
    int64_t tb = t0;
    for (; tb + U <= t1; tb += U) {
        uint4 raw[U];
#pragma unroll
        for (int u = 0; u < U; ++u) raw[u] = nxt[u];
        ATS_DX_FETCH(tb + U);      // the next pieces travel while these are used
#pragma unroll
        for (int u = 0; u < U; ++u) ATS_DX_TOKEN(raw[u], tb + u);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
        if (tb + u < t1) ATS_DX_TOKEN(nxt[u], tb + u);
#undef ATS_DX_FETCH
#undef ATS_DX_TOKEN
}

// ---------------------------------------------------------------- router weight gradient
// dWg[e, h] = sum_t dz[t, e] * x[t, h].  Tokens are split into chunks; a block owns one chunk
// and one group of columns, accumulates 8 experts at a time in registers and writes
// partial[chunk][e][h]; a second kernel adds the chunks in order.
constexpr int kDwExperts = 8;

template <typename T>
__global__ __launch_bounds__(256) void router_dw_partial_kernel(const float* __restrict__ dz, const T* __restrict__ x,
                                                                float* __restrict__ partial, int64_t Tn, int E, int H,
                                                                int chunk_tokens) {
    const int h = blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t t0 = (int64_t)blockIdx.y * chunk_tokens;
    const int64_t t1 = t0 + chunk_tokens < Tn ? t0 + chunk_tokens : Tn;
    if (h >= H) return;
    for (int e0 = 0; e0 < E; e0 += kDwExperts) {
        float acc[kDwExperts];
#pragma unroll
        for (int i = 0; i < kDwExperts; ++i) acc[i] = 0.f;
        for (int64_t t = t0; t < t1; ++t) {
            const float xv = Elem<T>::load(x + t * H + h);
            const float* dzt = dz + t * E + e0;
#pragma unroll
            for (int i = 0; i < kDwExperts; ++i)
                if (e0 + i < E) acc[i] += dzt[i] * xv;
        }
#pragma unroll
        for (int i = 0; i < kDwExperts; ++i)
            if (e0 + i < E) partial[((int64_t)blockIdx.y * E + e0 + i) * H + h] = acc[i];
    }
}

// The same sums with 16-byte loads: a thread owns V consecutive columns (H % V == 0, x 16-byte aligned) and asks
// for the next 8 tokens' pieces while it uses the current 8 (16 at a time measured no faster).  A token's 8
// gradients are wave uniform and come in as one scalar load: nothing in the loop over the experts is conditional
// (the sums of absent experts are formed and dropped), since a test per expert made every value a load of its
// own with a wait behind it.  Every column's sum runs over the tokens in the same order as in the kernel above
// (same bits).
template <typename T, bool FULL>   // FULL: E is a multiple of 8 (a token's 8 gradients are one 32-byte scalar load)
__global__ __launch_bounds__(256) void router_dw_partial_vec_kernel(const float* __restrict__ dz,
                                                                    const T* __restrict__ x,
                                                                    float* __restrict__ partial, int64_t Tn, int E,
                                                                    int H, int chunk_tokens) {
    constexpr int V = Elem<T>::kVec;
    constexpr int U = 8;
    const int h = (blockIdx.x * blockDim.x + threadIdx.x) * V;
    const int64_t t0 = (int64_t)blockIdx.y * chunk_tokens;
    const int64_t t1 = t0 + chunk_tokens < Tn ? t0 + chunk_tokens : Tn;
    if (h >= H) return;
    for (int e0 = 0; e0 < E; e0 += kDwExperts) {
        const int nv = E - e0 < kDwExperts ? E - e0 : kDwExperts;   // experts of this group that exist
        float acc[kDwExperts][V];
#pragma unroll
        for (int i = 0; i < kDwExperts; ++i)
#pragma unroll
            for (int j = 0; j < V; ++j) acc[i][j] = 0.f;
#define ATS_DW_TOKEN(raw_, t_)                                                                         \
    {                                                                                                  \
        float xv[V];                                                                                   \
        Elem<T>::unpack(raw_, xv);                                                                     \
        const float* dzt = dz + (t_) * E + e0;                                                         \
        float d[kDwExperts];                                                                           \
        _Pragma("unroll") for (int i = 0; i < kDwExperts; ++i) d[i] = dzt[FULL || i < nv ? i : nv - 1]; \
        _Pragma("unroll") for (int i = 0; i < kDwExperts; ++i) {                                       \
            _Pragma("unroll") for (int j = 0; j < V; ++j) acc[i][j] += d[i] * xv[j];                   \
        }                                                                                              \
    }
        uint4 nxt[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (t0 + u < t1) nxt[u] = *reinterpret_cast<const uint4*>(x + (t0 + u) * H + h);
        int64_t tb = t0;
        for (; tb + U <= t1; tb += U) {
            uint4 raw[U];
#pragma unroll
            for (int u = 0; u < U; ++u) raw[u] = nxt[u];
#pragma unroll
            for (int u = 0; u < U; ++u)      // the next pieces travel while these are used
                if (tb + U + u < t1) nxt[u] = *reinterpret_cast<const uint4*>(x + (tb + U + u) * H + h);
#pragma unroll
            for (int u = 0; u < U; ++u) ATS_DW_TOKEN(raw[u], tb + u);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (tb + u < t1) ATS_DW_TOKEN(nxt[u], tb + u);
#undef ATS_DW_TOKEN
#pragma unroll
        for (int i = 0; i < kDwExperts; ++i)
            if (i < nv) {
                float* dst = partial + ((int64_t)blockIdx.y * E + e0 + i) * H + h;
#pragma unroll
                for (int j = 0; j < V; ++j) dst[j] = acc[i][j];
            }
    }
}

__global__ __launch_bounds__(256) void router_dw_reduce_kernel(const float* __restrict__ partial, int n_chunks,
                                                               float* __restrict__ dwg, int64_t EH) {
    // a block owns 32 entries; 8 groups each add every 8th chunk, then the 8 sums are added in order
    __shared__ float part[8][32];
    const int col = threadIdx.x & 31, grp = threadIdx.x >> 5;
    const int64_t i = (int64_t)blockIdx.x * 32 + col;
    float s = 0.f;
    if (i < EH) {
#pragma unroll 8
        for (int c = grp; c < n_chunks; c += 8) s += partial[(int64_t)c * EH + i];
    }
    part[grp][col] = s;
    __syncthreads();
    if (grp == 0 && i < EH) {
        float t = part[0][col];
#pragma unroll
        for (int g = 1; g < 8; ++g) t += part[g][col];
        dwg[i] = t;
    }
}

static int dw_chunks(int64_t T, int* chunk_tokens) {
    int64_t n = (T + 127) / 128;
    if (n > 256) n = 256;
    if (n < 1) n = 1;
    *chunk_tokens = (int)((T + n - 1) / n);
    if (*chunk_tokens < 1) *chunk_tokens = 1;
    return (int)((T + *chunk_tokens - 1) / *chunk_tokens);
}

static int64_t ew_blocks(int64_t items) {
    int64_t b = (items + 255) / 256;
    if (b > 16384) b = 16384;
    return b < 1 ? 1 : b;
}

}  // namespace ats

extern "C" int ats_silu_mul_fwd(const void* a, int64_t lda, const void* b, int64_t ldb, void* out, int64_t ldo,
                                int64_t rows, const int32_t* rows_dev, int cols, int dtype, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(rows >= 0 && cols > 0 && lda >= cols && ldb >= cols && ldo >= cols, ATS_ERR_INVALID_ARG,
                "ats_silu_mul_fwd: rows=%lld cols=%d strides %lld/%lld/%lld", (long long)rows, cols, (long long)lda,
                (long long)ldb, (long long)ldo);
    ATS_REQUIRE(dtype == ATS_F32 || dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "ats_silu_mul_fwd: dtype tag %d", dtype);
    if (rows == 0) return ATS_OK;
    ATS_REQUIRE(a && b && out, ATS_ERR_INVALID_ARG, "ats_silu_mul_fwd: null pointer");
    const int V = dtype == ATS_F32 ? 4 : 8;
    const bool vec = cols % V == 0 && lda % V == 0 && ldb % V == 0 && ldo % V == 0 && aligned16(a) && aligned16(b) &&
                     aligned16(out);
    const int64_t blocks = vec ? (rows < 65536 ? rows : 65536) : ew_blocks(rows * cols);
    if (dtype == ATS_F32)
        hipLaunchKernelGGL((silu_mul_fwd_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const float*>(a), lda, static_cast<const float*>(b), ldb,
                           static_cast<float*>(out), ldo, rows, rows_dev, cols, vec);
    else
        hipLaunchKernelGGL((silu_mul_fwd_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const bf16_t*>(a), lda, static_cast<const bf16_t*>(b), ldb,
                           static_cast<bf16_t*>(out), ldo, rows, rows_dev, cols, vec);
    ATS_CHECK_LAUNCH("ats_silu_mul_fwd");
    return ATS_OK;
}

extern "C" int ats_silu_mul_bwd(const void* a, int64_t lda, const void* b, int64_t ldb, const void* dout, int64_t ldd,
                                void* da, int64_t ldda, void* db, int64_t lddb, int64_t rows, const int32_t* rows_dev,
                                int cols, int dtype, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(rows >= 0 && cols > 0 && lda >= cols && ldb >= cols && ldd >= cols && ldda >= cols && lddb >= cols,
                ATS_ERR_INVALID_ARG, "ats_silu_mul_bwd: rows=%lld cols=%d", (long long)rows, cols);
    ATS_REQUIRE(dtype == ATS_F32 || dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "ats_silu_mul_bwd: dtype tag %d", dtype);
    if (rows == 0) return ATS_OK;
    ATS_REQUIRE(a && b && dout && da && db, ATS_ERR_INVALID_ARG, "ats_silu_mul_bwd: null pointer");
    const int V = dtype == ATS_F32 ? 4 : 8;
    const bool vec = cols % V == 0 && lda % V == 0 && ldb % V == 0 && ldd % V == 0 && ldda % V == 0 && lddb % V == 0 &&
                     aligned16(a) && aligned16(b) && aligned16(dout) && aligned16(da) && aligned16(db);
    const int64_t blocks = vec ? (rows < 65536 ? rows : 65536) : ew_blocks(rows * cols);
    if (dtype == ATS_F32)
        hipLaunchKernelGGL((silu_mul_bwd_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const float*>(a), lda, static_cast<const float*>(b), ldb,
                           static_cast<const float*>(dout), ldd, static_cast<float*>(da), ldda,
                           static_cast<float*>(db), lddb, rows, rows_dev, cols, vec);
    else
        hipLaunchKernelGGL((silu_mul_bwd_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const bf16_t*>(a), lda, static_cast<const bf16_t*>(b), ldb,
                           static_cast<const bf16_t*>(dout), ldd, static_cast<bf16_t*>(da), ldda,
                           static_cast<bf16_t*>(db), lddb, rows, rows_dev, cols, vec);
    ATS_CHECK_LAUNCH("ats_silu_mul_bwd");
    return ATS_OK;
}

extern "C" int ats_combine_bwd(const void* dout, const void* y, const int32_t* token_map, const float* w, void* dy,
                               float* dw, int64_t n_rows, int64_t T, int k, int H, int y_dtype, int out_dtype,
                               ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(n_rows >= 0 && T >= 0 && k > 0 && H > 0, ATS_ERR_INVALID_ARG, "ats_combine_bwd: rows=%lld T=%lld k=%d H=%d",
                (long long)n_rows, (long long)T, k, H);
    ATS_REQUIRE((y_dtype == ATS_F32 || y_dtype == ATS_BF16) && (out_dtype == ATS_F32 || out_dtype == ATS_BF16),
                ATS_ERR_UNSUPPORTED, "ats_combine_bwd: dtype tags %d/%d", y_dtype, out_dtype);
    hipStream_t s = as_stream(stream);
    if (T > 0) {
        ATS_REQUIRE(dw, ATS_ERR_INVALID_ARG, "ats_combine_bwd: null pointer");
        hipLaunchKernelGGL(fill_f32_kernel, dim3((unsigned)ew_blocks(T * k)), dim3(256), 0, s, dw, T * k, 0.f);
    }
    if (n_rows > 0) {
        ATS_REQUIRE(dout && y && token_map && w && dy && dw, ATS_ERR_INVALID_ARG, "ats_combine_bwd: null pointer");
        const bool vec = H % 8 == 0 && aligned16(dout) && aligned16(y) && aligned16(dy);
        int64_t blocks = (n_rows + 3) / 4;
        if (blocks > 16384) blocks = 16384;
#define ATS_CB(TY, TO)                                                                                          \
    hipLaunchKernelGGL((combine_bwd_kernel<TY, TO>), dim3((unsigned)blocks), dim3(256), 0, s,                  \
                       static_cast<const TO*>(dout), static_cast<const TY*>(y), token_map, w, static_cast<TY*>(dy), \
                       dw, n_rows, k, H, vec)
        if (y_dtype == ATS_F32 && out_dtype == ATS_F32) ATS_CB(float, float);
        else if (y_dtype == ATS_BF16 && out_dtype == ATS_BF16) ATS_CB(bf16_t, bf16_t);
        else if (y_dtype == ATS_F32) ATS_CB(float, bf16_t);
        else ATS_CB(bf16_t, float);
#undef ATS_CB
    }
    ATS_CHECK_LAUNCH("ats_combine_bwd");
    return ATS_OK;
}

extern "C" int ats_route_bwd(const float* logits_route, const float* logits_aux, const int32_t* idx, const float* w,
                             const float* dw, const float* usage, float aux_scale, const float* aux_scale_dev,
                             float temperature, int mode, float* dlogits, int64_t T, int E, int k,
                             ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(T >= 0 && E > 0 && k > 0 && k <= E && temperature > 0.f && (mode == 0 || mode == 1),
                ATS_ERR_INVALID_ARG, "ats_route_bwd: T=%lld E=%d k=%d temperature=%g mode=%d", (long long)T, E, k,
                temperature, mode);
    if (T == 0) return ATS_OK;
    ATS_REQUIRE(logits_route && idx && w && dw && dlogits && (!usage || logits_aux), ATS_ERR_INVALID_ARG,
                "ats_route_bwd: null pointer");
    hipLaunchKernelGGL(route_bwd_kernel, dim3((unsigned)((T + 255) / 256)), dim3(256), 0, as_stream(stream),
                       logits_route, logits_aux, idx, w, dw, usage, aux_scale, aux_scale_dev, 1.0f / temperature, mode,
                       dlogits, T, E, k);
    ATS_CHECK_LAUNCH("ats_route_bwd");
    return ATS_OK;
}

extern "C" int ats_router_bwd_dx(const float* dlogits, const void* wg, const void* base, void* out, int64_t T, int E,
                                 int H, int dtype, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(T >= 0 && E > 0 && H > 0, ATS_ERR_INVALID_ARG, "ats_router_bwd_dx: T=%lld E=%d H=%d", (long long)T, E, H);
    ATS_REQUIRE(dtype == ATS_F32 || dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "ats_router_bwd_dx: dtype tag %d", dtype);
    if (T == 0) return ATS_OK;
    ATS_REQUIRE(dlogits && wg && out, ATS_ERR_INVALID_ARG, "ats_router_bwd_dx: null pointer");
    const int V = dtype == ATS_F32 ? 4 : 8;
    const bool vec = H % V == 0 && aligned16(wg) && aligned16(out) && (!base || aligned16(base));
    if (vec && E <= kDxExperts && T >= 4 * kDxChunk) {
        // (base may alias out: a thread reads its piece of a row before it writes it)
        const dim3 grid((unsigned)((H / V + 255) / 256), (unsigned)((T + kDxChunk - 1) / kDxChunk));
        if (dtype == ATS_F32)
            hipLaunchKernelGGL((router_dx_cols_kernel<float, false>), grid, dim3(256), 0, as_stream(stream), dlogits,
                               static_cast<const float*>(wg), static_cast<const float*>(base),
                               static_cast<float*>(out), T, E, H);
        else if (E == kDxExperts)
            hipLaunchKernelGGL((router_dx_cols_kernel<bf16_t, true>), grid, dim3(256), 0, as_stream(stream), dlogits,
                               static_cast<const bf16_t*>(wg), static_cast<const bf16_t*>(base),
                               static_cast<bf16_t*>(out), T, E, H);
        else
            hipLaunchKernelGGL((router_dx_cols_kernel<bf16_t, false>), grid, dim3(256), 0, as_stream(stream), dlogits,
                               static_cast<const bf16_t*>(wg), static_cast<const bf16_t*>(base),
                               static_cast<bf16_t*>(out), T, E, H);
        ATS_CHECK_LAUNCH("ats_router_bwd_dx");
        return ATS_OK;
    }
    int64_t blocks = (T + 3) / 4;
    if (blocks > 16384) blocks = 16384;
    if (dtype == ATS_F32)
        hipLaunchKernelGGL((router_dx_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), dlogits,
                           static_cast<const float*>(wg), static_cast<const float*>(base), static_cast<float*>(out), T,
                           E, H, vec);
    else
        hipLaunchKernelGGL((router_dx_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), dlogits,
                           static_cast<const bf16_t*>(wg), static_cast<const bf16_t*>(base),
                           static_cast<bf16_t*>(out), T, E, H, vec);
    ATS_CHECK_LAUNCH("ats_router_bwd_dx");
    return ATS_OK;
}

extern "C" size_t ats_router_bwd_dw_workspace(int64_t T, int E, int H) {
    int chunk_tokens;
    const int n = ats::dw_chunks(T > 0 ? T : 1, &chunk_tokens);
    return (size_t)n * (size_t)(E > 0 ? E : 0) * (size_t)(H > 0 ? H : 0) * sizeof(float);
}

extern "C" int ats_router_bwd_dw(const float* dlogits, const void* x, float* dwg, int64_t T, int E, int H, int dtype,
                                 void* workspace, size_t workspace_bytes, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(T >= 0 && E > 0 && H > 0, ATS_ERR_INVALID_ARG, "ats_router_bwd_dw: T=%lld E=%d H=%d", (long long)T, E, H);
    ATS_REQUIRE(dtype == ATS_F32 || dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "ats_router_bwd_dw: dtype tag %d", dtype);
    ATS_REQUIRE(dwg, ATS_ERR_INVALID_ARG, "ats_router_bwd_dw: null pointer");
    hipStream_t s = as_stream(stream);
    const int64_t EH = (int64_t)E * H;
    if (T == 0) {
        hipLaunchKernelGGL(fill_f32_kernel, dim3((unsigned)ew_blocks(EH)), dim3(256), 0, s, dwg, EH, 0.f);
        ATS_CHECK_LAUNCH("ats_router_bwd_dw");
        return ATS_OK;
    }
    ATS_REQUIRE(dlogits && x, ATS_ERR_INVALID_ARG, "ats_router_bwd_dw: null pointer");
    ATS_REQUIRE(workspace && workspace_bytes >= ats_router_bwd_dw_workspace(T, E, H), ATS_ERR_WORKSPACE,
                "ats_router_bwd_dw: workspace of %zu bytes, need %zu", workspace_bytes,
                ats_router_bwd_dw_workspace(T, E, H));
    int chunk_tokens;
    const int n_chunks = dw_chunks(T, &chunk_tokens);
    float* partial = static_cast<float*>(workspace);
    const int V = dtype == ATS_F32 ? 4 : 8;
    if (H % V == 0 && aligned16(x)) {
        const dim3 grid((unsigned)((H / V + 255) / 256), (unsigned)n_chunks);
        if (dtype == ATS_F32)
            hipLaunchKernelGGL((router_dw_partial_vec_kernel<float, false>), grid, dim3(256), 0, s, dlogits,
                               static_cast<const float*>(x), partial, T, E, H, chunk_tokens);
        else if (E % kDwExperts == 0)
            hipLaunchKernelGGL((router_dw_partial_vec_kernel<bf16_t, true>), grid, dim3(256), 0, s, dlogits,
                               static_cast<const bf16_t*>(x), partial, T, E, H, chunk_tokens);
        else
            hipLaunchKernelGGL((router_dw_partial_vec_kernel<bf16_t, false>), grid, dim3(256), 0, s, dlogits,
                               static_cast<const bf16_t*>(x), partial, T, E, H, chunk_tokens);
    } else {
        const dim3 grid((unsigned)((H + 255) / 256), (unsigned)n_chunks);
        if (dtype == ATS_F32)
            hipLaunchKernelGGL((router_dw_partial_kernel<float>), grid, dim3(256), 0, s, dlogits,
                               static_cast<const float*>(x), partial, T, E, H, chunk_tokens);
        else
            hipLaunchKernelGGL((router_dw_partial_kernel<bf16_t>), grid, dim3(256), 0, s, dlogits,
                               static_cast<const bf16_t*>(x), partial, T, E, H, chunk_tokens);
    }
    hipLaunchKernelGGL(router_dw_reduce_kernel, dim3((unsigned)((EH + 31) / 32)), dim3(256), 0, s, partial, n_chunks,
                       dwg, EH);
    ATS_CHECK_LAUNCH("ats_router_bwd_dw");
    return ATS_OK;
}
