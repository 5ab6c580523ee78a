// Router for gfx950: gate GEMM (tokens x experts, float32 logits) and the fused
// softmax / top-k / histogram / importance pass.
//
// Gate GEMM.  N = E is tiny, so the kernel is bound by reading x once from HBM.
// bf16: a block owns 16 tokens; its 4 or 8 waves split the hidden dimension (that many times
// more loads in flight than one wave per tile).  A wave loads 128 elements of its 16 token rows
// and of 16 gate rows per step with coalesced 16-byte loads (4 rows x 256 bytes per instruction),
// passes them through a wave-private piece of LDS into the operand layout of
// v_mfma_f32_16x16x32_bf16, and the waves' partial tiles are summed in a fixed order through LDS.
// f32 (and odd shapes): one wave per token with plain FMAs.
//
// Routing pass.  A group of G = pow2 >= min(E,64) lanes owns one token; values
// stay in registers, maxima / sums / arg-max run over DPP steps and row / half-wave swaps
// inside the group.  Per-block histogram and probability column sums go to a workspace and
// a second tiny kernel reduces them in a fixed order (bit-reproducible, no
// float atomics) and evaluates the auxiliary loss.
#include <limits.h>
#include <math.h>

#include "ats_common.hpp"

namespace ats {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8_t as_bf16x8(const u32x4_t& u) {
    union {
        u32x4_t u;
        bf16x8_t v;
    } cv;
    cv.u = u;
    return cv.v;
}

constexpr int kGateKC = 128;  // k elements consumed per wave per step

// NT = number of 16-wide expert tiles, KW = waves per block (each owns 1/KW of the hidden
// dimension).  With PF the loads of step s+1 are issued before the MFMAs of step s.
// A step's 16 x 128 elements of x and, tile after tile, of the gate reach the MFMA operand layout through a
// wave-private piece of LDS (see gate_gemm_bf16_flat_kernel: coalesced loads of whole cache lines instead of
// 16 rows x 64 bytes per instruction); a wave's LDS accesses complete in order, so no barrier is involved.
template <int NT, int KW, bool PF>
__global__ __launch_bounds__(KW * 64) void gate_gemm_bf16_kernel(const bf16_t* __restrict__ x,
                                                               const bf16_t* __restrict__ wg,
                                                               const float* __restrict__ bias,
                                                               float* __restrict__ logits, int64_t T, int H,
                                                               int E) {
    static_assert(NT <= 8, "a wave's partial tiles are parked in its 8 KB stage");
    __shared__ __align__(16) unsigned char stage[KW][2][16 * 256];   // per wave: one step of x rows, of 16 gate rows
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r = lane & 15;        // MFMA view: token row (A) / expert inside the tile (B) ...
    const int g = lane >> 4;        // ... and 8-element k group of each 32-element MFMA step
    const int lrow = lane >> 4;     // loader view: row 4 j + lrow of a 16-row tile ...
    const int lchunk = lane & 15;   // ... and 16-byte chunk of the step's 256-byte row piece
    const int64_t t0 = (int64_t)blockIdx.x * 16;

    // this wave's k range (whole steps; the tail is handled by predicates)
    const int steps_total = (H + kGateKC - 1) / kGateKC;
    const int steps_per_wave = (steps_total + KW - 1) / KW;
    const int s_begin = wave * steps_per_wave;
    const int s_end = min(steps_total, s_begin + steps_per_wave);

    f32x4_t acc[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) acc[n] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    const u32x4_t zero4 = {0u, 0u, 0u, 0u};
    u32x4_t a[PF ? 2 : 1][4], b[PF ? 2 : 1][NT][4];
    int woff[4], roff[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int row = 4 * j + lrow;
        woff[j] = row * 256 + ((lchunk ^ row) << 4);
        roff[j] = r * 256 + (((4 * j + g) ^ r) << 4);
    }
    unsigned char* const sx = stage[wave][0];
    unsigned char* const sg = stage[wave][1];

#define GG_LOAD(s_, buf_)                                                                              \
    {                                                                                                  \
        const int kk = (s_) * kGateKC + lchunk * 8;                                                    \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                                \
            const int64_t trow = t0 + 4 * j + lrow;                                                    \
            a[buf_][j] = zero4;                                                                        \
            if (trow < T && kk < H) a[buf_][j] = *reinterpret_cast<const u32x4_t*>(x + trow * (int64_t)H + kk); \
        }                                                                                              \
        _Pragma("unroll") for (int n = 0; n < NT; ++n) {                                               \
            _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                            \
                const int e = n * 16 + 4 * j + lrow;                                                   \
                b[buf_][n][j] = zero4;                                                                 \
                if (e < E && kk < H) b[buf_][n][j] = *reinterpret_cast<const u32x4_t*>(wg + (int64_t)e * H + kk); \
            }                                                                                          \
        }                                                                                              \
    }
// per output tile the order of accumulation is: steps ascending, the four 32-element pieces ascending
#define GG_MMA(buf_)                                                                                   \
    {                                                                                                  \
        u32x4_t fa[4];                                                                                 \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) *reinterpret_cast<u32x4_t*>(sx + woff[j]) = a[buf_][j]; \
        _Pragma("unroll") for (int n = 0; n < NT; ++n) {                                               \
            _Pragma("unroll") for (int j = 0; j < 4; ++j)                                              \
                *reinterpret_cast<u32x4_t*>(sg + woff[j]) = b[buf_][n][j];                             \
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                         \
            if (n == 0) {                                                                              \
                _Pragma("unroll") for (int i = 0; i < 4; ++i) fa[i] = *reinterpret_cast<const u32x4_t*>(sx + roff[i]); \
            }                                                                                          \
            _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                            \
                const u32x4_t fb = *reinterpret_cast<const u32x4_t*>(sg + roff[i]);                    \
                acc[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(fa[i]), as_bf16x8(fb), acc[n], 0, 0, 0); \
            }                                                                                          \
            asm volatile("" ::: "memory");                                                             \
        }                                                                                              \
    }
    if constexpr (PF) {
        if (s_begin < s_end) {
            GG_LOAD(s_begin, 0);
            int s = s_begin;
            for (; s + 2 < s_end; s += 2) {
                GG_LOAD(s + 1, 1);
                GG_MMA(0);
                GG_LOAD(s + 2, 0);
                GG_MMA(1);
            }
            if (s + 1 < s_end) {
                GG_LOAD(s + 1, PF ? 1 : 0);
                GG_MMA(0);
                GG_MMA(PF ? 1 : 0);
            } else {
                GG_MMA(0);
            }
        }
    } else {
        for (int s = s_begin; s < s_end; ++s) {
            GG_LOAD(s, 0);
            GG_MMA(0);
        }
    }
#undef GG_LOAD
#undef GG_MMA
    // D layout of the 16x16 tile: lane holds column (lane & 15), rows 4*(lane>>4) + v.  A wave parks its NT
    // partial tiles at the front of its own stage.
    float* const red = reinterpret_cast<float*>(stage[wave][0]);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int n = 0; n < NT; ++n) {
#pragma unroll
        for (int v = 0; v < 4; ++v) red[n * 256 + (4 * g + v) * 16 + r] = acc[n][v];
    }
    __syncthreads();
    for (int i = threadIdx.x; i < NT * 256; i += KW * 64) {
        const int n = i >> 8;
        const int row = (i & 255) >> 4;
        const int col = i & 15;
        const int e = n * 16 + col;
        const int64_t t = t0 + row;
        if (t < T && e < E) {
            float v = reinterpret_cast<const float*>(stage[0][0])[i];
#pragma unroll
            for (int w = 1; w < KW; ++w) v += reinterpret_cast<const float*>(stage[w][0])[i];
            if (bias) v += bias[e];
            logits[t * E + e] = v;
        }
    }
}

// Up to 16 experts and a hidden size of at most 8 x 4 x 128: the same split of K over 8 waves, but a wave
// asks for its whole K slice of the 16 token rows at once (up to 4 steps x 4 loads) before the first MFMA, so the
// block's bytes are all in flight after a few hundred cycles, which is what a kernel that lives for 20 us needs.
// The loads are coalesced - an instruction covers 4 rows x 256 bytes, whole cache lines - and a step's 16 x 128
// elements of x and of the gate go through a wave-private 4 KB piece of LDS each to reach the MFMA operand layout
// (lane (r, g) holds 8 elements of row r): loaded directly in that layout an instruction touches 16 rows x 64
// bytes, and the vector cache serves that pattern at a quarter of the rate (38 against 134 GB/s per CU from L2).
// LDS slot c ^ r holds the 16-byte chunk c of row r, so the 16 rows of a fragment read hit all banks.  The gate
// rows are fetched one step ahead of their use; order of accumulation as in gate_gemm_bf16_kernel: steps
// ascending, the four 32-element pieces ascending, the waves' partial sums in wave order.
__global__ __launch_bounds__(512) void gate_gemm_bf16_flat_kernel(const bf16_t* __restrict__ x,
                                                                  const bf16_t* __restrict__ wg,
                                                                  const float* __restrict__ bias,
                                                                  float* __restrict__ logits, int64_t T, int H, int E) {
    constexpr int KW = 8, S = 4;
    __shared__ __align__(16) unsigned char stage[KW][2][16 * 256];   // per wave: one step of x rows, of gate rows
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r = lane & 15;        // MFMA view: token row (A) / expert (B) ...
    const int g = lane >> 4;        // ... and 8-element k group of a 32-element piece
    const int lrow = lane >> 4;     // loader view: row 4 j + lrow of the tile ...
    const int lchunk = lane & 15;   // ... and 16-byte chunk of the step's 256-byte row piece
    const int64_t t0 = (int64_t)blockIdx.x * 16;
    const int steps_total = (H + kGateKC - 1) / kGateKC;
    const int steps_per_wave = (steps_total + KW - 1) / KW;      // <= S (host)
    const int s_begin = wave * steps_per_wave;
    const u32x4_t zero4 = {0u, 0u, 0u, 0u};
    u32x4_t a[S][4], b[2][4];
    // token rows first: they come from HBM, the gate rows from L2
#pragma unroll
    for (int st = 0; st < S; ++st) {
        const int kk = (s_begin + st) * kGateKC + lchunk * 8;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t trow = t0 + 4 * j + lrow;
            a[st][j] = zero4;
            if (st < steps_per_wave && trow < T && kk < H)
                a[st][j] = *reinterpret_cast<const u32x4_t*>(x + trow * (int64_t)H + kk);
        }
    }
#define GF_LOAD_B(st_, buf_)                                                                           \
    {                                                                                                  \
        const int kk = (s_begin + (st_)) * kGateKC + lchunk * 8;                                       \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                                \
            const int e = 4 * j + lrow;                                                                \
            b[buf_][j] = zero4;                                                                        \
            if ((st_) < steps_per_wave && e < E && kk < H)                                             \
                b[buf_][j] = *reinterpret_cast<const u32x4_t*>(wg + (int64_t)e * H + kk);              \
        }                                                                                              \
    }
    GF_LOAD_B(0, 0);
    int woff[4], roff[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int row = 4 * j + lrow;
        woff[j] = row * 256 + ((lchunk ^ row) << 4);
        roff[j] = r * 256 + (((4 * j + g) ^ r) << 4);
    }
    unsigned char* const sx = stage[wave][0];
    unsigned char* const sg = stage[wave][1];
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int st = 0; st < S; ++st) {
        if (st + 1 < S) GF_LOAD_B(st + 1, (st + 1) & 1);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            *reinterpret_cast<u32x4_t*>(sx + woff[j]) = a[st][j];
            *reinterpret_cast<u32x4_t*>(sg + woff[j]) = b[st & 1][j];
        }
        // the tile is private to the wave and a wave's LDS accesses complete in order: no barrier, the
        // compiler only has to keep the reads behind the writes (and the next step's writes behind the reads)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const u32x4_t fa = *reinterpret_cast<const u32x4_t*>(sx + roff[i]);
            const u32x4_t fb = *reinterpret_cast<const u32x4_t*>(sg + roff[i]);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(fa), as_bf16x8(fb), acc, 0, 0, 0);
        }
        asm volatile("" ::: "memory");
    }
#undef GF_LOAD_B
    // the waves' partial tiles, each in the front of its own stage
    float* const red = reinterpret_cast<float*>(stage[wave][0]);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int v = 0; v < 4; ++v) red[(4 * g + v) * 16 + r] = acc[v];
    __syncthreads();
    for (int i = threadIdx.x; i < 256; i += KW * 64) {
        const int row = i >> 4;
        const int col = i & 15;
        const int64_t t = t0 + row;
        if (t < T && col < E) {
            float v = reinterpret_cast<const float*>(stage[0][0])[i];
#pragma unroll
            for (int w = 1; w < KW; ++w) v += reinterpret_cast<const float*>(stage[w][0])[i];
            if (bias) v += bias[col];
            logits[t * E + col] = v;
        }
    }
}

// One wave per token, 8 experts at a time.  Works for every dtype / shape.
template <typename T>
__global__ __launch_bounds__(256) void gate_gemm_generic_kernel(const T* __restrict__ x, const T* __restrict__ wg,
                                                                const float* __restrict__ bias,
                                                                float* __restrict__ logits, int64_t Tn, int H,
                                                                int E) {
    const int lane = lane_id();
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
    for (int64_t t = wave; t < Tn; t += nwaves) {
        const T* xr = x + t * H;
        for (int e0 = 0; e0 < E; e0 += 8) {
            float acc[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = 0.f;
            for (int h = lane; h < H; h += kWave) {
                const float xv = Elem<T>::load(xr + h);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    if (e0 + j < E) acc[j] += xv * Elem<T>::load(wg + (int64_t)(e0 + j) * H + h);
                }
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float s = wave_sum(acc[j]);
                if (lane == 0 && e0 + j < E) logits[t * E + e0 + j] = s + (bias ? bias[e0 + j] : 0.f);
            }
        }
    }
}

// ------------------------------------------------------------------ routing pass
// Value of the partner lane in step S of an ascending butterfly over groups of 2^(S+1) lanes, without LDS:
// quad permutes for steps 0 and 1; mirrored half rows and rows for steps 2 and 3 (the lane 7-i or 15-i holds what
// lane i^4 or i^8 holds once the earlier steps have made quads / half rows uniform, which an ascending butterfly
// guarantees); swaps of 16-lane rows and of the wave's halves for steps 4 and 5.  All 64 lanes must be active.
template <int S>
__device__ __forceinline__ unsigned butterfly_partner(unsigned v) {
    if constexpr (S == 0) return dpp_u32<kDppSwapPairs>(v);
    else if constexpr (S == 1) return dpp_u32<kDppSwapQuadHalves>(v);
    else if constexpr (S == 2) return dpp_u32<kDppHalfMirror>(v);
    else if constexpr (S == 3) return dpp_u32<kDppRowMirror>(v);
    else if constexpr (S == 4) {
        const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);     // {even rows twice, odd rows twice}
        return (threadIdx.x & 16) ? r[0] : r[1];
    } else {
        const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);     // {low half twice, high half twice}
        return (threadIdx.x & 32) ? r[0] : r[1];
    }
}
template <int S>
__device__ __forceinline__ float butterfly_partner_f32(float v) {
    return __uint_as_float(butterfly_partner<S>(__float_as_uint(v)));
}
// Reductions over groups of G lanes (a power of two), the result in every lane of the group.
__device__ __forceinline__ float group_max(float v, int G) {
    if (G > 1) v = fmaxf(v, butterfly_partner_f32<0>(v));
    if (G > 2) v = fmaxf(v, butterfly_partner_f32<1>(v));
    if (G > 4) v = fmaxf(v, butterfly_partner_f32<2>(v));
    if (G > 8) v = fmaxf(v, butterfly_partner_f32<3>(v));
    if (G > 16) v = fmaxf(v, butterfly_partner_f32<4>(v));
    if (G > 32) v = fmaxf(v, butterfly_partner_f32<5>(v));
    return v;
}
__device__ __forceinline__ float group_sum(float v, int G) {
    if (G > 1) v += butterfly_partner_f32<0>(v);
    if (G > 2) v += butterfly_partner_f32<1>(v);
    if (G > 4) v += butterfly_partner_f32<2>(v);
    if (G > 8) v += butterfly_partner_f32<3>(v);
    if (G > 16) v += butterfly_partner_f32<4>(v);
    if (G > 32) v += butterfly_partner_f32<5>(v);
    return v;
}
// Order used for selection: larger value first, lower index among equals; NaN
// ranks above every number (as torch.topk does).
__device__ __forceinline__ bool key_before(float va, int ia, float vb, int ib) {
    const bool na = va != va, nb = vb != vb;
    if (na != nb) return na;
    if (!na && va != vb) return va > vb;
    return ia < ib;
}

constexpr int kRouteMaxK = 16;

// Selection key of key_before as an unsigned number: larger key = earlier in the order.  NaN is the largest
// key, -0 counts as +0, and 0 is below every value (used for lanes that hold no candidate).
__device__ __forceinline__ unsigned route_order_key(float v) {
    if (v != v) return 0xFFFFFFFFu;
    const unsigned u = (unsigned)__float_as_int(v + 0.0f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// One token per wave, one expert per lane (32 < E <= 64): the reductions of the softmax and the k arg-max rounds
// run on DPP and scalar reads instead of shuffles through LDS; an arg-max is the wave maximum of the keys,
// then the lowest lane that holds it.  Same selection, weights and statistics as route_topk_kernel, except that
// the sums of the softmax are formed in another (fixed) order.
__global__ __launch_bounds__(256) void route_topk_wave_kernel(const float* __restrict__ logits, int64_t T, int E, int k,
                                                              float temperature, int variant, int iters,
                                                              int32_t* __restrict__ idx_out, float* __restrict__ w_out,
                                                              int32_t* __restrict__ part_hist,
                                                              float* __restrict__ part_colsum) {
    extern __shared__ unsigned char smem_raw[];
    int* s_hist = reinterpret_cast<int*>(smem_raw);            // [E]
    float* s_col = reinterpret_cast<float*>(s_hist + E);        // [4][E]
    const bool want_stats = part_hist != nullptr;
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const bool has = lane < E;
    if (want_stats) {
        for (int i = threadIdx.x; i < E; i += 256) s_hist[i] = 0;
        __syncthreads();
    }
    float col = 0.f;
    const float neg_inf = -INFINITY;
    for (int it = 0; it < iters; ++it) {
        const int64_t t = ((int64_t)blockIdx.x * iters + it) * 4 + wave;
        if (t >= T) break;                                   // wave-uniform
        const float v = has ? logits[t * E + lane] : neg_inf;
        const float m0 = wave_max_f32(v);
        float p0 = has ? expf(v - m0) : 0.f;
        p0 = p0 / wave_sum_f32(p0);
        col += p0;
        float sv = v, p = p0;
        if (temperature != 1.0f) {
            sv = has ? __fdiv_rn(v, temperature) : neg_inf;
            const float m = wave_max_f32(sv);
            p = has ? expf(sv - m) : 0.f;
            p = p / wave_sum_f32(p);
        }
        unsigned key = has ? route_order_key(sv) : 0u;
        float sel_val = 0.f, sel_p = 0.f;
        int sel_idx = 0;
        for (int j = 0; j < k; ++j) {
            const unsigned best = wave_max_u32(key);
            const int first = __builtin_amdgcn_readfirstlane(__ffsll((long long)__ballot(key == best)) - 1);
            const float bv = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(sv), first));
            const float bp = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), first));
            if (lane == first) key = 0u;
            if (lane == j) {
                sel_val = bv;
                sel_p = bp;
                sel_idx = first;
            }
            if (want_stats && lane == 0) atomicAdd(&s_hist[first], 1);
        }
        float wsel;
        const bool is_sel = lane < k;
        if (variant == ATS_ROUTE_SOFTMAX_TOPK) {
            float tot = 0.f;
            for (int j = 0; j < k; ++j) tot += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(sel_p), j));
            wsel = sel_p / (tot + 1e-9f);
        } else {
            const float mx = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(sel_val), 0));
            const float ex = is_sel ? expf(sel_val - mx) : 0.f;
            float tot = 0.f;
            for (int j = 0; j < k; ++j) tot += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ex), j));
            wsel = ex / tot;
        }
        if (is_sel) {
            idx_out[t * k + lane] = sel_idx;
            w_out[t * k + lane] = wsel;
        }
    }
    if (want_stats) {
        if (has) s_col[wave * E + lane] = col;
        __syncthreads();
        for (int e = threadIdx.x; e < E; e += 256) {
            part_hist[(int64_t)blockIdx.x * E + e] = s_hist[e];
            part_colsum[(int64_t)blockIdx.x * E + e] = ((s_col[e] + s_col[E + e]) + s_col[2 * E + e]) + s_col[3 * E + e];
        }
    }
}

template <int VPL>
__global__ __launch_bounds__(256) void route_topk_kernel(const float* __restrict__ logits, int64_t T, int E, int k,
                                                         float temperature, int variant, int G, int iters,
                                                         int32_t* __restrict__ idx_out, float* __restrict__ w_out,
                                                         int32_t* __restrict__ part_hist,
                                                         float* __restrict__ part_colsum, float lbw,
                                                         int32_t* __restrict__ hist, float* __restrict__ colsum,
                                                         float* __restrict__ aux) {
    extern __shared__ unsigned char smem_raw[];
    int* s_hist = reinterpret_cast<int*>(smem_raw);            // [E]
    float* s_col = reinterpret_cast<float*>(s_hist + E);        // [4][E]  (then [E] terms of the auxiliary loss)
    const bool want_stats = part_hist != nullptr;
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int gl = lane & (G - 1);          // lane inside the group
    const int grp = lane / G;               // group inside the wave
    const int groups_per_wave = kWave / G;
    const int groups_per_block = 4 * groups_per_wave;

    if (want_stats) {
        for (int i = threadIdx.x; i < E; i += 256) s_hist[i] = 0;
        __syncthreads();
    }
    float col[VPL];
#pragma unroll
    for (int i = 0; i < VPL; ++i) col[i] = 0.f;

    const float neg_inf = -INFINITY;
    for (int it = 0; it < iters; ++it) {
        const int64_t t = ((int64_t)blockIdx.x * iters + it) * groups_per_block + wave * groups_per_wave + grp;
        const bool tok_ok = t < T;
        float v[VPL];
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            const int e = gl + i * G;
            v[i] = (tok_ok && e < E) ? logits[t * E + e] : neg_inf;
        }
        // softmax of the raw logits (importance term of the auxiliary loss)
        float m0 = neg_inf;
#pragma unroll
        for (int i = 0; i < VPL; ++i) m0 = fmaxf(m0, v[i]);
        m0 = group_max(m0, G);
        float p0[VPL];
        float s0 = 0.f;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            p0[i] = (gl + i * G < E) ? expf(v[i] - m0) : 0.f;
            s0 += p0[i];
        }
        s0 = group_sum(s0, G);
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            p0[i] = p0[i] / s0;
            if (tok_ok) col[i] += p0[i];
        }
        // tempered values and (variant 0) their softmax
        float sv[VPL], p[VPL];
        if (temperature == 1.0f) {
#pragma unroll
            for (int i = 0; i < VPL; ++i) {
                sv[i] = v[i];
                p[i] = p0[i];
            }
        } else {
            float m = neg_inf;
#pragma unroll
            for (int i = 0; i < VPL; ++i) {
                sv[i] = (gl + i * G < E) ? __fdiv_rn(v[i], temperature) : neg_inf;
                m = fmaxf(m, sv[i]);
            }
            m = group_max(m, G);
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < VPL; ++i) {
                p[i] = (gl + i * G < E) ? expf(sv[i] - m) : 0.f;
                s += p[i];
            }
            s = group_sum(s, G);
#pragma unroll
            for (int i = 0; i < VPL; ++i) p[i] = p[i] / s;
        }
        // k rounds of group-wide arg-max
        unsigned taken = 0;   // bit i: v[i] already selected
        float sel_term = 0.f; // lane j < k of the group keeps choice j: its unnormalised weight ...
        int sel_idx = 0;      // ... and expert id
        float tot = 0.f, first_val = 0.f;
        for (int j = 0; j < k; ++j) {
            float bv = neg_inf;
            int bi = INT_MAX;
            float bp = 0.f;
#pragma unroll
            for (int i = 0; i < VPL; ++i) {
                const int e = gl + i * G;
                if (e < E && !((taken >> i) & 1u) && key_before(sv[i], e, bv, bi)) {
                    bv = sv[i];
                    bi = e;
                    bp = p[i];
                }
            }
#define ROUTE_MERGE_STEP(S_)                                                       \
    if (G > (1 << (S_))) {                                                         \
        const float ov = butterfly_partner_f32<S_>(bv);                            \
        const int oi = (int)butterfly_partner<S_>((unsigned)bi);                   \
        const float op = butterfly_partner_f32<S_>(bp);                            \
        if (key_before(ov, oi, bv, bi)) {                                          \
            bv = ov;                                                               \
            bi = oi;                                                               \
            bp = op;                                                               \
        }                                                                          \
    }
            ROUTE_MERGE_STEP(0)
            ROUTE_MERGE_STEP(1)
            ROUTE_MERGE_STEP(2)
            ROUTE_MERGE_STEP(3)
            ROUTE_MERGE_STEP(4)
            ROUTE_MERGE_STEP(5)
#undef ROUTE_MERGE_STEP
            // owner marks its value as used
#pragma unroll
            for (int i = 0; i < VPL; ++i)
                if (gl + i * G == bi) taken |= 1u << i;
            // the round's choice is the same in every lane of the group, so the normaliser of the weights is
            // summed here, in rank order, instead of being gathered afterwards
            if (j == 0) first_val = bv;
            const float term = variant == ATS_ROUTE_SOFTMAX_TOPK ? bp : expf(bv - first_val);
            tot += term;
            // k <= G always holds: G >= min(E, 64) and k <= min(E, kRouteMaxK)
            if (gl == j) {
                sel_term = term;
                sel_idx = bi;
            }
            if (want_stats && tok_ok && gl == 0) atomicAdd(&s_hist[bi], 1);
        }
        // weights: lanes 0..k-1 of the group hold the choices in rank order
        const bool is_sel = gl < k;
        const float wsel = variant == ATS_ROUTE_SOFTMAX_TOPK ? sel_term / (tot + 1e-9f) : sel_term / tot;
        if (tok_ok && is_sel) {
            idx_out[t * k + gl] = sel_idx;
            w_out[t * k + gl] = wsel;
        }
    }
    if (want_stats) {
        // fold the groups of a wave together (fixed butterfly), then the 4 waves via LDS
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            float c = col[i];
            for (int off = 32; off >= G; off >>= 1) c += __shfl_xor(c, off, 64);
            const int e = gl + i * G;
            if (grp == 0 && e < E) s_col[wave * E + e] = c;
        }
        __syncthreads();
        if (gridDim.x > 1) {
            for (int e = threadIdx.x; e < E; e += 256) {
                part_hist[(int64_t)blockIdx.x * E + e] = s_hist[e];
                part_colsum[(int64_t)blockIdx.x * E + e] =
                    ((s_col[e] + s_col[E + e]) + s_col[2 * E + e]) + s_col[3 * E + e];
            }
        } else {
            // one block holds every token (a decoding step): its partials are the totals, so the statistics
            // and the auxiliary loss are finished here, with route_finalize_kernel's arithmetic
            float* s_term = s_col + 4 * E;
            for (int e = threadIdx.x; e < E; e += 256) {
                const int hsum = s_hist[e];
                const float csum = ((s_col[e] + s_col[E + e]) + s_col[2 * E + e]) + s_col[3 * E + e];
                hist[e] = hsum;
                colsum[e] = csum;
                const float usage = (float)hsum / (float)((double)T * k + 1e-9);
                const float importance = csum / (float)T;
                s_term[e] = usage * importance;
            }
            __syncthreads();
            if (threadIdx.x == 0 && aux) {
                float sum = 0.f;
                for (int e = 0; e < E; ++e) sum += s_term[e];
                aux[0] = fminf(sum * (float)E * lbw, 1.0f);
            }
        }
    }
}

// Reduces the per-block partials in a fixed order and evaluates the auxiliary loss.
// Thread (e, c) sums blocks c, c+TPE, ... of expert e (consecutive threads read consecutive
// experts: coalesced); the TPE partial sums of an expert are then added in ascending c.
__global__ __launch_bounds__(1024) void route_finalize_kernel(const int32_t* __restrict__ part_hist,
                                                             const float* __restrict__ part_colsum, int nblocks,
                                                             int E, int64_t T, int k, float lbw,
                                                             int32_t* __restrict__ hist, float* __restrict__ colsum,
                                                             float* __restrict__ aux) {
    extern __shared__ unsigned char smem_raw[];
    float* s_term = reinterpret_cast<float*>(smem_raw);          // [E]
    int* s_h = reinterpret_cast<int*>(s_term + E);               // [1024]
    float* s_c = reinterpret_cast<float*>(s_h + 1024);           // [1024]
    int tpe = 1;
    while (tpe * 2 * E <= 1024) tpe *= 2;  // threads per expert (power of two), 1 when E > 512
    for (int e0 = 0; e0 < E; e0 += 1024 / tpe) {
        const int e = e0 + (int)threadIdx.x % (1024 / tpe);
        const int c = (int)threadIdx.x / (1024 / tpe);
        int hsum = 0;
        float csum = 0.f;
        if (e < E) {
            for (int b = c; b < nblocks; b += tpe * 8) {   // 8 independent loads in flight, summed in order
                int hv[8];
                float cv[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int bb = b + u * tpe;
                    hv[u] = bb < nblocks ? part_hist[(int64_t)bb * E + e] : 0;
                    cv[u] = bb < nblocks ? part_colsum[(int64_t)bb * E + e] : 0.f;
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    hsum += hv[u];
                    csum += cv[u];
                }
            }
        }
        s_h[threadIdx.x] = hsum;
        s_c[threadIdx.x] = csum;
        __syncthreads();
        if (c == 0 && e < E) {
            for (int cc = 1; cc < tpe; ++cc) {
                hsum += s_h[cc * (1024 / tpe) + (int)threadIdx.x];
                csum += s_c[cc * (1024 / tpe) + (int)threadIdx.x];
            }
            hist[e] = hsum;
            colsum[e] = csum;
            const float usage = (float)hsum / (float)((double)T * k + 1e-9);
            const float importance = csum / (float)T;
            s_term[e] = usage * importance;
        }
        __syncthreads();
    }
    if (threadIdx.x == 0 && aux) {
        float s = 0.f;
        for (int e = 0; e < E; ++e) s += s_term[e];
        aux[0] = fminf(s * (float)E * lbw, 1.0f);
    }
}

static int route_grid(int64_t T, int E, int* G_out, int* iters_out) {
    int G = 1;
    while (G < E && G < kWave) G <<= 1;
    const int groups_per_block = 4 * (kWave / G);
    int64_t iters = (T + (int64_t)512 * groups_per_block - 1) / ((int64_t)512 * groups_per_block);
    if (iters < 1) iters = 1;
    if (iters > 64) iters = 64;
    const int64_t per_block = (int64_t)groups_per_block * iters;
    *G_out = G;
    // few tokens: one block takes them all in up to 16 passes and finishes the statistics itself
    const int64_t passes = (T + groups_per_block - 1) / groups_per_block;
    if (passes <= 16) {
        *iters_out = (int)(passes < 1 ? 1 : passes);
        return 1;
    }
    *iters_out = (int)iters;
    return (int)((T + per_block - 1) / per_block);
}

}  // namespace ats

extern "C" int ats_router_logits(const void* x, const void* wg, const float* bias, float* logits, int64_t T, int H,
                                 int E, int dtype, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(T >= 0 && H > 0 && E > 0, ATS_ERR_INVALID_ARG, "ats_router_logits: T=%lld H=%d E=%d", (long long)T, H,
                E);
    ATS_REQUIRE(dtype == ATS_F32 || dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "ats_router_logits: dtype tag %d", dtype);
    if (T == 0) return ATS_OK;
    ATS_REQUIRE(x && wg && logits, ATS_ERR_INVALID_ARG, "ats_router_logits: null pointer");
    hipStream_t s = as_stream(stream);
    const bool mfma_ok = dtype == ATS_BF16 && H % 8 == 0 && aligned16(x) && aligned16(wg) && E <= 128;
    if (mfma_ok) {
        const unsigned blocks = (unsigned)((T + 15) / 16);
        const bf16_t* xp = static_cast<const bf16_t*>(x);
        const bf16_t* wp = static_cast<const bf16_t*>(wg);
        const int nt = (E + 15) / 16;
        // Few experts: 8 waves split K (short dependent chains, 32 waves per CU resident);
        // more expert tiles need more registers per wave and use 4 waves with (NT <= 2) prefetch.
        // prefill-sized batches of a hidden size that 8 waves cover in 4 steps each: the flat kernel (one 16-token
        // tile per block: two blocks stay resident per CU; with two tiles per block the kernel ran 36 instead of 27 us
        // on [16384, 4096] x 8 experts, the looped kernel 37 us)
        if (nt <= 1 && H <= 8 * 4 * kGateKC && T >= 2048)
            hipLaunchKernelGGL(gate_gemm_bf16_flat_kernel, dim3(blocks), dim3(512), 0, s, xp, wp, bias, logits, T, H, E);
        else if (nt <= 1)
            hipLaunchKernelGGL((gate_gemm_bf16_kernel<1, 8, false>), dim3(blocks), dim3(512), 0, s, xp, wp, bias, logits, T, H, E);
        else if (nt <= 2)
            hipLaunchKernelGGL((gate_gemm_bf16_kernel<2, 4, true>), dim3(blocks), dim3(256), 0, s, xp, wp, bias, logits, T, H, E);
        else if (nt <= 4)
            hipLaunchKernelGGL((gate_gemm_bf16_kernel<4, 4, false>), dim3(blocks), dim3(256), 0, s, xp, wp, bias, logits, T, H, E);
        else
            hipLaunchKernelGGL((gate_gemm_bf16_kernel<8, 4, false>), dim3(blocks), dim3(256), 0, s, xp, wp, bias, logits, T, H, E);
    } else {
        int64_t blocks = (T + 3) / 4;
        if (blocks > 8192) blocks = 8192;
        if (dtype == ATS_F32)
            hipLaunchKernelGGL((gate_gemm_generic_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, s,
                               static_cast<const float*>(x), static_cast<const float*>(wg), bias, logits, T, H, E);
        else
            hipLaunchKernelGGL((gate_gemm_generic_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, s,
                               static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(wg), bias, logits, T, H, E);
    }
    ATS_CHECK_LAUNCH("ats_router_logits");
    return ATS_OK;
}

extern "C" size_t ats_route_topk_workspace(int64_t T, int E) {
    using namespace ats;
    if (T <= 0 || E <= 0) return 0;
    int G, iters;
    const int nblocks = route_grid(T, E, &G, &iters);
    return (size_t)nblocks * E * (sizeof(int32_t) + sizeof(float));
}

extern "C" int ats_route_topk(const float* logits, int64_t T, int E, int k, float temperature, int variant,
                              int32_t* idx_out, float* w_out, int32_t* hist, float* prob_colsum, float* aux,
                              float load_balancing_weight, void* workspace, size_t workspace_bytes,
                              ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(T >= 0 && E > 0 && E <= 1024 && k > 0 && k <= E && k <= kRouteMaxK, ATS_ERR_INVALID_ARG,
                "ats_route_topk: T=%lld E=%d k=%d (need 1 <= k <= min(E,%d), E <= 1024)", (long long)T, E, k,
                kRouteMaxK);
    ATS_REQUIRE(variant == ATS_ROUTE_SOFTMAX_TOPK || variant == ATS_ROUTE_TOPK_SOFTMAX, ATS_ERR_INVALID_ARG,
                "ats_route_topk: variant %d", variant);
    ATS_REQUIRE(temperature > 0.f, ATS_ERR_INVALID_ARG, "ats_route_topk: temperature %g", temperature);
    const bool stats = hist != nullptr;
    ATS_REQUIRE((hist != nullptr) == (prob_colsum != nullptr), ATS_ERR_INVALID_ARG,
                "ats_route_topk: hist and prob_colsum must be given together");
    ATS_REQUIRE(stats || aux == nullptr, ATS_ERR_INVALID_ARG, "ats_route_topk: aux needs hist and prob_colsum");
    if (T == 0) return ATS_OK;
    ATS_REQUIRE(logits && idx_out && w_out, ATS_ERR_INVALID_ARG, "ats_route_topk: null pointer");
    int G, iters;
    const int nblocks = route_grid(T, E, &G, &iters);
    int32_t* part_hist = nullptr;
    float* part_col = nullptr;
    if (stats) {
        const size_t need = (size_t)nblocks * E * (sizeof(int32_t) + sizeof(float));
        ATS_REQUIRE(workspace && workspace_bytes >= need, ATS_ERR_WORKSPACE,
                    "ats_route_topk: workspace %zu bytes, need %zu", workspace_bytes, need);
        part_hist = static_cast<int32_t*>(workspace);
        part_col = reinterpret_cast<float*>(part_hist + (size_t)nblocks * E);
    }
    hipStream_t s = as_stream(stream);
    const size_t smem = (size_t)E * 6 * sizeof(float);
    const int vpl = (E + G - 1) / G;
    if (G == kWave && vpl <= 1 && nblocks > 1)
        hipLaunchKernelGGL(route_topk_wave_kernel, dim3(nblocks), dim3(256), smem, s, logits, T, E, k, temperature,
                           variant, iters, idx_out, w_out, part_hist, part_col);
    else if (vpl <= 1)
        hipLaunchKernelGGL((route_topk_kernel<1>), dim3(nblocks), dim3(256), smem, s, logits, T, E, k, temperature,
                           variant, G, iters, idx_out, w_out, part_hist, part_col, load_balancing_weight, hist,
                           prob_colsum, aux);
    else if (vpl <= 4)
        hipLaunchKernelGGL((route_topk_kernel<4>), dim3(nblocks), dim3(256), smem, s, logits, T, E, k, temperature,
                           variant, G, iters, idx_out, w_out, part_hist, part_col, load_balancing_weight, hist,
                           prob_colsum, aux);
    else
        hipLaunchKernelGGL((route_topk_kernel<16>), dim3(nblocks), dim3(256), smem, s, logits, T, E, k, temperature,
                           variant, G, iters, idx_out, w_out, part_hist, part_col, load_balancing_weight, hist,
                           prob_colsum, aux);
    ATS_CHECK_LAUNCH("ats_route_topk");
    if (stats && nblocks > 1) {
        hipLaunchKernelGGL(route_finalize_kernel, dim3(1), dim3(1024), (size_t)(E + 2048) * sizeof(float), s, part_hist,
                           part_col, nblocks, E, T, k, load_balancing_weight, hist, prob_colsum, aux);
        ATS_CHECK_LAUNCH("ats_route_topk(finalize)");
    }
    return ATS_OK;
}
