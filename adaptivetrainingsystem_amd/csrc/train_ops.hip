// Training-step ops next to the sparse layer (gfx950, HBM-bound):
//   fused cross-entropy + accuracy (forward and the gradient w.r.t. the logits),
//   multi-tensor gradient norm + clipping.
// They replace fused_cross_entropy_accuracy_launcher (Src/Main_Scripts/training/fused_loss.cu:179-214)
// and fused_grad_clip_launcher (Src/Main_Scripts/training/fused_grad_clip.cu:117-175).  Differences by
// design: every sum runs in a fixed order (per-token / per-chunk partials and an ordered second pass
// instead of float atomics), nothing synchronises, bf16 logits and gradients are accepted, and the
// logits gradient exists (the reference's fused loss returns a value without a graph).
#include <math.h>

#include "ats_common.hpp"

namespace ats {

// exp through the hardware exp2 (about 1 ulp; the scaled argument adds a few 1e-7 relative for |x| < 30)
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }

// ---------------------------------------------------------------- cross entropy
struct MaxSum {
    float m, s;   // running maximum and sum of exp(x - m)
};
__device__ __forceinline__ MaxSum ms_merge(MaxSum a, MaxSum b) {
    if (b.m > a.m) {
        MaxSum t = a;
        a = b;
        b = t;
    }
    if (b.m == -INFINITY) return a;
    a.s += b.s * expf(b.m - a.m);
    return a;
}
struct ArgMax {
    float v;
    int i;
};
__device__ __forceinline__ ArgMax am_merge(ArgMax a, ArgMax b) {   // larger value, lower index among equals
    return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}

// One block (256 threads) per token: one pass over the row with an online max / sum-of-exponentials and
// arg-max per thread, then a block reduction.  Outputs per token: loss (0 for ignored tokens),
// lse = max + log(sum exp), correct (1.0 when the arg-max equals the label), valid (1.0 / 0.0).
// A token is ignored when its label equals pad_id or lies outside [0, V) (fused_loss.cu:83-84).
template <typename T>
__global__ __launch_bounds__(256) void cross_entropy_fwd_kernel(const T* __restrict__ logits,
                                                                const int64_t* __restrict__ labels, int64_t pad_id,
                                                                float* __restrict__ loss, float* __restrict__ lse,
                                                                float* __restrict__ correct, float* __restrict__ valid,
                                                                int V, bool vec) {
    constexpr int VW = Elem<T>::kVec;
    __shared__ MaxSum s_ms[4];
    __shared__ ArgMax s_am[4];
    const int64_t t = blockIdx.x;
    const int64_t label = labels[t];
    if (label == pad_id || label < 0 || label >= V) {
        if (threadIdx.x == 0) {
            loss[t] = 0.f;
            lse[t] = 0.f;
            correct[t] = 0.f;
            valid[t] = 0.f;
        }
        return;
    }
    const T* row = logits + t * V;
    MaxSum ms{-INFINITY, 0.f};
    ArgMax am{-INFINITY, 0x7fffffff};
    auto visit = [&](float x, int i) {
        if (x > ms.m) {
            ms.s = ms.s * expf(ms.m - x) + 1.f;
            ms.m = x;
        } else {
            ms.s += expf(x - ms.m);
        }
        if (x > am.v) {   // indices are visited in ascending order per thread: strict > keeps the first
            am.v = x;
            am.i = i;
        }
    };
    constexpr int kRegVecs = 16;   // rows of up to 256 * 16 vectors stay in registers: one pass over HBM,
                                   // all loads in flight at once, then max, then one exp per element
    const int nv = V / VW;
    if (vec && nv <= 256 * kRegVecs && V % VW == 0) {
        uint4 raw[kRegVecs];
#pragma unroll
        for (int q = 0; q < kRegVecs; ++q) {
            const int v = threadIdx.x + q * 256;
            if (v < nv) raw[q] = reinterpret_cast<const uint4*>(row)[v];
        }
        float mx = -INFINITY;
        int mi = 0x7fffffff;
#pragma unroll
        for (int q = 0; q < kRegVecs; ++q) {
            const int v = threadIdx.x + q * 256;
            if (v < nv) {
                float f[VW];
                Elem<T>::unpack(raw[q], f);
#pragma unroll
                for (int j = 0; j < VW; ++j)
                    if (f[j] > mx) {
                        mx = f[j];
                        mi = v * VW + j;
                    }
            }
        }
        float sum = 0.f;
#pragma unroll
        for (int q = 0; q < kRegVecs; ++q) {
            const int v = threadIdx.x + q * 256;
            if (v < nv) {
                float f[VW];
                Elem<T>::unpack(raw[q], f);
#pragma unroll
                for (int j = 0; j < VW; ++j) sum += fast_exp(f[j] - mx);
            }
        }
        ms = MaxSum{mx, sum};
        am = ArgMax{mx, mi};
    } else if (vec) {
        for (int v = threadIdx.x; v < nv; v += blockDim.x) {
            float f[VW];
            Elem<T>::unpack(reinterpret_cast<const uint4*>(row)[v], f);
#pragma unroll
            for (int j = 0; j < VW; ++j) visit(f[j], v * VW + j);
        }
        for (int i = nv * VW + threadIdx.x; i < V; i += blockDim.x) visit(Elem<T>::load(row + i), i);
    } else {
        for (int i = threadIdx.x; i < V; i += blockDim.x) visit(Elem<T>::load(row + i), i);
    }
    // wave reduction (fixed butterfly order), then the 4 waves in order
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        MaxSum o{__shfl_xor(ms.m, off, 64), __shfl_xor(ms.s, off, 64)};
        ArgMax p{__shfl_xor(am.v, off, 64), __shfl_xor(am.i, off, 64)};
        ms = ms_merge(ms, o);
        am = am_merge(am, p);
    }
    const int wave = threadIdx.x >> 6;
    if (lane_id() == 0) {
        s_ms[wave] = ms;
        s_am[wave] = am;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        MaxSum a = s_ms[0];
        ArgMax b = s_am[0];
        for (int w = 1; w < 4; ++w) {
            a = ms_merge(a, s_ms[w]);
            b = am_merge(b, s_am[w]);
        }
        const float l = a.m + logf(a.s);
        float tok = l - Elem<T>::load(row + label);
        if (isnan(tok) || isinf(tok)) tok = 10.0f;   // fused_loss.cu:121-124
        loss[t] = tok;
        lse[t] = l;
        correct[t] = b.i == (int)label ? 1.f : 0.f;
        valid[t] = 1.f;
    }
}

// sums[0] = sum w*loss, sums[1] = sum w (valid tokens), sums[2] = sum loss, sums[3] = sum correct,
// sums[4] = number of valid tokens; w = weights[t] (1 when weights == NULL).  Single block, fixed order.
__global__ __launch_bounds__(1024) void cross_entropy_sums_kernel(const float* __restrict__ loss,
                                                                 const float* __restrict__ correct,
                                                                 const float* __restrict__ valid,
                                                                 const float* __restrict__ weights, int64_t Tn,
                                                                 float* __restrict__ sums) {
    __shared__ float part[5][1024];
    float a[5] = {0.f, 0.f, 0.f, 0.f, 0.f};
    for (int64_t t = threadIdx.x; t < Tn; t += 1024) {
        const float v = valid[t];
        const float w = weights ? weights[t] * v : v;
        a[0] += w * loss[t];
        a[1] += w;
        a[2] += loss[t];
        a[3] += correct[t];
        a[4] += v;
    }
#pragma unroll
    for (int q = 0; q < 5; ++q) part[q][threadIdx.x] = a[q];
    __syncthreads();
    for (int stride = 512; stride > 0; stride >>= 1) {
        if ((int)threadIdx.x < stride) {
#pragma unroll
            for (int q = 0; q < 5; ++q) part[q][threadIdx.x] += part[q][threadIdx.x + stride];
        }
        __syncthreads();
    }
    if (threadIdx.x < 5) sums[threadIdx.x] = part[threadIdx.x][0];
}

// dlogits[t, v] = g_t * (exp(z - lse_t) - [v == label_t]),  g_t = scale[0] * w_t * valid_t / max(sums[1], 1e-8)
// (gradient of  sum_t w_t loss_t / sum_t w_t; scale[0] = upstream gradient of that mean).
template <typename T>
__global__ __launch_bounds__(256) void cross_entropy_bwd_kernel(const T* __restrict__ logits,
                                                                const int64_t* __restrict__ labels,
                                                                const float* __restrict__ lse,
                                                                const float* __restrict__ valid,
                                                                const float* __restrict__ weights,
                                                                const float* __restrict__ sums,
                                                                const float* __restrict__ scale,
                                                                T* __restrict__ dlogits, int V, bool vec) {
    constexpr int VW = Elem<T>::kVec;
    const int64_t t = blockIdx.x;
    const T* row = logits + t * V;
    T* out = dlogits + t * V;
    const float v = valid[t];
    const float g = v == 0.f ? 0.f : scale[0] * (weights ? weights[t] : 1.f) / fmaxf(sums[1], 1e-8f);
    const float l = lse[t];
    const int label = v == 0.f ? -1 : (int)labels[t];
    if (vec) {
        const int nv = V / VW;
        for (int i = threadIdx.x; i < nv; i += blockDim.x) {
            float f[VW];
            Elem<T>::unpack(reinterpret_cast<const uint4*>(row)[i], f);
#pragma unroll
            for (int j = 0; j < VW; ++j) {
                const float p = g == 0.f ? 0.f : fast_exp(f[j] - l);
                f[j] = g * (p - ((i * VW + j) == label ? 1.f : 0.f));
            }
            reinterpret_cast<uint4*>(out)[i] = Elem<T>::pack(f);
        }
        for (int i = nv * VW + threadIdx.x; i < V; i += blockDim.x) {
            const float p = g == 0.f ? 0.f : expf(Elem<T>::load(row + i) - l);
            Elem<T>::store(out + i, g * (p - (i == label ? 1.f : 0.f)));
        }
    } else {
        for (int i = threadIdx.x; i < V; i += blockDim.x) {
            const float p = g == 0.f ? 0.f : expf(Elem<T>::load(row + i) - l);
            Elem<T>::store(out + i, g * (p - (i == label ? 1.f : 0.f)));
        }
    }
}

// ---------------------------------------------------------------- gradient norm and clipping
// The tensors are cut into chunks of kClipChunk elements; chunk c belongs to the tensor whose
// chunk_start[] range contains c (chunk_start has n_tensors + 1 entries, built on the host).
constexpr int kClipChunk = 262144;

__device__ __forceinline__ int find_tensor(const int32_t* __restrict__ chunk_start, int n, int c) {
    int lo = 0, hi = n - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (chunk_start[mid] <= c) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

template <typename T>
__global__ __launch_bounds__(256) void grad_sumsq_kernel(const void* const* __restrict__ ptrs,
                                                         const int64_t* __restrict__ sizes,
                                                         const int32_t* __restrict__ chunk_start, int n_tensors,
                                                         float* __restrict__ partial) {
    __shared__ float s_part[4];
    const int c = blockIdx.x;
    const int ti = find_tensor(chunk_start, n_tensors, c);
    const T* g = static_cast<const T*>(ptrs[ti]);
    const int64_t begin = (int64_t)(c - chunk_start[ti]) * kClipChunk;
    const int64_t end = begin + kClipChunk < sizes[ti] ? begin + kClipChunk : sizes[ti];
    float acc = 0.f;
    constexpr int VW = Elem<T>::kVec;
    if ((reinterpret_cast<uintptr_t>(g) & 15u) == 0) {
        const int64_t nv = (end - begin) / VW;
        const uint4* gv = reinterpret_cast<const uint4*>(g + begin);
        for (int64_t i = threadIdx.x; i < nv; i += 256) {
            float f[VW];
            Elem<T>::unpack(gv[i], f);
#pragma unroll
            for (int j = 0; j < VW; ++j) acc += f[j] * f[j];
        }
        for (int64_t i = begin + nv * VW + threadIdx.x; i < end; i += 256) {
            const float f = Elem<T>::load(g + i);
            acc += f * f;
        }
    } else {
        for (int64_t i = begin + threadIdx.x; i < end; i += 256) {
            const float f = Elem<T>::load(g + i);
            acc += f * f;
        }
    }
    acc = wave_sum(acc);
    if (lane_id() == 0) s_part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) partial[c] = ((s_part[0] + s_part[1]) + s_part[2]) + s_part[3];
}

// norm_out[0] = sqrt(extra_sumsq + sum of the partials, in index order); norm_out[1] = that sum of squares.
__global__ __launch_bounds__(256) void grad_norm_finish_kernel(const float* __restrict__ partial, int n,
                                                               const float* __restrict__ extra_sumsq,
                                                               float* __restrict__ norm_out) {
    __shared__ float s[256];
    float acc = 0.f;
    for (int i = threadIdx.x; i < n; i += 256) acc += partial[i];
    s[threadIdx.x] = acc;
    __syncthreads();
    for (int stride = 128; stride > 0; stride >>= 1) {
        if ((int)threadIdx.x < stride) s[threadIdx.x] += s[threadIdx.x + stride];
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const float total = s[0] + (extra_sumsq ? extra_sumsq[0] : 0.f);
        norm_out[1] = total;
        norm_out[0] = sqrtf(total);
    }
}

// grads *= max_norm / (norm + 1e-6) when that factor is below 1 (fused_grad_clip.cu:66-91).
template <typename T>
__global__ __launch_bounds__(256) void grad_scale_kernel(void* const* __restrict__ ptrs,
                                                         const int64_t* __restrict__ sizes,
                                                         const int32_t* __restrict__ chunk_start, int n_tensors,
                                                         const float* __restrict__ norm, float max_norm) {
    const float coef = max_norm / (norm[0] + 1e-6f);
    if (!(coef < 1.0f)) return;
    const int c = blockIdx.x;
    const int ti = find_tensor(chunk_start, n_tensors, c);
    T* g = static_cast<T*>(ptrs[ti]);
    const int64_t begin = (int64_t)(c - chunk_start[ti]) * kClipChunk;
    const int64_t end = begin + kClipChunk < sizes[ti] ? begin + kClipChunk : sizes[ti];
    constexpr int VW = Elem<T>::kVec;
    if ((reinterpret_cast<uintptr_t>(g) & 15u) == 0) {
        const int64_t nv = (end - begin) / VW;
        uint4* gv = reinterpret_cast<uint4*>(g + begin);
        for (int64_t i = threadIdx.x; i < nv; i += 256) {
            float f[VW];
            Elem<T>::unpack(gv[i], f);
#pragma unroll
            for (int j = 0; j < VW; ++j) f[j] *= coef;
            gv[i] = Elem<T>::pack(f);
        }
        for (int64_t i = begin + nv * VW + threadIdx.x; i < end; i += 256) Elem<T>::store(g + i, Elem<T>::load(g + i) * coef);
    } else {
        for (int64_t i = begin + threadIdx.x; i < end; i += 256) Elem<T>::store(g + i, Elem<T>::load(g + i) * coef);
    }
}

}  // namespace ats

extern "C" int ats_cross_entropy_fwd(const void* logits, const int64_t* labels, int64_t pad_id, const float* weights,
                                     float* loss_tok, float* lse, float* correct, float* valid, float* sums, int64_t T,
                                     int V, int dtype, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(T >= 0 && T <= 0x7fffffffLL && V > 0, ATS_ERR_INVALID_ARG, "ats_cross_entropy_fwd: T=%lld V=%d", (long long)T, V);
    ATS_REQUIRE(dtype == ATS_F32 || dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "ats_cross_entropy_fwd: dtype tag %d", dtype);
    ATS_REQUIRE(sums && (T == 0 || (logits && labels && loss_tok && lse && correct && valid)), ATS_ERR_INVALID_ARG,
                "ats_cross_entropy_fwd: null pointer");
    hipStream_t s = as_stream(stream);
    const int VW = dtype == ATS_F32 ? 4 : 8;
    const bool vec = aligned16(logits) && V % VW == 0;
    if (T > 0) {
        if (dtype == ATS_F32)
            hipLaunchKernelGGL((cross_entropy_fwd_kernel<float>), dim3((unsigned)T), dim3(256), 0, s,
                               static_cast<const float*>(logits), labels, pad_id, loss_tok, lse, correct, valid, V, vec);
        else
            hipLaunchKernelGGL((cross_entropy_fwd_kernel<bf16_t>), dim3((unsigned)T), dim3(256), 0, s,
                               static_cast<const bf16_t*>(logits), labels, pad_id, loss_tok, lse, correct, valid, V, vec);
    }
    hipLaunchKernelGGL(cross_entropy_sums_kernel, dim3(1), dim3(1024), 0, s, loss_tok, correct, valid, weights, T, sums);
    ATS_CHECK_LAUNCH("ats_cross_entropy_fwd");
    return ATS_OK;
}

extern "C" int ats_cross_entropy_bwd(const void* logits, const int64_t* labels, const float* lse, const float* valid,
                                     const float* weights, const float* sums, const float* scale, void* dlogits,
                                     int64_t T, int V, int dtype, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(T >= 0 && T <= 0x7fffffffLL && V > 0, ATS_ERR_INVALID_ARG, "ats_cross_entropy_bwd: T=%lld V=%d", (long long)T, V);
    ATS_REQUIRE(dtype == ATS_F32 || dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "ats_cross_entropy_bwd: dtype tag %d", dtype);
    if (T == 0) return ATS_OK;
    ATS_REQUIRE(logits && labels && lse && valid && sums && scale && dlogits, ATS_ERR_INVALID_ARG,
                "ats_cross_entropy_bwd: null pointer");
    const int VW = dtype == ATS_F32 ? 4 : 8;
    const bool vec = aligned16(logits) && aligned16(dlogits) && V % VW == 0;
    if (dtype == ATS_F32)
        hipLaunchKernelGGL((cross_entropy_bwd_kernel<float>), dim3((unsigned)T), dim3(256), 0, as_stream(stream),
                           static_cast<const float*>(logits), labels, lse, valid, weights, sums, scale,
                           static_cast<float*>(dlogits), V, vec);
    else
        hipLaunchKernelGGL((cross_entropy_bwd_kernel<bf16_t>), dim3((unsigned)T), dim3(256), 0, as_stream(stream),
                           static_cast<const bf16_t*>(logits), labels, lse, valid, weights, sums, scale,
                           static_cast<bf16_t*>(dlogits), V, vec);
    ATS_CHECK_LAUNCH("ats_cross_entropy_bwd");
    return ATS_OK;
}

extern "C" int ats_grad_clip_chunk_elems(void) { return ats::kClipChunk; }

extern "C" int ats_grad_norm_clip(void* const* grad_ptrs, const int64_t* sizes, const int32_t* chunk_start,
                                  int n_tensors, int n_chunks, int dtype, const float* extra_sumsq, float* partial,
                                  float* norm_out, float max_norm, int do_clip, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(n_tensors >= 0 && n_chunks >= 0, ATS_ERR_INVALID_ARG, "ats_grad_norm_clip: n_tensors=%d n_chunks=%d",
                n_tensors, n_chunks);
    ATS_REQUIRE(dtype == ATS_F32 || dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "ats_grad_norm_clip: dtype tag %d", dtype);
    ATS_REQUIRE(norm_out && (n_chunks == 0 || (grad_ptrs && sizes && chunk_start && partial)), ATS_ERR_INVALID_ARG,
                "ats_grad_norm_clip: null pointer");
    hipStream_t s = as_stream(stream);
    if (do_clip == 2) {   // scale only: norm_out already holds the norm over all groups
        if (n_chunks > 0) {
            if (dtype == ATS_F32)
                hipLaunchKernelGGL((grad_scale_kernel<float>), dim3((unsigned)n_chunks), dim3(256), 0, s, grad_ptrs, sizes,
                                   chunk_start, n_tensors, norm_out, max_norm);
            else
                hipLaunchKernelGGL((grad_scale_kernel<bf16_t>), dim3((unsigned)n_chunks), dim3(256), 0, s, grad_ptrs, sizes,
                                   chunk_start, n_tensors, norm_out, max_norm);
        }
        ATS_CHECK_LAUNCH("ats_grad_norm_clip");
        return ATS_OK;
    }
    if (n_chunks > 0) {
        if (dtype == ATS_F32)
            hipLaunchKernelGGL((grad_sumsq_kernel<float>), dim3((unsigned)n_chunks), dim3(256), 0, s,
                               reinterpret_cast<const void* const*>(grad_ptrs), sizes, chunk_start, n_tensors, partial);
        else
            hipLaunchKernelGGL((grad_sumsq_kernel<bf16_t>), dim3((unsigned)n_chunks), dim3(256), 0, s,
                               reinterpret_cast<const void* const*>(grad_ptrs), sizes, chunk_start, n_tensors, partial);
    }
    hipLaunchKernelGGL(grad_norm_finish_kernel, dim3(1), dim3(256), 0, s, partial, n_chunks, extra_sumsq, norm_out);
    if (do_clip == 1 && n_chunks > 0) {
        if (dtype == ATS_F32)
            hipLaunchKernelGGL((grad_scale_kernel<float>), dim3((unsigned)n_chunks), dim3(256), 0, s, grad_ptrs, sizes,
                               chunk_start, n_tensors, norm_out, max_norm);
        else
            hipLaunchKernelGGL((grad_scale_kernel<bf16_t>), dim3((unsigned)n_chunks), dim3(256), 0, s, grad_ptrs, sizes,
                               chunk_start, n_tensors, norm_out, max_norm);
    }
    ATS_CHECK_LAUNCH("ats_grad_norm_clip");
    return ATS_OK;
}
