// Row softmax of materialised float32 attention scores, forward and backward.
//
// Float32 inputs take the route the reference's _standard_attention takes
// (Src/Main_Scripts/core/model.py:807-839): scores = q.k^T as a matrix per (batch, head), a row softmax, then
// weights.v -- here with the products on the float32 grouped GEMM kernels and the two passes below in between.
// The forward pass applies, in the reference's order, the scale, the causal fill with -1e4 (model.py:813-817),
// the additive (1 - mask) * -1e4 terms of a [B, Lk] or [B, 1, L, Lk] mask (819-824), the float32 softmax
// (827-829) and dropout on the weights (831-833, decisions by the hash of attention_extra.hpp).  The backward
// pass turns dP into dS = P * (dP' - sum_j P dP') * scale with dP' = keep * dP / (1 - p).
// One wave per row; a row is read three times at most (it stays in the XCD's L2).
#include <math.h>

#include "ats_common.hpp"
#include "attention_extra.hpp"

namespace ats {

// scores: [B * Hq, Lp, ld] (row r of head e at (e * Lp + r) * ld), raw q.k^T.  Columns >= Lk and rows >= L are
// padding: they are written as zeros.  weights_drop (optional, same layout): the weights after dropout.
__global__ __launch_bounds__(256) void attention_softmax_f32_kernel(float* __restrict__ scores, float* __restrict__ weights_drop,
                                                                    int Hq, int L, int Lp, int Lk, int ld, float scale,
                                                                    const float* __restrict__ key_bias, AttnExtra ex,
                                                                    int64_t n_rows) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);     // over [B * Hq, Lp]
    if (row >= n_rows) return;
    const int64_t e = row / Lp;
    const int i = (int)(row - e * Lp);
    const int b = (int)(e / Hq);
    float* srow = scores + row * ld;
    float* drow = weights_drop ? weights_drop + row * ld : nullptr;
    if (i >= L) {
        for (int j = lane; j < ld; j += 64) {
            srow[j] = 0.f;
            if (drow) drow[j] = 0.f;
        }
        return;
    }
    const int last_key = i + (Lk - L);      // keys after it are the query's future
    const float* kb = key_bias ? key_bias + (int64_t)b * Lk : nullptr;
    const float* pb = ex.bias_qk ? ex.bias_qk + (int64_t)b * ex.bias_sb + (int64_t)(e % Hq) * ex.bias_sh + (int64_t)i * Lk : nullptr;
    auto value = [&](int j) {
        float t = j > last_key ? -1e4f : srow[j] * scale;
        if (kb) t += kb[j];
        if (pb) t += pb[j];
        return t;
    };
    float mx = -INFINITY;
    for (int j = lane; j < Lk; j += 64) mx = fmaxf(mx, value(j));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    float sum = 0.f;
    for (int j = lane; j < Lk; j += 64) sum += expf(value(j) - mx);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
    const float inv = 1.0f / sum;
    const bool drop = ex.keep_scale > 0.f;
    const uint32_t head_key = attn_head_key(ex.seed_lo, ex.seed_hi, (uint32_t)e);
    for (int j = lane; j < ld; j += 64) {
        const float p = j < Lk ? expf(value(j) - mx) * inv : 0.f;
        srow[j] = p;
        if (drow) {
            const bool keep = !drop || attn_drop_hash(head_key, (uint32_t)i * (uint32_t)Lk + (uint32_t)j) >= ex.drop_threshold;
            drow[j] = (j < Lk && keep) ? p * (drop ? ex.keep_scale : 1.0f) : 0.f;
        }
    }
}

// weights: the undropped softmax output of the forward; dp: gradient of the dropped weights, overwritten with
// the gradient of the raw scores (q.k^T).
__global__ __launch_bounds__(256) void attention_softmax_bwd_f32_kernel(const float* __restrict__ weights, float* __restrict__ dp,
                                                                        int Hq, int L, int Lp, int Lk, int ld, float scale,
                                                                        AttnExtra ex, int64_t n_rows) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const int64_t e = row / Lp;
    const int i = (int)(row - e * Lp);
    const float* prow = weights + row * ld;
    float* grow = dp + row * ld;
    if (i >= L) {
        for (int j = lane; j < ld; j += 64) grow[j] = 0.f;
        return;
    }
    const bool drop = ex.keep_scale > 0.f;
    const uint32_t head_key = attn_head_key(ex.seed_lo, ex.seed_hi, (uint32_t)e);
    auto dweight = [&](int j) {
        float g = grow[j];
        if (drop)
            g = attn_drop_hash(head_key, (uint32_t)i * (uint32_t)Lk + (uint32_t)j) >= ex.drop_threshold ? g * ex.keep_scale : 0.f;
        return g;
    };
    float dot = 0.f;
    for (int j = lane; j < Lk; j += 64) dot += prow[j] * dweight(j);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) dot += __shfl_xor(dot, o, 64);
    for (int j = lane; j < ld; j += 64) grow[j] = j < Lk ? prow[j] * (dweight(j) - dot) * scale : 0.f;
}

}  // namespace ats

extern "C" int ats_attention_softmax_f32(float* scores, float* weights_drop, int B, int Hq, int L, int Lp, int Lk, int ld,
                                         float scale, const float* key_bias, const float* bias_qk, int64_t bias_sb,
                                         int64_t bias_sh, float dropout_p, uint64_t dropout_seed, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(B >= 0 && Hq > 0 && L >= 0 && Lp >= L && Lk >= L && ld >= Lk && scale > 0.f, ATS_ERR_INVALID_ARG,
                "ats_attention_softmax_f32: B=%d Hq=%d L=%d Lp=%d Lk=%d ld=%d scale=%g", B, Hq, L, Lp, Lk, ld, scale);
    if (B == 0 || Lp == 0) return ATS_OK;
    AttnExtra ex;
    bool extras = false;
    if (!make_attention_extra("ats_attention_softmax_f32", bias_qk, bias_sb, bias_sh, dropout_p, dropout_seed, L, Lk, &ex, &extras))
        return ATS_ERR_INVALID_ARG;
    ATS_REQUIRE(scores && (dropout_p == 0.f || weights_drop), ATS_ERR_INVALID_ARG,
                "ats_attention_softmax_f32: null pointer (dropout needs the second output)");
    const int64_t n_rows = (int64_t)B * Hq * Lp;
    ATS_REQUIRE((n_rows + 3) / 4 <= 0x7fffffff, ATS_ERR_UNSUPPORTED, "ats_attention_softmax_f32: %lld rows", (long long)n_rows);
    hipLaunchKernelGGL(attention_softmax_f32_kernel, dim3((unsigned)((n_rows + 3) / 4)), dim3(256), 0, as_stream(stream),
                       scores, weights_drop, Hq, L, Lp, Lk, ld, scale, key_bias, ex, n_rows);
    ATS_CHECK_LAUNCH("ats_attention_softmax_f32");
    return ATS_OK;
}

extern "C" int ats_attention_softmax_bwd_f32(const float* weights, float* dp, int B, int Hq, int L, int Lp, int Lk, int ld,
                                             float scale, float dropout_p, uint64_t dropout_seed, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(B >= 0 && Hq > 0 && L >= 0 && Lp >= L && Lk >= L && ld >= Lk && scale > 0.f, ATS_ERR_INVALID_ARG,
                "ats_attention_softmax_bwd_f32: B=%d Hq=%d L=%d Lp=%d Lk=%d ld=%d scale=%g", B, Hq, L, Lp, Lk, ld, scale);
    if (B == 0 || Lp == 0) return ATS_OK;
    AttnExtra ex;
    bool extras = false;
    if (!make_attention_extra("ats_attention_softmax_bwd_f32", nullptr, 0, 0, dropout_p, dropout_seed, L, Lk, &ex, &extras))
        return ATS_ERR_INVALID_ARG;
    ATS_REQUIRE(weights && dp, ATS_ERR_INVALID_ARG, "ats_attention_softmax_bwd_f32: null pointer");
    const int64_t n_rows = (int64_t)B * Hq * Lp;
    ATS_REQUIRE((n_rows + 3) / 4 <= 0x7fffffff, ATS_ERR_UNSUPPORTED, "ats_attention_softmax_bwd_f32: %lld rows",
                (long long)n_rows);
    hipLaunchKernelGGL(attention_softmax_bwd_f32_kernel, dim3((unsigned)((n_rows + 3) / 4)), dim3(256), 0, as_stream(stream),
                       weights, dp, Hq, L, Lp, Lk, ld, scale, ex, n_rows);
    ATS_CHECK_LAUNCH("ats_attention_softmax_bwd_f32");
    return ATS_OK;
}
